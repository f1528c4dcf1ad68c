// Shared device helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/lazyattn.h"

namespace lazyattn {

// Compute units of the caller's current device, asked once per device (the launch heuristics fill whole rounds of
// them).  256 -- an MI355X in its single-partition mode -- when no device can be asked.
int device_cus();

using bf16_t = __hip_bfloat16;
using f16_t = __half;
struct fp8e4m3_t { uint8_t v; };
struct fp8e5m2_t { uint8_t v; };

// ---- element <-> float -------------------------------------------------------
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return __bfloat162float(x); }
__device__ __forceinline__ float to_f32(f16_t x) { return __half2float(x); }
__device__ __forceinline__ float to_f32(fp8e4m3_t x) {
    // OCP e4m3fn: 1-4-3, bias 7, no inf, S.1111.111 = NaN
    const uint32_t s = x.v >> 7, e = (x.v >> 3) & 0xF, m = x.v & 7;
    float r;
    if (e == 0) r = (float)m * 0.001953125f;                 // m * 2^-9
    else if (e == 15 && m == 7) r = __builtin_nanf("");
    else r = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return s ? -r : r;
}
__device__ __forceinline__ float to_f32(fp8e5m2_t x) {
    // e5m2 is the top byte of an IEEE half
    return __half2float(__ushort_as_half((unsigned short)(x.v << 8)));
}

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return __float2bfloat16(x); }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float x) { return __float2half(x); }

// value of x after a round trip through T (models `.to(q.dtype)`)
template <typename T> __device__ __forceinline__ float round_to(float x) {
    return to_f32(from_f32<T>(x));
}

__device__ __forceinline__ int64_t load_index(const void *p, int64_t i, int bits) {
    return bits == 64 ? ((const int64_t *)p)[i] : (int64_t)((const int32_t *)p)[i];
}
// the same for entries known to be non-negative (offsets, lengths): a 32-bit entry is zero-extended, which pairs
// it with a zero register instead of computing on the loaded value
__device__ __forceinline__ int64_t load_index_nonneg(const void *p, int64_t i, int bits) {
    return bits == 64 ? ((const int64_t *)p)[i] : (int64_t)(uint32_t)((const int32_t *)p)[i];
}

// The low 32 bits of a wave-uniform entry below 2^31 (token offsets, lengths) as one scalar load, with no branch
// on the width: several of these in a row are in flight together, where load_index() compiles to a vector load
// and a wait per call.
__device__ __forceinline__ int64_t load_index_uniform(const void *p, int64_t i, int bits) {
    typedef const uint32_t __attribute__((address_space(4))) *sptr_u32;
    const char *a = (const char *)p + i * (int64_t)(bits >> 3);
    return (int64_t)*(sptr_u32)(const void *)a;
}

}  // namespace lazyattn
