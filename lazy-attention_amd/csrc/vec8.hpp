// Eight consecutive elements of a row as registers: 16-byte loads and stores (two for float),
// conversion to and from float.  Shared by the byte-shuffling kernels.
#pragma once
#include "common.hpp"

namespace lazyattn {

template <typename T> struct Vec8;                 // 8 consecutive elements
template <> struct Vec8<bf16_t> {
    uint4 v;
    __device__ void load(const bf16_t *p) { v = *reinterpret_cast<const uint4 *>(p); }
    __device__ void store(bf16_t *p) const { *reinterpret_cast<uint4 *>(p) = v; }
    __device__ void get(float *f) const {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { f[2 * i] = __uint_as_float(w[i] << 16); f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
    }
    __device__ void set(const float *f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bf16_t a = __float2bfloat16(f[2 * i]), b = __float2bfloat16(f[2 * i + 1]);
            w[i] = (uint32_t)*reinterpret_cast<const uint16_t *>(&a) | ((uint32_t)*reinterpret_cast<const uint16_t *>(&b) << 16);
        }
        v = make_uint4(w[0], w[1], w[2], w[3]);
    }
};
template <> struct Vec8<f16_t> {
    uint4 v;
    __device__ void load(const f16_t *p) { v = *reinterpret_cast<const uint4 *>(p); }
    __device__ void store(f16_t *p) const { *reinterpret_cast<uint4 *>(p) = v; }
    __device__ void get(float *f) const {
        const f16_t *h = reinterpret_cast<const f16_t *>(&v);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = __half2float(h[i]);
    }
    __device__ void set(const float *f) {
        f16_t *h = reinterpret_cast<f16_t *>(&v);
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = __float2half(f[i]);
    }
};
template <> struct Vec8<float> {
    float4 a, b;
    __device__ void load(const float *p) { a = *reinterpret_cast<const float4 *>(p); b = *reinterpret_cast<const float4 *>(p + 4); }
    __device__ void store(float *p) const { *reinterpret_cast<float4 *>(p) = a; *reinterpret_cast<float4 *>(p + 4) = b; }
    __device__ void get(float *f) const { f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w; }
    __device__ void set(const float *f) { a = make_float4(f[0], f[1], f[2], f[3]); b = make_float4(f[4], f[5], f[6], f[7]); }
};

}  // namespace lazyattn
