// The two 16-bit element types of the matrix kernels (bf16, float16): conversions, packing and the MFMA
// variants, so that a kernel is written once over `Elem<T>`.
#pragma once
#include "common.hpp"

namespace lazyattn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;

// Values travel as 32-bit words holding two elements; `mfma` is v_mfma_f32_32x32x16_{bf16,f16} and `mfma16`
// v_mfma_f32_16x16x32_{bf16,f16}, on 8-element operands given as four such words.
template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
    // largest P = 2^REBASE between two moves of the softmax reference: anything bf16's exponent carries
    static constexpr float REBASE = 16.f;
    // a lane's sum of 16 probabilities above this means some P is far from 1: time to move the reference
    // (2^40: decades below what bf16 and the fp32 sums hold)
    static constexpr float SUM_LIMIT = 1099511627776.f;
    static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        f32x2_t f = {a, b};
        bf16x2_t h = __builtin_convertvector(f, bf16x2_t);   // v_cvt_pk_bf16_f32, RNE
        return *reinterpret_cast<uint32_t *>(&h);
    }
    static __device__ __forceinline__ uint32_t splat(float w) { const uint32_t u = __float_as_uint(w) >> 16; return u | (u << 16); }
    // acc + lo(w) + hi(w) (v_dot2c_f32_bf16 against (1, 1))
    static __device__ __forceinline__ float dot2_ones(uint32_t w, float acc) {
        const uint32_t one = 0x3f803f80u;
        return __builtin_amdgcn_fdot2_f32_bf16(*reinterpret_cast<const bf16x2_t *>(&w),
                                               *reinterpret_cast<const bf16x2_t *>(&one), acc, false);
    }
    static __device__ __forceinline__ f32x16_t mfma(const uint4 &a, const uint4 &b, const f32x16_t &c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8_t *>(&a),
                                                       *reinterpret_cast<const bf16x8_t *>(&b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t mfma16(const uint4 &a, const uint4 &b, const f32x4_t &c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8_t *>(&a),
                                                       *reinterpret_cast<const bf16x8_t *>(&b), c, 0, 0, 0);
    }
};
template <> struct Elem<f16_t> {
    static constexpr float REBASE = 8.f;                      // P <= 256: far inside the half range
    static constexpr float SUM_LIMIT = 4096.f;                // every P below 2^12 then, the half range ends at 65504
    static __device__ __forceinline__ float lo(uint32_t w) { return (float)(*reinterpret_cast<const f16x2_t *>(&w))[0]; }
    static __device__ __forceinline__ float hi(uint32_t w) { return (float)(*reinterpret_cast<const f16x2_t *>(&w))[1]; }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        f32x2_t f = {a, b};
        f16x2_t h = __builtin_convertvector(f, f16x2_t);     // RNE
        return *reinterpret_cast<uint32_t *>(&h);
    }
    static __device__ __forceinline__ uint32_t splat(float w) { return pack(w, w); }
    static __device__ __forceinline__ float dot2_ones(uint32_t w, float acc) {
        const uint32_t one = 0x3c003c00u;
        return __builtin_amdgcn_fdot2(*reinterpret_cast<const f16x2_t *>(&w), *reinterpret_cast<const f16x2_t *>(&one), acc, false);
    }
    static __device__ __forceinline__ f32x16_t mfma(const uint4 &a, const uint4 &b, const f32x16_t &c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const f16x8_t *>(&a),
                                                      *reinterpret_cast<const f16x8_t *>(&b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t mfma16(const uint4 &a, const uint4 &b, const f32x4_t &c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const f16x8_t *>(&a),
                                                      *reinterpret_cast<const f16x8_t *>(&b), c, 0, 0, 0);
    }
};

}  // namespace lazyattn
