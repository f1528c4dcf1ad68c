// The step before the attention call, fused: NeoX rotary embedding of the new tokens' Q (and K,
// when the cache convention stores rotated keys) in place, and the scatter of K and V into
// the paged caches, in one launch.
//
// Replaces, for this path,
//   * the Q-only rotary of the un-rotated-cache variant (rotary_embedding.py:67-94, which
//     calls the third-party op rotary_embedding(positions, query, None, head_size,
//     cos_sin_cache, is_neox)), or the Q and K rotary of the other variant (:48-49);
//   * PagedAttention.write_to_paged_cache(key, value, key_cache, value_cache, slot_mapping,
//     kv_cache_dtype, k_scale, v_scale) (backends/triton_attn.py:100-109): token t goes to
//     slot_mapping[t] = block * block_size + offset (negative = skip), K as
//     [block, head, d / x, offset, d % x], V as [block, head, d, offset]; fp8 caches store
//     value / scale, saturated, rounded to e4m3.
// HBM-bound byte shuffling: every operand is touched once, 16 bytes per lane where the
// layouts allow it (everything except the V cache, whose token axis is innermost).
#include "common.hpp"
#include "vec8.hpp"

namespace lazyattn {

namespace {

typedef __attribute__((ext_vector_type(2))) float f32x2_t;

// value / scale -> fp8, saturating, round to nearest even; KIND 1: e4m3 (|x| <= 448), 2: e5m2 (|x| <= 57344).
// A true division (IEEE, as the writer it replaces does: a product with the reciprocal differs in the last
// place for about one value in a thousand); the clamp is NaN-propagating, so a NaN stays a NaN code.
template <int KIND> __device__ __forceinline__ uint8_t to_fp8(float x, float scale) {
    float y = __fdiv_rn(x, scale);
    const float top = KIND == 2 ? 57344.f : 448.f;
    y = __builtin_elementwise_minimum(__builtin_elementwise_maximum(y, -top), top);
    const int w = KIND == 2 ? __builtin_amdgcn_cvt_pk_bf8_f32(y, y, 0, false) : __builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0, false);
    return (uint8_t)(w & 0xff);
}

// Work items.  Per token, 8 elements each:
//   [0, Hq * C)            q chunk pairs   (C = rotary_dim / 16 pairs of 8-element chunks per head)
//   [.., + Hkv * C)        k chunk pairs: rotate (optional) + cache write of both chunks
//   [.., + Hkv * P)        k pass-through chunks (head_dim > rotary_dim): cache write only
// then, per run of RUN = 16 consecutive tokens: Hkv * D items, one (head, d) each, that move the
// run's V column.  The V cache keeps the token axis innermost; when the run fills 16 aligned slots of one
// page in order (the usual case: a prefill chunk is written page by page; pages of 16, 32, ... slots) the
// column is one 32-byte store, otherwise the item falls back to one store per token.
constexpr int RUN = 16;
template <typename T, typename TT, int FP8>
__global__ void __launch_bounds__(256)
rope_cache_write_kernel(const lazyattn_rope_write_params p) {
    const int D = p.head_dim, R = p.rotary_dim, HALF = R / 2;
    const int C = R / 16;                         // chunk pairs per head
    const int P = (D - R) / 8;                    // pass-through chunks per head
    const int n_q = p.num_q_heads * C, n_k = p.num_kv_heads * C, n_kp = p.num_kv_heads * P;
    const int per_token = n_q + n_k + n_kp;
    const int64_t n_tok_items = (int64_t)p.num_tokens * per_token;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    auto slot_of = [&](int64_t tok) -> int64_t {
        return p.slot_mapping ? (p.slot_bits == 64 ? ((const int64_t *)p.slot_mapping)[tok]
                                                   : (int64_t)((const int32_t *)p.slot_mapping)[tok]) : -1;
    };
    constexpr int CSZ = FP8 ? 1 : (int)sizeof(T);
    if (idx >= n_tok_items) {
        // ---- V column of one (run of tokens, head, d) ----
        if (!p.slot_mapping || !p.v_cache) return;
        const int64_t vi = idx - n_tok_items;
        const int per_run = p.num_kv_heads * D;
        const int64_t run = vi / per_run;
        if (run * RUN >= p.num_tokens) return;
        const int h = (int)(vi % per_run) / D, d = (int)(vi % per_run) % D;
        const int64_t t0 = run * RUN;
        const int n = p.num_tokens - t0 < RUN ? (int)(p.num_tokens - t0) : RUN;
        const float v_div = FP8 ? *p.v_scale : 1.f;
        const T *src = (const T *)p.v + t0 * p.v_stride[0] + (int64_t)h * p.v_stride[1] + d;
        const int64_t s0 = slot_of(t0);
        bool page = n == RUN && p.block_size % RUN == 0 && s0 >= 0 && s0 % RUN == 0 && p.vc_stride[3] == 1 &&
                    (((uintptr_t)p.v_cache | (uintptr_t)(p.vc_stride[0] * CSZ) | (uintptr_t)(p.vc_stride[1] * CSZ) |
                      (uintptr_t)(p.vc_stride[2] * CSZ)) & 15) == 0;
        for (int i = 1; page && i < RUN; ++i) page = slot_of(t0 + i) == s0 + i;
        if (page) {
            uint8_t *dst = (uint8_t *)p.v_cache + ((s0 / p.block_size) * p.vc_stride[0] + (int64_t)h * p.vc_stride[1] +
                                               (int64_t)d * p.vc_stride[2] + s0 % p.block_size) * CSZ;
            if (FP8) {
                __attribute__((aligned(16))) uint8_t b[RUN];
#pragma unroll
                for (int i = 0; i < RUN; ++i) b[i] = to_fp8<FP8 ? FP8 : 1>(to_f32(src[i * p.v_stride[0]]), v_div);
                *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(b);
            } else {
                __attribute__((aligned(16))) T col[RUN];
#pragma unroll
                for (int i = 0; i < RUN; ++i) col[i] = src[i * p.v_stride[0]];
                if (sizeof(T) == 2) {
                    reinterpret_cast<uint4 *>(dst)[0] = reinterpret_cast<const uint4 *>(col)[0];
                    reinterpret_cast<uint4 *>(dst)[1] = reinterpret_cast<const uint4 *>(col)[1];
                } else {
#pragma unroll
                    for (int i = 0; i < RUN * (int)sizeof(T) / 16; ++i)
                        reinterpret_cast<uint4 *>(dst)[i] = reinterpret_cast<const uint4 *>(col)[i];
                }
            }
            return;
        }
        for (int i = 0; i < n; ++i) {
            const int64_t sl = slot_of(t0 + i);
            if (sl < 0) continue;
            const int64_t o0 = (sl / p.block_size) * p.vc_stride[0] + (int64_t)h * p.vc_stride[1] + (int64_t)d * p.vc_stride[2] +
                               (sl % p.block_size) * p.vc_stride[3];
            if (FP8) ((uint8_t *)p.v_cache)[o0] = to_fp8<FP8 ? FP8 : 1>(to_f32(src[i * p.v_stride[0]]), v_div);
            else ((T *)p.v_cache)[o0] = src[i * p.v_stride[0]];
        }
        return;
    }
    const int64_t t = idx / per_token;
    int it = (int)(idx % per_token);

    const int64_t slot = slot_of(t);
    const bool write = slot >= 0 && p.k_cache != nullptr;
    const int64_t blk = write ? slot / p.block_size : 0;
    const int off = write ? (int)(slot % p.block_size) : 0;
    const float k_div = FP8 ? *p.k_scale : 1.f;

    // K chunk (8 consecutive d starting at d0) of head h -> [block, head, d / x, offset, d % x]
    auto put_k = [&](int h, int d0, const float *f, const Vec8<T> &raw) {
        uint8_t *dst = (uint8_t *)p.k_cache +
                       (blk * p.kc_stride[0] + (int64_t)h * p.kc_stride[1] + (int64_t)(d0 / p.x) * p.kc_stride[2] +
                        (int64_t)off * p.kc_stride[3] + (d0 % p.x)) * CSZ;
        if (FP8) {
            uint8_t b[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) b[i] = to_fp8<FP8 ? FP8 : 1>(f[i], k_div);
            *reinterpret_cast<uint2 *>(dst) = *reinterpret_cast<const uint2 *>(b);
        } else if (p.x % 8 == 0) {
            raw.store(reinterpret_cast<T *>(dst));
        } else {                                   // x = 4 (fp32 caches): two groups of four
            T tmp[8];
            Vec8<T> r = raw;
            r.store(tmp);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int d = d0 + i;
                ((T *)p.k_cache)[blk * p.kc_stride[0] + (int64_t)h * p.kc_stride[1] + (int64_t)(d / p.x) * p.kc_stride[2] +
                                 (int64_t)off * p.kc_stride[3] + (d % p.x)] = tmp[i];
            }
        }
    };

    if (it < n_q + n_k) {
        // ---- rotary chunk pair: elements d0..d0+7 and d0+HALF.. of one head ----
        const bool is_k = it >= n_q;
        if (is_k) it -= n_q;
        const int h = it / C, c = it % C, d0 = c * 8;
        T *base = is_k ? (T *)p.k + t * p.k_stride[0] + (int64_t)h * p.k_stride[1]
                       : (T *)p.q + t * p.q_stride[0] + (int64_t)h * p.q_stride[1];
        const bool rot = is_k ? p.rotate_k != 0 : p.rotate_q != 0;
        if (!rot && !(is_k && write)) return;
        Vec8<T> lo, hi;
        lo.load(base + d0);
        hi.load(base + d0 + HALF);
        float a[8], b[8];
        lo.get(a);
        hi.get(b);
        if (rot) {
            const int64_t pos = p.pos_bits == 64 ? ((const int64_t *)p.positions)[t] : (int64_t)((const int32_t *)p.positions)[t];
            const TT *row = (const TT *)p.cos_sin_cache + pos * p.table_stride;
            Vec8<TT> cv, sv;
            cv.load(row + d0);
            sv.load(row + HALF + d0);
            float cs[8], sn[8], x[8], y[8];
            cv.get(cs);
            sv.get(sn);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[e] = a[e] * cs[e] - b[e] * sn[e];
                y[e] = b[e] * cs[e] + a[e] * sn[e];
            }
            lo.set(x);
            hi.set(y);
            lo.store(base + d0);
            hi.store(base + d0 + HALF);
            // what goes to the cache is the rotated key as stored (rounded to T)
            lo.get(a);
            hi.get(b);
        }
        if (is_k && write) {
            put_k(h, d0, a, lo);
            put_k(h, d0 + HALF, b, hi);
        }
        return;
    }
    it -= n_q + n_k;
    if (it < n_kp) {
        // ---- K beyond the rotary dimensions: cache write only ----
        if (!write) return;
        const int h = it / P, d0 = R + (it % P) * 8;
        Vec8<T> r;
        r.load((const T *)p.k + t * p.k_stride[0] + (int64_t)h * p.k_stride[1] + d0);
        float f[8];
        r.get(f);
        put_k(h, d0, f, r);
        return;
    }
}

template <typename T, typename TT>
int launch_rw_cache(const lazyattn_rope_write_params &p, dim3 grid, hipStream_t stream) {
    if (p.cache_dtype == LAZYATTN_FP8_E4M3)
        hipLaunchKernelGGL((rope_cache_write_kernel<T, TT, 1>), grid, dim3(256), 0, stream, p);
    else if (p.cache_dtype == LAZYATTN_FP8_E5M2)
        hipLaunchKernelGGL((rope_cache_write_kernel<T, TT, 2>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((rope_cache_write_kernel<T, TT, 0>), grid, dim3(256), 0, stream, p);
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

template <typename T>
int launch_rw_table(const lazyattn_rope_write_params &p, dim3 grid, hipStream_t stream) {
    if (p.table_dtype == LAZYATTN_F32) return launch_rw_cache<T, float>(p, grid, stream);
    return launch_rw_cache<T, T>(p, grid, stream);
}

}  // namespace

int launch_rope_cache_write(const lazyattn_rope_write_params &p, hipStream_t stream) {
    const int D = p.head_dim, R = p.rotary_dim;
    const int64_t per_token = (int64_t)(p.num_q_heads + p.num_kv_heads) * (R / 16) + (int64_t)p.num_kv_heads * ((D - R) / 8);
    const int64_t runs = ((int64_t)p.num_tokens + RUN - 1) / RUN;
    const int64_t n = (int64_t)p.num_tokens * per_token + runs * p.num_kv_heads * D;
    if (n <= 0) return LAZYATTN_OK;
    const dim3 grid((unsigned)((n + 255) / 256));
    switch (p.dtype) {
        case LAZYATTN_F32: return launch_rw_table<float>(p, grid, stream);
        case LAZYATTN_BF16: return launch_rw_table<bf16_t>(p, grid, stream);
        case LAZYATTN_F16: return launch_rw_table<f16_t>(p, grid, stream);
        default: return LAZYATTN_E_DTYPE;
    }
}

}  // namespace lazyattn
