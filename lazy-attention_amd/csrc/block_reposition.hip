// Re-positioning of cached document blocks: copy a paged block (K and V) and re-rotate its keys
// from the positions they were stored at to the positions they take in the assembled sequence.
//
// Replaces the eager per-block loop of block_attn_vllm/gpu_model_runner.py:94-106, which for every
// layer and every (new_id, old_id, from_start, to_start) calls copy_paged_block and
// place_paged_block_keys (block_attn_vllm/utils.py:48-95): slot o of the block is un-rotated
// from position from_start + o to position 0 and then rotated to to_start + o, two explicit
// steps with the model's own cos/sin rows.  Here one launch handles all blocks of a layer; the
// two steps are kept (the table rows are rounded values, so R(to) R(-from) is not R(to - from) in
// general), evaluated in fp32 with one rounding at the end.
// K block [Hkv, D/x, BS, x]: an item is one (head, 8-d chunk pair (d, d + D/2), slot).
// V block [Hkv, D, BS]: copied 16 bytes at a time.
#include "common.hpp"
#include "vec8.hpp"

namespace lazyattn {

template <typename T, typename TT>
__global__ void __launch_bounds__(256)
block_reposition_kernel(T *k_cache, T *v_cache, const int32_t *items, const TT *table, int64_t table_stride,
                        int64_t kc_s0, int64_t kc_s1, int64_t kc_s2, int64_t kc_s3, int64_t vc_s0, int num_kv_heads,
                        int head_dim, int block_size, int x, int64_t v_block_elems) {
    const int item = blockIdx.y;
    const int new_id = items[4 * item], old_id = items[4 * item + 1];
    const int from_start = items[4 * item + 2], to_start = items[4 * item + 3];
    const int HALF = head_dim / 2, C = head_dim / 16;
    const int n_k = num_kv_heads * C * block_size;
    const int64_t n_v = v_block_elems * (int64_t)sizeof(T) / 16;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_k + n_v; i += (int64_t)gridDim.x * blockDim.x) {
        if (i < n_k) {
            const int o = (int)(i % block_size), c = (int)(i / block_size) % C, h = (int)(i / block_size) / C;
            const int d0 = c * 8;
            auto at = [&](int blk, int d) {
                return (int64_t)blk * kc_s0 + (int64_t)h * kc_s1 + (int64_t)(d / x) * kc_s2 + (int64_t)o * kc_s3 + (d % x);
            };
            float a[8], b[8];
            if (x % 8 == 0) {
                Vec8<T> lo, hi;
                lo.load(k_cache + at(old_id, d0));
                hi.load(k_cache + at(old_id, d0 + HALF));
                lo.get(a);
                hi.get(b);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) { a[e] = to_f32(k_cache[at(old_id, d0 + e)]); b[e] = to_f32(k_cache[at(old_id, d0 + HALF + e)]); }
            }
            Vec8<TT> cf, sf, ct, st;
            const TT *rf = table + (int64_t)(from_start + o) * table_stride, *rt = table + (int64_t)(to_start + o) * table_stride;
            cf.load(rf + d0); sf.load(rf + HALF + d0);
            ct.load(rt + d0); st.load(rt + HALF + d0);
            float c1[8], s1[8], c2[8], s2[8], xo[8], yo[8];
            cf.get(c1); sf.get(s1); ct.get(c2); st.get(s2);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                // R(-from): k cos - rotate_half(k) sin      (utils.py:84)
                const float u = a[e] * c1[e] + b[e] * s1[e];
                const float w = b[e] * c1[e] - a[e] * s1[e];
                // R(+to):   k cos + rotate_half(k) sin      (utils.py:86)
                xo[e] = u * c2[e] - w * s2[e];
                yo[e] = w * c2[e] + u * s2[e];
            }
            if (x % 8 == 0) {
                Vec8<T> lo, hi;
                lo.set(xo);
                hi.set(yo);
                lo.store(k_cache + at(new_id, d0));
                hi.store(k_cache + at(new_id, d0 + HALF));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    k_cache[at(new_id, d0 + e)] = from_f32<T>(xo[e]);
                    k_cache[at(new_id, d0 + HALF + e)] = from_f32<T>(yo[e]);
                }
            }
        } else if (new_id != old_id) {
            const int64_t j = i - n_k;
            reinterpret_cast<uint4 *>(v_cache + (int64_t)new_id * vc_s0)[j] = reinterpret_cast<const uint4 *>(v_cache + (int64_t)old_id * vc_s0)[j];
        }
    }
}

template <typename T, typename TT>
static int launch_rp(const lazyattn_reposition_params &p, hipStream_t stream) {
    const int64_t v_block_elems = (int64_t)p.num_kv_heads * p.head_dim * p.block_size;
    const int64_t work = (int64_t)p.num_kv_heads * (p.head_dim / 16) * p.block_size + v_block_elems * (int64_t)sizeof(T) / 16;
    const dim3 grid((unsigned)((work + 255) / 256), (unsigned)p.num_items);
    hipLaunchKernelGGL((block_reposition_kernel<T, TT>), grid, dim3(256), 0, stream, (T *)p.k_cache, (T *)p.v_cache, p.items,
                       (const TT *)p.cos_sin_cache, p.table_stride, p.kc_stride[0], p.kc_stride[1], p.kc_stride[2],
                       p.kc_stride[3], p.vc_stride[0], p.num_kv_heads, p.head_dim, p.block_size, p.x, v_block_elems);
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

int launch_block_reposition(const lazyattn_reposition_params &p, hipStream_t stream) {
    const bool t32 = p.table_dtype == LAZYATTN_F32;
    switch (p.dtype) {
        case LAZYATTN_F32: return launch_rp<float, float>(p, stream);
        case LAZYATTN_BF16: return t32 ? launch_rp<bf16_t, float>(p, stream) : launch_rp<bf16_t, bf16_t>(p, stream);
        case LAZYATTN_F16: return t32 ? launch_rp<f16_t, float>(p, stream) : launch_rp<f16_t, f16_t>(p, stream);
        default: return LAZYATTN_E_DTYPE;
    }
}

}  // namespace lazyattn
