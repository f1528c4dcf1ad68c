// Geometry-agnostic deferred-RoPE prefix-prefill kernel: fp32 arithmetic on the vector
// ALUs, any head_dim <= 256, any page size, any cache element type.  It is the kernel
// for float32 operands (where the result has to hold 1e-5 against an fp32 eager
// evaluation, so no reduced-precision matrix instruction may be used) and for shapes
// the MFMA kernel does not cover.
//
// One workgroup (256 threads) = one (request, q-head, 32-row query tile).  Keys are
// consumed in tiles of 32: K is gathered from the 5-D paged layout, rotated while it is
// written to LDS (old_ops/prefix_prefill.py:172-193,246-257), V is gathered next to it,
// then scores, online softmax (old_ops:287-313) and PV run out of LDS.
#include "common.hpp"

namespace lazyattn {

namespace {
constexpr int G_BM = 32;   // query rows per workgroup
constexpr int G_NT = 32;   // keys per tile
constexpr int G_THREADS = 256;
}  // namespace

template <int DMAX>
constexpr size_t generic_lds_bytes() {
    return sizeof(float) * (G_BM * (DMAX + 1) + G_NT * (DMAX + 1) + G_NT * DMAX + G_BM * (G_NT + 1)) +
           sizeof(int) * 2 * G_NT;
}

template <typename T, typename CT, typename TT, int DMAX>
__global__ void __launch_bounds__(G_THREADS)
prefill_generic_kernel(const lazyattn_prefill_params p, const int decode) {
    extern __shared__ float smem[];
    constexpr int LDQ = DMAX + 1;
    float *Qs = smem;
    float *Ks = Qs + G_BM * LDQ;
    float *Vs = Ks + G_NT * LDQ;
    float *Ss = Vs + G_NT * DMAX;
    int *kvalid = (int *)(Ss + G_BM * (G_NT + 1));
    int *kidx = kvalid + G_NT;

    const int tid = threadIdx.x;
    const int mt = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int D = p.head_dim, half = D / 2, BS = p.block_size, X = p.x;
    const int group = p.num_q_heads / p.num_kv_heads;
    const int g = h / group;

    const int64_t qs = load_index(p.b_start_loc, b, p.index_bits);
    const int64_t q_len = load_index(p.b_start_loc, b + 1, p.index_bits) - qs;
    const int64_t seq_len = load_index(p.b_seq_len, b, p.index_bits);
    int64_t ctx_len = seq_len - q_len;
    if (decode) {
        if (q_len != 1) return;               // old_ops/chunked_prefill_paged_decode.py:72-79
        ctx_len = seq_len;                    // every key comes from the cache
    } else {
        if (q_len <= 0) return;
        if (p.skip_decode && q_len == 1) return;   // old_ops/prefix_prefill.py:109-110
    }
    const int row0 = mt * G_BM;
    if (row0 >= q_len) return;                // block_mask, old_ops:322-328

    const bool lazy_b = p.is_lazy ? p.is_lazy[b] != 0 : true;
    const int pos_mode = p.pos_mode;
    const bool vanilla = pos_mode == LAZYATTN_POS_BLOCK_UNIFORM && !lazy_b;
    const bool rot_new = p.rotate_new_k && !vanilla;
    const int W = p.sliding_window > 0 ? p.sliding_window : 0;
    // position of query row 0 for the sliding window (decode: seq_len-1,
    // old_ops/chunked_prefill_paged_decode.py:237-241)
    const int64_t qpos0 = decode ? seq_len - 1 : ctx_len;
    const bool cache_fp8 = p.cache_dtype == LAZYATTN_FP8_E4M3 || p.cache_dtype == LAZYATTN_FP8_E5M2;
    const float ks = cache_fp8 ? *p.k_scale : 1.0f;
    const float vs = cache_fp8 ? *p.v_scale : 1.0f;

    const T *Q = (const T *)p.q;
    const T *Kn = (const T *)p.k;
    const T *Vn = (const T *)p.v;
    const CT *KC = (const CT *)p.k_cache;
    const CT *VC = (const CT *)p.v_cache;
    const TT *TAB = (const TT *)p.cos_sin_cache;

    // ---- Q tile -> LDS (rows past q_len are zero, old_ops:147-154) ----
    for (int i = tid; i < G_BM * D; i += G_THREADS) {
        const int r = i / D, d = i % D;
        float x = 0.f;
        if (row0 + r < q_len)
            x = to_f32(Q[(qs + row0 + r) * p.q_stride[0] + (int64_t)h * p.q_stride[1] + d * p.q_stride[2]]);
        Qs[r * LDQ + d] = x;
    }

    const int r = tid >> 3, c8 = tid & 7;
    const int64_t t_row = row0 + r;          // token index of this thread's row
    float m_i = -INFINITY, l_i = 0.f;
    float acc[DMAX / 8];
#pragma unroll
    for (int i = 0; i < DMAX / 8; ++i) acc[i] = 0.f;

    // number of new-token keys this tile can see (causal): up to the tile's last row
    int64_t new_end = 0;
    if (!decode) {
        new_end = row0 + G_BM;
        if (new_end > q_len) new_end = q_len;
    }
    const int64_t n_ctx_tiles = (ctx_len + G_NT - 1) / G_NT;
    const int64_t n_new_tiles = (new_end + G_NT - 1) / G_NT;

    for (int64_t tile = 0; tile < n_ctx_tiles + n_new_tiles; ++tile) {
        const bool is_new = tile >= n_ctx_tiles;
        const int64_t n0 = (is_new ? tile - n_ctx_tiles : tile) * G_NT;
        __syncthreads();   // previous tile fully consumed (and Q visible on the first pass)

        // ---- per-key validity ----
        if (tid < G_NT) {
            const int64_t n = n0 + tid;
            int ok;
            if (is_new) {
                ok = n < new_end;
            } else {
                ok = n < ctx_len;
                if (ok && !vanilla && p.q_mask) {
                    const int qm = p.q_mask[b * p.qm_stride[0] + (n / BS) * p.qm_stride[1]];
                    ok = (int)(n % BS) < BS - qm;                      // old_ops:165-167
                }
            }
            kvalid[tid] = ok;
            kidx[tid] = (int)n;
        }
        __syncthreads();   // masked slots are never loaded: they may hold anything, NaN included
        // ---- K tile: gather, rotate, store ----
        for (int i = tid; i < G_NT * half; i += G_THREADS) {
            const int kk = i / half, d1 = i % half, d2 = d1 + half;
            const int64_t n = n0 + kk;
            float k1 = 0.f, k2 = 0.f;
            int64_t pos = -1;
            if (is_new) {
                if (n < new_end) {
                    const int64_t base = (qs + n) * p.k_stride[0] + (int64_t)g * p.k_stride[1];
                    k1 = to_f32(Kn[base + d1 * p.k_stride[2]]);
                    k2 = to_f32(Kn[base + d2 * p.k_stride[2]]);
                    if (rot_new) pos = ctx_len + n;                    // old_ops:342-343
                }
            } else if (kvalid[kk]) {
                const int64_t j = n / BS;
                const int o = (int)(n % BS);
                const int64_t pb = p.block_table[b * p.bt_stride[0] + j * p.bt_stride[1]];
                const int64_t base = pb * p.kc_stride[0] + (int64_t)g * p.kc_stride[1] + o * p.kc_stride[3];
                k1 = to_f32(KC[base + (d1 / X) * p.kc_stride[2] + (d1 % X) * p.kc_stride[4]]);
                k2 = to_f32(KC[base + (d2 / X) * p.kc_stride[2] + (d2 % X) * p.kc_stride[4]]);
                if (cache_fp8) {                                        // old_ops:239-241
                    k1 = round_to<T>(k1 * ks);
                    k2 = round_to<T>(k2 * ks);
                }
                if (!vanilla) {
                    if (pos_mode == LAZYATTN_POS_NATURAL) {
                        pos = n;
                    } else {
                        int qo = p.q_offset ? p.q_offset[b * p.qo_stride[0] + j * p.qo_stride[1]] : 0;
                        // q_len == 1 rows: an offset of 0 keeps the previous page's rotation (ops/models/llama_v1.py:207-262)
                        if (decode && pos_mode == LAZYATTN_POS_BLOCK_UNIFORM && p.q_offset)
                            for (int64_t jj = j; qo == 0 && jj > 0;) qo = p.q_offset[b * p.qo_stride[0] + (--jj) * p.qo_stride[1]];
                        if (pos_mode == LAZYATTN_POS_OFFSET) pos = qo != 0 ? (int64_t)qo - 1 + o : n;
                        else pos = qo != 0 ? (int64_t)qo - 1 : 0;
                    }
                }
            }
            if (pos >= 0) {
                const float c = to_f32(TAB[pos * p.table_stride + d1]);
                const float s = to_f32(TAB[pos * p.table_stride + half + d1]);
                const float r1 = k1 * c - k2 * s;                       // old_ops:256
                const float r2 = k1 * s + k2 * c;                       // old_ops:257
                k1 = r1; k2 = r2;
            }
            Ks[kk * LDQ + d1] = k1;
            Ks[kk * LDQ + d2] = k2;
        }
        // ---- V tile ----
        for (int i = tid; i < G_NT * D; i += G_THREADS) {
            float x = 0.f;
            int kk, d;
            if (is_new) {
                kk = i / D; d = i % D;
                const int64_t n = n0 + kk;
                if (n < new_end)
                    x = to_f32(Vn[(qs + n) * p.v_stride[0] + (int64_t)g * p.v_stride[1] + d * p.v_stride[2]]);
            } else {
                kk = i % G_NT; d = i / G_NT;     // slots fastest: matches [.., D, BS]
                const int64_t n = n0 + kk;
                if (kvalid[kk]) {
                    const int64_t pb = p.block_table[b * p.bt_stride[0] + (n / BS) * p.bt_stride[1]];
                    x = to_f32(VC[pb * p.vc_stride[0] + (int64_t)g * p.vc_stride[1] + d * p.vc_stride[2] +
                                  (n % BS) * p.vc_stride[3]]);
                    if (cache_fp8) x = round_to<T>(x * vs);             // old_ops:304-305
                }
            }
            Vs[kk * DMAX + d] = x;
        }
        __syncthreads();

        // ---- scores for (row r, keys c8 + 8 i) ----
        float s[4] = {0.f, 0.f, 0.f, 0.f};
        for (int d = 0; d < D; ++d) {
            const float qv = Qs[r * LDQ + d];
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] = fmaf(qv, Ks[(c8 + 8 * i) * LDQ + d], s[i]);
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kk = c8 + 8 * i;
            const int64_t n = kidx[kk];
            bool ok = kvalid[kk] != 0;
            float v = s[i] * p.sm_scale;                                // old_ops:269
            if (is_new) {
                ok = ok && n <= t_row;                                  // old_ops:371-372
                if (W > 0 && t_row - n >= W) v = -10000.f;              // old_ops:373-376
            } else if (W > 0 && (qpos0 + t_row) - n >= W) {
                v = -10000.f;                                           // old_ops:282-284
            }
            s[i] = ok ? v : -INFINITY;
            tmax = fmaxf(tmax, s[i]);
        }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, off));
        const float m_new = fmaxf(m_i, tmax);
        float alpha = 1.f, lsum = 0.f;
        if (m_new != -INFINITY) {
            alpha = expf(m_i - m_new);                                  // old_ops:290
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float pr = expf(s[i] - m_new);
                Ss[r * (G_NT + 1) + c8 + 8 * i] = pr;
                lsum += pr;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) Ss[r * (G_NT + 1) + c8 + 8 * i] = 0.f;
        }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) lsum += __shfl_xor(lsum, off);
        l_i = l_i * alpha + lsum;                                       // old_ops:312
        m_i = m_new;
        __syncthreads();

        // ---- acc[r, c8 + 8 i] = acc * alpha + P V ----
#pragma unroll
        for (int i = 0; i < DMAX / 8; ++i) acc[i] *= alpha;
        for (int kk = 0; kk < G_NT; ++kk) {
            const float pr = Ss[r * (G_NT + 1) + kk];
#pragma unroll
            for (int i = 0; i < DMAX / 8; ++i) {
                const int d = c8 + 8 * i;
                if (d < D) acc[i] = fmaf(pr, Vs[kk * DMAX + d], acc[i]);
            }
        }
    }

    if (t_row < q_len) {
        T *O = (T *)p.o;
        const float inv = l_i > 0.f ? 1.f / l_i : 0.f;
#pragma unroll
        for (int i = 0; i < DMAX / 8; ++i) {
            const int d = c8 + 8 * i;
            if (d < D)
                O[(qs + t_row) * p.o_stride[0] + (int64_t)h * p.o_stride[1] + d * p.o_stride[2]] =
                    from_f32<T>(acc[i] * inv);
        }
    }
}

template <typename T, typename CT, typename TT>
static int launch_generic_dmax(const lazyattn_prefill_params &p, int decode, hipStream_t stream) {
    const int mt = decode ? 1 : (p.max_q_len + G_BM - 1) / G_BM;
    if (mt <= 0 || p.batch <= 0) return LAZYATTN_OK;
    dim3 grid(mt, p.num_q_heads, p.batch), block(G_THREADS);
    hipError_t e;
#define LAZYATTN_GENERIC_CASE(DM)                                                              \
    {                                                                                          \
        auto kern = prefill_generic_kernel<T, CT, TT, DM>;                                     \
        const size_t lds = generic_lds_bytes<DM>();                                            \
        if (lds > 48 * 1024) {                                                                 \
            e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds);                                                 \
            if (e != hipSuccess) return LAZYATTN_E_LAUNCH;                                     \
        }                                                                                      \
        hipLaunchKernelGGL(kern, grid, block, lds, stream, p, decode);                         \
    }
    if (p.head_dim <= 64) LAZYATTN_GENERIC_CASE(64)
    else if (p.head_dim <= 128) LAZYATTN_GENERIC_CASE(128)
    else LAZYATTN_GENERIC_CASE(256)
#undef LAZYATTN_GENERIC_CASE
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

template <typename T, typename TT>
static int launch_generic_cache(const lazyattn_prefill_params &p, int decode, hipStream_t stream) {
    if (p.cache_dtype == p.dtype) return launch_generic_dmax<T, T, TT>(p, decode, stream);
    if (p.cache_dtype == LAZYATTN_FP8_E4M3) return launch_generic_dmax<T, fp8e4m3_t, TT>(p, decode, stream);
    if (p.cache_dtype == LAZYATTN_FP8_E5M2) return launch_generic_dmax<T, fp8e5m2_t, TT>(p, decode, stream);
    return LAZYATTN_E_DTYPE;
}

template <typename T>
static int launch_generic_table(const lazyattn_prefill_params &p, int decode, hipStream_t stream) {
    if (p.table_dtype == p.dtype) return launch_generic_cache<T, T>(p, decode, stream);
    if (p.table_dtype == LAZYATTN_F32) return launch_generic_cache<T, float>(p, decode, stream);
    return LAZYATTN_E_DTYPE;
}

int launch_prefill_generic(const lazyattn_prefill_params &p, int decode, hipStream_t stream) {
    switch (p.dtype) {
        case LAZYATTN_F32: return launch_generic_table<float>(p, decode, stream);
        case LAZYATTN_BF16: return launch_generic_table<bf16_t>(p, decode, stream);
        case LAZYATTN_F16: return launch_generic_table<f16_t>(p, decode, stream);
        default: return LAZYATTN_E_DTYPE;
    }
}

}  // namespace lazyattn
