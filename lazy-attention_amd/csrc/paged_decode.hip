// q_len == 1 rows with the rotation fused in: bf16 / float16 (cache of the same type or fp8 e4m3), head sizes 128, 64 and
// other multiples of 16 below 128 (padded), pages of 16 or 32 slots, gfx950.
//
// Follows old_ops/chunked_prefill_paged_decode.py:23-280 (un-rotated cache, key n rotated
// at position n) and ops/models/llama_v1.py:18-637 (block-uniform rotation by q_offset-1,
// un-rotated branch for is_lazy == 0).  Every key, the new token included, is read from the
// paged cache (backends/triton_attn.py:100-109 writes it there before the call).
//
// The work is HBM-bound (each K/V byte is used by `group` query rows only), so the kernel is
// built around plain streaming: one wave owns one (request, kv head, slice of the pages) and
// walks its pages two at a time, entirely in registers -- no LDS, no barrier:
//   * a K page [D/8][16][8] is read with one 16-byte load per (token, 8-d chunk); lane
//     (token t = lane % 16, chunk group = lane / 16) receives exactly the A operand of
//     v_mfma_f32_16x16x32_bf16 for S^T = K . Q^T, and holds both halves (d, d + 64) of its
//     rotation pairs, so the rotation happens in place;
//   * the query heads of the group are the 16 columns of the MFMA (heads beyond the group are
//     zero columns; a group above 16 is cut into blocks of 16 heads, one wave each): the matrix
//     pipe is mostly idle here and that is fine;
//   * S^T comes out as (4 tokens per lane) x (head = lane % 16): each lane runs the online
//     softmax of one head, lanes 16 apart share a head and exchange the row max;
//   * P^T (two pages = 32 tokens) is the B operand of O^T += V^T . P^T as it stands if the
//     contraction index is ordered (page X tokens 4g..4g+3 | page Y tokens 4g..4g+3) per lane
//     group g, which is how the V rows [D][16] are read: 8 bytes per page, row and lane.
// fp8 e4m3 pages ([D/16][16][16] and [D][16] bytes) are read with 8- and 4-byte loads at the same lane mapping,
// converted, scaled and rounded to bf16 (old_ops/prefix_prefill.py:239-241 arithmetic), then treated alike.
// Slices of one request are merged by paged_decode_merge_kernel.
#include "common.hpp"
#include "elem16.hpp"
#include <type_traits>

namespace lazyattn {

namespace {


constexpr int BS = 16;
constexpr int WAVES = 4;            // independent waves per workgroup

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
template <typename T> __device__ __forceinline__ void unpack8(const uint4 &w, float *f) {
    f[0] = Elem<T>::lo(w.x); f[1] = Elem<T>::hi(w.x); f[2] = Elem<T>::lo(w.y); f[3] = Elem<T>::hi(w.y);
    f[4] = Elem<T>::lo(w.z); f[5] = Elem<T>::hi(w.z); f[6] = Elem<T>::lo(w.w); f[7] = Elem<T>::hi(w.w);
}

// two fp8 bytes (the low 16 bits of w) -> two floats; KIND 1: e4m3, 2: e5m2
template <int KIND> __device__ __forceinline__ f32x2_t cvt_fp8x2(uint32_t w) {
    if constexpr (KIND == 2) return __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
    else return __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
}
// 8 fp8 bytes -> (float * scale) rounded to the query type, as floats
template <typename T, int KIND> __device__ __forceinline__ void unpack8_fp8(uint32_t lo, uint32_t hi, float scale, float *f) {
    const f32x2_t a = cvt_fp8x2<KIND>(lo), b = cvt_fp8x2<KIND>(lo >> 16);
    const f32x2_t c = cvt_fp8x2<KIND>(hi), d = cvt_fp8x2<KIND>(hi >> 16);
    const float t[8] = {a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = round_to<T>(t[i] * scale);
}

// 8 consecutive cos (or sin) entries of one table row
template <typename TT> struct Tab8 {                        // a 16-bit table
    uint4 v;
    __device__ __forceinline__ void load(const uint8_t *row, int elem) { v = *reinterpret_cast<const uint4 *>(row + elem * 2); }
    __device__ __forceinline__ void get(float *f) const { unpack8<TT>(v, f); }
};
template <> struct Tab8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const uint8_t *row, int elem) {
        a = *reinterpret_cast<const float4 *>(row + elem * 4);
        b = *reinterpret_cast<const float4 *>(row + elem * 4 + 16);
    }
    __device__ __forceinline__ void get(float *f) const {
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
};

// what one page contributes, as loaded: the key side and the value side travel separately
// HD = head size (128 or 64): HD/32 key chunks per lane (one per MFMA of the scores), HD/64 rotation pair
// sets, HD/16 row blocks of V
template <typename TT, int HD> struct KeyRegs {
    uint4 k[HD / 32];           // chunks grp, 4 + grp, ... of token t; k[j] pairs with k[j + HD/64]
    Tab8<TT> c[HD / 64], s[HD / 64];   // cos / sin for d = 32 j + 8 grp ..
    int lim;                    // valid slots
    int first;                  // first slot inside the sliding window (<= 0: all)
    int tag;                    // computed cos/sin: what c and s currently hold (page or position), -1 = nothing
};
template <int HD> struct ValRegs {
    uint2 v[HD / 16];           // V[d = 16 blk + t][tokens 4 grp .. 4 grp + 3]
};

}  // namespace

// PAD: the head size is a multiple of 16 below HD = 128; the lane's chunks, the query and the V rows are laid out as
// for 128 with the two halves of the real head at (0 .., 64 ..) and zeros in between
// COMPUTE: cos/sin come from the inverse frequencies (p.rope_freqs) instead of the table; they are kept as the table
// would hold them, rounded to the element type (TT = T): half the registers of floats
template <typename T, typename TT, int FP8, int HD, bool PAD, bool COMPUTE>
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(2)))
paged_decode_kernel(const lazyattn_prefill_params p, const int nsplit) {
    static_assert(!COMPUTE || std::is_same<TT, T>::value, "computed cos/sin are kept in the element type");
    using E = Elem<T>;
    constexpr int D = HD, NM = HD / 32, NP = HD / 64, NBLK = HD / 16;
    constexpr int TSZ = sizeof(TT);
    const int Dr = PAD ? p.head_dim : D, HALFr = Dr / 2, CPr = Dr / 16, NBr = Dr / 16;   // real sizes
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int W = blockIdx.x * WAVES + wave;
    const int group = p.num_q_heads / p.num_kv_heads;
    // a wave takes 16 query heads of a kv head (the columns of its MFMAs): groups above 16 are cut into blocks
    // that walk the same pages side by side
    const int hblocks = (group + 15) >> 4;
    const int kvh = p.num_kv_heads * hblocks;
    if (W >= p.batch * kvh * nsplit) return;
    // (head block, then) kv heads vary fastest: the waves of a workgroup walk the same pages, whose heads are
    // adjacent 4 KB pieces of one cache block
    const int hb0 = (W % hblocks) * 16;                          // first head of this wave's block within the group
    const int g = (W % kvh) / hblocks;
    const int split = (W / kvh) % nsplit;
    const int b = W / (nsplit * kvh);

    const int64_t qs = load_index(p.b_start_loc, b, p.index_bits);
    const int q_len = (int)(load_index(p.b_start_loc, b + 1, p.index_bits) - qs);
    if (q_len != 1) return;                                      // old_ops/chunked_prefill_paged_decode.py:72-79
    const int seq_len = (int)load_index(p.b_seq_len, b, p.index_bits);
    const bool lazy_b = p.is_lazy ? p.is_lazy[b] != 0 : true;
    const bool vanilla = p.pos_mode == LAZYATTN_POS_BLOCK_UNIFORM && !lazy_b;
    const bool per_token = !vanilla && p.pos_mode == LAZYATTN_POS_NATURAL;
    // the packed table [block:32 | q_offset:16 | q_mask:16] is read as pairs of 32-bit words: the block is the
    // high word, offset and pad count share the low one
    const bool packed = p.packed_block_table != nullptr;
    const bool use_qmask = !vanilla && (packed || p.q_mask != nullptr);
    const bool use_qo = !vanilla && p.pos_mode == LAZYATTN_POS_BLOCK_UNIFORM;
    const int n_pages = seq_len > 0 ? (seq_len + BS - 1) / BS : 0;
    const int n_pairs = (n_pages + 1) / 2;
    // sliding window (old_ops/chunked_prefill_paged_decode.py:237-241): the row sits at position seq_len - 1 and
    // sees the keys at seq_len - window .. seq_len - 1; the page pairs before that are not visited
    const int first_key = p.sliding_window > 0 && seq_len > p.sliding_window ? seq_len - p.sliding_window : 0;
    const int first_pair = first_key / (2 * BS);
    const int pair_begin = first_pair + (int)((int64_t)(n_pairs - first_pair) * split / nsplit);
    const int pair_end = first_pair + (int)((int64_t)(n_pairs - first_pair) * (split + 1) / nsplit);

    const int t = lane & 15, grp = lane >> 4;

    // page metadata through the scalar unit
    typedef const int32_t __attribute__((address_space(4))) *sptr_i32;
    const int32_t *pk_words = packed ? (const int32_t *)(p.packed_block_table + b * p.pbt_stride[0]) : nullptr;
    const sptr_i32 pk_row = (sptr_i32)pk_words;                                      // low words
    const sptr_i32 bt_row = packed ? pk_row + 1 : (sptr_i32)(p.block_table + b * p.bt_stride[0]);
    const sptr_i32 qo_row = !use_qo ? bt_row : packed ? pk_row : (sptr_i32)(p.q_offset + b * p.qo_stride[0]);
    const sptr_i32 qm_row = !use_qmask ? bt_row : packed ? pk_row : (sptr_i32)(p.q_mask + b * p.qm_stride[0]);
    const int64_t bt_s1 = packed ? 2 * p.pbt_stride[1] : p.bt_stride[1];
    const int64_t qo_s1 = !use_qo ? bt_s1 : packed ? 2 * p.pbt_stride[1] : p.qo_stride[1];
    const int64_t qm_s1 = !use_qmask ? bt_s1 : packed ? 2 * p.pbt_stride[1] : p.qm_stride[1];
    const int qo_shift = use_qo && packed ? 16 : 0;
    const int qo_and = !use_qo ? 0 : packed ? 0xffff : -1, qm_and = !use_qmask ? 0 : packed ? 0xffff : -1;

    constexpr int CSZ = FP8 ? 1 : 2;                             // bytes per cache element
    const uint8_t *kc_base = (const uint8_t *)p.k_cache + (int64_t)g * p.kc_stride[1] * CSZ;
    const uint8_t *vc_base = (const uint8_t *)p.v_cache + (int64_t)g * p.vc_stride[1] * CSZ;
    const int64_t kc_page_bytes = p.kc_stride[0] * CSZ, vc_page_bytes = p.vc_stride[0] * CSZ;
    const float k_scale = FP8 ? *p.k_scale : 1.f, v_scale = FP8 ? *p.v_scale : 1.f;
    const uint8_t *tab = (const uint8_t *)p.cos_sin_cache;
    const int64_t row_bytes = p.table_stride * TSZ;
    // A cache page of 32 slots is read as two parts of 16: "page" j below is the j-th run of 16 slots of the
    // sequence, part j & 1 of cache page j >> 1 (pshift = 1); with pages of 16 slots the two coincide.
    const int pshift = p.block_size == 2 * BS ? 1 : 0;
    const int cache_bs = BS << pshift;
    // bf16: chunk 4 m + grp of token t at ((4 m + grp) * slots + t) * 16, 16 bytes
    // fp8 : the same 8 d are half (grp & 1) of 16-d chunk 2 m + grp / 2: ((2 m + grp / 2) * slots + t) * 16 + (grp & 1) * 8
    const uint32_t k_off = FP8 ? (uint32_t)(((grp >> 1) * cache_bs + t) * 16 + (grp & 1) * 8) : (uint32_t)((grp * cache_bs + t) * 16);
    const uint32_t K_STEP = (FP8 ? 512u : 1024u) << pshift;      // per m
    // V[d = 16 blk + t][tokens 4 grp ..]: 8 bytes (bf16) or 4 bytes (fp8) of the row
    const uint32_t v_off = FP8 ? (uint32_t)(t * cache_bs + grp * 4) : (uint32_t)(t * cache_bs * 2 + grp * 8);
    const uint32_t V_STEP = (FP8 ? 256u : 512u) << pshift;       // per blk

    // PAD: chunk 4 m + grp of the 128-wide layout is real chunk c (first half) or Dr/16 + c - 8 (second half), if c % 8
    // is below Dr/16; the others are read from chunk 0 and zeroed
    uint32_t pk_off[PAD ? NM : 1];
    bool pk_ok[PAD ? NM : 1];
    if constexpr (PAD) {
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            const int c = 4 * m + grp;
            pk_ok[m] = (c & 7) < CPr;
            const int rc = pk_ok[m] ? (c < 8 ? c : CPr + c - 8) : 0;
            pk_off[m] = FP8 ? (uint32_t)(((rc >> 1) * cache_bs + t) * 16 + (rc & 1) * 8) : (uint32_t)((rc * cache_bs + t) * 16);
        }
    }
    auto page_block = [&](int j) -> int {
        int jc = j < n_pages ? j : n_pages - 1;
        jc = jc < 0 ? 0 : jc;
        return bt_row[(jc >> pshift) * bt_s1];
    };
    // Block-uniform rotation: a page whose offset is 0 keeps the rotation of the page before it (the reference acts
    // only when the value changes and does nothing for 0, ops/models/llama_v1.py:207-262).  The pages of a slice
    // are visited in order, so the last non-zero offset is carried along; a slice that does not start at page 0
    // and whose first offset is 0 finds it by scanning backwards, 64 entries per step.
    int carry = 0;
    if (use_qo && pair_begin > 0 && pair_begin < pair_end) {
        int pj = (2 * pair_begin) >> pshift;
        if (((qo_row[pj * qo_s1] >> qo_shift) & qo_and) == 0) {
            const int32_t *row = packed ? pk_words : p.q_offset + b * p.qo_stride[0];
            for (int base = pj - 1; base >= 0 && carry == 0; base -= 64) {
                const int idx = base - lane;
                const int v = idx >= 0 ? (row[idx * qo_s1] >> qo_shift) & qo_and : 0;
                const uint64_t hit = __builtin_amdgcn_ballot_w64(v != 0);
                if (hit) carry = __builtin_amdgcn_readlane(v, __builtin_ctzll(hit));
            }
        }
    }
    // COMPUTE: this lane's inverse frequencies, in revolutions per position (d = 32 j + 8 grp + e)
    float frev[COMPUTE ? NP * 8 : 1];
    if constexpr (COMPUTE) {
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            const int e0 = PAD && 32 * j + 8 * grp >= HALFr ? 0 : 32 * j + 8 * grp;
#pragma unroll
            for (int e = 0; e < 8; ++e) frev[j * 8 + e] = p.rope_freqs[e0 + e] * 0.15915494309189535f;
        }
    }
    auto load_keys = [&](int j, KeyRegs<TT, HD> &r) {
        int jc = j < n_pages ? j : n_pages - 1;
        jc = jc < 0 ? 0 : jc;
        const int pj = jc >> pshift, part = jc & pshift;
        const int bt = bt_row[pj * bt_s1];
        int qo = (qo_row[pj * qo_s1] >> qo_shift) & qo_and;
        carry = qo ? qo : carry;
        qo = carry;
        const int qm = qm_row[pj * qm_s1] & qm_and;                                  // old_ops/chunked...:165-167 analogue
        const int ql = cache_bs - qm - (j & pshift) * BS;                            // valid slots of this part
        int l = seq_len - j * BS;
        l = l < ql ? l : ql;
        l = l > BS ? BS : l;
        r.lim = l < 0 ? 0 : l;
        r.first = first_key - j * BS;                                                // slots below it lie before the window
        const uint8_t *kb = kc_base + bt * kc_page_bytes + part * (BS * 16);
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            if constexpr (PAD) {
                uint4 w4;
                if (FP8) {
                    const uint2 w = *reinterpret_cast<const uint2 *>(kb + pk_off[m]);
                    w4 = make_uint4(w.x, w.y, 0, 0);
                } else {
                    w4 = *reinterpret_cast<const uint4 *>(kb + pk_off[m]);
                }
                r.k[m] = pk_ok[m] ? w4 : make_uint4(0, 0, 0, 0);
            } else if (FP8) {
                const uint2 w = *reinterpret_cast<const uint2 *>(kb + k_off + m * K_STEP);
                r.k[m] = make_uint4(w.x, w.y, 0, 0);
            } else {
                r.k[m] = *reinterpret_cast<const uint4 *>(kb + k_off + m * K_STEP);
            }
        }
        // position of this lane's token: its index in the sequence (un-rotated cache), or one
        // angle for the whole page (block-uniform), or row 0 = identity (un-rotated request)
        int pos = qo ? qo - 1 : 0;                                                   // ops/models/llama_v1.py:231-262
        if (per_token) {
            pos = j * BS + t;                                                        // old_ops/chunked...:203-233
            pos = pos < seq_len ? pos : seq_len - 1;     // slots past the end are masked; stay inside the table
            pos = pos < 0 ? 0 : pos;
        }
        if constexpr (COMPUTE) {
            // rope_cos_sin_from_freqs (model_executor/rope/cos_sin.py:62-66): cos / sin of position x frequency.  The
            // product is formed exactly (rounded product + its fma remainder) and reduced to one revolution before the
            // hardware sine and cosine, so the angle keeps float accuracy at positions in the tens of thousands.
            // Block-uniform pages repeat their position for a whole document: recomputed only when it changes.
            const int key = per_token ? j : pos;                                     // wave-uniform
            if (key != r.tag) {
                r.tag = key;
                const float P = (float)pos;
#pragma unroll
                for (int jj = 0; jj < NP; ++jj) {
                    float cs[8], sn[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float f = frev[jj * 8 + e];
                        const float hi = P * f, lo = fmaf(P, f, -hi);
                        const float rev = __builtin_amdgcn_fractf(hi) + lo;
                        cs[e] = __builtin_amdgcn_cosf(rev);
                        sn[e] = __builtin_amdgcn_sinf(rev);
                    }
                    r.c[jj].v = make_uint4(E::pack(cs[0], cs[1]), E::pack(cs[2], cs[3]), E::pack(cs[4], cs[5]), E::pack(cs[6], cs[7]));
                    r.s[jj].v = make_uint4(E::pack(sn[0], sn[1]), E::pack(sn[2], sn[3]), E::pack(sn[4], sn[5]), E::pack(sn[6], sn[7]));
                }
            }
        } else {
            const uint8_t *row = tab + (int64_t)pos * row_bytes;
#pragma unroll
            for (int j = 0; j < NP; ++j) {
                const int e = PAD && 32 * j + 8 * grp >= HALFr ? 0 : 32 * j + 8 * grp;   // (a padded chunk is zero: any angle will do)
                r.c[j].load(row, e);
                r.s[j].load(row, HALFr + e);
            }
        }
    };
    auto load_values = [&](int j, ValRegs<HD> &r) {
        int jv = j < n_pages ? j : n_pages - 1;
        jv = jv < 0 ? 0 : jv;
        const uint8_t *vb = vc_base + page_block(j) * vc_page_bytes + (jv & pshift) * (BS * CSZ);
#pragma unroll
        for (int blk = 0; blk < NBLK; ++blk) {
            const uint32_t vo = v_off + (PAD && blk >= NBr ? 0 : blk) * V_STEP;      // rows 16 blk .. of V; past the head: zeros
            uint2 w;
            if (FP8) w = make_uint2(*reinterpret_cast<const uint32_t *>(vb + vo), 0);
            else w = *reinterpret_cast<const uint2 *>(vb + vo);
            r.v[blk] = PAD && blk >= NBr ? make_uint2(0, 0) : w;
        }
    };
    // rotate the pair (lo, hi) = (d, d + 64) in fp32, one rounding to bf16
    auto rotate = [&](const uint4 &lo, const uint4 &hi, const Tab8<TT> &c, const Tab8<TT> &s, uint4 &xo, uint4 &yo) {
        float a[8], bb[8], cs[8], sn[8], x[8], y[8];
        if (FP8) {
            unpack8_fp8<T, FP8>(lo.x, lo.y, k_scale, a);
            unpack8_fp8<T, FP8>(hi.x, hi.y, k_scale, bb);
        } else {
            unpack8<T>(lo, a);
            unpack8<T>(hi, bb);
        }
        c.get(cs);
        s.get(sn);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x[e] = a[e] * cs[e] - bb[e] * sn[e];
            y[e] = a[e] * sn[e] + bb[e] * cs[e];
        }
        xo = make_uint4(E::pack(x[0], x[1]), E::pack(x[2], x[3]), E::pack(x[4], x[5]), E::pack(x[6], x[7]));
        yo = make_uint4(E::pack(y[0], y[1]), E::pack(y[2], y[3]), E::pack(y[4], y[5]), E::pack(y[6], y[7]));
    };

    // Q^T: column = head = t, contraction d = 32 m + 8 grp ..
    uint4 qf[NM];
    {
        const bool head_ok = hb0 + t < group;
        const T *qp = (const T *)p.q + qs * p.q_stride[0] + (int64_t)(g * group + (head_ok ? hb0 + t : 0)) * p.q_stride[1] + 8 * grp;
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            uint4 w = make_uint4(0, 0, 0, 0);
            if constexpr (PAD) {
                const int c = 32 * m + 8 * grp, lo = c & 63;               // column of the 128-wide layout
                if (head_ok && lo < HALFr) w = *reinterpret_cast<const uint4 *>(qp - 8 * grp + (c < 64 ? lo : HALFr + lo));
            } else {
                if (head_ok) w = *reinterpret_cast<const uint4 *>(qp + 32 * m);
            }
            qf[m] = w;
        }
    }
    const float cs2 = p.sm_scale * 1.4426950408889634f;
    float m_run = -INFINITY, l_run = 0.f;
    f32x4_t acc[NBLK];
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) acc[blk] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // scores of one page: S^T[token 4 grp + i][head t], masked
    auto scores = [&](const KeyRegs<TT, HD> &r) -> f32x4_t {
        uint4 kk[NM];
#pragma unroll
        for (int j = 0; j < NP; ++j) rotate(r.k[j], r.k[j + NP], r.c[j], r.s[j], kk[j], kk[j + NP]);
        f32x4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < NM; ++m) s = E::mfma16(kk[m], qf[m], s);
        if (r.lim < BS || r.first > 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] = (4 * grp + i < r.lim && 4 * grp + i >= r.first) ? s[i] : -INFINITY;
        }
        return s;
    };
    // V words of a page with the masked tokens zeroed (a masked slot may hold anything)
    auto masked_v = [&](const ValRegs<HD> &r, int lim, int blk) -> uint2 {
        uint2 w = r.v[blk];
        if (FP8) {
            const f32x2_t lo = cvt_fp8x2<FP8>(w.x), hi = cvt_fp8x2<FP8>(w.x >> 16);
            w = make_uint2(E::pack(lo[0] * v_scale, lo[1] * v_scale), E::pack(hi[0] * v_scale, hi[1] * v_scale));
        }
        if (lim < BS) {
            if (4 * grp + 0 >= lim) w.x &= 0xffff0000u;
            if (4 * grp + 1 >= lim) w.x &= 0x0000ffffu;
            if (4 * grp + 2 >= lim) w.y &= 0xffff0000u;
            if (4 * grp + 3 >= lim) w.y &= 0x0000ffffu;
        }
        return w;
    };

    // The key side of pair i+1 is requested as soon as the scores of pair i have consumed the
    // registers it lands in, the value side of pair i at the top of its iteration: every load has
    // about half an iteration of other work between issue and use, at no extra registers.
    KeyRegs<TT, HD> KX, KY;
    KX.tag = KY.tag = -1;
    if (pair_begin < pair_end) {
        load_keys(2 * pair_begin, KX);
        load_keys(2 * pair_begin + 1, KY);
    }
    for (int pr = pair_begin; pr < pair_end; ++pr) {
        ValRegs<HD> X, Y;
        load_values(2 * pr, X);
        load_values(2 * pr + 1, Y);
        const f32x4_t sx = scores(KX), sy = scores(KY);
        const int lim_x = KX.lim, lim_y = KY.lim;
        if (pr + 1 < pair_end) {
            load_keys(2 * pr + 2, KX);
            load_keys(2 * pr + 3, KY);
        }
        // online softmax of head t over the 32 tokens; lanes t, t+16, t+32, t+48 share the head
        float mx = fmaxf(fmaxf(fmaxf(sx[0], sx[1]), fmaxf(sx[2], sx[3])), fmaxf(fmaxf(sy[0], sy[1]), fmaxf(sy[2], sy[3])));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_safe) * cs2);
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
            for (int blk = 0; blk < NBLK; ++blk) acc[blk] *= alpha;
            l_run *= alpha;
        }
        m_run = m_new;
        const float mc = m_safe * cs2;
        float px[4], py[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            px[i] = __builtin_amdgcn_exp2f(fmaf(sx[i], cs2, -mc));
            py[i] = __builtin_amdgcn_exp2f(fmaf(sy[i], cs2, -mc));
        }
        l_run += (px[0] + px[1]) + (px[2] + px[3]) + (py[0] + py[1]) + (py[2] + py[3]);
        const uint4 pf = make_uint4(E::pack(px[0], px[1]), E::pack(px[2], px[3]), E::pack(py[0], py[1]), E::pack(py[2], py[3]));
#pragma unroll
        for (int blk = 0; blk < NBLK; ++blk) {
            const uint2 vx = masked_v(X, lim_x, blk), vy = masked_v(Y, lim_y, blk);
            acc[blk] = E::mfma16(make_uint4(vx.x, vx.y, vy.x, vy.y), pf, acc[blk]);
        }
    }

    // ---- epilogue: lane (head t, grp) holds O^T[d = 16 blk + 4 grp + i][head t] ----
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);
    if (hb0 + t >= group) return;
    const int h = g * group + hb0 + t;
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    if (nsplit == 1) {
        T *op = (T *)p.o + qs * p.o_stride[0] + (int64_t)h * p.o_stride[1] + 4 * grp;
#pragma unroll
        for (int blk = 0; blk < NBLK; ++blk) {
            if (PAD && blk >= NBr) continue;
            *reinterpret_cast<uint2 *>(op + 16 * blk) =
                make_uint2(E::pack(acc[blk][0] * inv, acc[blk][1] * inv), E::pack(acc[blk][2] * inv, acc[blk][3] * inv));
        }
        return;
    }
    // partial of this slice: normalised O and log2-sum-exp, indexed by (slice, request, head)
    float *wo = (float *)p.workspace;
    float *wl = wo + (int64_t)nsplit * p.batch * p.num_q_heads * D;
    const int64_t r_idx = ((int64_t)split * p.batch + b) * p.num_q_heads + h;
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk)
        *reinterpret_cast<float4 *>(wo + r_idx * D + 16 * blk + 4 * grp) =
            make_float4(acc[blk][0] * inv, acc[blk][1] * inv, acc[blk][2] * inv, acc[blk][3] * inv);
    if (grp == 0) wl[r_idx] = l_run > 0.f ? m_run * cs2 + __builtin_amdgcn_logf(l_run) : -INFINITY;
}

// merge of the slices: one 32-lane group per (request, q head); it is given the few fields it
// needs rather than the whole parameter block
struct DecodeMergeArgs {
    const void *workspace, *b_start_loc;
    void *o;
    int64_t o_stride[2];
    int32_t batch, num_q_heads, index_bits;
    int32_t head_dim;              // elements of an output row (below HD when the partial rows are padded)
};
template <typename T, int HD, int NB>
__global__ void __launch_bounds__(256)
paged_decode_merge_kernel(const DecodeMergeArgs p, const int nsplit) {
    using E = Elem<T>;
    constexpr int D = HD, LPR = HD / 4;                       // lanes per row (4 elements each)
    const int64_t r = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    if (r >= (int64_t)p.batch * p.num_q_heads) return;
    const int b = (int)(r / p.num_q_heads), h = (int)(r % p.num_q_heads);
    // (the two offsets without a branch on their width -- their low words; they are below 2^31 -- so that both
    // loads are in flight together)
    const int es = p.index_bits >> 3;
    const uint32_t qs32 = *(const uint32_t *)((const char *)p.b_start_loc + (int64_t)b * es);
    const uint32_t qe32 = *(const uint32_t *)((const char *)p.b_start_loc + (int64_t)(b + 1) * es);
    const int64_t qs = qs32;
    if (qe32 - qs32 != 1) return;
    const int d = (threadIdx.x % LPR) * 4;
    if (d >= p.head_dim) return;
    const float *wo = (const float *)p.workspace;
    const float *wl = wo + (int64_t)nsplit * p.batch * p.num_q_heads * D;
    const int64_t rows = (int64_t)p.batch * p.num_q_heads;
    // NB slices per batch (8, or 32 when there are more than 8 slices: a short single request is cut into up to
    // 64), log-sum-exps and partial rows requested together: one memory round trip per batch; batches are
    // chained by a running maximum
    float mx = -INFINITY, wsum = 0.f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < nsplit; s0 += NB) {
        float e[NB];
        float4 v[NB];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int64_t ri = (int64_t)(s0 + j < nsplit ? s0 + j : nsplit - 1) * rows + r;
            e[j] = wl[ri];
            v[j] = *reinterpret_cast<const float4 *>(wo + ri * D + d);
        }
        float bm = e[0];
#pragma unroll
        for (int j = 1; j < NB; ++j) bm = fmaxf(bm, e[j]);
        const float m_new = fmaxf(mx, bm);
        if (m_new == -INFINITY) continue;
        const float keep = __builtin_amdgcn_exp2f(mx - m_new);
        o.x *= keep; o.y *= keep; o.z *= keep; o.w *= keep;
        wsum *= keep;
        mx = m_new;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const float w = s0 + j < nsplit ? __builtin_amdgcn_exp2f(e[j] - mx) : 0.f;
            o.x = fmaf(w, v[j].x, o.x); o.y = fmaf(w, v[j].y, o.y); o.z = fmaf(w, v[j].z, o.z); o.w = fmaf(w, v[j].w, o.w);
            wsum += w;
        }
    }
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
    T *op = (T *)p.o + qs * p.o_stride[0] + (int64_t)h * p.o_stride[1] + d;
    *reinterpret_cast<uint2 *>(op) = make_uint2(E::pack(o.x * inv, o.y * inv), E::pack(o.z * inv, o.w * inv));
}

// The same merge for a handful of rows and many slices (one or a few requests cut into up to 64 slices): a whole
// workgroup per row, its 256 lanes = G groups of HD/4; group g takes slices g, g + G, ... (at most eight: all of
// their loads are in flight together), and the G partial results meet in LDS.  With one 32-lane group per row the
// four workgroups of a single request's 32 rows each pulled 160 KB through one CU in two dependent rounds.
template <typename T, int HD>
__global__ void __launch_bounds__(256)
paged_decode_merge_wide_kernel(const DecodeMergeArgs p, const int nsplit) {
    using E = Elem<T>;
    constexpr int D = HD, LPR = HD / 4, G = 256 / LPR, PER = 64 / G;      // PER: slices per group when there are 64
    __shared__ float sm[G][LPR][4];
    __shared__ float se[G][2];
    const int64_t r = blockIdx.x;
    const int b = (int)(r / p.num_q_heads), h = (int)(r % p.num_q_heads);
    const int es = p.index_bits >> 3;
    const uint32_t qs32 = *(const uint32_t *)((const char *)p.b_start_loc + (int64_t)b * es);
    const uint32_t qe32 = *(const uint32_t *)((const char *)p.b_start_loc + (int64_t)(b + 1) * es);
    if (qe32 - qs32 != 1) return;                               // (the whole workgroup: one row)
    const int g = threadIdx.x / LPR, ln = threadIdx.x % LPR, d = ln * 4;
    const float *wo = (const float *)p.workspace;
    const float *wl = wo + (int64_t)nsplit * p.batch * p.num_q_heads * D;
    const int64_t rows = (int64_t)p.batch * p.num_q_heads;
    float e[PER];
    float4 v[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int sl = g + j * G;
        const int64_t ri = (int64_t)(sl < nsplit ? sl : nsplit - 1) * rows + r;
        e[j] = wl[ri];
        v[j] = *reinterpret_cast<const float4 *>(wo + ri * D + d);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; ++j) mx = fmaxf(mx, g + j * G < nsplit ? e[j] : -INFINITY);
    float wsum = 0.f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    if (mx != -INFINITY) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const float w = g + j * G < nsplit ? __builtin_amdgcn_exp2f(e[j] - mx) : 0.f;
            o.x = fmaf(w, v[j].x, o.x); o.y = fmaf(w, v[j].y, o.y); o.z = fmaf(w, v[j].z, o.z); o.w = fmaf(w, v[j].w, o.w);
            wsum += w;
        }
    }
    *reinterpret_cast<float4 *>(&sm[g][ln][0]) = o;
    if (ln == 0) { se[g][0] = mx; se[g][1] = wsum; }
    __syncthreads();
    if (g != 0 || d >= p.head_dim) return;
    float m_all = -INFINITY;
#pragma unroll
    for (int k = 0; k < G; ++k) m_all = fmaxf(m_all, se[k][0]);
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    float w_all = 0.f;
    if (m_all != -INFINITY) {
#pragma unroll
        for (int k = 0; k < G; ++k) {
            const float c = __builtin_amdgcn_exp2f(se[k][0] - m_all);        // (a group without keys: exp2(-inf) = 0)
            const float4 ok = *reinterpret_cast<const float4 *>(&sm[k][ln][0]);
            t.x = fmaf(c, ok.x, t.x); t.y = fmaf(c, ok.y, t.y); t.z = fmaf(c, ok.z, t.z); t.w = fmaf(c, ok.w, t.w);
            w_all = fmaf(c, se[k][1], w_all);
        }
    }
    const float inv = w_all > 0.f ? 1.f / w_all : 0.f;
    T *op = (T *)p.o + (int64_t)qs32 * p.o_stride[0] + (int64_t)h * p.o_stride[1] + d;
    *reinterpret_cast<uint2 *>(op) = make_uint2(E::pack(t.x * inv, t.y * inv), E::pack(t.z * inv, t.w * inv));
}

// ------------------------------------------------------------------ host side
// width of the lane layout and of a partial row: the head size, or 128 for the head sizes that are padded to it
static int decode_tile_dim(const lazyattn_prefill_params &p) { return p.head_dim == 64 ? 64 : 128; }

bool decode_mfma_supports(const lazyattn_prefill_params &p) {
    const bool fp8 = p.cache_dtype == LAZYATTN_FP8_E4M3 || p.cache_dtype == LAZYATTN_FP8_E5M2;
    if ((p.dtype != LAZYATTN_BF16 && p.dtype != LAZYATTN_F16) || !(p.cache_dtype == p.dtype || fp8)) return false;
    if (p.table_dtype != p.dtype && p.table_dtype != LAZYATTN_F32) return false;
    // 128, 64, or a multiple of 16 below 128 (padded to 128)
    if (p.head_dim < 16 || p.head_dim > 128 || p.head_dim % 16 || p.rotary_dim != p.head_dim) return false;
    if ((p.block_size != BS && p.block_size != 2 * BS) || p.x != (fp8 ? 16 : 8)) return false;
    if (p.pos_mode != LAZYATTN_POS_NATURAL && p.pos_mode != LAZYATTN_POS_BLOCK_UNIFORM) return false;
    if (p.q_stride[2] != 1 || p.o_stride[2] != 1) return false;
    if (p.kc_stride[4] != 1 || p.kc_stride[3] != p.x || p.kc_stride[2] != (int64_t)p.block_size * p.x) return false;
    if (p.vc_stride[3] != 1 || p.vc_stride[2] != p.block_size) return false;
    const int64_t al[] = {p.q_stride[0], p.q_stride[1], p.o_stride[0], p.o_stride[1], p.kc_stride[0], p.kc_stride[1],
                          p.vc_stride[0], p.vc_stride[1], p.rope_freqs ? 0 : p.table_stride};
    for (int64_t s : al)
        if (s % 16) return false;                      // 16-byte rows whatever the element size
    const void *ptrs[] = {p.q, p.o, p.k_cache, p.v_cache, p.cos_sin_cache};
    for (const void *q : ptrs)
        if (((uintptr_t)q) & 15) return false;
    if (((uintptr_t)p.packed_block_table & 7) || ((uintptr_t)p.rope_freqs & 3)) return false;
    return true;
}

// Slices of the page axis per (request, kv head).  A workgroup is four independent waves, one work item each; the
// launch is fastest when its workgroups fit the chip's CUs (256 where these were measured) in one round with none left over -- a few CUs with a
// second workgroup make the tail of the launch (32 requests of 5 K keys: 4 / 6 / 8 slices = 256 / 384 / 512
// workgroups take 118 / 141 / 123 us; 12 requests: 8 / 12 / 16 slices = 192 / 288 / 384 workgroups 49 / 60 / 50 us) --
// so: as many slices as keep the work items at or below 1 024, of at least five pages each (5 K keys, call = both
// launches: one request 16 / 32 / 64 slices 27.4 / 19.8 / 13.7 us).
static int decode_splits(const lazyattn_prefill_params &p) {
    if (p.num_splits > 0) return p.num_splits > 64 ? 64 : p.num_splits;
    const int64_t natural = (int64_t)p.batch * p.num_kv_heads * ((p.num_q_heads / p.num_kv_heads + 15) / 16);
    if (natural <= 0) return 1;
    // (or at or below two, three, four times as many -- whole rounds -- when that fills the rounds at least a tenth
    // better: 48 requests = 384 items, 2 / 5 slices fill 75 % of one / 94 % of two rounds: 189 / 181 us)
    const int64_t round = (int64_t)device_cus() * WAVES;
    int64_t s = round / natural;
    double fill = (double)(natural * s) / (double)round;
    for (int64_t k = 2; k <= 4; ++k) {
        const int64_t sk = k * round / natural;
        const double fk = (double)(natural * sk) / (double)(k * round);
        if (fk > fill * 1.1) { s = sk; fill = fk; }
    }
    const int64_t pages = p.max_seq_len > 0 ? (p.max_seq_len + BS - 1) / BS : 64;
    if (s > pages / 5) s = pages / 5;
    if (s > 64) s = 64;
    return s < 1 ? 1 : (int)s;
}

size_t decode_workspace_bytes(const lazyattn_prefill_params &p) {
    const int ns = decode_splits(p);
    if (ns <= 1) return 0;
    return (size_t)ns * (size_t)p.batch * p.num_q_heads * (decode_tile_dim(p) + 1) * sizeof(float);
}

int launch_decode_mfma(const lazyattn_prefill_params &p, hipStream_t stream) {
    int nsplit = decode_splits(p);
    if (nsplit > 1) {
        // without room for the partials the call still runs, one slice per request and kv head
        const size_t need = (size_t)nsplit * (size_t)p.batch * p.num_q_heads * (decode_tile_dim(p) + 1) * sizeof(float);
        if (!p.workspace || (size_t)p.workspace_bytes < need || (((uintptr_t)p.workspace) & 15)) nsplit = 1;
    }
    const int phases = p.phases ? p.phases : LAZYATTN_PHASE_ALL;
    const int64_t waves = (int64_t)p.batch * p.num_kv_heads * ((p.num_q_heads / p.num_kv_heads + 15) / 16) * nsplit;
    const unsigned nblocks = (unsigned)((waves + WAVES - 1) / WAVES);
    if (phases & LAZYATTN_PHASE_MAIN) {
        const bool t32 = p.table_dtype == LAZYATTN_F32;
        const int fp8 = p.cache_dtype == LAZYATTN_FP8_E4M3 ? 1 : p.cache_dtype == LAZYATTN_FP8_E5M2 ? 2 : 0;   // kind of cache page
        const dim3 grid(nblocks), block(WAVES * 64);
        auto launch = [&](auto elem, auto hd, auto pad) {
            using T = decltype(elem);
            constexpr int HD = decltype(hd)::value;
            constexpr bool PAD = decltype(pad)::value;
            if (p.rope_freqs) {
                if (fp8 == 1) hipLaunchKernelGGL((paged_decode_kernel<T, T, 1, HD, PAD, true>), grid, block, 0, stream, p, nsplit);
                else if (fp8 == 2) hipLaunchKernelGGL((paged_decode_kernel<T, T, 2, HD, PAD, true>), grid, block, 0, stream, p, nsplit);
                else hipLaunchKernelGGL((paged_decode_kernel<T, T, 0, HD, PAD, true>), grid, block, 0, stream, p, nsplit);
            }
            else if (fp8 == 1 && t32) hipLaunchKernelGGL((paged_decode_kernel<T, float, 1, HD, PAD, false>), grid, block, 0, stream, p, nsplit);
            else if (fp8 == 1) hipLaunchKernelGGL((paged_decode_kernel<T, T, 1, HD, PAD, false>), grid, block, 0, stream, p, nsplit);
            else if (fp8 == 2 && t32) hipLaunchKernelGGL((paged_decode_kernel<T, float, 2, HD, PAD, false>), grid, block, 0, stream, p, nsplit);
            else if (fp8 == 2) hipLaunchKernelGGL((paged_decode_kernel<T, T, 2, HD, PAD, false>), grid, block, 0, stream, p, nsplit);
            else if (t32) hipLaunchKernelGGL((paged_decode_kernel<T, float, 0, HD, PAD, false>), grid, block, 0, stream, p, nsplit);
            else hipLaunchKernelGGL((paged_decode_kernel<T, T, 0, HD, PAD, false>), grid, block, 0, stream, p, nsplit);
        };
        using hd128 = std::integral_constant<int, 128>;
        using hd64 = std::integral_constant<int, 64>;
        using yes = std::true_type;
        using no = std::false_type;
        if (p.head_dim == 64) { if (p.dtype == LAZYATTN_F16) launch(f16_t{}, hd64{}, no{}); else launch(bf16_t{}, hd64{}, no{}); }
        else if (p.head_dim == 128) { if (p.dtype == LAZYATTN_F16) launch(f16_t{}, hd128{}, no{}); else launch(bf16_t{}, hd128{}, no{}); }
        else { if (p.dtype == LAZYATTN_F16) launch(f16_t{}, hd128{}, yes{}); else launch(bf16_t{}, hd128{}, yes{}); }
        if (hipGetLastError() != hipSuccess) return LAZYATTN_E_LAUNCH;
    }
    if (nsplit > 1 && (phases & LAZYATTN_PHASE_COMBINE)) {
        const int64_t rows = (int64_t)p.batch * p.num_q_heads;
        const DecodeMergeArgs m{p.workspace, p.b_start_loc, p.o, {p.o_stride[0], p.o_stride[1]}, p.batch, p.num_q_heads, p.index_bits, p.head_dim};
        const int rows_wg = 256 / (decode_tile_dim(p) / 4);
        const dim3 mgrid((unsigned)((rows + rows_wg - 1) / rows_wg));
        const bool f16 = p.dtype == LAZYATTN_F16;
#define LAZYATTN_DECODE_MERGE(HD, NB)                                                                                   \
    {                                                                                                                   \
        if (f16) hipLaunchKernelGGL((paged_decode_merge_kernel<f16_t, HD, NB>), mgrid, dim3(256), 0, stream, m, nsplit); \
        else hipLaunchKernelGGL((paged_decode_merge_kernel<bf16_t, HD, NB>), mgrid, dim3(256), 0, stream, m, nsplit);    \
    }
        if (nsplit > 8 && rows <= 512) {
            // few rows, many slices: a workgroup per row
            const dim3 wgrid((unsigned)rows);
            if (p.head_dim == 64) {
                if (f16) hipLaunchKernelGGL((paged_decode_merge_wide_kernel<f16_t, 64>), wgrid, dim3(256), 0, stream, m, nsplit);
                else hipLaunchKernelGGL((paged_decode_merge_wide_kernel<bf16_t, 64>), wgrid, dim3(256), 0, stream, m, nsplit);
            } else {
                if (f16) hipLaunchKernelGGL((paged_decode_merge_wide_kernel<f16_t, 128>), wgrid, dim3(256), 0, stream, m, nsplit);
                else hipLaunchKernelGGL((paged_decode_merge_wide_kernel<bf16_t, 128>), wgrid, dim3(256), 0, stream, m, nsplit);
            }
        } else if (p.head_dim == 64) {
            if (nsplit <= 8) LAZYATTN_DECODE_MERGE(64, 8) else LAZYATTN_DECODE_MERGE(64, 32)
        } else {
            if (nsplit <= 8) LAZYATTN_DECODE_MERGE(128, 8) else LAZYATTN_DECODE_MERGE(128, 32)
        }
#undef LAZYATTN_DECODE_MERGE
        if (hipGetLastError() != hipSuccess) return LAZYATTN_E_LAUNCH;
    }
    return LAZYATTN_OK;
}

}  // namespace lazyattn
