// Deferred-RoPE prefix-prefill attention on the gfx950 matrix cores (bf16 MFMA).
//
// Work decomposition.  The query rows that share one kv-head -- `group` q-heads x q_len
// tokens -- are cut into units of 32 rows (one q-head, 32 consecutive tokens).  A
// workgroup of NW waves owns NW consecutive units (unit = chunk * group + head_in_group,
// so with group = 4 the four heads of one token chunk sit side by side) and a slice of
// the key axis (split-KV).  Every 64-key tile of paged K is therefore gathered from HBM,
// rotated and written to LDS ONCE for all NW*32 rows, instead of once per q-head as the
// reference's grid (batch, q_head, m_tile) does (ops/prefix_prefill.py:681-682).
//
// Per 64-key tile:
//   gather   4 pages of K ([D/x][16][x], 4 KB each for bf16) with 16-byte loads, the
//            matching cos/sin rows, and 4 pages of V ([D][16]);
//   rotate   k1*c - k2*s, k1*s + k2*c in fp32 registers, one rounding to bf16
//            (old_ops/prefix_prefill.py:248-257 with FORCE_FP32_ROTARY), write to LDS in
//            the cache's own [page][D/8][slot][8] order, which is exactly the A-operand
//            order of v_mfma_f32_32x32x16_bf16;
//   S^T      = K . Q^T (keys x rows), 32x32x16 MFMA, Q fragments stay in registers;
//   softmax  per lane one query row; row max via one v_permlane32_swap; exp2 with
//            sm_scale*log2(e) folded into one fma (old_ops:287-291);
//   O^T     += V^T . P^T: the S^T accumulator registers ARE the B operand (the k index of
//            the MFMA is permuted so that no shuffle is needed), V^T comes from LDS.
// The new tokens' K/V (old_ops:326-396) are appended as further tiles with a causal mask.
// With more than one split every workgroup writes (O/l, log2-sum-exp) partials and a
// second kernel merges them.
#include "common.hpp"

namespace lazyattn {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;

constexpr int D = 128;          // head_dim
constexpr int HALF = 64;
constexpr int BS = 16;          // page size (tokens)
constexpr int NT = 64;          // keys per tile
constexpr int PAGES = NT / BS;  // pages per tile
constexpr int UNIT = 32;        // query rows per wave
// LDS tile layouts (bytes)
constexpr int K_PAGE = 4096;            // [d8 = 16][slot = 16][8 bf16]
constexpr int K_TILE = PAGES * K_PAGE;  // 16 KB
constexpr int V_SG = 1024 + 64;         // [sg = slot/4][d = 128][4 slots], padded
constexpr int V_PAGE = 4 * V_SG;
constexpr int V_TILE = PAGES * V_PAGE;  // 17 KB
constexpr int LDS_BYTES = 2 * (K_TILE + V_TILE);

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
// value of x in the partner lane (lane ^ 32) of a 64-wide wave, via v_permlane32_swap.
// The two operands are kept distinct registers on purpose.
__device__ __forceinline__ float partner32(float x) {
    uint32_t a = __float_as_uint(x), b = a;
    asm volatile("" : "+v"(b));
    auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    // r[0] = {a.lo, b.lo}, r[1] = {a.hi, b.hi}: lanes < 32 want r[1], lanes >= 32 want r[0]
    return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    f32x2_t f = {a, b};
    bf16x2_t h = __builtin_convertvector(f, bf16x2_t);   // v_cvt_pk_bf16_f32, RNE
    return *reinterpret_cast<uint32_t *>(&h);
}

// 8 consecutive table entries as floats
template <typename TT> struct TabVec;
template <> struct TabVec<bf16_t> {
    uint4 v;
    __device__ __forceinline__ void load(const void *p) { v = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ void identity(bool cosine) {
        const uint32_t w = cosine ? 0x3f803f80u : 0u;
        v = make_uint4(w, w, w, w);
    }
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = (&v.x)[i >> 1];
        return (i & 1) ? bf16_hi(w) : bf16_lo(w);
    }
};
template <> struct TabVec<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const void *p) {
        a = reinterpret_cast<const float4 *>(p)[0];
        b = reinterpret_cast<const float4 *>(p)[1];
    }
    __device__ __forceinline__ void identity(bool cosine) {
        const float w = cosine ? 1.f : 0.f;
        a = make_float4(w, w, w, w); b = a;
    }
    __device__ __forceinline__ float get(int i) const { return i < 4 ? (&a.x)[i] : (&b.x)[i - 4]; }
};

// one K work item: 8 (d, d+64) pairs of one key
template <typename TT> struct KItem {
    uint4 k1, k2;        // raw: 8 bf16 each, or 8 fp8 in .x/.y
    TabVec<TT> c, s;
    int lds_off;         // byte offset of chunk d8 inside the K tile; chunk d8+8 is +8*256
    int kind;            // 0 = zero fill, 1 = bf16, 2 = fp8 e4m3
};
struct VItem {
    uint4 v;             // ctx bf16: 8 slots of one d; ctx fp8: 16 slots of one d; new: 8 d of one key
    int a0, a1;          // ctx: LDS byte offsets; new: (page, slot) packed
    int lim;             // valid slots in the page (ctx) / 1 = valid (new)
    int kind;            // -1 no item, 1 ctx bf16, 2 ctx fp8, 3 new-token row
};

struct Ctx {
    const lazyattn_prefill_params *p;
    int b, g;
    int64_t qs, q_len, ctx_len;
    int n_pages;         // pages holding context keys
    int pos_mode;
    bool vanilla, rot_new;
    float k_scale, v_scale;
    int t_end;           // new-token keys this workgroup can see: [0, t_end)
};

// valid slots of context page j: slot < lim
__device__ __forceinline__ int page_limit(const Ctx &c, int j) {
    if (j >= c.n_pages) return 0;
    int64_t lim = c.ctx_len - (int64_t)j * BS;
    if (lim > BS) lim = BS;
    if (!c.vanilla && c.p->q_mask) {
        const int qm = c.p->q_mask[c.b * c.p->qm_stride[0] + j * c.p->qm_stride[1]];   // old_ops:165-167
        if (BS - qm < lim) lim = BS - qm;
    }
    return lim < 0 ? 0 : (int)lim;
}

template <typename TT>
__device__ __forceinline__ void load_table(const Ctx &c, KItem<TT> &it, int64_t pos, int cp) {
    const TT *tab = (const TT *)c.p->cos_sin_cache + pos * c.p->table_stride + cp * 8;
    it.c.load(tab);
    it.s.load(tab + HALF);
}

// ---- issue the global loads of one K item of tile `tile` ----
template <bool FP8, typename TT>
__device__ __forceinline__ void load_k_item(const Ctx &c, KItem<TT> &it, int tile, int n_ctx_tiles, int idx) {
    const lazyattn_prefill_params &p = *c.p;
    it.kind = 0;
    it.k1 = make_uint4(0, 0, 0, 0); it.k2 = it.k1;
    if (tile < n_ctx_tiles) {
        const int o = idx & 15, cp = (idx >> 4) & 7, pg = idx >> 7;
        const int j = tile * PAGES + pg;
        it.lds_off = pg * K_PAGE + cp * 256 + o * 16;
        if (j >= c.n_pages) return;
        const int64_t pb = p.block_table[c.b * p.bt_stride[0] + j * p.bt_stride[1]];
        int64_t pos = -1;
        if (!c.vanilla) {
            if (c.pos_mode == LAZYATTN_POS_NATURAL) {
                pos = (int64_t)j * BS + o;                                          // old_ops:183-184
            } else {
                const int qo = p.q_offset[c.b * p.qo_stride[0] + j * p.qo_stride[1]];
                if (c.pos_mode == LAZYATTN_POS_OFFSET) pos = qo ? (int64_t)qo - 1 + o : (int64_t)j * BS + o;
                else pos = qo ? (int64_t)qo - 1 : 0;                                // ops:180-186
            }
        }
        if (FP8) {
            // [D/16][16 slots][16]: this item takes 8 bytes of chunk cp/2 and of chunk cp/2+4
            const uint8_t *kc = (const uint8_t *)p.k_cache + pb * p.kc_stride[0] + (int64_t)c.g * p.kc_stride[1] +
                                (cp >> 1) * p.kc_stride[2] + o * 16 + (cp & 1) * 8;
            const uint2 a = *reinterpret_cast<const uint2 *>(kc);
            const uint2 b2 = *reinterpret_cast<const uint2 *>(kc + 4 * p.kc_stride[2]);
            it.k1.x = a.x; it.k1.y = a.y; it.k2.x = b2.x; it.k2.y = b2.y;
            it.kind = 2;
        } else {
            const bf16_t *kc = (const bf16_t *)p.k_cache + pb * p.kc_stride[0] + (int64_t)c.g * p.kc_stride[1] +
                               cp * p.kc_stride[2] + o * 8;
            it.k1 = *reinterpret_cast<const uint4 *>(kc);
            it.k2 = *reinterpret_cast<const uint4 *>(kc + 8 * p.kc_stride[2]);
            it.kind = 1;
        }
        if (pos >= 0) load_table<TT>(c, it, pos, cp);
        else { it.c.identity(true); it.s.identity(false); }
    } else {
        // new-token keys: [T, Hkv, D] rows
        const int cp = idx & 7, kl = idx >> 3;
        const int m = (tile - n_ctx_tiles) * NT + kl;
        it.lds_off = (kl >> 4) * K_PAGE + cp * 256 + (kl & 15) * 16;
        if (m >= c.t_end) return;
        const bf16_t *kn = (const bf16_t *)p.k + (c.qs + m) * p.k_stride[0] + (int64_t)c.g * p.k_stride[1] + cp * 8;
        it.k1 = *reinterpret_cast<const uint4 *>(kn);
        it.k2 = *reinterpret_cast<const uint4 *>(kn + HALF);
        it.kind = 1;
        if (c.rot_new) load_table<TT>(c, it, c.ctx_len + m, cp);                    // old_ops:342-343
        else { it.c.identity(true); it.s.identity(false); }
    }
}

__device__ __forceinline__ void fp8x8_to_f32(uint32_t lo, uint32_t hi, float scale, float *out) {
    // (the word-select form of the conversion crashes this compiler's copy propagation)
    f32x2_t a = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false), b = __builtin_amdgcn_cvt_pk_f32_fp8(lo >> 16, false);
    f32x2_t c2 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false), d2 = __builtin_amdgcn_cvt_pk_f32_fp8(hi >> 16, false);
    out[0] = a[0] * scale; out[1] = a[1] * scale; out[2] = b[0] * scale; out[3] = b[1] * scale;
    out[4] = c2[0] * scale; out[5] = c2[1] * scale; out[6] = d2[0] * scale; out[7] = d2[1] * scale;
}

// ---- rotate one K item in fp32 and write both chunks to the LDS tile ----
template <typename TT>
__device__ __forceinline__ void rotate_store_k(const KItem<TT> &it, uint8_t *ktile, float k_scale) {
    uint4 r1, r2;
    if (it.kind == 0) {
        r1 = make_uint4(0, 0, 0, 0); r2 = r1;
    } else {
        float a[8], b[8];
        if (it.kind == 2) {
            fp8x8_to_f32(it.k1.x, it.k1.y, k_scale, a);
            fp8x8_to_f32(it.k2.x, it.k2.y, k_scale, b);
#pragma unroll
            for (int i = 0; i < 8; ++i) {          // (x.f32 * k_scale).to(bf16): old_ops:239-241
                a[i] = round_to<bf16_t>(a[i]);
                b[i] = round_to<bf16_t>(b[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w1 = (&it.k1.x)[i], w2 = (&it.k2.x)[i];
                a[2 * i] = bf16_lo(w1); a[2 * i + 1] = bf16_hi(w1);
                b[2 * i] = bf16_lo(w2); b[2 * i + 1] = bf16_hi(w2);
            }
        }
        float x[8], y[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float cs = it.c.get(i), sn = it.s.get(i);
            x[i] = a[i] * cs - b[i] * sn;                                           // old_ops:253
            y[i] = a[i] * sn + b[i] * cs;                                           // old_ops:254
        }
        r1 = make_uint4(pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(x[4], x[5]), pack_bf16(x[6], x[7]));
        r2 = make_uint4(pack_bf16(y[0], y[1]), pack_bf16(y[2], y[3]), pack_bf16(y[4], y[5]), pack_bf16(y[6], y[7]));
    }
    *reinterpret_cast<uint4 *>(ktile + it.lds_off) = r1;
    *reinterpret_cast<uint4 *>(ktile + it.lds_off + 8 * 256) = r2;
}

// ---- V items ----
template <bool FP8>
__device__ __forceinline__ void load_v_item(const Ctx &c, VItem &it, int tile, int n_ctx_tiles, int idx) {
    const lazyattn_prefill_params &p = *c.p;
    it.kind = 0;
    it.v = make_uint4(0, 0, 0, 0);
    if (tile < n_ctx_tiles) {
        if (FP8) {
            // [D][16 slots] bytes: one item = all 16 slots of one d
            const int d = idx & 127, pg = idx >> 7;
            const int j = tile * PAGES + pg;
            it.a0 = pg * V_PAGE + d * 8;
            it.lim = page_limit(c, j);
            it.kind = 2;
            if (it.lim <= 0) return;                     // stored as zeros
            const int64_t pb = p.block_table[c.b * p.bt_stride[0] + j * p.bt_stride[1]];
            const uint8_t *vc = (const uint8_t *)p.v_cache + pb * p.vc_stride[0] + (int64_t)c.g * p.vc_stride[1] + d * 16;
            it.v = *reinterpret_cast<const uint4 *>(vc);
            it.kind = 2;
        } else {
            // [D][16 slots] bf16: one item = 8 slots (half a row) of one d
            const int d = idx & 127, hf = (idx >> 7) & 1, pg = idx >> 8;
            const int j = tile * PAGES + pg;
            it.a0 = pg * V_PAGE + (2 * hf) * V_SG + d * 8;
            it.a1 = hf;
            it.lim = page_limit(c, j);
            it.kind = 1;
            if (it.lim <= 0) return;                     // stored as zeros
            const int64_t pb = p.block_table[c.b * p.bt_stride[0] + j * p.bt_stride[1]];
            const bf16_t *vc = (const bf16_t *)p.v_cache + pb * p.vc_stride[0] + (int64_t)c.g * p.vc_stride[1] +
                               d * 16 + hf * 8;
            it.v = *reinterpret_cast<const uint4 *>(vc);
            it.kind = 1;
        }
    } else {
        const int dc = idx & 15, kl = idx >> 4;          // 8 d of one new-token key
        const int m = (tile - n_ctx_tiles) * NT + kl;
        it.a0 = (kl >> 4) * V_PAGE + ((kl & 15) >> 2) * V_SG + (dc * 8) * 8 + (kl & 3) * 2;
        it.kind = 3;
        if (m >= c.t_end) return;                        // stays zero
        const bf16_t *vn = (const bf16_t *)p.v + (c.qs + m) * p.v_stride[0] + (int64_t)c.g * p.v_stride[1] + dc * 8;
        it.v = *reinterpret_cast<const uint4 *>(vn);
    }
}

__device__ __forceinline__ void store_v_item(const VItem &it, uint8_t *vtile, float v_scale) {
    if (it.kind == 3) {
        // one key, 8 d: scatter 2-byte entries into [sg][d][slot%4]
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = (&it.v.x)[i];
            *reinterpret_cast<uint16_t *>(vtile + it.a0 + (2 * i) * 8) = (uint16_t)(w & 0xffffu);
            *reinterpret_cast<uint16_t *>(vtile + it.a0 + (2 * i + 1) * 8) = (uint16_t)(w >> 16);
        }
        return;
    }
    if (it.kind == 2) {
        // 16 fp8 slots of one d -> bf16, four 8-byte groups of 4 slots
        const uint32_t *w = &it.v.x;
#pragma unroll
        for (int sg = 0; sg < 4; ++sg) {
            f32x2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[sg], false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[sg] >> 16, false);
            float f[4] = {lo[0] * v_scale, lo[1] * v_scale, hi[0] * v_scale, hi[1] * v_scale};
#pragma unroll
            for (int s = 0; s < 4; ++s)
                if (sg * 4 + s >= it.lim) f[s] = 0.f;    // masked slots contribute nothing, whatever they hold
            uint2 out = make_uint2(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]));
            *reinterpret_cast<uint2 *>(vtile + it.a0 + sg * V_SG) = out;
        }
        return;
    }
    uint4 v = it.v;
    if (it.lim < BS) {
        const int first = it.a1 * 8;                     // slot of element 0
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t w = (&v.x)[i];
            if (first + 2 * i >= it.lim) w &= 0xffff0000u;
            if (first + 2 * i + 1 >= it.lim) w &= 0x0000ffffu;
            (&v.x)[i] = w;
        }
    }
    *reinterpret_cast<uint2 *>(vtile + it.a0) = make_uint2(v.x, v.y);
    *reinterpret_cast<uint2 *>(vtile + it.a0 + V_SG) = make_uint2(v.z, v.w);
}

}  // namespace

template <int NW, bool FP8, typename TT>
__global__ void __launch_bounds__(NW * 64)
prefill_mfma_kernel(const lazyattn_prefill_params p, const int nsplit, const int n_mt) {
    constexpr int NTHREADS = NW * 64;
    constexpr int K_ITEMS = (NT * 8) / NTHREADS;                 // 512 K items per tile
    constexpr int V_TOTAL = FP8 ? PAGES * D : PAGES * D * 2;     // ctx V items per tile
    constexpr int V_ITEMS = (PAGES * D * 2) / NTHREADS;          // new-token tiles: 64 keys x 16 chunks
    static_assert(K_ITEMS >= 1 && V_ITEMS >= 1, "tile too small for the workgroup");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, gh = lane >> 5;

    // ---- which work item: consecutive m-tiles of one (request, kv-head, split) share an XCD ----
    const int n_groups = p.batch * p.num_kv_heads * nsplit;
    int mt, kvgrp;
    {
        const int L = blockIdx.x;
        if ((n_groups & 7) == 0) {
            const int xcd = L & 7, q = L >> 3;
            mt = q % n_mt;
            kvgrp = (q / n_mt) * 8 + xcd;
        } else {
            mt = L % n_mt;
            kvgrp = L / n_mt;
        }
    }
    const int split = kvgrp % nsplit;
    const int g = (kvgrp / nsplit) % p.num_kv_heads;
    const int b = kvgrp / (nsplit * p.num_kv_heads);
    const int group = p.num_q_heads / p.num_kv_heads;

    Ctx c;
    c.p = &p; c.b = b; c.g = g;
    c.qs = load_index(p.b_start_loc, b, p.index_bits);
    c.q_len = load_index(p.b_start_loc, b + 1, p.index_bits) - c.qs;
    c.ctx_len = load_index(p.b_seq_len, b, p.index_bits) - c.q_len;
    if (c.q_len <= 0 || c.ctx_len < 0) return;
    if (p.skip_decode && c.q_len == 1) return;                   // old_ops:109-110
    const int n_chunks = (int)((c.q_len + UNIT - 1) / UNIT);
    const int n_units = n_chunks * group;
    if (mt * NW >= n_units) return;                              // block_mask, old_ops:322-328
    const bool lazy_b = p.is_lazy ? p.is_lazy[b] != 0 : true;
    c.pos_mode = p.pos_mode;
    c.vanilla = p.pos_mode == LAZYATTN_POS_BLOCK_UNIFORM && !lazy_b;   // ops:398
    c.rot_new = p.rotate_new_k && !c.vanilla;
    c.n_pages = (int)((c.ctx_len + BS - 1) / BS);
    c.k_scale = FP8 ? *p.k_scale : 1.f;
    c.v_scale = FP8 ? *p.v_scale : 1.f;
    {
        int last_unit = mt * NW + NW - 1;
        if (last_unit > n_units - 1) last_unit = n_units - 1;
        int64_t te = (int64_t)(last_unit / group + 1) * UNIT;
        c.t_end = (int)(te < c.q_len ? te : c.q_len);
    }

    // ---- this wave's rows ----
    const int unit = mt * NW + wave;
    const bool active = unit < n_units;
    const int chunk = active ? unit / group : 0;
    const int h = g * group + (active ? unit % group : 0);
    const int t0 = chunk * UNIT;
    const int64_t row = t0 + l32;                                // token index of this lane's query row
    const bool row_ok = active && row < c.q_len;

    // Q^T fragments: B operand of S^T = K.Q^T, lane = (row l32, d = ks*16 + gh*8 .. +8)
    bf16x8_t qf[8];
    {
        const bf16_t *qp = (const bf16_t *)p.q + (c.qs + row) * p.q_stride[0] + (int64_t)h * p.q_stride[1] + gh * 8;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (row_ok) v = *reinterpret_cast<const uint4 *>(qp + ks * 16);
            qf[ks] = *reinterpret_cast<bf16x8_t *>(&v);
        }
    }

    const int n_ctx_tiles = (c.n_pages + PAGES - 1) / PAGES;
    const int n_new_tiles = (c.t_end + NT - 1) / NT;
    const int n_tiles = n_ctx_tiles + n_new_tiles;
    const int tile_begin = (int)((int64_t)n_tiles * split / nsplit);
    const int tile_end = (int)((int64_t)n_tiles * (split + 1) / nsplit);

    const float cs2 = p.sm_scale * 1.4426950408889634f;          // scores to log2 units
    float m_run = -INFINITY, l_run = 0.f;
    f32x16_t acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

    KItem<TT> kit[K_ITEMS];
    VItem vit[V_ITEMS];

    if (tile_begin < tile_end) {
        // ---- prologue: first tile into buffer 0 ----
#pragma unroll
        for (int i = 0; i < K_ITEMS; ++i) load_k_item<FP8, TT>(c, kit[i], tile_begin, n_ctx_tiles, tid + i * NTHREADS);
        {
            const bool ctx_t = tile_begin < n_ctx_tiles;
#pragma unroll
            for (int i = 0; i < V_ITEMS; ++i) {
                const int idx = tid + i * NTHREADS;
                if (!ctx_t || idx < V_TOTAL) load_v_item<FP8>(c, vit[i], tile_begin, n_ctx_tiles, idx);
                else vit[i] = VItem{make_uint4(0, 0, 0, 0), 0, 0, 0, -1};
            }
        }
#pragma unroll
        for (int i = 0; i < K_ITEMS; ++i) rotate_store_k<TT>(kit[i], lds, c.k_scale);
#pragma unroll
        for (int i = 0; i < V_ITEMS; ++i)
            if (vit[i].kind >= 0) store_v_item(vit[i], lds + 2 * K_TILE, c.v_scale);
    }
    __syncthreads();

    for (int tile = tile_begin; tile < tile_end; ++tile) {
        const int cur = (tile - tile_begin) & 1;
        const uint8_t *ktile = lds + cur * K_TILE;
        const uint8_t *vtile = lds + 2 * K_TILE + cur * V_TILE;
        uint8_t *ktile_n = lds + (cur ^ 1) * K_TILE;
        uint8_t *vtile_n = lds + 2 * K_TILE + (cur ^ 1) * V_TILE;
        const bool has_next = tile + 1 < tile_end;
        const bool is_ctx = tile < n_ctx_tiles;
        const bool next_ctx = tile + 1 < n_ctx_tiles;

        if (has_next) {
#pragma unroll
            for (int i = 0; i < K_ITEMS; ++i) load_k_item<FP8, TT>(c, kit[i], tile + 1, n_ctx_tiles, tid + i * NTHREADS);
#pragma unroll
            for (int i = 0; i < V_ITEMS; ++i) {
                const int idx = tid + i * NTHREADS;
                if (!next_ctx || idx < V_TOTAL) load_v_item<FP8>(c, vit[i], tile + 1, n_ctx_tiles, idx);
                else vit[i] = VItem{make_uint4(0, 0, 0, 0), 0, 0, 0, -1};
            }
        }

        // keys of this tile that exist: bit kk of `valid`
        uint64_t valid;
        int m0 = 0;
        if (is_ctx) {
            valid = 0;
#pragma unroll
            for (int pg = 0; pg < PAGES; ++pg) {
                const int lim = page_limit(c, tile * PAGES + pg);
                valid |= (uint64_t)((1u << lim) - 1u) << (pg * BS);
            }
        } else {
            m0 = (tile - n_ctx_tiles) * NT;
            const int n = c.t_end - m0;
            valid = n >= 64 ? ~0ull : ((1ull << n) - 1ull);
        }
        // a new-token tile entirely in this wave's future contributes nothing (causal)
        const bool compute = active && (is_ctx || m0 <= t0 + UNIT - 1);

        if (compute) {
            // ---- S^T = K . Q^T ----
            f32x16_t s[2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[sub][i] = 0.f;
                const uint8_t *kp = ktile + (sub * 2 + (l32 >> 4)) * K_PAGE + gh * 256 + (l32 & 15) * 16;
#pragma unroll
                for (int ks = 0; ks < 8; ++ks) {
                    const bf16x8_t a = *reinterpret_cast<const bf16x8_t *>(kp + ks * 512);
                    s[sub] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s[sub], 0, 0, 0);
                }
            }
            // ---- masks: register i of sub-tile `sub` holds key sub*32 + 8*(i/4) + 4*gh + i%4 ----
            const bool need_mask = (valid != ~0ull) || (!is_ctx && m0 + NT - 1 > t0);
            if (need_mask) {
#pragma unroll
                for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int kk = sub * 32 + 8 * (i >> 2) + 4 * gh + (i & 3);
                        bool ok = (valid >> kk) & 1ull;
                        if (!is_ctx) ok = ok && (m0 + kk <= row);                     // old_ops:371-372
                        if (!ok) s[sub][i] = -INFINITY;
                    }
            }
            // ---- online softmax (old_ops:287-291,312-313) ----
            float mx = s[0][0];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[sub][i]);
            mx = fmaxf(mx, partner32(mx));
            const float m_new = fmaxf(m_run, mx);
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_safe) * cs2);      // -inf -> 0
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[dt][i] *= alpha;
                l_run *= alpha;
            }
            m_run = m_new;
            const float mc = m_safe * cs2;
            float lsum = 0.f;
            bf16x8_t pf[4];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                float pr[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    pr[i] = __builtin_amdgcn_exp2f(fmaf(s[sub][i], cs2, -mc));
                    lsum += pr[i];
                }
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    uint4 w = make_uint4(pack_bf16(pr[8 * t + 0], pr[8 * t + 1]), pack_bf16(pr[8 * t + 2], pr[8 * t + 3]),
                                         pack_bf16(pr[8 * t + 4], pr[8 * t + 5]), pack_bf16(pr[8 * t + 6], pr[8 * t + 7]));
                    pf[sub * 2 + t] = *reinterpret_cast<bf16x8_t *>(&w);
                }
            }
            l_run += lsum;

            if (has_next) {
#pragma unroll
                for (int i = 0; i < K_ITEMS; ++i) rotate_store_k<TT>(kit[i], ktile_n, c.k_scale);
            }

            // ---- O^T += V^T . P^T ; k index j of step kt <-> slots 4*gh + j (j<4), 8 + 4*gh + j-4 ----
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                const uint8_t *vp = vtile + kt * V_PAGE + gh * V_SG + l32 * 8;
#pragma unroll
                for (int dt = 0; dt < 4; ++dt) {
                    const uint2 lo = *reinterpret_cast<const uint2 *>(vp + dt * 256);
                    const uint2 hi = *reinterpret_cast<const uint2 *>(vp + dt * 256 + 2 * V_SG);
                    uint4 w = make_uint4(lo.x, lo.y, hi.x, hi.y);
                    const bf16x8_t a = *reinterpret_cast<bf16x8_t *>(&w);
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[kt], acc[dt], 0, 0, 0);
                }
            }
        } else if (has_next) {
#pragma unroll
            for (int i = 0; i < K_ITEMS; ++i) rotate_store_k<TT>(kit[i], ktile_n, c.k_scale);
        }
        if (has_next) {
#pragma unroll
            for (int i = 0; i < V_ITEMS; ++i)
                if (vit[i].kind >= 0) store_v_item(vit[i], vtile_n, c.v_scale);
        }
        __syncthreads();
    }

    // ---- epilogue ----
    l_run += partner32(l_run);
    if (!row_ok) return;
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    if (nsplit == 1) {
        bf16_t *op = (bf16_t *)p.o + (c.qs + row) * p.o_stride[0] + (int64_t)h * p.o_stride[1];
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int d = dt * 32 + 8 * i4 + 4 * gh;
                uint2 w = make_uint2(pack_bf16(acc[dt][4 * i4] * inv, acc[dt][4 * i4 + 1] * inv),
                                     pack_bf16(acc[dt][4 * i4 + 2] * inv, acc[dt][4 * i4 + 3] * inv));
                *reinterpret_cast<uint2 *>(op + d) = w;
            }
    } else {
        const int64_t T = p.num_tokens;
        float *wo = (float *)p.workspace;
        float *wl = wo + (int64_t)nsplit * T * p.num_q_heads * D;
        const int64_t r_idx = ((int64_t)split * T + (c.qs + row)) * p.num_q_heads + h;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int d = dt * 32 + 8 * i4 + 4 * gh;
                *reinterpret_cast<float4 *>(wo + r_idx * D + d) =
                    make_float4(acc[dt][4 * i4] * inv, acc[dt][4 * i4 + 1] * inv, acc[dt][4 * i4 + 2] * inv,
                                acc[dt][4 * i4 + 3] * inv);
            }
        if (gh == 0) wl[r_idx] = l_run > 0.f ? m_run * cs2 + __builtin_amdgcn_logf(l_run) : -INFINITY;
    }
}

// ---- merge split-KV partials: one 32-lane group per (token, q-head) row ----
__global__ void __launch_bounds__(256)
prefill_combine_kernel(const lazyattn_prefill_params p, const int nsplit) {
    const int b = blockIdx.y;
    const int64_t qs = load_index(p.b_start_loc, b, p.index_bits);
    const int64_t q_len = load_index(p.b_start_loc, b + 1, p.index_bits) - qs;
    if (q_len <= 0 || (p.skip_decode && q_len == 1)) return;
    const int64_t r = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (r >= q_len * p.num_q_heads) return;
    const int64_t tok = qs + r / p.num_q_heads;
    const int h = (int)(r % p.num_q_heads);
    const int d = (threadIdx.x & 31) * 4;
    const int64_t T = p.num_tokens;
    const float *wo = (const float *)p.workspace;
    const float *wl = wo + (int64_t)nsplit * T * p.num_q_heads * D;
    float mx = -INFINITY;
    for (int s = 0; s < nsplit; ++s) mx = fmaxf(mx, wl[((int64_t)s * T + tok) * p.num_q_heads + h]);
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    float wsum = 0.f;
    if (mx != -INFINITY) {
        for (int s = 0; s < nsplit; ++s) {
            const int64_t ri = ((int64_t)s * T + tok) * p.num_q_heads + h;
            const float w = __builtin_amdgcn_exp2f(wl[ri] - mx);
            const float4 v = *reinterpret_cast<const float4 *>(wo + ri * D + d);
            o.x = fmaf(w, v.x, o.x); o.y = fmaf(w, v.y, o.y); o.z = fmaf(w, v.z, o.z); o.w = fmaf(w, v.w, o.w);
            wsum += w;
        }
    }
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
    bf16_t *op = (bf16_t *)p.o + tok * p.o_stride[0] + (int64_t)h * p.o_stride[1] + d;
    *reinterpret_cast<uint2 *>(op) = make_uint2(pack_bf16(o.x * inv, o.y * inv), pack_bf16(o.z * inv, o.w * inv));
}

// ------------------------------------------------------------------ host side
static int mfma_mtiles(const lazyattn_prefill_params &p, int nw) {
    const int group = p.num_q_heads / p.num_kv_heads;
    const int units = ((p.max_q_len + UNIT - 1) / UNIT) * group;
    return (units + nw - 1) / nw;
}

static int mfma_waves(const lazyattn_prefill_params &p) {
    if (p.cache_dtype == LAZYATTN_FP8_E4M3 && p.table_dtype == LAZYATTN_F32) return 8;
    const int group = p.num_q_heads / p.num_kv_heads;
    const int units = ((p.max_q_len + UNIT - 1) / UNIT) * group;
    return units >= 8 ? 8 : 4;
}

static int mfma_splits(const lazyattn_prefill_params &p, int nw) {
    if (p.num_splits > 0) return p.num_splits > 64 ? 64 : p.num_splits;
    const int64_t natural = (int64_t)p.batch * p.num_kv_heads * mfma_mtiles(p, nw);
    const int64_t ctx_tiles = p.max_seq_len > 0 ? (p.max_seq_len + NT - 1) / NT : 1;
    int64_t s = (256 + natural - 1) / natural;        // one workgroup per CU
    if (s > ctx_tiles / 2) s = ctx_tiles / 2;        // at least two tiles per split
    if (s > 64) s = 64;
    return s < 1 ? 1 : (int)s;
}

bool mfma_supports(const lazyattn_prefill_params &p) {
    const bool fp8 = p.cache_dtype == LAZYATTN_FP8_E4M3;
    if (p.dtype != LAZYATTN_BF16) return false;
    if (!(p.cache_dtype == LAZYATTN_BF16 || fp8)) return false;
    if (p.table_dtype != LAZYATTN_BF16 && p.table_dtype != LAZYATTN_F32) return false;
    if (p.head_dim != D || p.block_size != BS || p.x != (fp8 ? 16 : 8)) return false;
    if (p.sliding_window > 0) return false;
    if (p.q_stride[2] != 1 || p.k_stride[2] != 1 || p.v_stride[2] != 1 || p.o_stride[2] != 1) return false;
    if (p.kc_stride[4] != 1 || p.kc_stride[3] != p.x || p.kc_stride[2] != (int64_t)BS * p.x) return false;
    if (p.vc_stride[3] != 1 || p.vc_stride[2] != BS) return false;
    const int64_t al[] = {p.q_stride[0], p.q_stride[1], p.k_stride[0], p.k_stride[1], p.v_stride[0], p.v_stride[1],
                          p.o_stride[0], p.o_stride[1], p.kc_stride[0], p.kc_stride[1], p.vc_stride[0], p.vc_stride[1],
                          p.table_stride};
    for (int64_t s : al)
        if (s % 8) return false;
    const void *ptrs[] = {p.q, p.k, p.v, p.o, p.k_cache, p.v_cache, p.cos_sin_cache};
    for (const void *q : ptrs)
        if (((uintptr_t)q) & 15) return false;
    if (p.num_tokens <= 0) return false;
    return true;
}

size_t mfma_workspace_bytes(const lazyattn_prefill_params &p) {
    const int nw = mfma_waves(p);
    const int ns = mfma_splits(p, nw);
    if (ns <= 1) return 0;
    return (size_t)ns * (size_t)p.num_tokens * p.num_q_heads * (D + 1) * sizeof(float);
}

template <int NW, bool FP8, typename TT>
static int launch_mfma_t(const lazyattn_prefill_params &p, int nsplit, int n_mt, hipStream_t stream) {
    auto kern = prefill_mfma_kernel<NW, FP8, TT>;
    static bool attr_set = false;
    if (!attr_set) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess)
            return LAZYATTN_E_LAUNCH;
        attr_set = true;
    }
    const unsigned nblocks = (unsigned)(p.batch * p.num_kv_heads * nsplit * n_mt);
    hipLaunchKernelGGL(kern, dim3(nblocks), dim3(NW * 64), LDS_BYTES, stream, p, nsplit, n_mt);
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

template <int NW>
static int launch_mfma_nw(const lazyattn_prefill_params &p, int nsplit, int n_mt, hipStream_t stream) {
    const bool fp8 = p.cache_dtype == LAZYATTN_FP8_E4M3;
    const bool t32 = p.table_dtype == LAZYATTN_F32;
    if (fp8) {
        // <4 waves, fp8 cache, f32 table> is not instantiated (it crashes this compiler);
        // launch_prefill_mfma() routes that combination to the 8-wave kernel.
        if constexpr (NW == 8) {
            if (t32) return launch_mfma_t<8, true, float>(p, nsplit, n_mt, stream);
        }
        return launch_mfma_t<NW, true, bf16_t>(p, nsplit, n_mt, stream);
    }
    return t32 ? launch_mfma_t<NW, false, float>(p, nsplit, n_mt, stream)
               : launch_mfma_t<NW, false, bf16_t>(p, nsplit, n_mt, stream);
}

int launch_prefill_mfma(const lazyattn_prefill_params &p, hipStream_t stream) {
    const int nw = mfma_waves(p);
    const int nsplit = mfma_splits(p, nw);
    const int n_mt = mfma_mtiles(p, nw);
    const int phases = p.phases ? p.phases : LAZYATTN_PHASE_ALL;
    if (nsplit > 1) {
        const size_t need = (size_t)nsplit * (size_t)p.num_tokens * p.num_q_heads * (D + 1) * sizeof(float);
        if (!p.workspace || (size_t)p.workspace_bytes < need) return LAZYATTN_E_WORKSPACE;
        if (((uintptr_t)p.workspace) & 15) return LAZYATTN_E_WORKSPACE;
    }
    if (phases & LAZYATTN_PHASE_MAIN) {
        const int rc = nw == 8 ? launch_mfma_nw<8>(p, nsplit, n_mt, stream) : launch_mfma_nw<4>(p, nsplit, n_mt, stream);
        if (rc != LAZYATTN_OK) return rc;
    }
    if (nsplit > 1 && (phases & LAZYATTN_PHASE_COMBINE)) {
        const int64_t rows = (int64_t)p.max_q_len * p.num_q_heads;
        hipLaunchKernelGGL(prefill_combine_kernel, dim3((unsigned)((rows + 7) / 8), p.batch), dim3(256), 0, stream, p,
                           nsplit);
        if (hipGetLastError() != hipSuccess) return LAZYATTN_E_LAUNCH;
    }
    return LAZYATTN_OK;
}

}  // namespace lazyattn
