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
//   gather   4 pages of K ([D/x][16][x], one contiguous 4 KB run per page and kv-head for
//            bf16) with 16-byte loads off a wave-uniform base, the matching cos/sin rows,
//            and 4 pages of V ([D][16]);
//   rotate   k1*c - k2*s, k1*s + k2*c in fp32 registers, one rounding to bf16
//            (old_ops/prefix_prefill.py:248-257 with FORCE_FP32_ROTARY), write to LDS in
//            the cache's own [page][D/8][slot][8] order, which is exactly the A-operand
//            order of v_mfma_f32_32x32x16_bf16;
//   S^T      = K . Q^T (keys x rows) in two 32-key halves, Q fragments re-read from LDS;
//   softmax  per lane one query row; Q carries sm_scale*log2(e) and the accumulators start at
//            minus a per-row reference, so P = exp2(S) directly; the row max (one
//            v_permlane32_swap) only decides when that reference moves (old_ops:287-291);
//   O^T     += V^T . P^T: the S^T accumulator registers ARE the B operand (the k index of
//            the MFMA is permuted so that no shuffle is needed), V^T comes from LDS.
// Tiles come in three kinds: full context tiles (no masking code at all), edge context
// tiles (pad slots / end of context) and new-token tiles (old_ops:326-396, causal mask).
// With more than one split every workgroup writes (O/l, log2-sum-exp) partials and a
// second kernel merges them.
//
// This header holds the kernel template and its launch dispatch.  One translation unit per (element type, kind of
// cache page) instantiates it (prefill_mfma_<type>[_<fp8 kind>].hip), so the 120 instantiations compile side by
// side; prefill_mfma.hip holds the host-side choices (workgroup shape, split count) and the merge kernel.
#pragma once
#include "common.hpp"
#include "elem16.hpp"
#include "fastdiv.hpp"
#include "batch_plan.hpp"
#include <atomic>
#include <type_traits>

namespace lazyattn {

namespace {


constexpr int BS = 16;          // page size (tokens)
constexpr int NT = 64;          // keys per tile
constexpr int PAGES = NT / BS;  // pages per tile
constexpr int UNIT = 32;        // query rows per wave
// LDS tiles (bytes).  K: [page][d8 = 16][slot = 16][8 bf16].
// V: [page][d = 128][2 chunks of 8 slots] -- a cache page's own [d][16 slots] order, 32 bytes per row of d, with the
// two 16-byte chunks of a row swapped where bit 3 of d is set (so that lanes writing both chunks of their own row, as
// the fp8 conversion does, spread over all banks).  A chunk is the 16 bytes one lane feeds to the PV MFMA as its A
// operand: the computing waves read K slot s of a page as MFMA row (s with bits 2 and 3 swapped), which puts the
// scores of slots 8*gh .. 8*gh+7 of a page into one lane's accumulator registers -- chunk gh of the V rows.
// A V tile in LDS is therefore a byte-for-byte copy of four cache pages, and full pages of 16-bit caches go there by
// global -> LDS loads that pass through no register.
// V has three buffers (the loads of tile t+2 land while tile t is read and tile t+1 waits), K two (its way leads
// through the gathering waves' registers, which are the third stage).
// Sizes that follow from the head size HD (128 or 64); a K page is HD * 32 bytes, a V page as well.
template <int HD> struct Geo {
    static constexpr int K_PAGE = HD * 32, K_TILE = PAGES * K_PAGE;
    static constexpr int V_PAGE = HD * 32, V_TILE = PAGES * V_PAGE;
    static constexpr int V_BUFS = 3;
    static constexpr int KV_BYTES = 2 * K_TILE + V_BUFS * V_TILE; // V tiles (first: low LDS addresses), then K tiles: 80 KB at 128
    static constexpr int Q_WAVE = HD * 64;                        // Q^T fragments of one computing wave
    static constexpr int KS = HD / 16, DT = HD / 32;              // k-steps of K.Q^T, 32-row blocks of O^T
    static constexpr int K_ITEMS = HD / 64, V_ITEMS = HD / 32;    // 16-byte items per gathering lane and page
    static constexpr int PAIR = (HD / 16) * 256;                  // bytes from the chunk of d to the chunk of d + HD/2 (16-bit cache)
    static constexpr int PAIR8 = (HD / 32) * 256;                 // ... in an fp8 page
};

enum { TILE_FULL = 0, TILE_EDGE = 1, TILE_NEW = 2 };

// value of x in the partner lane (lane ^ 32) of the wave, via v_permlane32_swap
// IEEE-754 maximum of three (v_maximum3_f32): NaN-propagating, so no canonicalising pre-pass
__device__ __forceinline__ float max3(float a, float b, float c) {
    return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}
__device__ __forceinline__ float partner32(float x, bool upper) {
    uint32_t a = __float_as_uint(x), b = a;
    asm volatile("" : "+v"(b));      // two distinct registers for the swap
    auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    // r[0] = {a.lo, b.lo}, r[1] = {a.hi, b.hi}
    return __uint_as_float(upper ? r[0] : r[1]);
}
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// the divisors of the kernel's prologue
struct MfmaDivs { FastDiv n_mt, nsplit, kv_heads, group; };


typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ldg16(const uint8_t *base, uint32_t off) {
    return *reinterpret_cast<const uint4 *>(base + off);
}
__device__ __forceinline__ u32x4_t ldg16v(const uint8_t *base, uint32_t off) {
    return *reinterpret_cast<const u32x4_t *>(base + off);
}
__device__ __forceinline__ uint2 ldg8(const uint8_t *base, uint32_t off) {
    return *reinterpret_cast<const uint2 *>(base + off);
}
// The same 16-byte load, written as asm: the compiler does not count it among the loads it waits for, and takes the
// value to be there at once.  Whoever uses this owns the wait: settle() below, before anything reads `dst`.
__device__ __forceinline__ void ldg16_uncounted(u32x4_t &dst, const uint8_t *sbase, uint32_t voff) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void ldg16_uncounted_hi(u32x4_t &dst, const uint8_t *sbase, uint32_t voff) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
// 16 bytes per lane from global memory straight into LDS: lane i's bytes (scalar base + its own 32-bit offset) go to
// lds_addr + i * 16.  m0 carries the LDS address; a scalar write of m0 needs one wait state before such a load reads it.
__device__ __forceinline__ void dma16(const uint8_t *sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(sbase), "v"(voff), "s"(lds_addr) : "memory", "m0");
}
// wait until at most N of this wave's vector memory loads are outstanding (they complete in order)
template <int N> __device__ __forceinline__ void wait_vmem() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

// 8 consecutive cos (or sin) table entries
template <typename TT> struct TabVec {                     // a 16-bit table
    u32x4_t v;
    static constexpr int LOADS = 1;
    __device__ __forceinline__ void load(const uint8_t *base, uint32_t off) { v = ldg16v(base, off); }
    __device__ __forceinline__ void load_uncounted(const uint8_t *base, uint32_t off) { ldg16_uncounted(v, base, off); }
    __device__ __forceinline__ void fill(float w) { const uint32_t u = Elem<TT>::splat(w); v = u32x4_t{u, u, u, u}; }
    __device__ __forceinline__ void get(float *f) const {
        f[0] = Elem<TT>::lo(v[0]); f[1] = Elem<TT>::hi(v[0]); f[2] = Elem<TT>::lo(v[1]); f[3] = Elem<TT>::hi(v[1]);
        f[4] = Elem<TT>::lo(v[2]); f[5] = Elem<TT>::hi(v[2]); f[6] = Elem<TT>::lo(v[3]); f[7] = Elem<TT>::hi(v[3]);
    }
};
template <> struct TabVec<float> {
    u32x4_t a, b;
    static constexpr int LOADS = 2;
    __device__ __forceinline__ void load(const uint8_t *base, uint32_t off) {
        a = ldg16v(base, off);
        b = ldg16v(base, off + 16);
    }
    __device__ __forceinline__ void load_uncounted(const uint8_t *base, uint32_t off) {
        ldg16_uncounted(a, base, off);
        ldg16_uncounted_hi(b, base, off);
    }
    __device__ __forceinline__ void fill(float w) { const uint32_t u = __float_as_uint(w); a = u32x4_t{u, u, u, u}; b = a; }
    __device__ __forceinline__ void get(float *f) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) { f[i] = __uint_as_float(a[i]); f[4 + i] = __uint_as_float(b[i]); }
    }
};

template <typename T> __device__ __forceinline__ void unpack8(const uint4 &w, float *f) {
    f[0] = Elem<T>::lo(w.x); f[1] = Elem<T>::hi(w.x); f[2] = Elem<T>::lo(w.y); f[3] = Elem<T>::hi(w.y);
    f[4] = Elem<T>::lo(w.z); f[5] = Elem<T>::hi(w.z); f[6] = Elem<T>::lo(w.w); f[7] = Elem<T>::hi(w.w);
}
template <typename T> __device__ __forceinline__ void unpack8(const u32x4_t &w, float *f) {
    f[0] = Elem<T>::lo(w[0]); f[1] = Elem<T>::hi(w[0]); f[2] = Elem<T>::lo(w[1]); f[3] = Elem<T>::hi(w[1]);
    f[4] = Elem<T>::lo(w[2]); f[5] = Elem<T>::hi(w[2]); f[6] = Elem<T>::lo(w[3]); f[7] = Elem<T>::hi(w[3]);
}
// two fp8 bytes (the low 16 bits of w) -> two floats; KIND 1: e4m3, 2: e5m2
template <int KIND> __device__ __forceinline__ f32x2_t cvt_fp8x2(uint32_t w) {
    if constexpr (KIND == 2) return __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
    else return __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
}
// 8 fp8 bytes -> floats, unscaled
template <int KIND> __device__ __forceinline__ void unpack8_fp8_raw(uint32_t lo, uint32_t hi, float *f) {
    f32x2_t a, b, c, d;
    if constexpr (KIND == 2) {
        a = __builtin_amdgcn_cvt_pk_f32_bf8(lo, false); b = __builtin_amdgcn_cvt_pk_f32_bf8(lo, true);
        c = __builtin_amdgcn_cvt_pk_f32_bf8(hi, false); d = __builtin_amdgcn_cvt_pk_f32_bf8(hi, true);
    } else {
        a = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false); b = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
        c = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false); d = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
    }
    f[0] = a[0]; f[1] = a[1]; f[2] = b[0]; f[3] = b[1]; f[4] = c[0]; f[5] = c[1]; f[6] = d[0]; f[7] = d[1];
}
// two fp8 bytes (low or high half of w) -> two bf16 in one word, exact (every fp8 value is a bf16 value)
template <int KIND, bool HIGH> __device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t w) {
    if constexpr (KIND == 2) return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(w, 1.0f, HIGH));
    else return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, HIGH));
}
// 8 fp8 bytes -> (float * scale) rounded to the query type, as floats  (old_ops:239-241)
template <typename T, int KIND> __device__ __forceinline__ void unpack8_fp8(uint32_t lo, uint32_t hi, float scale, float *f) {
    const f32x2_t a = cvt_fp8x2<KIND>(lo), b = cvt_fp8x2<KIND>(lo >> 16);
    const f32x2_t c = cvt_fp8x2<KIND>(hi), d = cvt_fp8x2<KIND>(hi >> 16);
    const float t[8] = {a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = round_to<T>(t[i] * scale);
}

// one K item in flight: 8 (d, d+64) pairs of one key
template <typename TT> struct KRegs {
    u32x4_t k1, k2;
    TabVec<TT> c, s;
    uint32_t lds_off;
};
// Wait until at most N vector memory loads of this wave are outstanding; the item's registers count as written
// here, so that nothing that reads them can be placed before the wait.
template <int N> __device__ __forceinline__ void settle(KRegs<float> &r) {
    asm volatile("s_waitcnt vmcnt(%6)" : "+v"(r.k1), "+v"(r.k2), "+v"(r.c.a), "+v"(r.c.b), "+v"(r.s.a), "+v"(r.s.b) : "n"(N) : "memory");
}
template <int N, typename TT> __device__ __forceinline__ void settle(KRegs<TT> &r) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(r.k1), "+v"(r.k2), "+v"(r.c.v), "+v"(r.s.v) : "n"(N) : "memory");
}

}  // namespace

// Workgroup = NC computing waves (32 query rows each) followed by the gathering waves.  The
// hardware places wave w on SIMD w % 4, so every SIMD hosts computing and gathering
// waves: the gather's address arithmetic, fp32 rotation and LDS writes run in
// the shadow of the other waves' MFMAs, and neither role ever waits for the other's
// memory latency -- they only meet at one barrier per tile.
// NC = computing waves = 32-row units per workgroup: 8 for long key ranges, 4 when the call is small and more,
// lighter workgroups fill the chip with fewer key-axis splits.  Either way twelve waves (three per SIMD, 168
// registers each) at head size 128: 8 + 4 or 4 + 8; the Q^T fragments then live in LDS and are re-read every tile.
// At head size 64 the four-unit shape has eight waves, two per SIMD, and keeps Q^T in registers.
// Gathering waves: four, one per 16-key page of a tile -- or eight, two per page with half of its items each, for
// the four-unit shape at head size 128: there the gathering wave's serial instruction stream is the longest of a
// SIMD's (one computing + one gathering wave), and two half-length streams beside it are shorter than one.  Twelve
// waves leave 168 registers each, so that shape reads Q^T from LDS as well.
constexpr int gather_waves(int nc, int hd) { return nc == 4 && hd == 128 ? 8 : 4; }
constexpr bool q_in_registers(int nc, int hd) { return nc == 4 && gather_waves(nc, hd) == 4; }
template <int HD> constexpr int lds_bytes(int nc) {      // K and V tiles + Q^T fragments (if in LDS) + page limits
    return Geo<HD>::KV_BYTES + (q_in_registers(nc, HD) ? 0 : nc * Geo<HD>::Q_WAVE) + 2 * PAGES * 4;
}

// WIN: built with the sliding-window code (calls without a window run the instantiation without it)
// PAD: the head size is a multiple of 16 below HD = 128: Q, K and V sit zero-padded in the 128-wide tiles, the two
// halves of the real head at (0 .., 64 ..) so that the rotation pairs stay (d, 64 + d)
template <int NC, int HD, int FP8, bool WIN, bool PAD, typename T, typename TT>
__global__ void __launch_bounds__((NC + gather_waves(NC, HD)) * 64)
prefill_mfma_kernel(const lazyattn_prefill_params p, const int nsplit, const int n_mt, const BatchShape bal, const MfmaDivs dv) {
    using G = Geo<HD>;
    constexpr int D = HD, HALF = HD / 2;
    const int Dr = PAD ? p.head_dim : D, HALFr = Dr / 2, CPr = Dr / 16;   // real head size, its half, its chunk pairs
    constexpr int K_PAGE = G::K_PAGE, K_TILE = G::K_TILE, V_PAGE = G::V_PAGE, V_TILE = G::V_TILE, V_BUFS = G::V_BUFS;
    constexpr int KV_BYTES = G::KV_BYTES, KS = G::KS, DT = G::DT;
    // a page has HD K items (HD/16 chunk pairs x 16 slots) and 2 HD V items (an fp8 page row of 16 slots is one
    // 16-byte item): per lane of the NH gathering waves that share the page.  Item i of a wave's registers is item
    // i * NH + half of the page.
    constexpr int NG = gather_waves(NC, HD), NH = NG / 4;
    constexpr int KI = G::K_ITEMS / NH, VI = G::V_ITEMS / NH;
    constexpr int VI_CTX = FP8 ? VI / 2 : VI;
    static_assert(KI >= 1 && VI_CTX >= 1, "a page's items do not split over this many gathering waves");
    // fp8 pages under bf16 operands: the cache scales leave the gather.  Rotation and P.V are linear, so
    // k_scale goes into the factor Q is multiplied by anyway and v_scale into the final 1/l; the pages' bytes are
    // converted and used as they are (fp8 -> bf16 is exact), and the few new-token keys and values, which are
    // not quantised, are divided by the scales instead.  Against scaling every element and rounding it to bf16
    // first (old_ops:239-241) this saves the gathering waves a multiply and a rounding per element and differs by
    // less than that one rounding (nothing at all for power-of-two scales, 1.0 included).  float16 operands keep
    // the element-wise scaling: raw e5m2 values can leave the half range.
    constexpr bool FOLD = FP8 != 0 && std::is_same<T, bf16_t>::value;
    constexpr uint32_t TSZ = sizeof(TT);
    using E = Elem<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = uniform(tid >> 6);              // in an SGPR: everything derived from it stays scalar
    const bool gatherer = wave >= NC;

    // ---- work item: the m-tiles of one (request, kv-head, split) land on the same XCD ----
    const int group = p.num_q_heads / p.num_kv_heads;
    // mt, split, g, b: this workgroup's m-tile, key-axis split, kv head and request; nsplit_wg: the splits of its
    // request; witem: its number among the work items of its kv head (where its partial rows go)
    int mt, split, g, b, nsplit_wg = nsplit, witem;
    uint32_t split_mul = 0;                          // ceil(2^32 / nsplit_wg) under the balanced list (0: one split)
    if (bal.items_cap > 0) {
        // Balanced list: the grid holds (kv head, I) for I below the number of work items the host made room for; which
        // (request, m-tile, split) item I is, follows from all the requests' lengths (batch_plan.hpp): the first wave
        // works it out and leaves it in LDS for the others, which meanwhile form the per-lane constants below.
        // Workgroups of one kv head stay on one XCD.
        const int L = blockIdx.x, hkv = p.num_kv_heads;
        if ((hkv & 7) == 0) { g = (L & 7) + 8 * ((L >> 3) % (hkv >> 3)); witem = (L >> 3) / (hkv >> 3); }
        else { g = L % hkv; witem = L / hkv; }
        int *found = reinterpret_cast<int *>(lds + lds_bytes<HD>(NC) - 24);      // (behind the page limits, unused otherwise)
        if (wave == 0) {
            const PlanTables tabs{p.b_start_loc, p.b_seq_len, p.batch, p.index_bits};
            PlanItem it;
            if (p.batch <= 64) {                                 // one request per lane: a quarter of the arithmetic
                const PlanLane<1> reqs = plan_load<1>(tabs, bal, lane);
                it = plan_locate(reqs, bal, plan_target(reqs, bal), witem, lane);
            } else if (p.batch <= PLAN_MAX_BATCH) {
                const PlanLane<4> reqs = plan_load<4>(tabs, bal, lane);
                it = plan_locate(reqs, bal, plan_target(reqs, bal), witem, lane);
            } else {
                it = plan_locate_chunks(tabs, bal, witem, lane);
            }
            if (lane == 0) {
                found[0] = it.b; found[1] = it.mt; found[2] = it.split; found[3] = it.nsplit;
                found[4] = it.nsplit > 1 ? (int)(0xffffffffu / (uint32_t)it.nsplit + 1u) : 0;
                // the first work item of a request tells the merge where the request's items start and how many
                // splits it has
                if (it.b >= 0 && it.mt == 0 && it.split == 0 && g == 0 && bal.table_bytes > 0)
                    reinterpret_cast<PlanRecord *>(p.workspace)[it.b] = PlanRecord{it.item_base, it.nsplit, 0, 0};
            }
        }
        __syncthreads();
        b = uniform(found[0]); mt = uniform(found[1]); split = uniform(found[2]); nsplit_wg = uniform(found[3]);
        split_mul = (uint32_t)uniform(found[4]);
        if (b < 0) return;
    } else {
        const int n_groups = p.batch * p.num_kv_heads * nsplit;
        int kvgrp;
        const int L = blockIdx.x;
        if (((p.batch * p.num_kv_heads) & 7) == 0) {
            // every split and m-tile of one (request, kv-head) on one XCD: they share K/V through its L2
            const int xcd = L & 7, q = L >> 3;
            const int r = (int)dv.n_mt.quot(q);
            mt = (int)dv.n_mt.rem(q, r);
            const int rs = (int)dv.nsplit.quot(r);
            kvgrp = (rs * 8 + xcd) * nsplit + (int)dv.nsplit.rem(r, rs);
        } else if ((n_groups & 7) == 0) {
            const int xcd = L & 7, q = L >> 3;
            const int r = (int)dv.n_mt.quot(q);
            mt = (int)dv.n_mt.rem(q, r);
            kvgrp = r * 8 + xcd;
        } else {
            kvgrp = (int)dv.n_mt.quot(L);
            mt = (int)dv.n_mt.rem(L, kvgrp);
        }
        const int bg = (int)dv.nsplit.quot(kvgrp);               // (request, kv head)
        split = (int)dv.nsplit.rem(kvgrp, bg);
        b = (int)dv.kv_heads.quot(bg);
        g = (int)dv.kv_heads.rem(bg, b);
        witem = (b * n_mt + mt) * nsplit + split;
    }

    // The request's lengths are requested here, ahead of the gathering waves' per-lane constants: nothing in
    // those depends on the lengths, and they are a couple of hundred instructions from a cold instruction cache.
    // (Measured against scalar loads of the three entries in flight together, with and without all kernel
    // arguments fetched at entry: this form, a vector load per entry, is the fastest of the three by 1-1.5 %.)
    const int64_t qs = load_index_nonneg(p.b_start_loc, b, p.index_bits);
    const int64_t qe = load_index_nonneg(p.b_start_loc, b + 1, p.index_bits);
    const int64_t seq = load_index_nonneg(p.b_seq_len, b, p.index_bits);
    const float k_scale = FP8 ? *p.k_scale : 1.f;
    const float v_scale = FP8 ? *p.v_scale : 1.f;
    const uint8_t lazy_raw = p.is_lazy ? p.is_lazy[b] : (uint8_t)1;
    __builtin_amdgcn_sched_barrier(0);
    const int pos_mode = p.pos_mode;
    // A cache page of 32 slots is handled as two parts of 16: "page" j below is the j-th run of 16 context
    // slots, part j & 1 of cache page j >> 1.  Its valid slots follow from the page's pad count.
    const int pshift = p.block_size == 2 * BS ? 1 : 0, part_mask = pshift;
    const int cache_bs = BS << pshift;
    const int gw = (wave - NC) & 3;                              // gathering waves: this wave's page of every tile
    const int half = NH == 2 ? (wave - NC) >> 2 : 0;             // ... and which of the page's items
    auto item = [&](int i) { return i * NH + half; };
    // (an un-rotated request of the block-uniform mode reads row 0 for every page, like the mode's other requests
    // read one row per page: what depends on the request's own flag is decided later)
    const int nat_step = pos_mode == LAZYATTN_POS_BLOCK_UNIFORM ? 0 : BS;
    const bool per_token = pos_mode != LAZYATTN_POS_BLOCK_UNIFORM;
    const uint8_t *tab_base = (const uint8_t *)p.cos_sin_cache;
    const uint32_t row_bytes = (uint32_t)p.table_stride * TSZ;
    // per-token rotation of context pages reads the packed table [2][D/16][rows][8]: the 16
    // slots of a page are 16 consecutive 16-byte chunks there
    const bool packed_tab = p.cos_sin_packed != nullptr && per_token;
    // this wave's part of its cache pages (pages of 32 slots: the tile's pages 0, 1 are the two parts of
    // one cache page, 2, 3 of the next): first slot, and the position step that goes with it
    const int slot0 = (gw & part_mask) * BS;
    // K items of a page: 128 = (8 chunks of 8 (d, d+64) pairs) x 16 slots, two per lane
    uint32_t k_toff[KI];
    // Cache offsets of a lane's items: item i = item 0 + i * (a wave-uniform stride), so one offset register
    // serves all of them and the strides go into the scalar page base.
    // K bf16: [D/8][slots][8] -> item (cp, o) at (cp*slots + o)*16 bytes, cp = lane/16 + 4 i
    //   fp8 : [D/16][slots][16] -> 8 bytes at chunk cp/2, half cp&1
    // V bf16: item = one 16-byte chunk of a row, in the order the chunks take in LDS (position lane + 64 i: row
    //   d = position / 2, chunk = (position & 1) ^ bit 3 of d); fp8: row d = lane + 64 i, 16 slots
    uint32_t k_goff = FP8 ? (uint32_t)(((lane >> 5) * cache_bs + slot0 + (lane & 15)) * 16 + ((lane >> 4) & 1) * 8)
                          : (uint32_t)(((lane >> 4) * cache_bs + slot0 + (lane & 15)) * 16);
    uint32_t v_goff = FP8 ? (uint32_t)(lane * cache_bs + slot0)
                          : (uint32_t)((lane >> 1) * cache_bs * 2 + slot0 * 2 + ((lane ^ (lane >> 4)) & 1) * 16);
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int idx = lane + item(i) * 64;
        const int o = idx & 15, cp = PAD && (idx >> 4) >= CPr ? 0 : idx >> 4;   // (a padded chunk reads chunk 0 and is zeroed)
        // block-uniform rotation and un-rotated requests use one table row for the whole page
        k_toff[i] = packed_tab ? ((uint32_t)cp * (uint32_t)p.packed_rows + (uint32_t)o) * 8 * TSZ
                               : (per_token ? (uint32_t)o * row_bytes : 0u) + (uint32_t)cp * 8 * TSZ;
    }
    // PAD: per-item cache offsets (the chunk of d + Dr/2 is not a fixed distance away in an fp8 page) and
    // which of the lane's items exist
    uint32_t pk1[PAD ? KI : 1], pk2[PAD ? KI : 1], pv[PAD ? VI_CTX : 1];
    bool pk_ok[PAD ? KI : 1], pv_ok[PAD ? VI_CTX : 1];
    if constexpr (PAD) {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            const int idx = lane + item(i) * 64, o = idx & 15;
            pk_ok[i] = (idx >> 4) < CPr;
            const int c1 = pk_ok[i] ? idx >> 4 : 0, c2 = CPr + c1;                  // 8-element chunks of d and d + Dr/2
            pk1[i] = FP8 ? (uint32_t)(((c1 >> 1) * cache_bs + slot0 + o) * 16 + (c1 & 1) * 8) : (uint32_t)((c1 * cache_bs + slot0 + o) * 16);
            pk2[i] = FP8 ? (uint32_t)(((c2 >> 1) * cache_bs + slot0 + o) * 16 + (c2 & 1) * 8) : (uint32_t)((c2 * cache_bs + slot0 + o) * 16);
        }
#pragma unroll
        for (int i = 0; i < VI_CTX; ++i) {
            const int idx = lane + item(i) * 64;
            const int d = FP8 ? idx : idx >> 1;
            pv_ok[i] = d < Dr;
            const int dc = pv_ok[i] ? d : 0;
            pv[i] = FP8 ? (uint32_t)(dc * cache_bs + slot0) : (uint32_t)(dc * cache_bs * 2 + slot0 * 2 + ((idx ^ (idx >> 4)) & 1) * 16);
        }
    }
    // (pinned here: the values are only used by the gathering waves' code further down, and the compiler would
    // otherwise move their computation there, behind the wait for the lengths)
    asm volatile("" : "+v"(k_goff), "+v"(v_goff));
#pragma unroll
    for (int i = 0; i < KI; ++i) asm volatile("" : "+v"(k_toff[i]));
    if constexpr (PAD) {
#pragma unroll
        for (int i = 0; i < KI; ++i) asm volatile("" : "+v"(pk1[i]), "+v"(pk2[i]));
#pragma unroll
        for (int i = 0; i < VI_CTX; ++i) asm volatile("" : "+v"(pv[i]));
    }
    __builtin_amdgcn_sched_barrier(0);
    const int q_len = (int)(qe - qs);
    const int ctx_len = (int)(seq - q_len);
    if (q_len <= 0 || ctx_len < 0) return;
    if (p.skip_decode && q_len == 1) return;                     // old_ops:109-110
    const int n_chunks = (q_len + UNIT - 1) / UNIT;
    const int n_units = n_chunks * group;
    if (mt * NC >= n_units) return;                              // block_mask, old_ops:322-328
    const bool lazy_b = lazy_raw != 0;
    const bool vanilla = pos_mode == LAZYATTN_POS_BLOCK_UNIFORM && !lazy_b;   // ops:398
    const bool use_qmask = !vanilla && p.q_mask != nullptr;
    const int n_pages = (ctx_len + BS - 1) / BS;
    int t_end;                                                   // new-token keys [0, t_end) are visible here
    {
        int last_unit = mt * NC + NC - 1;
        if (last_unit > n_units - 1) last_unit = n_units - 1;
        const int te = ((int)dv.group.quot(last_unit) + 1) * UNIT;
        t_end = te < q_len ? te : q_len;
    }
    const int n_ctx_tiles = (n_pages + PAGES - 1) / PAGES;
    const int n_new_tiles = (t_end + NT - 1) / NT;
    // The key axis is cut into nsplit ranges of equal estimated cost.  A new-token tile costs about
    // three context tiles (element-wise V scatter, per-row causal masks, branchy loads), and all of them
    // sit at the end: with equal tile counts the last split was the tail of every launch.
    constexpr int NEW_COST = 3;
    // Sliding window (old_ops:270-284, 373-376): the row at sequence position P sees the keys at positions
    // P - window + 1 .. P only.  Positions: context slot n -> n, new token m -> ctx_len + m.  The tiles that
    // lie entirely before the window of the workgroup's first row are not visited at all.
    const int window = WIN ? p.sliding_window : 0;
    int skip_ctx = 0, skip_new = 0;                 // whole context / new-token tiles before every window
    if (window) {
        const int first_row = (int)dv.group.quot(mt * NC) * UNIT;
        const int lo_min = ctx_len + first_row - window + 1;
        if (lo_min > 0) {
            skip_ctx = lo_min < ctx_len ? lo_min / NT : n_ctx_tiles;
            if (lo_min >= ctx_len) skip_new = (lo_min - ctx_len) / NT;
            if (skip_new > n_new_tiles) skip_new = n_new_tiles;
        }
    }
    const int live_ctx = n_ctx_tiles - skip_ctx, live_new = n_new_tiles - skip_new;
    const uint32_t cost = (uint32_t)live_ctx + (uint32_t)NEW_COST * (uint32_t)live_new;   // (tiles: far below 2^25; splits <= 64)
    auto tile_at = [&](uint32_t c) -> int {        // first tile whose cost interval ends after c
        return skip_ctx + skip_new + (c <= (uint32_t)live_ctx ? (int)c : live_ctx + (int)((c - (uint32_t)live_ctx) / NEW_COST));
    };
    // Equal shares of the cost, the first (cost mod splits) of them one longer.  The split count is the request's own
    // under the balanced list, where no multiplier can come from the host: the wave that located the work item left
    // ceil(2^32 / splits), exact for costs below 2^26 and at most 64 splits.  (A division here -- forty instructions
    // from a cold instruction cache on every wave's way to its first memory request -- cost 0.5 us of an 18 us launch.)
    const uint32_t share = bal.items_cap > 0 ? (split_mul ? FastDiv::mulhi(cost, split_mul) : cost) : dv.nsplit.quot(cost);
    const uint32_t longer = cost - share * (uint32_t)nsplit_wg;
    const uint32_t c_lo = (uint32_t)split * share + ((uint32_t)split < longer ? (uint32_t)split : longer);
    const uint32_t c_hi = c_lo + share + ((uint32_t)split < longer ? 1u : 0u);
    const int tile_begin = tile_at(c_lo);
    const int tile_end = split + 1 == nsplit_wg ? n_ctx_tiles + n_new_tiles : tile_at(c_hi);

    // ---- page metadata, fetched ahead of its use ----
    // Gathering wave w owns page w of every tile, so it needs one block-table entry, one
    // q_offset and one q_mask per tile.  They are read through the scalar unit (constant address
    // space): the values are wave-uniform, land in SGPRs, and waiting for them never drains the
    // vector loads in flight.  Branch-free on purpose (a branch around a load makes the compiler
    // drain every outstanding load at the join): pages past the context read entry n_pages-1
    // and get limit 0; an absent q_offset / q_mask array is replaced by the block table, masked to 0.
    struct PageMeta { int bt, qo, lim; };      // physical block, q_offset, number of valid slots
    typedef const int32_t __attribute__((address_space(4))) *sptr_i32;
    const bool use_qo = !vanilla && pos_mode != LAZYATTN_POS_NATURAL;
    const sptr_i32 bt_row = (sptr_i32)(p.block_table + b * p.bt_stride[0]);
    const sptr_i32 qo_row = use_qo ? (sptr_i32)(p.q_offset + b * p.qo_stride[0]) : bt_row;
    const sptr_i32 qm_row = use_qmask ? (sptr_i32)(p.q_mask + b * p.qm_stride[0]) : bt_row;
    const int64_t bt_s1 = p.bt_stride[1];
    const int64_t qo_s1 = use_qo ? p.qo_stride[1] : p.bt_stride[1];
    const int64_t qm_s1 = use_qmask ? p.qm_stride[1] : p.bt_stride[1];
    const int qo_and = use_qo ? -1 : 0, qm_and = use_qmask ? -1 : 0;
    auto load_page = [&](int j) -> PageMeta {
        PageMeta m;
        int jc = j < n_pages ? j : n_pages - 1;
        jc = jc < 0 ? 0 : jc;
        const int pj = jc >> pshift;
        m.bt = bt_row[pj * bt_s1];
        m.qo = qo_row[pj * qo_s1] & qo_and;
        const int qm = qm_row[pj * qm_s1] & qm_and;                                  // old_ops:165-167
        const int ql = cache_bs - qm - (j & part_mask) * BS;                         // valid slots of this part
        int l = ctx_len - j * BS;
        l = l < ql ? l : ql;
        l = l > BS ? BS : l;
        m.lim = l < 0 ? 0 : l;
        return m;
    };
    // Valid-slot counts of the four pages of a context tile, one byte per page and LDS buffer (a word per tile:
    // the computing waves compare it with four times BS to tell a full tile): written by the gathering waves
    // with the tile, read by the computing waves for the masks.
    constexpr bool QREG = q_in_registers(NC, HD);
    constexpr int Q_BYTES = QREG ? 0 : NC * G::Q_WAVE;
    uint8_t *page_lims = lds + KV_BYTES + Q_BYTES;

    if (gatherer) {
        // ====================================================================== gather
        // The block-table entries of the first three tiles are requested before anything else: the scalar
        // loads are a memory round trip.
        const PageMeta pm0 = load_page(tile_begin * PAGES + gw);
        const PageMeta pm1 = load_page((tile_begin + 1) * PAGES + gw);
        PageMeta pm_pend = load_page((tile_begin + 2) * PAGES + gw);
        const bool rot_new = p.rotate_new_k && !vanilla;
        const float k_unscale = FOLD ? 1.f / k_scale : 1.f, v_unscale = FOLD ? 1.f / v_scale : 1.f;
        const uint8_t *kc_base = (const uint8_t *)p.k_cache + (int64_t)g * p.kc_stride[1] * (FP8 ? 1 : 2);
        const uint8_t *vc_base = (const uint8_t *)p.v_cache + (int64_t)g * p.vc_stride[1] * (FP8 ? 1 : 2);
        const int64_t kc_page_bytes = p.kc_stride[0] * (FP8 ? 1 : 2);
        const int64_t vc_page_bytes = p.vc_stride[0] * (FP8 ? 1 : 2);
        const uint8_t *ctab_base = packed_tab ? (const uint8_t *)p.cos_sin_packed : tab_base;
        const uint32_t pos_bytes = packed_tab ? 8 * TSZ : row_bytes;       // bytes per unit of position
        const uint32_t sin_delta = packed_tab ? (uint32_t)(HALFr / 8) * (uint32_t)p.packed_rows * 8 * TSZ : HALFr * TSZ;
        const int part_pos = nat_step ? slot0 : 0;               // block-uniform: one position for the whole page
        const uint32_t k_item = (uint32_t)((FP8 ? 2 : 4) * cache_bs * 16);
        const uint32_t v_item = (uint32_t)(64 * cache_bs);
        // bytes from the chunk of d to the chunk of d + HD/2 in the cache page
        const uint32_t pair = (uint32_t)(FP8 ? G::PAIR8 : G::PAIR) << pshift;
        KRegs<TT> kr[KI];
        uint4 vr[VI];

        // ---- loads of a context page: no branch, no zero fill ----
        // Position of the page's first slot.  Natural: j*16 (old_ops:183-184); offset: q_offset-1 if
        // set, else natural (old_ops:186-191); block-uniform: q_offset-1 if set, else 0 (ops:180-186);
        // un-rotated requests read row 0 of the table (cos 1, sin 0): exact identity.  pm.qo is 0
        // wherever q_offset is not consulted, nat_step is 0 wherever the fallback is row 0.
        // A page past the context (its slots are all masked) takes the last page's position: the
        // table only has to cover the positions of real keys.
        // The lane offsets are handed out as fresh 32-bit values per page: a load then is "scalar base + 32-bit
        // lane offset" as it stands.  Left to itself the compiler widens the loop-invariant offsets to 64 bits
        // once, outside the loop, and then forms every address with a 64-bit vector add.
        struct PageBase { const uint8_t *kb, *tb, *ts, *vb; uint32_t ko, vo, to[KI]; };
        auto page_base = [&](int tile, const PageMeta &pm) -> PageBase {
            const int j = tile * PAGES + gw;
            const int jp = j < n_pages ? j : n_pages - 1;
            const int pos0 = pm.qo ? pm.qo - 1 + part_pos : jp * nat_step;
            PageBase pb;
            pb.kb = kc_base + pm.bt * kc_page_bytes;
            pb.tb = ctab_base + (int64_t)pos0 * pos_bytes;
            pb.ts = pb.tb + sin_delta;
            pb.vb = vc_base + pm.bt * vc_page_bytes;
            pb.ko = k_goff; pb.vo = v_goff;
            asm volatile("" : "+v"(pb.ko), "+v"(pb.vo));
#pragma unroll
            for (int i = 0; i < KI; ++i) { pb.to[i] = k_toff[i]; asm volatile("" : "+v"(pb.to[i])); }
            return pb;
        };
        auto load_k_item = [&](int i, const PageBase &pb) {
            const uint8_t *kb = pb.kb;
            kr[i].lds_off = (uint32_t)(gw * K_PAGE + (lane + item(i) * 64) * 16);
            if constexpr (PAD) {
                u32x4_t k1, k2;
                if (FP8) {
                    const uint2 a = ldg8(kb, pk1[i]), a2 = ldg8(kb, pk2[i]);
                    k1 = u32x4_t{a.x, a.y, 0, 0};
                    k2 = u32x4_t{a2.x, a2.y, 0, 0};
                } else {
                    k1 = ldg16v(kb, pk1[i]);
                    k2 = ldg16v(kb, pk2[i]);
                }
                const u32x4_t z = {0, 0, 0, 0};
                kr[i].k1 = pk_ok[i] ? k1 : z;
                kr[i].k2 = pk_ok[i] ? k2 : z;
            } else if (FP8) {
                const uint2 a = ldg8(kb + item(i) * k_item, pb.ko), a2 = ldg8(kb + item(i) * k_item + pair, pb.ko);
                kr[i].k1 = u32x4_t{a.x, a.y, 0, 0};
                kr[i].k2 = u32x4_t{a2.x, a2.y, 0, 0};
            } else {
                kr[i].k1 = ldg16v(kb + item(i) * k_item, pb.ko);
                kr[i].k2 = ldg16v(kb + item(i) * k_item + pair, pb.ko);
            }
            kr[i].c.load(pb.tb, pb.to[i]);
            kr[i].s.load(pb.ts, pb.to[i]);
        };
        // the same four loads (full page of a 16-bit cache) outside the compiler's count: the steady state below
        // places its own waits, because the V loads that go straight to LDS are outside that count anyway
        auto load_k_item_uncounted = [&](int i, const PageBase &pb) {
            kr[i].lds_off = (uint32_t)(gw * K_PAGE + (lane + item(i) * 64) * 16);
            ldg16_uncounted(kr[i].k1, pb.kb + item(i) * k_item, pb.ko);
            ldg16_uncounted(kr[i].k2, pb.kb + item(i) * k_item + pair, pb.ko);
            kr[i].c.load_uncounted(pb.tb, pb.to[i]);
            kr[i].s.load_uncounted(pb.ts, pb.to[i]);
        };
        auto load_v_item = [&](int i, const PageBase &pb) {
            if constexpr (PAD) {
                const uint4 t = ldg16(pb.vb, pv[i]);
                vr[i] = pv_ok[i] ? t : make_uint4(0, 0, 0, 0);
            } else {
                vr[i] = ldg16(pb.vb + item(i) * v_item, pb.vo);
            }
        };
        auto issue_loads_ctx = [&](int tile, const PageMeta &pm) {
            const PageBase pb = page_base(tile, pm);
#pragma unroll
            for (int i = 0; i < KI; ++i) load_k_item(i, pb);
#pragma unroll
            for (int i = 0; i < VI_CTX; ++i) load_v_item(i, pb);
        };
        // ---- loads of this wave's 16 keys of a new-token tile ----
        auto issue_loads_new = [&](int tile) {
            const int m0 = (tile - n_ctx_tiles) * NT + gw * BS;
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                const int idx = lane + item(i) * 64;
                const int cp = idx & (D / 16 - 1), kl = idx / (D / 16), m = m0 + kl;
                kr[i].lds_off = (uint32_t)(gw * K_PAGE + cp * 256 + kl * 16);
                u32x4_t k1 = {0, 0, 0, 0}, k2 = k1;
                TabVec<TT> c, sn;
                c.fill(1.f); sn.fill(0.f);
                if (m < t_end && (!PAD || cp < CPr)) {
                    const T *kn = (const T *)p.k + (qs + m) * p.k_stride[0] + (int64_t)g * p.k_stride[1] + cp * 8;
                    k1 = *reinterpret_cast<const u32x4_t *>(kn);
                    k2 = *reinterpret_cast<const u32x4_t *>(kn + HALFr);
                    if (rot_new) {                                               // old_ops:342-343
                        const uint8_t *tb = tab_base + (int64_t)(ctx_len + m) * row_bytes;
                        c.load(tb, (uint32_t)cp * 8 * TSZ);
                        sn.load(tb, (uint32_t)cp * 8 * TSZ + HALFr * TSZ);
                    }
                }
                kr[i].k1 = k1; kr[i].k2 = k2; kr[i].c = c; kr[i].s = sn;
            }
#pragma unroll
            for (int i = 0; i < VI; ++i) {
                const int idx = lane + item(i) * 64;
                const int dc = idx & (D / 8 - 1), m = m0 + idx / (D / 8);
                // (the value is chosen before the one store: a store under the branch lets the compiler merge
                // the iterations' stores behind a pointer phi, and the array then stays in scratch memory)
                uint4 t = make_uint4(0, 0, 0, 0);
                if (m < t_end && (!PAD || dc * 8 < Dr))
                    t = *reinterpret_cast<const uint4 *>((const T *)p.v + (qs + m) * p.v_stride[0] +
                                                         (int64_t)g * p.v_stride[1] + dc * 8);
                vr[i] = t;
            }
        };
        // kind of this wave's part of a tile, and its loads
        auto issue_loads = [&](int tile, const PageMeta &pm) -> int {
            if (tile >= n_ctx_tiles) { issue_loads_new(tile); return TILE_NEW; }
            issue_loads_ctx(tile, pm);                     // pages past the context re-read the last page: harmless
            if (pm.lim == BS) return TILE_FULL;
            if (tile * PAGES + gw >= n_pages) {
#pragma unroll
                for (int i = 0; i < KI; ++i) { kr[i].k1 = u32x4_t{0, 0, 0, 0}; kr[i].k2 = kr[i].k1; }
            }
            return TILE_EDGE;
        };
        // ---- rotate the K items in fp32 and write them to a K tile ----
        auto store_k_item = [&](int i, uint8_t *ktile, int kind) {
            float a[8], bb[8], cs[8], sn[8];
            if (FOLD && kind != TILE_NEW) {
                unpack8_fp8_raw<FP8>(kr[i].k1[0], kr[i].k1[1], a);
                unpack8_fp8_raw<FP8>(kr[i].k2[0], kr[i].k2[1], bb);
            } else if (FP8 && kind != TILE_NEW) {
                unpack8_fp8<T, FP8>(kr[i].k1[0], kr[i].k1[1], k_scale, a);
                unpack8_fp8<T, FP8>(kr[i].k2[0], kr[i].k2[1], k_scale, bb);
            } else {
                unpack8<T>(kr[i].k1, a);
                unpack8<T>(kr[i].k2, bb);
            }
            kr[i].c.get(cs);
            kr[i].s.get(sn);
            float x[8], y[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[e] = a[e] * cs[e] - bb[e] * sn[e];                             // old_ops:253
                y[e] = a[e] * sn[e] + bb[e] * cs[e];                             // old_ops:254
            }
            if (FOLD && kind == TILE_NEW) {
#pragma unroll
                for (int e = 0; e < 8; ++e) { x[e] *= k_unscale; y[e] *= k_unscale; }
            }
            *reinterpret_cast<uint4 *>(ktile + kr[i].lds_off) = make_uint4(
                E::pack(x[0], x[1]), E::pack(x[2], x[3]), E::pack(x[4], x[5]), E::pack(x[6], x[7]));
            *reinterpret_cast<uint4 *>(ktile + kr[i].lds_off + G::PAIR) = make_uint4(
                E::pack(y[0], y[1]), E::pack(y[2], y[3]), E::pack(y[4], y[5]), E::pack(y[6], y[7]));
        };
        auto store_k = [&](uint8_t *ktile, int kind) {
#pragma unroll
            for (int i = 0; i < KI; ++i) store_k_item(i, ktile, kind);
        };
        // one V item of a context page -> the page's rows in LDS ([d][2 chunks of 8 slots], chunks swapped where bit 3
        // of d is set)
        auto store_v_item = [&](int i, uint8_t *vtile, int kind, int lim) {
            const int idx = lane + item(i) * 64;
            if (FP8) {
                // 16 fp8 slots of one d -> both chunks of its row
                const int d = idx;
                const uint32_t w[4] = {vr[i].x, vr[i].y, vr[i].z, vr[i].w};
                uint32_t o2[4][2];                               // o2[q][h]: slots 4q + 2h, 4q + 2h + 1
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    if constexpr (FOLD) {
                        o2[q4][0] = fp8x2_to_bf16x2<FP8, false>(w[q4]);
                        o2[q4][1] = fp8x2_to_bf16x2<FP8, true>(w[q4]);
                        if (kind == TILE_EDGE) {                 // masked slots contribute nothing, whatever they hold
#pragma unroll
                            for (int s = 0; s < 4; ++s)
                                if (q4 * 4 + s >= lim) o2[q4][s >> 1] &= (s & 1) ? 0x0000ffffu : 0xffff0000u;
                        }
                        continue;
                    }
                    const f32x2_t lo = cvt_fp8x2<FP8>(w[q4]);
                    const f32x2_t hi = cvt_fp8x2<FP8>(w[q4] >> 16);
                    float f[4] = {lo[0] * v_scale, lo[1] * v_scale, hi[0] * v_scale, hi[1] * v_scale};
                    if (kind == TILE_EDGE) {
#pragma unroll
                        for (int s = 0; s < 4; ++s)
                            if (q4 * 4 + s >= lim) f[s] = 0.f;   // masked slots contribute nothing, whatever they hold
                    }
                    o2[q4][0] = E::pack(f[0], f[1]);
                    o2[q4][1] = E::pack(f[2], f[3]);
                }
                uint8_t *dst = vtile + gw * V_PAGE + d * 32;
                const int sw = ((d >> 3) & 1) * 16;
                *reinterpret_cast<uint4 *>(dst + sw) = make_uint4(o2[0][0], o2[0][1], o2[1][0], o2[1][1]);
                *reinterpret_cast<uint4 *>(dst + (sw ^ 16)) = make_uint4(o2[2][0], o2[2][1], o2[3][0], o2[3][1]);
            } else {
                // 8 slots (8*hf ..) of one d, already the chunk that belongs at position idx
                const int hf = (idx ^ (idx >> 4)) & 1;
                uint4 v = vr[i];
                if (kind == TILE_EDGE) {
                    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (hf * 8 + 2 * e >= lim) w[e] &= 0xffff0000u;
                        if (hf * 8 + 2 * e + 1 >= lim) w[e] &= 0x0000ffffu;
                    }
                    v = make_uint4(w[0], w[1], w[2], w[3]);
                }
                *reinterpret_cast<uint4 *>(vtile + gw * V_PAGE + idx * 16) = v;
            }
        };
        // ---- write the V items to a V tile; lim = valid slots of the page ----
        auto store_v = [&](uint8_t *vtile, int kind, int lim) {
            if (kind == TILE_NEW) {
                // item = 8 d of one new-token key: scatter 2-byte entries
#pragma unroll
                for (int i = 0; i < VI; ++i) {
                    const int idx = lane + item(i) * 64;
                    const int dc = idx & (D / 8 - 1), slot = idx / (D / 8);
                    uint8_t *dst = vtile + gw * V_PAGE + (dc * 8) * 32 + (((slot >> 3) ^ dc) & 1) * 16 + (slot & 7) * 2;
                    uint32_t w[4] = {vr[i].x, vr[i].y, vr[i].z, vr[i].w};
                    if constexpr (FOLD) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = E::pack(E::lo(w[e]) * v_unscale, E::hi(w[e]) * v_unscale);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        *reinterpret_cast<uint16_t *>(dst + (2 * e) * 32) = (uint16_t)(w[e] & 0xffffu);
                        *reinterpret_cast<uint16_t *>(dst + (2 * e + 1) * 32) = (uint16_t)(w[e] >> 16);
                    }
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < VI_CTX; ++i) store_v_item(i, vtile, kind, lim);
        };
        uint8_t *const kt0 = lds + V_BUFS * V_TILE;             // the two K tiles follow the three V tiles
        // K tile + the page's limit -> K buffer `kbuf`; V (unless it is already on its way there) -> V buffer `vb`
        auto store_tile = [&](int kbuf, int vb, int kind, int lim, bool with_v) {
            store_k(kt0 + kbuf * K_TILE, kind);
            if (with_v) store_v(lds + vb * V_TILE, kind, lim);
            if (lane == 0 && half == 0) page_lims[kbuf * PAGES + gw] = (uint8_t)lim;
        };
        // Full pages of a 16-bit cache need nothing done to V: their bytes go from the cache to the V tile by
        // global -> LDS loads (lane i of a load brings 16 bytes to i * 16 of a 1 KB stretch; which 16 bytes, is the
        // lane's own offset).  They are written as asm, outside the compiler's count of loads in flight: counted,
        // every later LDS store of this wave would be made to wait for them.  The steady state therefore issues its
        // K loads the same way and places the waits itself.  Loads complete in order; per tile the wave issues
        //   K item 0 (LPI loads) | V (VI loads) | K items 1 .. KI-1
        // so when item i of the next tile is needed, (KI-1) * LPI + VI younger loads have been issued since, and when
        // V of the next tile must have landed (the barrier at the end of the tile after the one it was issued in),
        // (2 KI - 1) * LPI + VI.
        constexpr bool VDMA = !FP8 && !PAD;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
        auto dma_v = [&](const PageBase &pb, int vb) {
#pragma unroll
            for (int i = 0; i < VI; ++i)
                dma16(pb.vb + item(i) * v_item, pb.vo, lds0 + (uint32_t)(vb * V_TILE + gw * V_PAGE + item(i) * 1024));
        };
        constexpr int LPI = 2 + 2 * TabVec<TT>::LOADS;
        constexpr int ITEM_YOUNGER = (KI - 1) * LPI + VI, V_YOUNGER = (2 * KI - 1) * LPI + VI;
        static_assert(V_YOUNGER < 64, "the wait counter holds 6 bits");

        // At the top of iteration `tile` the raw K/V of tile+1 sit in registers (loaded during
        // the previous iteration); they are rotated into the other LDS buffer while the
        // computing waves work on `tile`, then the loads of tile+2 are issued.  V buffers go round in threes:
        // vcur holds V of `tile`.
        int nxt_kind = TILE_FULL, nxt_lim = BS;
        int vcur = 0;
        bool v_sent = false;                 // V of tile+1 went (or is going) straight to its LDS buffer
        auto vnext = [](int v) { return v == V_BUFS - 1 ? 0 : v + 1; };
        if (tile_begin < tile_end) {
            const int k0 = issue_loads(tile_begin, pm0);
            if (k0 == TILE_FULL && tile_begin + 1 < n_ctx_tiles && tile_begin + 1 < tile_end && pm1.lim == BS) {
                // two full context tiles: as in the steady state below, each item of the second tile is requested
                // into the registers its counterpart of the first has just left, so the requests pass through the
                // CU's memory pipeline while the first tile is rotated instead of in one burst before the barrier
                const PageBase pb = page_base(tile_begin + 1, pm1);
                uint8_t *kt = kt0, *vt = lds;
#pragma unroll
                for (int i = 0; i < KI; ++i) {
                    store_k_item(i, kt, TILE_FULL);
                    load_k_item(i, pb);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int i = 0; i < VI_CTX; ++i) {
                    store_v_item(i, vt, TILE_FULL, BS);
                    load_v_item(i, pb);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (lane == 0 && half == 0) page_lims[gw] = (uint8_t)BS;
            } else {
                store_tile(0, 0, k0, pm0.lim, true);
                if (tile_begin + 1 < tile_end) {
                    nxt_kind = issue_loads(tile_begin + 1, pm1);
                    nxt_lim = pm1.lim;
                }
            }
        }
        __syncthreads();
        int tile = tile_begin;
        while (tile < tile_end) {
            // steady state: this wave's pages of tile+1 (in registers) and tile+2 (to load) are full context pages
            while (tile + 2 < n_ctx_tiles && tile + 2 < tile_end && nxt_kind == TILE_FULL && pm_pend.lim == BS) {
                const int cur = (tile - tile_begin) & 1;
                const PageMeta pm_new = load_page((tile + 3) * PAGES + gw);      // scalar loads, land during the rotation
                // Item by item: as soon as an item of tile+1 has left its registers for LDS, the same item of
                // tile+2 is requested into them.  The four gathering waves' loads then reach the CU's memory
                // pipeline spread over the tile instead of in one burst at its end (in a burst each of the twelve
                // loads of a wave waited tens of cycles to be accepted, all of it on this wave's critical path).
                const PageBase pb = page_base(tile + 2, pm_pend);
                const int vn = vnext(vcur), vnn = vnext(vn);
                uint8_t *kt = kt0 + (cur ^ 1) * K_TILE, *vt = lds + vn * V_TILE;
                if constexpr (VDMA) {
                    if (!v_sent) {
                        // first round: K and V of tile+1 came through counted loads; V leaves its registers first,
                        // while the compiler's count is still right
#pragma unroll
                        for (int i = 0; i < VI_CTX; ++i) store_v_item(i, vt, TILE_FULL, BS);
                    }
#pragma unroll
                    for (int i = 0; i < KI; ++i) {
                        settle<ITEM_YOUNGER>(kr[i]);
                        store_k_item(i, kt, TILE_FULL);
                        load_k_item_uncounted(i, pb);
                        __builtin_amdgcn_sched_barrier(0);
                        // V of tile+2 sets out behind the first K item's loads: it has this tile and the next to land
                        if (i == 0) {
                            dma_v(pb, vnn);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                    if (v_sent) wait_vmem<V_YOUNGER>();                      // V of tile+1 has landed
                    v_sent = true;
                } else {
#pragma unroll
                    for (int i = 0; i < KI; ++i) {
                        store_k_item(i, kt, TILE_FULL);
                        load_k_item(i, pb);
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int i = 0; i < VI_CTX; ++i) {
                        store_v_item(i, vt, TILE_FULL, BS);
                        load_v_item(i, pb);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if (lane == 0 && half == 0) page_lims[(cur ^ 1) * PAGES + gw] = (uint8_t)BS;
                pm_pend = pm_new;
                ++tile;
                vcur = vn;
                __syncthreads();
            }
            if (tile >= tile_end) break;
            const int cur = (tile - tile_begin) & 1;
            const int vn = vnext(vcur);
            if (v_sent) {
                // out of the steady state: K of tile+1 is in flight uncounted, V on its way to LDS; nothing else
#pragma unroll
                for (int i = 0; i < KI; ++i) settle<0>(kr[i]);
            }
            if (tile + 1 < tile_end) store_tile(cur ^ 1, vn, nxt_kind, nxt_lim, !v_sent);
            v_sent = false;
            int new_kind = TILE_FULL;
            if (tile + 2 < tile_end) new_kind = issue_loads(tile + 2, pm_pend);
            nxt_kind = new_kind;
            nxt_lim = pm_pend.lim;
            pm_pend = load_page((tile + 3) * PAGES + gw);
            ++tile;
            vcur = vn;
            __syncthreads();
        }
        return;
    }

    // ========================================================================== compute
    const int l32 = lane & 31, gh = lane >> 5;
    const int unit = mt * NC + wave;
    const bool active = unit < n_units;
    const int chunk = active ? (int)dv.group.quot(unit) : 0;
    const int h = g * group + (active ? unit - chunk * group : 0);
    const int t0 = chunk * UNIT;
    const int row = t0 + l32;                                    // token index of this lane's query row
    const bool row_ok = active && row < q_len;

    // Q^T fragments: B operand of S^T = K.Q^T, lane = (row l32, d = ks*16 + gh*8 .. +8).
    // Eight computing waves: they live in this wave's own LDS slice (three waves share a SIMD's register
    // file) and are re-read for every tile.  Four: 32 registers per lane, no LDS traffic for Q at all.
    // Q is multiplied by sm_scale * log2(e) here, once, and rounded to bf16 again: the MFMA then
    // delivers the scores in log2 units and no per-score multiply is left in the tile loop (the
    // reference scales the fp32 scores, old_ops:287; the extra rounding of Q is one more relative
    // 2^-9 per element, like the one the rotated K already carries).
    const float cs2 = p.sm_scale * 1.4426950408889634f * (FOLD ? k_scale : 1.f);
    uint8_t *qlds = lds + KV_BYTES + (QREG ? 0 : wave * G::Q_WAVE) + lane * 16;
    uint4 qreg[QREG ? KS : 1];
    {
        const T *qp = (const T *)p.q + (qs + row) * p.q_stride[0] + (int64_t)h * p.q_stride[1] + gh * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if constexpr (PAD) {
                // tile column c = ks*16 + gh*8: real element c (first half of the head) or Dr/2 + c - 64 (second)
                const int c = ks * 16 + gh * 8, lo = c & 63;
                if (row_ok && lo < HALFr) v = *reinterpret_cast<const uint4 *>(qp - gh * 8 + (c < 64 ? lo : HALFr + lo));
            } else {
                if (row_ok) v = *reinterpret_cast<const uint4 *>(qp + ks * 16);
            }
            float f[8];
            unpack8<T>(v, f);
            const uint4 qs4 = make_uint4(E::pack(f[0] * cs2, f[1] * cs2), E::pack(f[2] * cs2, f[3] * cs2),
                                         E::pack(f[4] * cs2, f[5] * cs2), E::pack(f[6] * cs2, f[7] * cs2));
            if constexpr (QREG) qreg[ks] = qs4;
            else *reinterpret_cast<uint4 *>(qlds + ks * 1024) = qs4;
        }
    }
    // Online softmax against a reference m_ref per row that moves rarely.  The MFMA accumulators of S^T
    // start at -m_ref, so the scores arrive already relative to it and P = exp2(S) needs no subtraction.
    // m_ref is moved (and O, l rescaled, old_ops:287-291) only when a row's tile maximum exceeds it by more
    // than REBASE, or when the row sees its first valid key; in between P may exceed 1 (by at most
    // 2^REBASE), which fp32 accumulation and bf16's exponent range carry without loss.
    // Once every row of the wave has seen a key, full tiles do not compute the row maximum at all: P = exp2(S)
    // is formed at once and the rows' sums of P -- needed anyway -- tell whether any P left the range the
    // element type and the fp32 accumulators carry comfortably (SUM_LIMIT); only then is the maximum taken
    // and the reference moved, before the P.V step that would use those P.
    constexpr float REBASE = E::REBASE, SUM_LIMIT = E::SUM_LIMIT;
    float m_ref = 0.f, l_run = 0.f;
    bool seen = false;                                              // the row has had a valid key
    f32x16_t cinit;                                                 // -m_ref in every element
#pragma unroll
    for (int i = 0; i < 16; ++i) cinit[i] = 0.f;
    f32x16_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

    // ---- S^T = K . Q^T for 32 keys of a tile (pages 2*sub, 2*sub+1) ----
    // Operands are requested two k-steps ahead of their MFMAs (a ring of three sets): one step ahead leaves the
    // LDS latency exposed in every step.  `between(ks)` is vector work of this wave placed behind the MFMA of
    // step ks in the instruction stream: the wave runs it while the matrix pipe works (the exponentials of the
    // other half, see the tile loop).
    auto qk_half = [&](const uint8_t *ktile, int sub, f32x16_t &s, auto between) {
        // MFMA row l32 takes slot (l32 with bits 2 and 3 swapped) of page l32 / 16: a lane's accumulator registers
        // then hold the scores of slots 8*gh .. 8*gh+7 of each page, the order of a V row's chunk gh
        const int kslot = (l32 & 3) | ((l32 & 4) << 1) | ((l32 & 8) >> 1);
        const uint8_t *kp = ktile + (sub * 2 + (l32 >> 4)) * K_PAGE + gh * 256 + kslot * 16;
        uint4 a[3], q[QREG ? 1 : 3];
        auto fetch = [&](int ks) {
            a[ks % 3] = *reinterpret_cast<const uint4 *>(kp + ks * 512);
            if constexpr (!QREG) q[ks % 3] = *reinterpret_cast<const uint4 *>(qlds + ks * 1024);
        };
        fetch(0);
        fetch(1);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + 2 < KS) fetch(ks + 2);
            const uint4 &qf = QREG ? qreg[QREG ? ks : 0] : q[QREG ? 0 : ks % 3];
            s = E::mfma(a[ks % 3], qf, ks ? s : cinit);
            between(ks);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // ---- masks: register i of half `sub` holds key sub*32 + 16*(i/8) + 8*gh + i%8 ----
    // key0 = sequence position of the tile's first key (only used under a sliding window)
    auto mask_half = [&](f32x16_t &s, uint32_t vbits, int sub, int kind, int m0, int key0) {
        const uint32_t w = vbits >> (8 * gh);
        // causal: key m0 + kk <= row  <=>  16*(i/8) + i%8 <= row - m0 - sub*32 - 8*gh   (old_ops:371-372)
        const int lim = kind == TILE_NEW ? row - m0 - sub * 32 - 8 * gh : 64;
        // window: key0 + sub*32 + 8*gh + kb >= ctx_len + row - window + 1
        const int lb = window ? ctx_len + row - window + 1 - key0 - sub * 32 - 8 * gh : -64;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int kb = 16 * (i >> 3) + (i & 7);
            const bool ok = ((w >> kb) & 1u) && kb <= lim && (!WIN || kb >= lb);
            s[i] = ok ? s[i] : -INFINITY;
        }
    };
    // ---- tile maximum per row; move the reference if a row needs it (rare after its first tile) ----
    auto rebase = [&](f32x16_t &s0, f32x16_t &s1) {
        // v_maximum3_f32: no quieting pre-pass over the MFMA results, NaN scores stay NaN
        float ma = max3(s0[0], s0[1], s0[2]), mb = max3(s1[0], s1[1], s1[2]);
#pragma unroll
        for (int i = 3; i < 15; i += 2) { ma = max3(ma, s0[i], s0[i + 1]); mb = max3(mb, s1[i], s1[i + 1]); }
        float mx = max3(ma, mb, s0[15]);
        mx = max3(mx, s1[15], s1[15]);
        mx = max3(mx, partner32(mx, gh != 0), mx);                  // relative to m_ref; -inf: no valid key in this tile
        const bool valid = mx > -INFINITY;                          // false for NaN too: NaN rows stay NaN below
        const float delta = (valid && (!seen || mx > REBASE)) ? mx : 0.f;
        if (__builtin_amdgcn_ballot_w64(delta != 0.f)) {
            const float alpha = seen ? __builtin_amdgcn_exp2f(-delta) : 1.f;   // nothing accumulated before the first key
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) acc[dt] *= alpha;
            l_run *= alpha;
            s0 -= delta;
            s1 -= delta;
            m_ref += delta;
#pragma unroll
            for (int i = 0; i < 16; ++i) cinit[i] = -m_ref;
        }
        seen = seen || valid;
    };
    // ---- the rare step of the lazy path: the P of `sa` left the comfortable range; move the reference to the
    // maximum of those 32 keys.  `sb`: scores still to be used that were formed against the old reference;
    // `hsum`: row sum of a half already added to O under the old reference ----
    auto bump = [&](f32x16_t &sa, f32x16_t *sb, float *hsum) {
        float mx = max3(sa[0], sa[1], sa[2]);
#pragma unroll
        for (int i = 3; i < 15; i += 2) mx = max3(mx, sa[i], sa[i + 1]);
        mx = max3(mx, sa[15], sa[15]);
        mx = max3(mx, partner32(mx, gh != 0), mx);
        const float delta = mx > 0.f ? mx : 0.f;                    // (NaN: 0, the row stays NaN)
        const float alpha = __builtin_amdgcn_exp2f(-delta);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[dt] *= alpha;
        l_run *= alpha;
        if (hsum) *hsum *= alpha;
        sa -= delta;
        if (sb) *sb -= delta;
        m_ref += delta;
#pragma unroll
        for (int i = 0; i < 16; ++i) cinit[i] = -m_ref;
    };
    // ---- P = exp2(S) for 32 keys (S is relative to m_ref), packed as the two B operands of the PV steps ----
    // One eighth of a half at a time (two exponentials, one pack, one partial row sum), so that the pieces can be
    // placed between MFMAs: w[] collects the packed probabilities, ta / tb the two chains of the lane's row sum
    // (of the rounded probabilities, two per instruction; old_ops:312 sums them unrounded).
    struct HalfP { uint32_t w[8]; float ta, tb; };
    auto exp_piece = [&](const f32x16_t &s, HalfP &h, int i) {
        h.w[i] = E::pack(__builtin_amdgcn_exp2f(s[2 * i]), __builtin_amdgcn_exp2f(s[2 * i + 1]));
        if (i & 1) h.tb = E::dot2_ones(h.w[i], i == 1 ? 0.f : h.tb);
        else h.ta = E::dot2_ones(h.w[i], i == 0 ? 0.f : h.ta);
        // (the sums count as used where they are formed: the first set of a tile is only read on the lazy path, and
        // the compiler would otherwise collect its eight dot instructions in front of that path's check, between
        // two MFMA phases, instead of leaving them behind the MFMAs)
        if (i & 1) asm volatile("" : "+v"(h.tb));
        else asm volatile("" : "+v"(h.ta));
    };
    auto exp_half = [&](const f32x16_t &s, HalfP &h) {
#pragma unroll
        for (int i = 0; i < 8; ++i) exp_piece(s, h, i);
    };
    // ---- O^T += V^T . P^T for 32 keys (pages 2*sub, 2*sub+1 of the tile) ----
    // k index j of a 16-key step <-> slot 8*gh + j of the page: chunk gh of every row of d, as it lies in the cache
    auto pv_half = [&](const uint8_t *vtile, int sub, const HalfP &h, auto between) {
        const uint8_t *vp = vtile + (sub * 2) * V_PAGE + l32 * 32 + ((gh ^ (l32 >> 3)) & 1) * 16;
        const uint4 p0 = make_uint4(h.w[0], h.w[1], h.w[2], h.w[3]), p1 = make_uint4(h.w[4], h.w[5], h.w[6], h.w[7]);
        // 2 DT MFMAs: the 32-row blocks of d for the first page of the half, then for the second;
        // their V^T operands are requested two MFMAs ahead
        uint4 a[3];
        auto fetch = [&](int j) { a[j % 3] = *reinterpret_cast<const uint4 *>(vp + (j / DT) * V_PAGE + (j % DT) * 1024); };
        fetch(0);
        fetch(1);
#pragma unroll
        for (int j = 0; j < 2 * DT; ++j) {
            if (j + 2 < 2 * DT) fetch(j + 2);
            acc[j % DT] = E::mfma(a[j % 3], j < DT ? p0 : p1, acc[j % DT]);
            between(j);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // which of the tile's 64 keys exist: new-token tiles from the token count, context tiles from the
    // page limits the gathering waves left beside the tile
    struct Desc { int kind; uint32_t vlo, vhi; int m0, key0; };
    static_assert(PAGES == 4 && BS < 256, "a tile's page limits travel as the four bytes of one word");
    constexpr uint32_t FULL_LIMS = (uint32_t)BS * 0x01010101u;
    auto describe_ctx = [&](int tile, uint32_t limw) -> Desc {
        Desc td{TILE_FULL, ~0u, ~0u, 0, tile * NT};
        if (limw != FULL_LIMS) {
            const uint32_t l0 = limw & 0xffu, l1 = (limw >> 8) & 0xffu, l2 = (limw >> 16) & 0xffu, l3 = limw >> 24;
            td.kind = TILE_EDGE;
            td.vlo = ((1u << l0) - 1u) | (((1u << l1) - 1u) << BS);
            td.vhi = ((1u << l2) - 1u) | (((1u << l3) - 1u) << BS);
        }
        // a tile that starts before the window of this wave's last row needs the per-row lower bound
        if (window && td.kind == TILE_FULL && td.key0 < ctx_len + t0 + UNIT - window) td.kind = TILE_EDGE;
        return td;
    };
    auto describe_new = [&](int tile) -> Desc {
        Desc td{TILE_NEW, ~0u, ~0u, (tile - n_ctx_tiles) * NT, 0};
        td.key0 = ctx_len + td.m0;
        const int n = t_end - td.m0;
        const uint64_t valid = n >= 64 ? ~0ull : (n <= 0 ? 0ull : ((1ull << n) - 1ull));
        td.vlo = (uint32_t)valid; td.vhi = (uint32_t)(valid >> 32);
        return td;
    };
    // The tile body, in the order the instructions are issued.  A wave's own vector work sits behind its own
    // MFMAs wherever the data allow it, so that a single wave keeps the matrix pipe busy through the whole tile
    // and the waves of a SIMD need not be out of step with each other to fill it:
    //   A  S0 = K0.Q^T                       8 MFMAs
    //   B  S1 = K1.Q^T                       8 MFMAs, behind each: two exponentials of S0, pack, row sum
    //      (head size 64: four MFMAs per phase, twice the vector work behind each)
    //   C  O += V0^T.P0^T                    8 MFMAs, behind each: the same for S1
    //   D  O += V1^T.P1^T                    8 MFMAs
    // That is the path of a full tile whose rows have all seen a key (no masks, no row maximum).  Any other
    // tile computes S1 first, masks, takes the maximum over both halves (the reference may move), and then forms
    // P0 in one go; from C on the two paths are the same instructions.
    // Context tiles and new-token tiles run the same body from two loops: the context loop carries none of the
    // new-token bookkeeping (between the two score phases a full tile now has a compare and a branch where the
    // common loop had some thirty scalar instructions, an eighth of the tile's time with one computing wave per SIMD).
    bool all_seen = false;       // wave-uniform: every row of this wave has met a key (full tiles then need no maximum)
    auto tile_body = [&](int tile, const uint8_t *vtile, auto new_tile) {
        constexpr bool NEWT = decltype(new_tile)::value;
        const int cur = (tile - tile_begin) & 1;
        const uint8_t *ktile = lds + V_BUFS * V_TILE + cur * K_TILE;
        // valid-slot counts of the tile's pages: requested now, looked at after phase A
        uint32_t limw = FULL_LIMS;
        if constexpr (!NEWT) limw = *reinterpret_cast<const uint32_t *>(page_lims + cur * PAGES);
        f32x16_t s0, s1;
        HalfP h0, h1;
        __builtin_amdgcn_s_setprio(2);
        qk_half(ktile, 0, s0, [](int) {});
        Desc td;
        bool lazy = false;
        if constexpr (NEWT) {
            td = describe_new(tile);
            qk_half(ktile, 1, s1, [](int) {});
        } else {
            td = describe_ctx(tile, (uint32_t)uniform((int)limw));
            lazy = td.kind == TILE_FULL && all_seen;
            // (the exponentials of S0 are formed behind these MFMAs on every tile: a tile that is not lazy forms
            // them again after its masks and maximum, and the first set, possibly garbage, is dropped)
            qk_half(ktile, 1, s1, [&](int ks) {
#pragma unroll
                for (int i = 0; i < 8 / KS; ++i) exp_piece(s0, h0, ks * (8 / KS) + i);
            });
        }
        // The maximum is needed when the tile is not lazy, or when a lazy tile's row sums say that some P of
        // the first half left the comfortable range: one path for both (then P0 is formed again).
        bool slow = !lazy;
        if constexpr (!NEWT) {
            if (lazy) slow = __builtin_amdgcn_ballot_w64(!(h0.ta + h0.tb <= SUM_LIMIT)) != 0;
        }
        if (slow) {
            // (the first set of P0 counts as used here too: otherwise the compiler moves its exponentials
            // out from behind the MFMAs into the branch that keeps them)
            if constexpr (!NEWT) {
#pragma unroll
                for (int i = 0; i < 8; ++i) asm volatile("" ::"v"(h0.w[i]));
            }
            __builtin_amdgcn_s_setprio(0);
            if (td.kind != TILE_FULL) {
                mask_half(s0, td.vlo, 0, td.kind, td.m0, td.key0);
                mask_half(s1, td.vhi, 1, td.kind, td.m0, td.key0);
            }
            rebase(s0, s1);
            all_seen = __builtin_amdgcn_ballot_w64(!seen) == 0;
            exp_half(s0, h0);
            __builtin_amdgcn_s_setprio(2);
        }
        float sum0 = h0.ta + h0.tb;
        pv_half(vtile, 0, h0, [&](int j) {
#pragma unroll
            for (int i = 0; i < 8 / (2 * DT); ++i) exp_piece(s1, h1, j * (8 / (2 * DT)) + i);
        });
        if constexpr (!NEWT) {
            if (lazy && __builtin_amdgcn_ballot_w64(!(h1.ta + h1.tb <= SUM_LIMIT))) {
                // (the scores are made opaque here: otherwise half of the row maximum below is computed ahead
                // of the branch, on every tile)
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(s1[i]));
                bump(s1, nullptr, &sum0);
                exp_half(s1, h1);
            }
        }
        pv_half(vtile, 1, h1, [](int) {});
        __builtin_amdgcn_s_setprio(0);
        l_run += sum0 + (h1.ta + h1.tb);
    };
    __syncthreads();
    int tile = tile_begin;
    const int ctx_stop = tile_end < n_ctx_tiles ? tile_end : n_ctx_tiles;
    const uint8_t *vtile = lds, *const v_wrap = lds + V_BUFS * V_TILE;   // V buffers go round in threes
    auto v_advance = [&] { vtile += V_TILE; if (vtile == v_wrap) vtile = lds; };
    for (; tile < ctx_stop; ++tile) {
        tile_body(tile, vtile, std::false_type{});
        v_advance();
        __syncthreads();
    }
    for (; tile < tile_end; ++tile) {
        // Rows of an idle wave are all-zero queries (harmless, never stored); a new-token tile
        // entirely in this wave's future contributes nothing (causal) and is skipped.
        if ((tile - n_ctx_tiles) * NT <= t0 + UNIT - 1) tile_body(tile, vtile, std::true_type{});
        v_advance();
        __syncthreads();
    }

    // ---- epilogue ----
    // (Measured and dropped, twice each way: staging the rows through LDS so that they leave as whole 256-byte rows
    // -- this once-per-wave code runs from a cold instruction cache and the staging cost what the better store
    // pattern gained; and merging the splits here, by the last workgroup of a set to arrive -- device-scope stores
    // and loads for the partial rows plus one release/acquire ticket per workgroup made the call 1 us shorter at
    // 5 K keys and 5 % longer at 65 K, where every finishing workgroup's cache invalidation hits the others.)
    l_run += partner32(l_run, gh != 0);
    if (!row_ok) return;
    const float out_scale = FOLD ? v_scale : 1.f;
    const float inv = l_run > 0.f ? out_scale / l_run : 0.f;
    if (nsplit_wg == 1) {
        T *op = (T *)p.o + (qs + row) * p.o_stride[0] + (int64_t)h * p.o_stride[1];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int d = dt * 32 + 8 * i4 + 4 * gh;
                if (PAD && d >= Dr) continue;                                  // padding columns of the tile
                *reinterpret_cast<uint2 *>(op + d) =
                    make_uint2(E::pack(acc[dt][4 * i4] * inv, acc[dt][4 * i4 + 1] * inv),
                               E::pack(acc[dt][4 * i4 + 2] * inv, acc[dt][4 * i4 + 3] * inv));
            }
    } else {
        // Partial row = 128 halves sharing one power-of-two scale (the row's largest |O/l| lands in
        // [0.5, 1)) + (log2-sum-exp, scale) as two floats: half the bytes of an fp32 row, written by every
        // workgroup at the same moment and read back by the merge, for an error of at most 2^-12 of the
        // row's largest element -- an eighth of the rounding of the bf16 output.
        float am = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; i += 2) am = max3(am, fabsf(acc[dt][i]), fabsf(acc[dt][i + 1]));
        am = fmaxf(am, partner32(am, gh != 0)) * inv;
        uint32_t eb = (__float_as_uint(am) >> 23) & 0xffu;           // biased exponent: am in [2^(eb-127), 2^(eb-126))
        eb = eb > 252u ? 252u : eb;
        const float down = __uint_as_float((253u - eb) << 23) * inv;   // 2^-(eb-126) / l
        const float up = __uint_as_float((eb + 1u) << 23);            // 2^(eb-126)
        // Where the rows go: every computing wave of every work item has a slot of 32 rows, numbered
        // (kv head, work item of that kv head, wave); inside it the R rows of the unit (R < 32 only at a request's
        // end) are laid out [piece][gh][row][4]: one store instruction of this wave then writes one contiguous run
        // (512 bytes for a full unit) instead of 32 runs of 16 bytes a row apart -- the partial rows leave in a
        // quarter of the time (measured with the bytes kept and only the addresses changed: 1.8 of the 3.2 us the
        // stores cost at 5 K keys).  The merge kernel reads with the same lane mapping.  (piece = the 8 columns
        // dt*32 + 8*i4 .. +7, gh its half)
        const int64_t items_per_kv = bal.items_cap > 0 ? (int64_t)bal.items_split_cap : (int64_t)p.batch * n_mt * nsplit;
        const int64_t slots = (int64_t)p.num_kv_heads * items_per_kv * NC;
        const int64_t slot = ((int64_t)g * items_per_kv + witem) * NC + wave;
        _Float16 *wo = (_Float16 *)((uint8_t *)p.workspace + bal.table_bytes);
        float2 *wl = reinterpret_cast<float2 *>(wo + slots * UNIT * D);
        const int R = q_len - t0 < UNIT ? q_len - t0 : UNIT;
        _Float16 *wb = wo + slot * UNIT * D + (gh * R + l32) * 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const f32x2_t lo = {acc[dt][4 * i4] * down, acc[dt][4 * i4 + 1] * down};
                const f32x2_t hi = {acc[dt][4 * i4 + 2] * down, acc[dt][4 * i4 + 3] * down};
                const f16x2_t hl = __builtin_convertvector(lo, f16x2_t), hh = __builtin_convertvector(hi, f16x2_t);   // RNE
                *reinterpret_cast<uint2 *>(wb + (dt * 4 + i4) * (2 * R * 4)) =
                    make_uint2(*reinterpret_cast<const uint32_t *>(&hl), *reinterpret_cast<const uint32_t *>(&hh));
            }
        if (gh == 0)
            wl[slot * UNIT + l32] = make_float2(l_run > 0.f ? m_ref + __builtin_amdgcn_logf(l_run) : -INFINITY, up);
    }
}

template <int NC, int HD, int FP8, bool WIN, bool PAD, typename T, typename TT>
int launch_mfma_t(const lazyattn_prefill_params &p, int nsplit, int n_mt, const BatchShape &bal, hipStream_t stream) {
    auto kern = prefill_mfma_kernel<NC, HD, FP8, WIN, PAD, T, TT>;
    constexpr int LDS_BYTES = lds_bytes<HD>(NC);
    // the attribute belongs to the device's copy of the kernel: once per device, on the caller's current device
    // (any host thread may call: the flag is atomic, and setting the attribute twice is harmless)
    static std::atomic<bool> attr_set[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LAZYATTN_E_LAUNCH;
    if (!attr_set[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess)
            return LAZYATTN_E_LAUNCH;
        attr_set[dev].store(true, std::memory_order_release);
    }
    const int64_t nb = (int64_t)p.num_kv_heads * (bal.items_cap > 0 ? (int64_t)bal.items_cap : (int64_t)nsplit * p.batch * n_mt);
    if (nb <= 0 || nb > 0x7fffffff) return LAZYATTN_E_SHAPE;
    const MfmaDivs dv{FastDiv((uint32_t)n_mt), FastDiv((uint32_t)nsplit), FastDiv((uint32_t)p.num_kv_heads),
                      FastDiv((uint32_t)(p.num_q_heads / p.num_kv_heads))};
    hipLaunchKernelGGL(kern, dim3((unsigned)nb), dim3((NC + gather_waves(NC, HD)) * 64), LDS_BYTES, stream, p, nsplit, n_mt, bal, dv);
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

// table type: the element type or float
template <int NC, int HD, int FP8, bool WIN, bool PAD, typename T>
int launch_mfma_table(const lazyattn_prefill_params &p, int nsplit, int n_mt, const BatchShape &bal, hipStream_t stream) {
    if (p.table_dtype == LAZYATTN_F32) return launch_mfma_t<NC, HD, FP8, WIN, PAD, T, float>(p, nsplit, n_mt, bal, stream);
    return launch_mfma_t<NC, HD, FP8, WIN, PAD, T, T>(p, nsplit, n_mt, bal, stream);
}
// head size and sliding window
template <int NC, int FP8, typename T>
int launch_mfma_shape(const lazyattn_prefill_params &p, int nsplit, int n_mt, const BatchShape &bal, hipStream_t stream) {
    if (p.head_dim == 64)
        return p.sliding_window > 0 ? launch_mfma_table<NC, 64, FP8, true, false, T>(p, nsplit, n_mt, bal, stream)
                                    : launch_mfma_table<NC, 64, FP8, false, false, T>(p, nsplit, n_mt, bal, stream);
    // other head sizes: the 128-wide kernel with padding (built with the window code, which a window of 0 switches off)
    if (p.head_dim != 128) return launch_mfma_table<NC, 128, FP8, true, true, T>(p, nsplit, n_mt, bal, stream);
    if (p.sliding_window > 0) return launch_mfma_table<NC, 128, FP8, true, false, T>(p, nsplit, n_mt, bal, stream);
    return launch_mfma_table<NC, 128, FP8, false, false, T>(p, nsplit, n_mt, bal, stream);
}
// Every kernel of one (element type, cache page kind: 0 the element type, 1 fp8 e4m3, 2 fp8 e5m2); nw = computing
// waves per workgroup (4 or 8).  Explicitly instantiated, one translation unit each.
template <typename T, int FP8>
int launch_mfma_family(const lazyattn_prefill_params &p, int nw, int nsplit, int n_mt, const BatchShape &bal, hipStream_t stream) {
    return nw == 8 ? launch_mfma_shape<8, FP8, T>(p, nsplit, n_mt, bal, stream)
                   : launch_mfma_shape<4, FP8, T>(p, nsplit, n_mt, bal, stream);
}

}  // namespace lazyattn
