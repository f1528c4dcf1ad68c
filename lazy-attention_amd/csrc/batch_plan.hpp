// How a batch of requests with different lengths is cut into work items of about equal length, decided on the device.
//
// The host knows the number of requests, of new tokens and the two maxima the caller passes; the lengths themselves
// live in device memory (b_start_loc, b_seq_len).  A split count chosen on the host is therefore the same for every
// request and sized for the longest one: a batch of ragged requests then leaves most compute units idle behind the
// few workgroups of its long requests.  For calls with more than one request the host only fixes the number of work
// items per kv head the grid has room for; the first wave of every workgroup of the main kernel reads all the
// lengths -- one memory round trip, which its own lengths cost anyway -- and derives, identically everywhere:
//   m_j     m-tiles (workgroups per kv head and split) of request j
//   c_j     cost of its key axis in 64-key tiles (a new-token tile counts as three)
//   T       tiles per work item: the work items of a launch run in rounds of one per compute unit, and being of
//           about T tiles each they finish round by round; for every number of rounds r the grid has room for, the
//           batch's W = sum m_j c_j tiles give the T that fills r rounds, W / (r rounds' items - half the m-tiles),
//           and r (T tile time + a work item's fixed time) estimates the launch; for the r with the lowest estimate,
//           T starts at the value whose item count fits for certain, W / (items - m-tiles), and is lowered in up to
//           three probes of the real item count toward the value that fills the rounds exactly
//   s_j     = ceil(c_j / T) key-axis splits of request j (at least two tiles each, at most 64)
// and from the prefix sums of m_j s_j which (request, m-tile, split) its work item is.  The first work item of every
// request leaves (first item, splits) of the request in a small table at the head of the workspace, where the merge
// kernel finds them with one scalar load.
// The arithmetic per request is plain C++ (also compiled for the host, where a unit test checks its invariants).
#pragma once
#include <stdint.h>

#include "fastdiv.hpp"

namespace lazyattn {

constexpr int PLAN_UNIT = 32;          // query rows per computing wave
constexpr int PLAN_TILE = 64;          // keys per tile
constexpr int PLAN_PAGE = 16;          // slots per run of context the kernel calls a page
constexpr int PLAN_NEW_COST = 3;       // a new-token tile costs about three context tiles
constexpr int PLAN_MAX_SPLITS = 64;

struct BatchShape {
    int32_t group;          // q-heads per kv-head
    int32_t nc;             // 32-row units per workgroup (4 or 8)
    int32_t n_mt_cap;       // m-tiles the caller's max_q_len allows per request (rows beyond are not computed)
    int32_t skip_decode;    // requests with one new token are left out
    int32_t items_cap;      // work items per kv head the grid has room for (at least the m-tiles)
    int32_t items_target;   // work items per kv head that fill one round of the chip's compute units
    int32_t items_split_cap;    // most work items per kv head of a batch that is split: what the partial rows have room for
    int32_t forced_splits;  // > 0: every request gets this many splits (the caller's num_splits, or the host's for a large batch)
    int32_t table_bytes;    // the requests' records at the head of the workspace (a multiple of 256); the partial rows follow
};

// (lengths are below 2^31: 32-bit arithmetic, shifts for the powers of two -- this runs at the head of every workgroup)
LAZYATTN_HD int plan_mtiles(int32_t q_len, int32_t ctx_len, const BatchShape &s) {
    if (q_len <= 0 || ctx_len < 0 || (s.skip_decode && q_len == 1)) return 0;
    const uint32_t chunks = ((uint32_t)q_len + PLAN_UNIT - 1) / PLAN_UNIT;           // < 2^26
    const uint32_t cap = (uint32_t)s.n_mt_cap;
    if (chunks > (cap << (s.nc == 8 ? 3 : 2))) return (int)cap;                        // (also keeps the product below in range)
    const uint32_t units = chunks * (uint32_t)s.group;
    const uint32_t m = s.nc == 8 ? (units + 7) >> 3 : (units + 3) >> 2;
    return (int)(m < cap ? m : cap);
}
// What the host can say of the m-tiles of a whole batch from its totals alone (the lengths are on the device): an
// upper bound.  A request with work has at least one new token (two when one-token requests are skipped), so at most
// R = min(batch, tokens / that) requests have any; each may end with a partly filled 32-row chunk -- the chunks
// together are at most (tokens + 31 R) / 32 -- and, unless the workgroup's units divide the q-heads of a kv head, with
// a partly filled m-tile; and none has more m-tiles than n_mt_cap.
LAZYATTN_HD int64_t plan_mtiles_bound(int64_t tokens, int64_t batch, const BatchShape &s) {
    const int64_t least = s.skip_decode ? 2 : 1;
    const int64_t with_work = tokens / least < batch ? tokens / least : batch;
    const int64_t chunks = (tokens + (PLAN_UNIT - 1) * with_work) / PLAN_UNIT;
    const int64_t by_chunks = (chunks * s.group + s.nc - 1) / s.nc + (s.group % s.nc ? with_work : 0);
    const int64_t by_requests = with_work * s.n_mt_cap;
    return by_chunks < by_requests ? by_chunks : by_requests;
}
// tiles of the key axis, weighted (below 2^24 for every context a 32-bit length can describe)
LAZYATTN_HD uint32_t plan_cost(int32_t q_len, int32_t ctx_len) {
    const uint32_t pages = ((uint32_t)ctx_len + PLAN_PAGE - 1) / PLAN_PAGE;
    const uint32_t ctx_tiles = (pages + PLAN_TILE / PLAN_PAGE - 1) / (PLAN_TILE / PLAN_PAGE);
    const uint32_t new_tiles = ((uint32_t)q_len + PLAN_TILE - 1) / PLAN_TILE;
    const uint32_t c = ctx_tiles + PLAN_NEW_COST * new_tiles;
    return c < (1u << 24) - 1 ? c : (1u << 24) - 1;
}
// n / d for n, d below 2^24, d > 0, through one float reciprocal and an integer correction (exact)
LAZYATTN_HD uint32_t plan_udiv(uint32_t n, uint32_t d) {
    uint32_t q = (uint32_t)((float)n * (1.0f / (float)d));
    // (the float product is off by less than two for such operands: two corrections each way, and no loop that
    // operands out of range could keep going)
    q -= q * d > n;
    q -= q * d > n;
    q += (q + 1) * d <= n;
    q += (q + 1) * d <= n;
    return q;
}
// splits of a request of `cost` tiles when a work item is to have at most T tiles (T = 0: no request is split)
LAZYATTN_HD int plan_splits(uint32_t cost, uint32_t T, const BatchShape &s) {
    uint32_t n;
    if (s.forced_splits > 0) n = (uint32_t)s.forced_splits;
    else if (T == 0) n = 1;
    else { n = plan_udiv(cost, T); n += n * T < cost; }
    const uint32_t most = cost / 2 > 1 ? cost / 2 : 1;             // at least two tiles per split
    n = n < most ? n : most;
    n = n < (uint32_t)PLAN_MAX_SPLITS ? n : (uint32_t)PLAN_MAX_SPLITS;
    return (int)(n < 1 ? 1 : n);
}

// Per workgroup a 64-key tile takes about 1.34 us in the four-unit shape and 1.98 us in the eight-unit shape, and a
// work item some 6 us of prologue, first-tile latency, epilogue and this planning (measured on an MI355X with 16-bit
// operands at head size 128).
constexpr float PLAN_ITEM_US = 6.f;
constexpr int PLAN_PROBES = 3;
LAZYATTN_HD float plan_tile_us(const BatchShape &s) { return s.nc == 8 ? 1.98f : 1.34f; }
LAZYATTN_HD float plan_ratio(float a, float b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return a * __builtin_amdgcn_rcpf(b);                 // (every workgroup forms the same value; what must hold is checked by counting)
#else
    return a / b;
#endif
}
LAZYATTN_HD uint32_t plan_clamp_tiles(float t, uint32_t c_max) {
    const uint32_t T = t < 2.f ? 2u : (t < 16777216.f ? (uint32_t)t : (1u << 24));
    return T < c_max ? T : c_max;
}
// T for the whole batch (0: no request is split).  W: sum of m_j c_j, M: sum of m_j, c_max: largest c_j,
// count(T): the work items per kv head a given T makes -- on the device a reduction over the scanning wave.
// Whatever the approximations in W and the quotients: a T is only returned after count(T) was seen to fit.
template <class Count>
LAZYATTN_HD uint32_t plan_choose_tiles(float W, int M, uint32_t c_max, const BatchShape &s, Count count) {
    if (s.forced_splits > 0 || c_max < 4 || M <= 0 || s.items_target <= 0 || M >= s.items_split_cap) return 0;
    const int target = s.items_target;
    int r = 1, lim = target;                              // the fewest rounds the m-tiles leave room to split in
    while (lim <= M) { ++r; lim += target; }
    if (lim > s.items_split_cap) return 0;
    const float tile_us = plan_tile_us(s);
    float best = 0.f;
    int lim_best = 0;
    for (; lim <= s.items_split_cap; ++r, lim += target) {
        const uint32_t T0 = plan_clamp_tiles(plan_ratio(W, (float)(lim - (M >> 1))) + 1.f, c_max);
        const float e = (float)r * ((float)T0 * tile_us + PLAN_ITEM_US);
        if (lim_best == 0 || e < best) { best = e; lim_best = lim; }
    }
    lim = lim_best;
    uint32_t T = plan_clamp_tiles(plan_ratio(W, (float)(lim - M)) + 1.f, c_max);
    int n = count(T);
    for (int i = 0; i < 4 && n > lim; ++i) {              // (only if W was off)
        if (T >= c_max) return 0;
        T = plan_clamp_tiles(plan_ratio((float)T * (float)n, (float)lim) + 1.f, c_max);
        n = count(T);
    }
    if (n > lim) return 0;
    for (int i = 0; i < PLAN_PROBES; ++i) {
        uint32_t T1 = plan_clamp_tiles(plan_ratio((float)T * (float)n, (float)lim), c_max);
        if (T1 >= T) break;
        int n1 = count(T1);
        if (n1 > lim) {
            T1 = (T + T1 + 1) >> 1;
            if (T1 >= T) break;
            n1 = count(T1);
            if (n1 > lim) break;
        }
        T = T1; n = n1;
    }
    return T >= c_max ? 0u : T;
}

// What the first work item of a request leaves for the merge kernel (one entry per request at the head of the workspace).
struct PlanRecord { int32_t item_base, nsplit, m, pad; };      // (m, pad: zero; 16 bytes, one scalar load)

#if defined(__HIPCC__)
// ---------------------------------------------------------------------------------------- one wave scans the batch
struct PlanTables { const void *b_start_loc, *b_seq_len; int32_t batch, index_bits; };

// The low 32 bits of an offset or length (all below 2^31), whatever the width of the entries: one load and no
// branch, so that the nine of a lane are in flight together.
__device__ __forceinline__ int32_t plan_index(const void *p, int64_t i, int bits) {
    return *reinterpret_cast<const int32_t *>((const char *)p + i * (int64_t)(bits >> 3));
}
// Inclusive prefix sum / running maximum over the 64 lanes of a wave in six data-parallel steps (shifts by 1, 2, 4, 8
// inside the rows of 16 lanes, then the last lane of a row combined into the rows after it): vector instructions, no
// trip through the LDS crossbar as a shuffle takes.  Values are non-negative (the identity is 0).
#define LAZYATTN_PLAN_SCAN(OP)                                                                       \
    v = OP(v, __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false)); /* row_shr:1 */            \
    v = OP(v, __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false)); /* row_shr:2 */            \
    v = OP(v, __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false)); /* row_shr:4 */            \
    v = OP(v, __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false)); /* row_shr:8 */            \
    v = OP(v, __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false)); /* row_bcast:15 -> rows 1, 3 */ \
    v = OP(v, __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false)); /* row_bcast:31 -> rows 2, 3 */
__device__ __forceinline__ int plan_add(int a, int b) { return a + b; }
__device__ __forceinline__ int plan_max(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ int plan_wave_scan(int v) { LAZYATTN_PLAN_SCAN(plan_add) return v; }
__device__ __forceinline__ int plan_wave_sum(int v) { return __builtin_amdgcn_readlane(plan_wave_scan(v), 63); }
__device__ __forceinline__ int plan_wave_max(int v) { LAZYATTN_PLAN_SCAN(plan_max) return __builtin_amdgcn_readlane(v, 63); }
#undef LAZYATTN_PLAN_SCAN

// T is chosen on the device for batches of up to 256 requests (four per lane of the scanning wave); larger batches
// are scanned 256 requests at a time for the split count the host fixed.
constexpr int PLAN_MAX_BATCH = 256;
// The requests R lane .. R lane + R - 1 (R = 1 for batches of up to 64 requests, else 4): their m-tile counts and
// costs (0 beyond the batch).  2 R + 1 loads per lane, requested together.
template <int R> struct PlanLane { int m[R]; uint32_t c[R]; };
template <int R> __device__ __forceinline__ PlanLane<R> plan_load(const PlanTables &t, const BatchShape &s, int lane, int first = 0) {
    const int r0 = first + lane * R;
    int32_t off[R + 1], seq[R];
#pragma unroll
    for (int j = 0; j < R + 1; ++j) {
        const int rb = r0 + j;
        off[j] = plan_index(t.b_start_loc, rb < t.batch ? rb : t.batch, t.index_bits);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int rb = r0 + j;
        seq[j] = plan_index(t.b_seq_len, rb < t.batch ? rb : t.batch - 1, t.index_bits);
    }
    PlanLane<R> r;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int32_t ql = r0 + j < t.batch ? off[j + 1] - off[j] : 0;
        const int32_t ctx = seq[j] - ql;
        r.m[j] = plan_mtiles(ql, ctx, s);
        r.c[j] = r.m[j] ? plan_cost(ql, ctx) : 0;
    }
    return r;
}

// plan_splits() for a T the whole wave shares: the reciprocal is formed once, the quotient needs one correction each
// way (cost and T are below 2^24, so the float product is off by less than one)
struct PlanDivisor { uint32_t T; float inv; };
__device__ __forceinline__ PlanDivisor plan_divisor(uint32_t T) { return PlanDivisor{T, T ? 1.0f / (float)T : 0.f}; }
__device__ __forceinline__ int plan_splits_fast(uint32_t cost, const PlanDivisor &d, const BatchShape &s) {
    uint32_t n;
    if (s.forced_splits > 0) n = (uint32_t)s.forced_splits;
    else if (d.T == 0) n = 1;
    else {
        uint32_t q = (uint32_t)((float)cost * d.inv);
        q -= q * d.T > cost;
        q += (q + 1) * d.T <= cost;
        n = q + (q * d.T < cost);
    }
    const uint32_t most = cost / 2 > 1 ? cost / 2 : 1;
    n = n < most ? n : most;
    n = n < (uint32_t)PLAN_MAX_SPLITS ? n : (uint32_t)PLAN_MAX_SPLITS;
    return (int)(n < 1 ? 1 : n);
}
// work items per kv head when a work item is to have at most T tiles (wave-uniform)
template <int R> __device__ __forceinline__ int plan_count(const PlanLane<R> &r, const BatchShape &s, uint32_t T) {
    const PlanDivisor d = plan_divisor(T);
    int n = 0;
#pragma unroll
    for (int j = 0; j < R; ++j) n += r.m[j] ? r.m[j] * plan_splits_fast(r.c[j], d, s) : 0;
    return plan_wave_sum(n);
}
template <int R> __device__ __forceinline__ uint32_t plan_target(const PlanLane<R> &r, const BatchShape &s) {
    if (s.forced_splits > 0) return 0;
    int cm = 0, ws = 0, ms = 0;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        cm = plan_max(cm, (int)r.c[j]);
        ws += (int)(((uint32_t)r.m[j] * r.c[j]) >> 4);             // (m c < 2^24 * m-tiles: sixteenths keep 256 requests' sum in range)
        ms += r.m[j];
    }
    const uint32_t c_max = (uint32_t)plan_wave_max(cm);
    const float W = 16.f * (float)(uint32_t)plan_wave_sum(ws);
    const int M = plan_wave_sum(ms);
    return plan_choose_tiles(W, M, c_max, s, [&](uint32_t T) { return plan_count(r, s, T); });
}

struct PlanItem { int b, mt, split, nsplit, item_base; };      // b < 0: the item is beyond the batch's work
// which (request, m-tile, split) work item `item` of a kv head is (wave-uniform result); the lanes hold the requests
// first .. first + 64 R - 1, whose work items start at item_base; *total: the work items of these requests
template <int R>
__device__ __forceinline__ PlanItem plan_locate(const PlanLane<R> &r, const BatchShape &s, uint32_t T, int item, int lane,
                                                int first = 0, int item_base = 0, int *total = nullptr) {
    PlanItem out{-1, 0, 0, 1, 0};
    const PlanDivisor d = plan_divisor(T);
    int ns[R], cn[R], tot = 0;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        ns[j] = r.m[j] ? plan_splits_fast(r.c[j], d, s) : 0;
        cn[j] = r.m[j] * ns[j];
        tot += cn[j];
    }
    const int incl = plan_wave_scan(tot);
    if (total) *total = __builtin_amdgcn_readlane(incl, 63);
    // (an item before these requests' first is not theirs: without this test the first lane would claim it with a
    // negative remainder -- and the division below does not end for such operands)
    const uint64_t hit = item >= item_base ? __builtin_amdgcn_ballot_w64(item_base + incl > item) : 0ull;
    if (!hit) return out;
    const int idx = __builtin_ctzll(hit);
    int first_item = item_base + __builtin_amdgcn_readlane(incl - tot, idx);
    int rem = item - first_item;
    int j = 0, nsel = __builtin_amdgcn_readlane(ns[0], idx);
#pragma unroll
    for (int k = 0; k + 1 < R; ++k) {
        const int ck = __builtin_amdgcn_readlane(cn[k], idx), nk = __builtin_amdgcn_readlane(ns[k + 1], idx);
        if (j == k && rem >= ck) { rem -= ck; first_item += ck; j = k + 1; nsel = nk; }
    }
    out.b = first + idx * R + j;
    out.nsplit = nsel;
    out.item_base = first_item;
    out.mt = (int)plan_udiv((uint32_t)rem, (uint32_t)nsel);
    out.split = rem - out.mt * nsel;
    return out;
}
// The same for a batch of any size, 256 requests at a time, for the split count the host fixed (T is not chosen on
// the device for such batches).
__device__ __forceinline__ PlanItem plan_locate_chunks(const PlanTables &t, const BatchShape &s, int item, int lane) {
    PlanItem out{-1, 0, 0, 1, 0};
    int base = 0;
#pragma nounroll
    for (int first = 0; first < t.batch; first += PLAN_MAX_BATCH) {
        const PlanLane<4> reqs = plan_load<4>(t, s, lane, first);
        int total = 0;
        out = plan_locate(reqs, s, 0, item, lane, first, base, &total);
        if (out.b >= 0) break;
        base += total;
    }
    return out;
}
#endif  // __HIPCC__

}  // namespace lazyattn
