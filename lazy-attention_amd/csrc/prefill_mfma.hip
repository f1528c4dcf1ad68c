// Host side of the matrix-core prefill path: which workgroup shape and how many key-axis splits a call gets, the
// merge of the split partials, and the launch.  The kernel itself is in prefill_mfma_kernel.hpp.
#include "prefill_mfma_kernel.hpp"
#include <cmath>

namespace lazyattn {

// instantiated in prefill_mfma_<type>[_<fp8 kind>].hip
extern template int launch_mfma_family<bf16_t, 0>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
extern template int launch_mfma_family<bf16_t, 1>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
extern template int launch_mfma_family<bf16_t, 2>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
extern template int launch_mfma_family<f16_t, 0>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
extern template int launch_mfma_family<f16_t, 1>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
extern template int launch_mfma_family<f16_t, 2>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);

// ---- merge split-KV partials ----
// The few fields the merge needs, not the whole parameter block.
struct MergeArgs {
    const void *workspace, *b_start_loc, *b_seq_len;
    void *o;
    int64_t o_stride[2];
    int64_t items_per_kv;           // work items per kv head the partial rows are numbered by
    int32_t num_q_heads, num_kv_heads, index_bits, skip_decode;
    int32_t batch, head_dim;        // head_dim: elements of an output row (below HD when the partial rows are padded)
    int32_t group, nc, n_mt;        // q-heads per kv-head; 32-row units per workgroup of the main kernel; its m-tiles per request
    int32_t nsplit;                 // splits of every request (the plain grid)
    // xcd_map: one-dimensional grid in which the workgroups of a (request, kv-head) go to the XCD whose L2 the main
    // kernel's workgroups of that (request, kv-head) wrote the partial rows through (consecutive workgroup ids go
    // round the eight XCDs; a hint only: any placement gives the same result)
    int32_t xcd_map;
    BatchShape bal;                 // items_cap > 0: the main kernel ran the balanced list, splits differ per request
    FastDiv by_group, by_windows, by_kv_heads;
};

// One workgroup = 32 consecutive tokens of one request x one q-head; wave dt merges the columns dt*32 .. +31, lane
// (gh, l32) the 4-column groups 8*i4 + 4*gh of token l32 -- the mapping of the main kernel's accumulators, so that a
// load instruction reads one contiguous run of the partial rows as the main kernel wrote them (see its epilogue: the
// R rows of a unit are stored [piece][gh][row][4 halves] in the slot of (kv head, work item, wave)).
// Log-sum-exps and row pieces of NB splits (2, 4 or 8, the smallest that covers the request's splits; more only
// beyond eight) are requested together and before the first use: one memory round trip per batch; batches are
// chained like the tiles of the main kernel, by a running maximum.  The merged tile is turned through LDS (rows
// padded by 8 bytes: conflict-free both ways) so that the output leaves as whole rows, 32 bytes per thread.
template <int D, int NB>
__device__ __forceinline__ void merge_splits(const _Float16 *wb, const float2 *we, int64_t split_stride_rows, int R,
                                             int nsplit, float (&o)[16], float &wsum) {
    float mx = -INFINITY;
    for (int s0 = 0; s0 < nsplit; s0 += NB) {
        float2 e[NB];                                        // (log2-sum-exp, scale of the row's halves)
        uint2 v[NB][4];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int64_t so = (int64_t)(s0 + j < nsplit ? s0 + j : nsplit - 1) * split_stride_rows;
            e[j] = we[so];
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
                const u32x2_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(wb + so * D + i4 * (2 * R * 4)));
                v[j][i4] = make_uint2(t[0], t[1]);
            }
        }
        float bm = e[0].x;
#pragma unroll
        for (int j = 1; j < NB; ++j) bm = fmaxf(bm, e[j].x);
        const float m_new = fmaxf(mx, bm);
        if (m_new == -INFINITY) continue;                    // nothing visible so far
        const float keep = __builtin_amdgcn_exp2f(mx - m_new);   // mx = -inf -> 0
#pragma unroll
        for (int i = 0; i < 16; ++i) o[i] *= keep;
        wsum *= keep;
        mx = m_new;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const float w = s0 + j < nsplit ? __builtin_amdgcn_exp2f(e[j].x - mx) : 0.f;
            const float ws = w * e[j].y;
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const f16x2_t a = *reinterpret_cast<const f16x2_t *>(&v[j][i4].x), c = *reinterpret_cast<const f16x2_t *>(&v[j][i4].y);
                o[4 * i4] = fmaf(ws, (float)a[0], o[4 * i4]);
                o[4 * i4 + 1] = fmaf(ws, (float)a[1], o[4 * i4 + 1]);
                o[4 * i4 + 2] = fmaf(ws, (float)c[0], o[4 * i4 + 2]);
                o[4 * i4 + 3] = fmaf(ws, (float)c[1], o[4 * i4 + 3]);
            }
            wsum += w;
        }
    }
}

template <typename T, int HD>
__global__ void __launch_bounds__(HD * 2)
prefill_combine_kernel(const MergeArgs p) {
    using E = Elem<T>;
    constexpr int D = HD, ROW = HD * 2 + 8;                   // bytes of a tile row in LDS
    __shared__ __attribute__((aligned(16))) uint8_t tile[UNIT * ROW];
    __shared__ int row_ok[UNIT];
    const int lane = threadIdx.x & 63, dt = threadIdx.x >> 6, l32 = lane & 31, gh = lane >> 5;
    int h, b, nsplit = p.nsplit;
    int64_t win;                                              // first token of the window, in its request
    int64_t item0;                                            // first work item of the request (balanced) or of (request, m-tile 0)
    int m_req = p.n_mt;                                       // m-tiles of the request the main grid covered
    if (p.xcd_map) {
        const uint32_t L = blockIdx.x, xcd = L & 7u, q = L >> 3;
        const uint32_t t = p.by_group.quot(q), hh = p.by_group.rem(q, t);
        const uint32_t r = p.by_windows.quot(t), w = p.by_windows.rem(t, r);
        const uint32_t bg = r * 8u + xcd;                     // (request, kv-head): what the main kernel keeps on one XCD
        b = (int)p.by_kv_heads.quot(bg);
        h = (int)(p.by_kv_heads.rem(bg, (uint32_t)b) * (uint32_t)p.group + hh);
        win = (int64_t)w * UNIT;
        item0 = (int64_t)b * p.n_mt * p.nsplit;
    } else {
        h = (int)(blockIdx.x % (unsigned)p.num_q_heads);
        win = (int64_t)(blockIdx.x / (unsigned)p.num_q_heads) * UNIT;
        b = blockIdx.y;
        item0 = (int64_t)b * p.n_mt * p.nsplit;
    }
    // Exactly the rows the main kernel wrote partials for: anything else would merge whatever an earlier call
    // left in the workspace.
    // (the request is the same for the whole workgroup and its three entries come as scalar loads in flight
    // together -- this kernel is a chain of memory round trips and little else)
    const int64_t qs = load_index_uniform(p.b_start_loc, b, p.index_bits);
    const int64_t qe = load_index_uniform(p.b_start_loc, b + 1, p.index_bits);
    const int64_t seq = load_index_uniform(p.b_seq_len, b, p.index_bits);
    const int64_t q_len = qe - qs;
    if (p.bal.items_cap > 0) {
        // balanced list: where the request's work items start and how many splits it has was left at the head of the
        // workspace by its first work item (a request without work has no record: its rows are not valid below,
        // whatever an older call left in its place)
        typedef const int32_t __attribute__((address_space(4))) *sptr_record;
        const sptr_record rec = (sptr_record)((const int32_t *)p.workspace + (int64_t)b * 4);
        item0 = rec[0];
        nsplit = rec[1];
        m_req = plan_mtiles((int32_t)q_len, (int32_t)(seq - q_len), p.bal);
        if (m_req > 0 && nsplit <= 1) return;                 // its rows were written directly
        if (nsplit < 1 || nsplit > PLAN_MAX_SPLITS || item0 < 0 || item0 + (int64_t)m_req * nsplit > p.items_per_kv) m_req = 0;
    }
    const int64_t row = win + l32;
    const int unit = (int)(win / UNIT) * p.group + h % p.group;
    const int mt = unit / p.nc, wave = unit % p.nc;
    const bool valid = q_len > 0 && !(p.skip_decode && q_len == 1) && row < q_len && mt < m_req &&   // (past the grid sized by max_q_len)
                       seq - q_len >= 0;
    float o[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) o[i] = 0.f;
    float wsum = 0.f;
    if (valid) {
        const int R = (int)(q_len - win < UNIT ? q_len - win : UNIT);
        const int64_t slots = (int64_t)p.num_kv_heads * p.items_per_kv * p.nc;
        const int64_t slot = ((int64_t)(h / p.group) * p.items_per_kv + item0 + (int64_t)mt * nsplit) * p.nc + wave;   // split 0
        const _Float16 *wo = (const _Float16 *)((const uint8_t *)p.workspace + p.bal.table_bytes);
        const float2 *wl = reinterpret_cast<const float2 *>(wo + slots * UNIT * D);
        const _Float16 *wb = wo + slot * UNIT * D + (dt * 4 * 2 * R + gh * R + l32) * 4;
        const float2 *we = wl + slot * UNIT + l32;
        const int64_t stride = (int64_t)p.nc * UNIT;             // rows from one split's slot to the next
        if (nsplit <= 2) merge_splits<D, 2>(wb, we, stride, R, nsplit, o, wsum);
        else if (nsplit <= 4) merge_splits<D, 4>(wb, we, stride, R, nsplit, o, wsum);
        else merge_splits<D, 8>(wb, we, stride, R, nsplit, o, wsum);
    }
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4)
        *reinterpret_cast<uint2 *>(tile + l32 * ROW + (dt * 32 + 8 * i4 + 4 * gh) * 2) =
            make_uint2(E::pack(o[4 * i4] * inv, o[4 * i4 + 1] * inv), E::pack(o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv));
    if (dt == 0 && gh == 0) row_ok[l32] = valid;
    __syncthreads();
    // whole rows out: 32 bytes per thread, HD/16 threads per row
    const int r = threadIdx.x / (HD / 16), seg = threadIdx.x % (HD / 16);
    if (row_ok[r] && seg * 16 < p.head_dim) {                 // (beyond head_dim: padding columns of the partial rows)
        const uint4 a = *reinterpret_cast<const uint4 *>(tile + r * ROW + seg * 32);
        const uint4 c = *reinterpret_cast<const uint4 *>(tile + r * ROW + seg * 32 + 16);
        T *op = (T *)p.o + (qs + win + r) * p.o_stride[0] + (int64_t)h * p.o_stride[1] + seg * 16;
        *reinterpret_cast<uint4 *>(op) = a;
        *reinterpret_cast<uint4 *>(op + 8) = c;
    }
}

// ------------------------------------------------------------------ host side
// a split-KV partial row: 128 halves + (log2-sum-exp, scale)
// width of the tiles and of a partial row: the head size, or 128 for the head sizes that are padded to it
static int tile_dim(const lazyattn_prefill_params &p) { return p.head_dim == 64 ? 64 : 128; }
static size_t partial_row_bytes(const lazyattn_prefill_params &p) { return (size_t)tile_dim(p) * sizeof(_Float16) + 2 * sizeof(float); }
static int mfma_units(const lazyattn_prefill_params &p) {
    const int group = p.num_q_heads / p.num_kv_heads;
    return ((p.max_q_len + UNIT - 1) / UNIT) * group;
}
static int mfma_mtiles(const lazyattn_prefill_params &p, int nw) { return (mfma_units(p) + nw - 1) / nw; }

// M-tiles (workgroups per kv head and split) the call has, estimated from what the host knows -- the token
// count, the request count and the longest request -- by taking every request to have either one new token or
// max_q_len of them.  Exact for uniform batches and for one long request among one-token requests, the two
// shapes a serving batch usually has; it only steers the split count and the workgroup shape.
static int64_t mfma_mtiles_estimate(const lazyattn_prefill_params &p, int nw) {
    const int64_t per_req = mfma_mtiles(p, nw);
    if (p.batch <= 1 || p.max_q_len <= 1) return (int64_t)p.batch * per_req;
    int64_t longs = ((int64_t)p.num_tokens - p.batch + p.max_q_len - 2) / (p.max_q_len - 1);
    longs = longs < 1 ? 1 : (longs > p.batch ? p.batch : longs);
    const int group = p.num_q_heads / p.num_kv_heads;
    const int64_t per_short = (group + nw - 1) / nw;             // a one-token request, unless it is skipped
    return longs * per_req + (p.skip_decode ? 0 : (p.batch - longs) * per_short);
}
// Upper bound on the same number (batch_plan.hpp).
static int64_t mfma_mtiles_bound(const lazyattn_prefill_params &p, int nw) {
    BatchShape s{};
    s.group = p.num_q_heads / p.num_kv_heads;
    s.nc = nw;
    s.n_mt_cap = mfma_mtiles(p, nw);
    s.skip_decode = p.skip_decode;
    return plan_mtiles_bound(p.num_tokens, p.batch, s);
}
// A list of work items with a fixed split count pays a scan of the lengths per workgroup where the plain grid pays
// nothing: taken when it at least halves the grid (requests with one new token beside long ones).
static bool mfma_compact(const lazyattn_prefill_params &p, int nw) {
    return p.batch > 1 && mfma_mtiles_bound(p, nw) * 2 <= (int64_t)p.batch * mfma_mtiles(p, nw);
}

static int mfma_splits(const lazyattn_prefill_params &p, int nw);

// units (computing waves) per workgroup: the shape with the lower estimated time.  Per workgroup a 64-key tile takes
// about 1.34 us in the four-unit shape (128 rows) and 1.98 us in the eight-unit shape (256 rows: a third less per
// row), a workgroup has some 8 us of launch, prologue, first-tile latency and epilogue, the workgroups run in rounds
// of one per compute unit (256 on the part these figures were taken on), and split partials cost about 2 us plus half a microsecond per split to write and merge.  (Measured on
// this part with bf16 operands at head size 128; the other element types and head sizes shift both shapes alike.)
static int mfma_waves(const lazyattn_prefill_params &p) {
    if (p.kernel == LAZYATTN_KERNEL_MFMA4) return 4;
    if (p.kernel == LAZYATTN_KERNEL_MFMA8) return 8;
    if (mfma_units(p) <= 4) return 4;
    if (p.batch > 1 && p.batch <= PLAN_MAX_BATCH && p.num_splits <= 0) {
        // Several requests, cut into work items on the device: the wider workgroup (a third less time per row) when
        // the average request fills most of it and the batch has rows for a few dozen of them; else its rows would
        // stand empty, or the few workgroups would need many splits.  (Measured over thirty ragged batches at
        // Llama-3-8B geometry: the better shape in all but two, those within 7 %.)
        const int group = p.num_q_heads / p.num_kv_heads;
        const int64_t avg_units = (((int64_t)p.num_tokens / p.batch + UNIT - 1) / UNIT) * group;
        const int64_t all_units = (((int64_t)p.num_tokens + UNIT - 1) / UNIT) * group;
        return avg_units >= 6 && all_units >= 32 ? 8 : 4;
    }
    const int64_t tiles = p.max_seq_len > 0 ? (p.max_seq_len + NT - 1) / NT : 64;
    auto cost = [&](int nw, double tile_us) {
        const int64_t s = mfma_splits(p, nw);
        const int64_t cus = device_cus();
        const int64_t wgs = p.num_kv_heads * mfma_mtiles_estimate(p, nw) * s, rounds = (wgs + cus - 1) / cus;
        return (double)rounds * ((double)((tiles + s - 1) / s) * tile_us + 8.0) + (s > 1 ? 2.0 + 0.5 * (double)s : 0.0);
    };
    return cost(8, 1.98) <= cost(4, 1.34) ? 8 : 4;
}

static int mfma_splits(const lazyattn_prefill_params &p, int nw) {
    if (p.num_splits > 0) return p.num_splits > 64 ? 64 : p.num_splits;
    const int64_t natural = p.num_kv_heads * mfma_mtiles_estimate(p, nw);
    const int64_t ctx_tiles = p.max_seq_len > 0 ? (p.max_seq_len + NT - 1) / NT : 1;
    // One workgroup per CU and none left over: a CU holds one workgroup at a time, so a few workgroups beyond the
    // chip's CUs (256 where these figures were taken) are a second round that most CUs sit out (3 requests of 128 new tokens over 5 K keys, 96
    // workgroups per split: 2 / 3 splits = 192 / 288 workgroups take 55 / 77 us; 6 x 64 over 8 K, 48 per split:
    // 5 / 6 splits 65 / 90 us).  Long workgroups (64 tiles and more) may take two to four whole rounds when that
    // fills the rounds at least a fifth better (3 x 512 new tokens over 16 K keys, 192 per split: 1 / 4 splits =
    // 75 % of one round / three full rounds: 448 / 427 us).
    const int64_t CUS = device_cus();
    int64_t s = natural <= CUS ? CUS / natural : 1;
    auto fill = [&](int64_t sp) {
        const int64_t w = natural * sp, rounds = (w + CUS - 1) / CUS;
        return (double)w / (double)(rounds * CUS);
    };
    if (ctx_tiles / s >= 64) {
        double best = fill(s);
        for (int64_t k = 2; k <= 4; ++k) {
            const int64_t sk = k * CUS / natural;
            if (sk > s && fill(sk) > best * 1.2) { s = sk; best = fill(sk); }
        }
    }
    // A split more costs about half a microsecond (its partial rows written, read and merged) and saves
    // tiles / s^2 tile times: past s = sqrt(2 tiles tile_us) the launch gets longer even with compute units to spare
    // (32 new tokens over 5.4 K keys, 8 workgroups per split: 16 / 32 splits take 21.0 / 24.0 us).
    const double s_most = std::sqrt(2.0 * (double)ctx_tiles * (nw == 8 ? 1.98 : 1.34));
    if ((double)s > s_most) s = (int64_t)(s_most + 0.5);
    if (s > ctx_tiles / 2) s = ctx_tiles / 2;        // at least two tiles per split
    if (s > 64) s = 64;
    return s < 1 ? 1 : (int)s;
}

// Why the matrix-core kernel does not take a call (nullptr: it does).
const char *mfma_unsupported_reason(const lazyattn_prefill_params &p) {
    const bool fp8 = p.cache_dtype == LAZYATTN_FP8_E4M3 || p.cache_dtype == LAZYATTN_FP8_E5M2;
    if (p.dtype != LAZYATTN_BF16 && p.dtype != LAZYATTN_F16) return "operands are not bfloat16 or float16";
    if (!(p.cache_dtype == p.dtype || fp8)) return "the cache type is neither the operand type nor fp8";
    if (p.table_dtype != p.dtype && p.table_dtype != LAZYATTN_F32) return "the cos/sin table is neither of the operand type nor float32";
    // 128, 64, or a multiple of 16 below 128 (padded to 128)
    if (p.head_dim < 16 || p.head_dim > 128 || p.head_dim % 16) return "head size above 128 or not a multiple of 16";
    if (p.rotary_dim != p.head_dim) return "rotary_dim differs from the head size";
    if (p.block_size != BS && p.block_size != 2 * BS) return "cache pages of neither 16 nor 32 slots";
    if (p.x != (fp8 ? 16 : 8)) return "the key cache's innermost axis is not 16 bytes";
    if (p.q_stride[2] != 1 || p.k_stride[2] != 1 || p.v_stride[2] != 1 || p.o_stride[2] != 1) return "q/k/v/o rows are not contiguous";
    if (p.kc_stride[4] != 1 || p.kc_stride[3] != p.x || p.kc_stride[2] != (int64_t)p.block_size * p.x)
        return "a key cache page of one head is not contiguous";
    if (p.vc_stride[3] != 1 || p.vc_stride[2] != p.block_size) return "a value cache page of one head is not contiguous";
    const int64_t al[] = {p.q_stride[0], p.q_stride[1], p.k_stride[0], p.k_stride[1], p.v_stride[0], p.v_stride[1],
                          p.o_stride[0], p.o_stride[1], p.kc_stride[0], p.kc_stride[1], p.vc_stride[0], p.vc_stride[1],
                          p.table_stride};
    for (int64_t s : al)
        if (s % 16) return "a stride is not a multiple of 16 elements";
    const void *ptrs[] = {p.q, p.k, p.v, p.o, p.k_cache, p.v_cache, p.cos_sin_cache};
    for (const void *q : ptrs)
        if (((uintptr_t)q) & 15) return "a tensor is not 16-byte aligned";
    if (p.num_tokens <= 0) return "num_tokens is not set";
    return nullptr;
}
bool mfma_supports(const lazyattn_prefill_params &p) { return mfma_unsupported_reason(p) == nullptr; }



// What one call launches: the workgroup shape, and either the plain grid (request, kv head, split, m-tile) with one
// split count for every request -- a single request, or a fixed split count (the caller's, or the host's for more
// than 256 requests) on a batch without many one-token requests -- or the list of work items (batch_plan.hpp): with
// the splits decided per request on the device (up to 256 requests, no count from the caller) or with the fixed count.
struct MfmaLaunch {
    int nw, n_mt, nsplit;           // nsplit: of the plain grid (1 under the balanced list)
    BatchShape bal;                 // items_cap > 0: balanced list
    int64_t items_per_kv;           // work items per kv head the partial rows are numbered by (0: no partial rows)
};
static MfmaLaunch mfma_launch_shape(const lazyattn_prefill_params &p) {
    MfmaLaunch L{};
    L.nw = mfma_waves(p);
    L.n_mt = mfma_mtiles(p, L.nw);
    const int group = p.num_q_heads / p.num_kv_heads;
    int forced = p.num_splits > 0 ? (p.num_splits > PLAN_MAX_SPLITS ? PLAN_MAX_SPLITS : p.num_splits) : 0;
    // The list of work items replaces the plain grid when the device chooses the splits (up to 256 requests, no count
    // from the caller), else when it at least halves the grid (requests with one new token beside long ones).
    const bool device_splits = p.batch <= PLAN_MAX_BATCH && forced == 0;
    const bool balanced = p.batch > 1 && (device_splits || mfma_compact(p, L.nw));
    auto plain = [&] {
        L.nsplit = mfma_splits(p, L.nw);
        L.items_per_kv = L.nsplit > 1 ? (int64_t)p.batch * L.n_mt * L.nsplit : 0;
        return L;
    };
    if (!balanced) return plain();
    L.nsplit = 1;
    const int64_t m_bound = mfma_mtiles_bound(p, L.nw);             // at least the m-tiles the batch really has
    if (!device_splits && forced == 0) {
        // one count for every request, from the host's estimate of the work -- as far as the partial rows of that
        // many splits of every m-tile the batch may have (the bound, not the estimate) stay within a quarter GB
        forced = mfma_splits(p, L.nw);
        const size_t per_item = (size_t)p.num_kv_heads * L.nw * UNIT * partial_row_bytes(p);
        while (forced > 1 && (size_t)m_bound * (size_t)forced * per_item > ((size_t)256 << 20)) --forced;
    }
    // One round of the chip's compute units is what the device cuts a batch for (batch_plan.hpp); a batch with more
    // m-tiles than that is not split, and the grid has room for it.
    // Room beyond one round -- up to every m-tile cut in four, and three rounds at most -- is made when one round
    // could not even cut every m-tile in two: it would then leave the long requests whole.  (Work items the
    // device does not use return after their scan of the batch: they cost a little at the launch's end, so the grid
    // is not made larger than the device can be expected to fill.)
    const int64_t target = (device_cus() + p.num_kv_heads - 1) / p.num_kv_heads;
    int64_t split_cap = target;
    if (forced) split_cap = m_bound * forced;
    else if (2 * m_bound > target) split_cap = 4 * m_bound < 3 * target ? 4 * m_bound : 3 * target;
    const int64_t cap = split_cap < m_bound ? m_bound : split_cap;
    // (no records when nothing is split: there is no merge to read them, and no workspace to hold them)
    const int64_t table_bytes = forced == 1 ? 0 : ((int64_t)p.batch * (int64_t)sizeof(PlanRecord) + 255) / 256 * 256;
    if (cap > 0x3fffffff || table_bytes > 0x3fffffff) return plain();     // (beyond any real batch)
    L.bal = BatchShape{group, L.nw, L.n_mt, p.skip_decode, (int32_t)cap, (int32_t)target, (int32_t)split_cap, forced,
                       (int32_t)table_bytes};
    // the slots of the partial rows: a batch that is split has at most split_cap items per kv head
    L.items_per_kv = forced == 1 ? 0 : split_cap;
    return L;
}
// the requests' records (balanced list) and the partial rows
static size_t mfma_partial_bytes(const lazyattn_prefill_params &p, const MfmaLaunch &L) {
    if (L.items_per_kv <= 0) return 0;
    return (size_t)L.bal.table_bytes + (size_t)p.num_kv_heads * (size_t)L.items_per_kv * L.nw * UNIT * partial_row_bytes(p);
}

size_t mfma_workspace_bytes(const lazyattn_prefill_params &p) { return mfma_partial_bytes(p, mfma_launch_shape(p)); }

// the choices a call gets: computing waves per workgroup (4 or 8) and key-axis splits (0: decided per request on the device)
void mfma_choices(const lazyattn_prefill_params &p, int *waves, int *splits) {
    const MfmaLaunch L = mfma_launch_shape(p);
    *waves = L.nw;
    *splits = L.bal.items_cap > 0 ? L.bal.forced_splits : L.nsplit;
}

int launch_prefill_mfma(const lazyattn_prefill_params &p, hipStream_t stream) {
    const MfmaLaunch L = mfma_launch_shape(p);
    const int nw = L.nw, nsplit = L.nsplit, n_mt = L.n_mt;
    const int phases = p.phases ? p.phases : LAZYATTN_PHASE_ALL;
    if (mfma_partial_bytes(p, L) > 0) {
        const size_t need = mfma_partial_bytes(p, L);
        if (!p.workspace || (size_t)p.workspace_bytes < need) return LAZYATTN_E_WORKSPACE;
        if (((uintptr_t)p.workspace) & 15) return LAZYATTN_E_WORKSPACE;
    }
    if (phases & LAZYATTN_PHASE_MAIN) {
        const bool f16 = p.dtype == LAZYATTN_F16;
        int rc;
        if (p.cache_dtype == LAZYATTN_FP8_E4M3)
            rc = f16 ? launch_mfma_family<f16_t, 1>(p, nw, nsplit, n_mt, L.bal, stream) : launch_mfma_family<bf16_t, 1>(p, nw, nsplit, n_mt, L.bal, stream);
        else if (p.cache_dtype == LAZYATTN_FP8_E5M2)
            rc = f16 ? launch_mfma_family<f16_t, 2>(p, nw, nsplit, n_mt, L.bal, stream) : launch_mfma_family<bf16_t, 2>(p, nw, nsplit, n_mt, L.bal, stream);
        else
            rc = f16 ? launch_mfma_family<f16_t, 0>(p, nw, nsplit, n_mt, L.bal, stream) : launch_mfma_family<bf16_t, 0>(p, nw, nsplit, n_mt, L.bal, stream);
        if (rc != LAZYATTN_OK) return rc;
    }
    if (L.items_per_kv > 0 && (phases & LAZYATTN_PHASE_COMBINE)) {
        const int group = p.num_q_heads / p.num_kv_heads;
        // 32 tokens x one q-head per workgroup: windows per request x requests
        const int64_t windows = ((int64_t)p.max_q_len + UNIT - 1) / UNIT;
        // (the condition under which the main kernel gives a (request, kv-head) to one XCD; under the balanced list
        // a kv head stays on one XCD, which the same numbering gives when the kv heads are a multiple of eight)
        const int xcd_map = ((p.batch * p.num_kv_heads) & 7) == 0 && windows * p.num_q_heads * p.batch <= 0x7fffffff;
        if (windows * p.num_q_heads > 0x7fffffff) return LAZYATTN_E_SHAPE;
        const MergeArgs m{p.workspace, p.b_start_loc, p.b_seq_len, p.o, {p.o_stride[0], p.o_stride[1]}, L.items_per_kv,
                          p.num_q_heads, p.num_kv_heads, p.index_bits, p.skip_decode, p.batch, p.head_dim, group, nw, n_mt,
                          nsplit, xcd_map, L.bal,
                          FastDiv((uint32_t)group), FastDiv((uint32_t)windows), FastDiv((uint32_t)p.num_kv_heads)};
        const dim3 grid = xcd_map ? dim3((unsigned)(windows * p.num_q_heads * p.batch))
                                  : dim3((unsigned)(windows * p.num_q_heads), p.batch);
        const bool f16 = p.dtype == LAZYATTN_F16;
        if (tile_dim(p) == 64) {
            if (f16) hipLaunchKernelGGL((prefill_combine_kernel<f16_t, 64>), grid, dim3(128), 0, stream, m);
            else hipLaunchKernelGGL((prefill_combine_kernel<bf16_t, 64>), grid, dim3(128), 0, stream, m);
        } else {
            if (f16) hipLaunchKernelGGL((prefill_combine_kernel<f16_t, 128>), grid, dim3(256), 0, stream, m);
            else hipLaunchKernelGGL((prefill_combine_kernel<bf16_t, 128>), grid, dim3(256), 0, stream, m);
        }
        if (hipGetLastError() != hipSuccess) return LAZYATTN_E_LAUNCH;
    }
    return LAZYATTN_OK;
}

}  // namespace lazyattn
