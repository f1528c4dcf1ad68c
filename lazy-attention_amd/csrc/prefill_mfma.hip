// Host side of the matrix-core prefill path: which workgroup shape and how many key-axis splits a call gets, the
// merge of the split partials, and the launch.  The kernel itself is in prefill_mfma_kernel.hpp.
#include "prefill_mfma_kernel.hpp"

namespace lazyattn {

// instantiated in prefill_mfma_<type>[_<fp8 kind>].hip
extern template int launch_mfma_family<bf16_t, 0>(const lazyattn_prefill_params &, int, int, int, int, hipStream_t);
extern template int launch_mfma_family<bf16_t, 1>(const lazyattn_prefill_params &, int, int, int, int, hipStream_t);
extern template int launch_mfma_family<bf16_t, 2>(const lazyattn_prefill_params &, int, int, int, int, hipStream_t);
extern template int launch_mfma_family<f16_t, 0>(const lazyattn_prefill_params &, int, int, int, int, hipStream_t);
extern template int launch_mfma_family<f16_t, 1>(const lazyattn_prefill_params &, int, int, int, int, hipStream_t);
extern template int launch_mfma_family<f16_t, 2>(const lazyattn_prefill_params &, int, int, int, int, hipStream_t);

// ---- merge split-KV partials ----
// The few fields the merge needs, not the whole parameter block.
struct MergeArgs {
    const void *workspace, *b_start_loc, *b_seq_len;
    void *o;
    int64_t o_stride[2];
    int32_t num_tokens, num_q_heads, index_bits, skip_decode;
    int32_t batch, token_grid;      // token_grid: the 32-token windows are cut over all tokens instead of per request
    int32_t head_dim;               // elements of an output row (below HD when the partial rows are padded)
    int32_t group, unit_cap;        // q-heads per kv-head; 32-row units per (request, kv-head) the main grid covers
    // xcd_map: one-dimensional grid in which the workgroups of a (request, kv-head) go to the XCD whose L2 the main
    // kernel's workgroups of that (request, kv-head) wrote the partial rows through (consecutive workgroup ids go
    // round the eight XCDs; a hint only: any placement gives the same result)
    int32_t xcd_map;
    FastDiv by_group, by_windows, by_kv_heads;
};
// One workgroup = 32 consecutive tokens x one q-head; wave dt merges the columns dt*32 .. +31, lane (gh, l32) the
// 4-column groups 8*i4 + 4*gh of token l32 -- the mapping of the main kernel's accumulators, so that a load
// instruction reads one contiguous run of the partial rows as the main kernel wrote them (see its epilogue: the R
// rows of a request's 32-token chunk are stored [head][piece][gh][row][4 halves]).  Log-sum-exps and row pieces of NB
// splits (2, 4 or 8, the smallest that covers nsplit; more only when nsplit > 8) are requested together and before
// the first use: one memory round trip per batch; batches are chained like the tiles of the main kernel, by a
// running maximum.  The merged tile is turned through LDS (rows padded by 8 bytes: conflict-free both ways) so
// that the output leaves as whole rows, 32 bytes per thread.  The windows are cut per request (grid y = request),
// or over all tokens of the call when that grid is at most half as large (one long request among one-token
// requests): then the 32 tokens of a workgroup need not belong to one request, and every lane finds its own by a
// binary search of the offsets.
template <typename T, int HD, int NB>
__global__ void __launch_bounds__(HD * 2)
prefill_combine_kernel(const MergeArgs p, const int nsplit) {
    using E = Elem<T>;
    constexpr int D = HD, ROW = HD * 2 + 8;                   // bytes of a tile row in LDS
    __shared__ __attribute__((aligned(16))) uint8_t tile[UNIT * ROW];
    __shared__ int row_ok[UNIT];
    const int lane = threadIdx.x & 63, dt = threadIdx.x >> 6, l32 = lane & 31, gh = lane >> 5;
    int h, b;
    int64_t win;                                              // first token of the window
    if (p.xcd_map) {
        const uint32_t L = blockIdx.x, xcd = L & 7u, q = L >> 3;
        const uint32_t t = p.by_group.quot(q), hh = p.by_group.rem(q, t);
        const uint32_t r = p.by_windows.quot(t), w = p.by_windows.rem(t, r);
        const uint32_t bg = r * 8u + xcd;                     // (request, kv-head): what the main kernel keeps on one XCD
        b = (int)p.by_kv_heads.quot(bg);
        h = (int)(p.by_kv_heads.rem(bg, (uint32_t)b) * (uint32_t)p.group + hh);
        win = (int64_t)w * UNIT;
    } else {
        h = (int)(blockIdx.x % (unsigned)p.num_q_heads);
        win = (int64_t)(blockIdx.x / (unsigned)p.num_q_heads) * UNIT;
        b = blockIdx.y;
    }
    bool valid = true;
    if (p.token_grid) {
        valid = win + l32 < load_index(p.b_start_loc, p.batch, p.index_bits);
        int lo = 0, hi = p.batch;                             // offsets[lo] <= token < offsets[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (load_index(p.b_start_loc, mid, p.index_bits) <= win + l32) lo = mid; else hi = mid;
        }
        b = lo;
    }
    // Exactly the rows the main kernel wrote partials for: anything else would merge whatever an earlier call
    // left in the workspace.
    // (per-request windows: the request is the same for the whole workgroup and its three entries come as scalar
    // loads in flight together -- this kernel is a chain of memory round trips and little else)
    int64_t qs, qe, seq;
    if (p.token_grid) {
        qs = load_index(p.b_start_loc, b, p.index_bits);
        qe = load_index(p.b_start_loc, b + 1, p.index_bits);
        seq = load_index(p.b_seq_len, b, p.index_bits);
    } else {
        qs = load_index_uniform(p.b_start_loc, b, p.index_bits);
        qe = load_index_uniform(p.b_start_loc, b + 1, p.index_bits);
        seq = load_index_uniform(p.b_seq_len, b, p.index_bits);
    }
    const int64_t q_len = qe - qs;
    const int64_t tok0 = p.token_grid ? win : qs + win;       // token of the window's row 0
    const int64_t row = tok0 + l32 - qs;
    valid = valid && q_len > 0 && !(p.skip_decode && q_len == 1) && row < q_len &&
            (row / UNIT) * p.group + h % p.group < p.unit_cap &&                 // (past the grid sized by max_q_len)
            seq - q_len >= 0;
    float o[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) o[i] = 0.f;
    float wsum = 0.f;
    if (valid) {
        const int64_t t0 = (row / UNIT) * UNIT;
        const int R = (int)(q_len - t0 < UNIT ? q_len - t0 : UNIT), lr = (int)(row - t0);
        const int64_t NTOK = p.num_tokens, split_rows = NTOK * p.num_q_heads;
        const _Float16 *wo = (const _Float16 *)p.workspace;
        const float2 *wl = reinterpret_cast<const float2 *>(wo + (int64_t)nsplit * split_rows * D);
        const int64_t blk = (qs + t0) * p.num_q_heads + (int64_t)h * R;                  // in rows, split 0
        const _Float16 *wb = wo + blk * D + (dt * 4 * 2 * R + gh * R + lr) * 4;
        const float2 *we = wl + blk + lr;
        float mx = -INFINITY;
        for (int s0 = 0; s0 < nsplit; s0 += NB) {
            float2 e[NB];                                        // (log2-sum-exp, scale of the row's halves)
            uint2 v[NB][4];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int64_t so = (int64_t)(s0 + j < nsplit ? s0 + j : nsplit - 1) * split_rows;
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
        T *op = (T *)p.o + (tok0 + r) * p.o_stride[0] + (int64_t)h * p.o_stride[1] + seg * 16;
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
// Upper bound on the same number: every request may end with a partly filled 32-row chunk and a partly filled
// m-tile.  The compact work list is sized by it.
static int64_t mfma_mtiles_bound(const lazyattn_prefill_params &p, int nw) {
    const int group = p.num_q_heads / p.num_kv_heads;
    const int64_t chunks = ((int64_t)p.num_tokens + UNIT - 1) / UNIT + p.batch;
    return (chunks * group + nw - 1) / nw + p.batch;
}
// The compact list pays a scan of the token offsets per workgroup: taken when it at least halves the grid.
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

// the choices launch_prefill_mfma() makes for a call: computing waves per workgroup (4 or 8) and key-axis splits
void mfma_choices(const lazyattn_prefill_params &p, int *waves, int *splits) {
    *waves = mfma_waves(p);
    *splits = mfma_splits(p, *waves);
}

size_t mfma_workspace_bytes(const lazyattn_prefill_params &p) {
    const int nw = mfma_waves(p);
    const int ns = mfma_splits(p, nw);
    if (ns <= 1) return 0;
    return (size_t)ns * (size_t)p.num_tokens * p.num_q_heads * partial_row_bytes(p);
}

int launch_prefill_mfma(const lazyattn_prefill_params &p, hipStream_t stream) {
    const int nw = mfma_waves(p);
    const int nsplit = mfma_splits(p, nw);
    const int n_mt = mfma_mtiles(p, nw);
    const int64_t bound = mfma_mtiles_bound(p, nw);
    const int mt_total = mfma_compact(p, nw) && bound <= 0x7fffffff ? (int)bound : 0;
    const int phases = p.phases ? p.phases : LAZYATTN_PHASE_ALL;
    if (nsplit > 1) {
        const size_t need = (size_t)nsplit * (size_t)p.num_tokens * p.num_q_heads * partial_row_bytes(p);
        if (!p.workspace || (size_t)p.workspace_bytes < need) return LAZYATTN_E_WORKSPACE;
        if (((uintptr_t)p.workspace) & 15) return LAZYATTN_E_WORKSPACE;
    }
    if (phases & LAZYATTN_PHASE_MAIN) {
        const bool f16 = p.dtype == LAZYATTN_F16;
        int rc;
        if (p.cache_dtype == LAZYATTN_FP8_E4M3)
            rc = f16 ? launch_mfma_family<f16_t, 1>(p, nw, nsplit, n_mt, mt_total, stream) : launch_mfma_family<bf16_t, 1>(p, nw, nsplit, n_mt, mt_total, stream);
        else if (p.cache_dtype == LAZYATTN_FP8_E5M2)
            rc = f16 ? launch_mfma_family<f16_t, 2>(p, nw, nsplit, n_mt, mt_total, stream) : launch_mfma_family<bf16_t, 2>(p, nw, nsplit, n_mt, mt_total, stream);
        else
            rc = f16 ? launch_mfma_family<f16_t, 0>(p, nw, nsplit, n_mt, mt_total, stream) : launch_mfma_family<bf16_t, 0>(p, nw, nsplit, n_mt, mt_total, stream);
        if (rc != LAZYATTN_OK) return rc;
    }
    if (nsplit > 1 && (phases & LAZYATTN_PHASE_COMBINE)) {
        // windows per request x requests, or windows over all tokens when that is at most half as many
        const int token_grid = p.batch > 1 && 2 * (int64_t)p.num_tokens <= (int64_t)p.batch * p.max_q_len;
        // 32 tokens x one q-head per workgroup
        const int64_t windows = ((int64_t)(token_grid ? p.num_tokens : p.max_q_len) + UNIT - 1) / UNIT;
        const int group = p.num_q_heads / p.num_kv_heads;
        // (the condition under which the main kernel gives a (request, kv-head) to one XCD)
        const int xcd_map = !token_grid && mt_total == 0 && ((p.batch * p.num_kv_heads) & 7) == 0 &&
                            windows * p.num_q_heads * p.batch <= 0x7fffffff;
        const MergeArgs m{p.workspace, p.b_start_loc, p.b_seq_len, p.o, {p.o_stride[0], p.o_stride[1]}, p.num_tokens, p.num_q_heads,
                          p.index_bits, p.skip_decode, p.batch, token_grid, p.head_dim, group,
                          mt_total > 0 ? 0x7fffffff : n_mt * nw, xcd_map,
                          FastDiv((uint32_t)group), FastDiv((uint32_t)windows), FastDiv((uint32_t)p.num_kv_heads)};
        const dim3 grid = xcd_map ? dim3((unsigned)(windows * p.num_q_heads * p.batch))
                                  : dim3((unsigned)(windows * p.num_q_heads), token_grid ? 1 : p.batch);
        const bool f16 = p.dtype == LAZYATTN_F16;
#define LAZYATTN_COMBINE(HD, NB)                                                                                  \
    {                                                                                                             \
        if (f16) hipLaunchKernelGGL((prefill_combine_kernel<f16_t, HD, NB>), grid, dim3(HD * 2), 0, stream, m, nsplit); \
        else hipLaunchKernelGGL((prefill_combine_kernel<bf16_t, HD, NB>), grid, dim3(HD * 2), 0, stream, m, nsplit);    \
    }
        if (p.head_dim == 64) {
            if (nsplit <= 2) LAZYATTN_COMBINE(64, 2) else if (nsplit <= 4) LAZYATTN_COMBINE(64, 4) else LAZYATTN_COMBINE(64, 8)
        } else {
            if (nsplit <= 2) LAZYATTN_COMBINE(128, 2) else if (nsplit <= 4) LAZYATTN_COMBINE(128, 4) else LAZYATTN_COMBINE(128, 8)
        }
#undef LAZYATTN_COMBINE
        if (hipGetLastError() != hipSuccess) return LAZYATTN_E_LAUNCH;
    }
    return LAZYATTN_OK;
}

}  // namespace lazyattn
