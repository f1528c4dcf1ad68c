"""The arithmetic that cuts a ragged batch into work items on the device (csrc/batch_plan.hpp), compiled for the
host: no split is shorter than two tiles, no request is cut into more than 64, more splits of the longest request
never mean fewer work items, the small-number division is exact, and the tiles per work item chosen for a batch
never make more work items than the grid has room for -- also when the totals it starts from are off -- and the
host's bound on a batch's m-tiles holds.  No GPU needed."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SRC = r'''
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>
#include "batch_plan.hpp"
using namespace lazyattn;
int main() {
    // exact division for numerators and divisors below 2^24
    std::mt19937 rng(7);
    for (int i = 0; i < 2000000; ++i) {
        const uint32_t n = rng() & 0xffffff, d = (rng() & 0xffffff) | 1u;
        const uint32_t dd = i % 3 == 0 ? (d & 0xff) | 1u : d;
        if (plan_udiv(n, dd) != n / dd) { printf("udiv %u %u\n", n, dd); return 1; }
    }
    for (uint32_t d = 1; d < 3000; ++d)
        for (uint32_t n : {0u, 1u, d - 1, d, d + 1, 2 * d - 1, 2 * d, 16777215u, 16777215u / d * d, 16777215u / d * d - 1})
            if (n < (1u << 24) && plan_udiv(n, d) != n / d) { printf("udiv edge %u %u\n", n, d); return 1; }
    // random batches, every candidate the planning kernel looks at (the longest request cut into k = 1 .. 64):
    // every request with work gets between 1 and 64 splits of at least two tiles, none longer than the candidate's
    // item length unless one of those bounds holds it back; k = 1 splits nothing; more splits never mean fewer items
    for (int trial = 0; trial < 3000; ++trial) {
        BatchShape s{};
        s.group = 1 << (rng() % 4);
        s.nc = (rng() & 1) ? 8 : 4;
        s.n_mt_cap = 1 + rng() % 64;
        s.skip_decode = rng() & 1;
        const int batch = 1 + rng() % 40;
        std::vector<int> m(batch);
        std::vector<uint32_t> c(batch);
        std::vector<int64_t> ql_of(batch);
        uint64_t W = 0;
        uint32_t M = 0, c_max = 0;
        for (int j = 0; j < batch; ++j) {
            const int64_t ql = (rng() % 5 == 0) ? 1 : (rng() % 4 == 0 ? 2 + rng() % 3 : 1 + rng() % 600);
            const int64_t ctx = (rng() % 7 == 0) ? 0 : rng() % (1 << (8 + rng() % 12));
            ql_of[j] = ql;
            m[j] = plan_mtiles(ql, ctx, s);
            c[j] = m[j] ? plan_cost(ql, ctx) : 0;
            W += (uint64_t)m[j] * c[j];
            M += m[j];
            c_max = c[j] > c_max ? c[j] : c_max;
        }
        {   // the host's bound on the m-tiles, from the totals alone
            int64_t tokens = 0;
            for (int j = 0; j < batch; ++j) tokens += ql_of[j];
            if ((int64_t)M > plan_mtiles_bound(tokens, batch, s)) {
                printf("%u m-tiles, bound %lld (tokens %lld, batch %d, group %d, nc %d, cap %d, skip %d)\n", M,
                       (long long)plan_mtiles_bound(tokens, batch, s), (long long)tokens, batch, s.group, s.nc, s.n_mt_cap, s.skip_decode);
                return 1;
            }
        }
        if (!c_max) continue;
        uint64_t prev = 0;
        for (uint32_t k = 1; k <= 64; ++k) {
            const uint32_t T = (c_max + k - 1) / k;
            uint64_t items = 0;
            uint32_t longest = 0;
            for (int j = 0; j < batch; ++j) {
                if (!m[j]) continue;
                const uint32_t ns = (uint32_t)plan_splits(c[j], T, s);
                const uint32_t len = (c[j] + ns - 1) / ns;
                if (ns < 1 || ns > 64 || (ns > 1 && c[j] / ns < 2)) { printf("splits %u cost %u T %u\n", ns, c[j], T); return 1; }
                if (len > T && ns != 64 && c[j] / (ns + 1) >= 2) { printf("item of %u tiles for T %u (cost %u, %u splits)\n", len, T, c[j], ns); return 1; }
                items += (uint64_t)m[j] * ns;
                longest = len > longest ? len : longest;
            }
            if (k == 1 && items != M) { printf("k = 1 splits something\n"); return 1; }
            if (items < prev) { printf("fewer items for more splits\n"); return 1; }
            prev = items;
        }
        // the choice of T: whatever it is, the items it makes fit the rounds the grid has room for; every candidate
        // it was offered is counted with the real counts; totals off by a quarter either way change nothing in that
        s.items_target = 1 + rng() % 40;
        s.items_split_cap = s.items_target * (1 + rng() % 3) + rng() % 3;
        s.items_cap = s.items_split_cap > (int)M ? s.items_split_cap : (int)M;
        for (float off : {1.0f, 0.75f, 1.25f}) {
            int probes = 0;
            auto count = [&](uint32_t T) {
                ++probes;
                int n = 0;
                for (int j = 0; j < batch; ++j) n += m[j] ? m[j] * plan_splits(c[j], T, s) : 0;
                return n;
            };
            const uint32_t T = plan_choose_tiles((float)W * off, (int)M, c_max, s, count);
            if (probes > 5 + 2 * PLAN_PROBES) { printf("%d probes\n", probes); return 1; }
            const int n = count(T);
            if (T == 0 ? n != (int)M : (n > s.items_split_cap || T < 2 || T >= c_max)) {
                printf("T %u makes %d items (m-tiles %u, room %d, c_max %u)\n", T, n, M, s.items_split_cap, c_max);
                return 1;
            }
            // a batch that fits half a round and has a request worth cutting is cut
            if (off == 1.0f && T == 0 && (int)M * 2 <= s.items_target && c_max >= 64 && s.items_target >= 8) {
                printf("nothing split: m-tiles %u of %d, c_max %u\n", M, s.items_target, c_max);
                return 1;
            }
        }
        s.forced_splits = 1 + rng() % 70;
        for (int j = 0; j < batch; ++j)
            if (m[j]) {
                const int ns = plan_splits(c[j], 0, s);
                const int want = s.forced_splits > 64 ? 64 : s.forced_splits;
                if (ns > want || ns < 1 || (ns < want && c[j] / (ns + 1) >= 2)) { printf("forced %d -> %d (cost %u)\n", s.forced_splits, ns, c[j]); return 1; }
            }
    }
    printf("ok\n");
    return 0;
}
'''


def test_batch_partition_arithmetic(tmp_path):
    src = tmp_path / "plan.cpp"
    src.write_text(SRC)
    exe = tmp_path / "plan"
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "lazy-attention_amd", "csrc"), str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)]).decode()
    assert out.strip() == "ok", out
