"""Pins for the CPU oracle (no GPU).  Each test is chosen so that a plausible mistake
in the oracle (a wrong sign in the rotation, a transposed cache index, an off-by-one
in the q_offset bias, a dropped pad mask, a wrong causal edge) fails it.

Reference vectors used: lazy_attn/tests/core/test_scheduler.py:49-50,
tests/core/test_rotation_offset_bound.py:18-75, tests/worker/test_q_offset_range.py:71-79.
The reference stores no numeric vectors for the attention kernels themselves; those
are pinned by brute force, an independent C restatement, torch's SDPA on pre-rotated
keys (the construction of tests/kernels/test_prefix_prefill.py:107-134,238-289), and
invariants of rotary attention.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import deferred_rope as orc
from lazy_amd import workloads as wl
from cref import run_c_ref


def run_oracle(w, **kw):
    return orc.prefix_prefill(
        w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
        w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode,
        rotate_new_k=w.rotate_new_k, kv_cache_dtype=w.kv_cache_dtype,
        k_scale=w.k_scale, v_scale=w.v_scale, **kw)


def tiny(variant, seed=0, dtype=torch.float32, doc_lens=(5, 8, 3), q_lens=(3, 1, 4), bs=4, **kw):
    reqs = [[2, 0], [1], [0, 1, 2]][:len(q_lens)]
    return wl.make_workload("tiny", dtype=dtype, hq=4, hkv=2, d=8, theta=10000.0, block_size=bs,
                            doc_lens=list(doc_lens), requests=reqs, q_lens=list(q_lens),
                            variant=variant, seed=seed, keep_aux=True, **kw)


# ---------------------------------------------------------------- metadata (KAT)
def test_metadata_known_answer():
    # lazy_attn/tests/core/test_scheduler.py:16-23,49-50
    q_offset, q_mask = orc.metadata_for_lazy_attention([6, 15, 8, 2], [8, 16, 8, 8], 8)
    assert q_offset == [10, 16, 16, 31, 39, 1]
    assert q_mask == [2, 0, 1, 0, 6, 0]
    q_offset, q_mask2 = orc.metadata_for_mepic([6, 15, 8, 2], [8, 16, 8, 8], 8)
    assert q_offset == [0] * 6 and q_mask2 == q_mask


@pytest.mark.parametrize("lens", [[6], [16, 16], [6, 15, 8, 2], [1] * 5, [4096, 17], [100] * 32])
def test_metadata_closed_form(lens):
    # lazy_attn/tests/core/test_rotation_offset_bound.py:18-44
    padded = [((n + 15) // 16) * 16 for n in lens]
    q_offset, _ = orc.metadata_for_lazy_attention(lens, padded, 16)
    assert orc.max_rotation_offset(lens, padded) == max(q_offset)


def test_metadata_bound_examples():
    # test_rotation_offset_bound.py:47-75
    huge = 0xFFFF * 4
    assert orc.max_rotation_offset([huge], [huge]) == 1
    assert orc.max_rotation_offset([1024] * 64, [1024] * 64) == 1024 * 63 + 1
    assert orc.max_rotation_offset([1] * 8, [16] * 8) == 8 * 15 + 7 + 1


def test_workload_metadata_matches_producer():
    w = tiny("block_uniform", doc_lens=(6, 15, 8, 2), q_lens=(3,), bs=8)
    # request 0 uses documents [2, 0] -> true [8, 6], padded [8, 8]
    qo, qm = orc.metadata_for_lazy_attention([8, 6], [8, 8], 8)
    assert w.q_offset[0, :len(qo)].tolist() == qo
    assert w.q_mask[0, :len(qm)].tolist() == qm


# ---------------------------------------------------------------- cos/sin table
def test_table_closed_form():
    t = orc.build_cos_sin_table(300, 64, 500000.0, dtype=torch.float64, math_dtype=torch.float64)
    assert t.shape == (300, 64)
    assert torch.equal(t[0], torch.cat([torch.ones(32), torch.zeros(32)]).double())
    for p, i in [(1, 0), (7, 5), (123, 31), (299, 17)]:
        inv = 500000.0 ** (-2.0 * i / 64)
        assert abs(t[p, i].item() - math.cos(p * inv)) < 1e-12
        assert abs(t[p, 32 + i].item() - math.sin(p * inv)) < 1e-12
    assert torch.allclose(t[:, :32] ** 2 + t[:, 32:] ** 2, torch.ones(300, 32).double(), atol=1e-12)
    # angle addition: R(a)R(b) = R(a+b)
    a, b = 37, 101
    ca, sa, cb, sb = t[a, :32], t[a, 32:], t[b, :32], t[b, 32:]
    assert torch.allclose(ca * cb - sa * sb, t[a + b, :32], atol=1e-12)
    assert torch.allclose(sa * cb + ca * sb, t[a + b, 32:], atol=1e-12)


def test_llama3_inv_freq_regions():
    # cos_sin.py:44-58: short wavelengths untouched, long ones divided by the factor,
    # the band between interpolated; monotone non-increasing.
    kw = dict(scaling_factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, orig_max_position=8192)
    plain = orc.plain_inv_freq(128, 500000.0)
    l3 = orc.llama3_inv_freq(128, 500000.0, **kw)
    wl_ = 2 * math.pi / plain
    hi = wl_ < 8192 / 4.0
    lo = wl_ > 8192 / 1.0
    assert hi.any() and lo.any() and (~hi & ~lo).any()
    assert torch.equal(l3[hi], plain[hi])
    assert torch.allclose(l3[lo], plain[lo] / 8.0)
    mid = ~hi & ~lo
    assert ((l3[mid] < plain[mid]) & (l3[mid] > plain[mid] / 8.0)).all()
    i = int(torch.nonzero(mid)[0])
    s = (8192 / wl_[i] - 1.0) / 3.0
    assert abs(l3[i] - ((1 - s) * plain[i] / 8.0 + s * plain[i])) < 1e-15
    assert workloads_table_matches(kw)


def workloads_table_matches(kw):
    a = wl.cos_sin_table(64, 128, 500000.0, torch.float32, llama3=kw)
    b = orc.build_cos_sin_table(64, 128, 500000.0, llama3=kw, dtype=torch.float32)
    return torch.allclose(a, b, atol=1e-6)


def test_rotation_is_norm_preserving_and_sign_correct():
    t = orc.build_cos_sin_table(50, 8, 10000.0, dtype=torch.float64, math_dtype=torch.float64)
    x = torch.randn(50, 3, 8, dtype=torch.float64)
    y = orc.rotate_at(x, torch.arange(50), t)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
    assert torch.equal(y[0], x[0])
    # pair (i, i+D/2) is rotated counter-clockwise by p*inv[i]: e_i -> cos e_i + sin e_{i+D/2}
    e = torch.zeros(1, 1, 8, dtype=torch.float64); e[0, 0, 1] = 1.0
    r = orc.rotate_at(e, torch.tensor([5]), t)[0, 0]
    inv = 10000.0 ** (-2.0 / 8)
    assert abs(r[1] - math.cos(5 * inv)) < 1e-12 and abs(r[5] - math.sin(5 * inv)) < 1e-12


# ---------------------------------------------------------------- brute force
@pytest.mark.parametrize("variant", ["natural", "offset", "block_uniform"])
@pytest.mark.parametrize("sliding_window", [0, 5])
def test_oracle_equals_brute_force(variant, sliding_window):
    w = tiny(variant, seed=3)
    got = run_oracle(w, sliding_window=sliding_window, compute_dtype=torch.float64)
    ref = orc.brute_force_prefix_prefill(
        w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table.tolist(), w.b_start_loc, w.b_seq_len,
        w.cos_sin_cache, w.q_offset.tolist(), w.q_mask.tolist(), pos_mode=w.pos_mode,
        rotate_new_k=w.rotate_new_k, sliding_window=sliding_window)
    assert (got.double() - ref).abs().max() < 1e-6


def test_oracle_vanilla_branch_equals_brute_force():
    w = tiny("block_uniform", seed=4)
    lazy = torch.tensor([True, False, False])
    got = run_oracle(w, is_lazy=lazy, compute_dtype=torch.float64)
    ref = orc.brute_force_prefix_prefill(
        w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table.tolist(), w.b_start_loc, w.b_seq_len,
        w.cos_sin_cache, w.q_offset.tolist(), w.q_mask.tolist(), pos_mode=w.pos_mode,
        rotate_new_k=w.rotate_new_k, is_lazy=lazy.tolist())
    assert (got.double() - ref).abs().max() < 1e-6
    # and the vanilla rows differ from the rotated ones (the flag is not a no-op)
    assert (got - run_oracle(w, compute_dtype=torch.float64)).abs().max() > 1e-3


# ---------------------------------------------------------------- C restatement
@pytest.mark.parametrize("variant", ["natural", "offset", "block_uniform"])
def test_oracle_equals_c_restatement(c_ref, variant):
    w = wl.make_workload("mid", dtype=torch.float32, hq=8, hkv=2, d=32, theta=500000.0,
                         block_size=16, doc_lens=[40, 16, 33, 70], requests=[[3, 1, 0], [2], [0, 2, 3, 1]],
                         q_lens=[70, 1, 9], variant=variant, seed=11)
    for sw in (0, 37):
        a = run_oracle(w, sliding_window=sw)
        b = run_c_ref(c_ref, w, sliding_window=sw)
        assert (a - b).abs().max() < 2e-6, (variant, sw)
    a = run_oracle(w, skip_decode=True, out=torch.full_like(w.q, 7.0))
    b = run_c_ref(c_ref, w, skip_decode=True)
    assert torch.all(a[70] == 7.0)              # the q_len==1 request is left untouched
    keep = torch.ones(80, dtype=torch.bool); keep[70] = False
    assert (a[keep] - b[keep]).abs().max() < 2e-6


def test_c_restatement_config1_full(c_ref):
    w = wl.config(1)
    assert w.q.shape == (64, 32, 64) and w.k_cache.shape == (64, 8, 16, 16, 4)
    assert abs(w.flops / 1e9 - 0.2855) < 1e-3
    a = run_oracle(w)
    b = run_c_ref(c_ref, w)
    assert (a - b).abs().max() < 1e-5


# ---------------------------------------------------------------- SDPA on pre-rotated keys
def sdpa_reference(w, dtype=torch.float64):
    """Standard attention: rotate the un-rotated logical keys at their effective
    positions, append the new keys, bottom-right causal mask, GQA by head repeat
    (tests/kernels/test_prefix_prefill.py:242-272), torch's own SDPA."""
    table = w.cos_sin_cache.to(dtype)
    hq, d = w.q.shape[1], w.q.shape[2]
    group = hq // w.k.shape[1]
    out = torch.zeros(w.q.shape, dtype=dtype)
    for b, a in enumerate(w.aux):
        qs, qe = int(w.b_start_loc[b]), int(w.b_start_loc[b + 1])
        kc = orc.rotate_at(a["k_ctx"].to(dtype), a["eff_pos"], table)[a["valid"]]
        vc = a["v_ctx"].to(dtype)[a["valid"]]
        kn = orc.rotate_at(a["k_new_unrot"].to(dtype), a["q_pos"], table)
        keys = torch.cat([kc, kn]); vals = torch.cat([vc, w.v[qs:qe].to(dtype)])
        tq, tk = qe - qs, keys.shape[0]
        mask = torch.ones(tq, tk, dtype=torch.bool).tril(diagonal=tk - tq)
        o = F.scaled_dot_product_attention(
            w.q[qs:qe].to(dtype).permute(1, 0, 2)[None],
            keys.permute(1, 0, 2).repeat_interleave(group, 0)[None],
            vals.permute(1, 0, 2).repeat_interleave(group, 0)[None], attn_mask=mask[None, None])
        out[qs:qe] = o[0].permute(1, 0, 2)
    return out


@pytest.mark.parametrize("variant", ["natural", "offset", "block_uniform"])
def test_deferred_equals_prerotated_sdpa(variant):
    w = wl.make_workload("sdpa", dtype=torch.float32, hq=8, hkv=4, d=16, theta=10000.0,
                         block_size=8, doc_lens=[13, 8, 21, 5], requests=[[1, 3, 0, 2], [2, 2], [0]],
                         q_lens=[11, 5, 1], variant=variant, seed=5, keep_aux=True)
    got = run_oracle(w, compute_dtype=torch.float64)
    ref = sdpa_reference(w)
    tol = 1e-5 if variant == "block_uniform" else 1e-6   # cache holds f32-rounded rotated keys
    assert (got.double() - ref).abs().max() < tol


def test_offset_and_block_uniform_agree_and_differ_from_natural_when_padded():
    a = tiny("offset", seed=9); b = tiny("block_uniform", seed=9); c = tiny("natural", seed=9)
    oa = run_oracle(a, compute_dtype=torch.float64)
    ob = run_oracle(b, compute_dtype=torch.float64)
    oc = run_oracle(c, compute_dtype=torch.float64)
    assert (oa - ob).abs().max() < 1e-5
    assert (oa - oc).abs().max() > 1e-3


# ---------------------------------------------------------------- invariants
def test_relative_position_identity():
    """Shifting every key base and the query by the same amount changes nothing
    (docs/design.md:37-47)."""
    w = tiny("offset", seed=6)
    base = run_oracle(w, compute_dtype=torch.float64)
    shift = 9
    big = orc.build_cos_sin_table(128, 8, 10000.0, dtype=torch.float32)
    w.cos_sin_cache = big
    # un-rotate q (rows of the table are exact inverses under sin -> -sin), re-rotate shifted
    half = 4
    for b, a in enumerate(w.aux):
        qs, qe = int(w.b_start_loc[b]), int(w.b_start_loc[b + 1])
        rows = big[a["q_pos"]].double()
        c, s = rows[:, None, :half], rows[:, None, half:]
        qu = orc.neox_rotate(w.q[qs:qe].double(), c, -s)
        w.q[qs:qe] = orc.rotate_at(qu, a["q_pos"] + shift, big.double()).float()
    w.q_offset = torch.where(w.q_offset != 0, w.q_offset + shift, w.q_offset)
    # new-token keys are rotated at ctx_len+m inside the op, which does not shift:
    # compare only the context contribution by making the new keys invisible except self
    got = run_oracle(w, compute_dtype=torch.float64)
    # rows t=0 see only context keys + themselves; the self key's position did not shift,
    # so restrict to requests' first rows with the self score removed is not possible here.
    # Instead verify on a context-only variant: q_len==1 rows where the single new key is
    # rotated at ctx_len (unshifted) -- its score changes, so drop it by comparing against
    # an oracle run whose new key is zeroed in both cases.
    w0 = tiny("offset", seed=6); w0.k.zero_()
    w.k.zero_()
    assert (run_oracle(w, compute_dtype=torch.float64) -
            run_oracle(w0, compute_dtype=torch.float64)).abs().max() < 1e-5
    assert (got - base).abs().max() > 1e-4      # with real new keys the shift is visible


def test_page_permutation_invariance():
    w = tiny("natural", seed=7)
    base = run_oracle(w, compute_dtype=torch.float64)
    nb = w.k_cache.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm); inv[perm] = torch.arange(nb)
    w.k_cache = w.k_cache[perm]; w.v_cache = w.v_cache[perm]
    w.block_table = inv[w.block_table.long()].to(torch.int32)
    assert torch.equal(run_oracle(w, compute_dtype=torch.float64), base)


def test_pad_slots_are_inert_and_equal_truncation():
    w = tiny("natural", seed=8)
    base = run_oracle(w, compute_dtype=torch.float64)
    # poison every masked slot with NaN: output unchanged
    bs = 4
    for b in range(3):
        q_len = int(w.b_start_loc[b + 1] - w.b_start_loc[b]); ctx = int(w.b_seq_len[b]) - q_len
        for j in range(ctx // bs):
            m = int(w.q_mask[b, j])
            if m:
                pb = int(w.block_table[b, j])
                w.k_cache[pb, :, :, bs - m:, :] = float("nan")
                w.v_cache[pb, :, :, bs - m:] = float("nan")
    assert int(w.q_mask.sum()) > 0
    assert torch.equal(run_oracle(w, compute_dtype=torch.float64), base)
    # dropping the mask instead lets the NaNs through
    w.q_mask.zero_()
    assert run_oracle(w, compute_dtype=torch.float64).isnan().any()


def test_causal_edge_first_row_sees_only_itself():
    w = wl.make_workload("nocontext", dtype=torch.float32, hq=2, hkv=1, d=8, theta=10000.0,
                         block_size=4, doc_lens=[4], requests=[[]], q_lens=[5], variant="natural",
                         seed=2, keep_aux=True)
    o = run_oracle(w, compute_dtype=torch.float64)
    assert torch.allclose(o[0], w.v[0].expand(2, 8), atol=1e-6)   # softmax over one key
    assert not torch.allclose(o[1], w.v[1].expand(2, 8), atol=1e-3)


def test_fp8_dequant_matches_torch_conversion():
    w = wl.make_workload("fp8", dtype=torch.bfloat16, hq=4, hkv=2, d=16, theta=10000.0, block_size=16,
                         doc_lens=[32, 16], requests=[[1, 0]], q_lens=[8], variant="natural",
                         kv_cache_dtype="fp8", seed=3)
    assert w.k_cache.dtype == torch.uint8 and w.k_cache.shape[-1] == 16
    got = run_oracle(w)
    # same op on a bf16 cache holding the dequantised values
    w2 = wl.make_workload("fp8", dtype=torch.bfloat16, hq=4, hkv=2, d=16, theta=10000.0, block_size=16,
                          doc_lens=[32, 16], requests=[[1, 0]], q_lens=[8], variant="natural",
                          kv_cache_dtype="fp8", seed=3)
    kd = (w2.k_cache.view(torch.float8_e4m3fn).float() * w2.k_scale).to(torch.bfloat16)
    vd = (w2.v_cache.view(torch.float8_e4m3fn).float() * w2.v_scale).to(torch.bfloat16)
    # x = 16 layout -> same 5-D indexing works on the dequantised tensor
    ref = orc.prefix_prefill(w2.q, w2.k, w2.v, kd, vd, w2.block_table, w2.b_start_loc, w2.b_seq_len,
                             w2.cos_sin_cache, w2.q_offset, w2.q_mask, pos_mode=w2.pos_mode,
                             rotate_new_k=True)
    assert torch.equal(got, ref)


def test_decode_oracle_equals_prefill_with_token_in_cache():
    """q_len==1 kernel (old_ops/chunked_prefill_paged_decode.py:68-280): the new token's K
    sits in the cache; same result as the prefill op given that K as the new key."""
    w = wl.make_workload("dec", dtype=torch.float32, hq=4, hkv=2, d=8, theta=10000.0, block_size=4,
                         doc_lens=[8, 6], requests=[[1, 0], [0]], q_lens=[1, 1], variant="natural", seed=12)
    pre = run_oracle(w, compute_dtype=torch.float64)
    # write the new token into its page (slot ctx % bs of page ctx // bs)
    for b in range(2):
        ctx = int(w.b_seq_len[b]) - 1
        pb = int(w.block_table[b, ctx // 4]); o_ = ctx % 4
        w.k_cache[pb, :, :, o_, :] = w.k[b].view(2, 2, 4)
        w.v_cache[pb, :, :, o_] = w.v[b]
    dec = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                           w.cos_sin_cache, w.q_mask, compute_dtype=torch.float64)
    assert (dec - pre).abs().max() < 1e-6


def test_lazy_decode_rotating_keys_equals_derotating_query():
    """ops/models/llama_v1.py:231-262 rotates Q backwards by q_offset-1 per page; the oracle
    rotates the page's keys forwards.  Both give the same scores: check on one request by
    brute force over pages."""
    w = wl.make_workload("ldec", dtype=torch.float32, hq=4, hkv=2, d=8, theta=10000.0, block_size=4,
                         doc_lens=[7, 8], requests=[[1, 0]], q_lens=[1], variant="block_uniform", seed=13)
    ctx = int(w.b_seq_len[0]) - 1
    pb = int(w.block_table[0, ctx // 4])
    w.k_cache[pb, :, :, ctx % 4, :] = w.k[0].view(2, 2, 4)
    w.v_cache[pb, :, :, ctx % 4] = w.v[0]
    got = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                           w.cos_sin_cache, w.q_mask, q_offset=w.q_offset, pos_mode=orc.POS_BLOCK_UNIFORM,
                           compute_dtype=torch.float64)
    tab = w.cos_sin_cache.double()
    seq = ctx + 1
    scores = torch.full((4, seq), float("-inf"), dtype=torch.float64)
    vals = torch.zeros(seq, 2, 8, dtype=torch.float64)
    for n in range(seq):
        j, o_ = divmod(n, 4)
        if o_ >= 4 - int(w.q_mask[0, j]):
            continue
        blk = int(w.block_table[0, j])
        kvec = w.k_cache[blk, :, :, o_, :].reshape(2, 8).double()
        vals[n] = w.v_cache[blk, :, :, o_].double()
        qo = int(w.q_offset[0, j])
        rows = tab[qo - 1] if qo > 1 else tab[0]
        c, s_ = rows[:4], rows[4:]
        qrot = orc.neox_rotate(w.q[0].double(), c, -s_)           # rotate Q backwards
        for h in range(4):
            scores[h, n] = (qrot[h] * kvec[h // 2]).sum() / math.sqrt(8)
    p = torch.softmax(scores, dim=-1)
    ref = torch.stack([(p[h][:, None] * vals[:, h // 2]).sum(0) for h in range(4)])
    assert (got[0].double() - ref).abs().max() < 1e-6


def _token_into_cache(w, bs):
    """Write every request's (single) new token where the attention backend leaves it (backends/triton_attn.py:100-109)."""
    hkv, x = w.k_cache.shape[1], w.k_cache.shape[4]
    for b in range(w.b_seq_len.numel()):
        ctx = int(w.b_seq_len[b]) - 1
        pb = int(w.block_table[b, ctx // bs]); o_ = ctx % bs
        w.k_cache[pb, :, :, o_, :] = w.k[int(w.b_start_loc[b])].view(hkv, -1, x)
        w.v_cache[pb, :, :, o_] = w.v[int(w.b_start_loc[b])]


@pytest.mark.parametrize("window", [3, 6, 50])
def test_decode_oracle_sliding_window_equals_prefill_oracle(window):
    """paged_decode(sliding_window=w): the same rows through the prefill oracle, whose window branch is pinned by
    the brute force above (old_ops/chunked_prefill_paged_decode.py:237-241 vs old_ops/prefix_prefill.py:270-284)."""
    w = wl.make_workload("decw", dtype=torch.float32, hq=4, hkv=2, d=8, theta=10000.0, block_size=4,
                         doc_lens=[8, 6, 5], requests=[[1, 0, 2], [0]], q_lens=[1, 1], variant="natural", seed=14)
    pre = run_oracle(w, compute_dtype=torch.float64, sliding_window=window)
    _token_into_cache(w, 4)
    dec = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                           w.cos_sin_cache, w.q_mask, compute_dtype=torch.float64, sliding_window=window)
    assert (dec - pre).abs().max() < 1e-6
    if window < 8:
        unwindowed = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                                      w.cos_sin_cache, w.q_mask, compute_dtype=torch.float64)
        assert (dec - unwindowed).abs().max() > 1e-3                # the window does cut something


def test_decode_oracle_unrotated_requests_equal_prefill_oracle():
    """paged_decode(is_lazy[b] == 0) under the block-uniform mode (ops/models/llama_v1.py:290-434): no rotation, no
    pad mask -- the same rows through the prefill oracle's un-rotated branch, which the brute force pins."""
    w = wl.make_workload("decv", dtype=torch.float32, hq=4, hkv=2, d=8, theta=10000.0, block_size=4,
                         doc_lens=[7, 6, 5], requests=[[1, 0, 2], [0], [2, 1]], q_lens=[1, 1, 1],
                         variant="block_uniform", seed=15)
    lazy = torch.tensor([False, True, False])
    pre = run_oracle(w, compute_dtype=torch.float64, is_lazy=lazy)
    _token_into_cache(w, 4)
    dec = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len, w.cos_sin_cache,
                           w.q_mask, q_offset=w.q_offset, is_lazy=lazy, pos_mode=orc.POS_BLOCK_UNIFORM,
                           compute_dtype=torch.float64)
    assert (dec - pre).abs().max() < 1e-6
    all_lazy = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len, w.cos_sin_cache,
                                w.q_mask, q_offset=w.q_offset, pos_mode=orc.POS_BLOCK_UNIFORM, compute_dtype=torch.float64)
    assert (dec[0] - all_lazy[0]).abs().max() > 1e-3 and (dec[1] - all_lazy[1]).abs().max() < 1e-12


def test_lazy_decode_zero_offset_keeps_the_previous_rotation():
    """The page walk of ops/models/llama_v1.py:149-262 restated literally -- Q de-rotated when the page's offset
    differs from the previous page's, 1 = the query as given, 0 = leave Q as it is -- on a table with zeros after
    offsets above 1 (which the scheduler never emits, but the kernel defines)."""
    w = wl.make_workload("carry", dtype=torch.float32, hq=4, hkv=2, d=8, theta=10000.0, block_size=4,
                         doc_lens=[8, 8, 4], requests=[[1, 0, 2]], q_lens=[1], variant="block_uniform", seed=16)
    _token_into_cache(w, 4)
    seq = int(w.b_seq_len[0])
    npages = (seq + 3) // 4
    qo = w.q_offset.clone()
    assert qo[0, :npages].tolist()[:5] == [1, 1, 9, 9, 17]
    qo[0, 1] = 0          # after a 1: identity either way
    qo[0, 3] = 0          # after a 9: keeps the rotation by 8
    qo[0, 5] = 0          # the query page (was 1): keeps the rotation by 16 of page 4
    got = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len, w.cos_sin_cache,
                           w.q_mask, q_offset=qo, pos_mode=orc.POS_BLOCK_UNIFORM, compute_dtype=torch.float64)
    tab = w.cos_sin_cache.double()
    q_full = w.q[0].double()
    q_rot = q_full
    prev = -1
    scores = torch.full((4, seq), float("-inf"), dtype=torch.float64)
    vals = torch.zeros(seq, 2, 8, dtype=torch.float64)
    for j in range(npages):
        val = int(qo[0, j])
        if val != prev:
            if val == 1:
                q_rot = q_full
            elif val != 0:
                rows = tab[val - 1]
                q_rot = orc.neox_rotate(q_full, rows[:4], -rows[4:])
            prev = val
        blk = int(w.block_table[0, j])
        for o_ in range(4):
            n = j * 4 + o_
            if n >= seq or o_ >= 4 - int(w.q_mask[0, j]):
                continue
            kvec = w.k_cache[blk, :, :, o_, :].reshape(2, 8).double()
            vals[n] = w.v_cache[blk, :, :, o_].double()
            for h in range(4):
                scores[h, n] = (q_rot[h] * kvec[h // 2]).sum() / math.sqrt(8)
    p = torch.softmax(scores, dim=-1)
    ref = torch.stack([(p[h][:, None] * vals[:, h // 2]).sum(0) for h in range(4)])
    assert (got[0].double() - ref).abs().max() < 1e-6
    # and the carry matters: reading 0 as "no rotation" gives something else
    naive = orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len, w.cos_sin_cache,
                             w.q_mask, q_offset=torch.where(qo == 0, torch.ones_like(qo), qo),
                             pos_mode=orc.POS_BLOCK_UNIFORM, compute_dtype=torch.float64)
    assert (got - naive).abs().max() > 1e-3


def test_paged_cache_write_is_inverse_of_gather_and_matches_layout_formula():
    """K[block, h, d // x, off, d % x], V[block, h, d, off] (the third-party reshape_and_cache layout the
    reference's kernels index at old_ops/prefix_prefill.py:172-181,196-199): element-wise formula on a
    small case, and the round trip through gather_pages."""
    g = torch.Generator().manual_seed(1)
    t, hkv, d, bs, x, nb = 20, 2, 16, 4, 8, 7
    k = torch.randn(t, hkv, d, generator=g); v = torch.randn(t, hkv, d, generator=g)
    kc = torch.zeros(nb, hkv, d // x, bs, x); vc = torch.zeros(nb, hkv, d, bs)
    slots = torch.randperm(nb * bs, generator=g)[:t]
    slots[5] = -1
    orc.paged_cache_write(k, v, kc, vc, slots)
    for tok in range(t):
        s_ = int(slots[tok])
        if s_ < 0:
            continue
        for h in range(hkv):
            for dd in range(d):
                assert kc[s_ // bs, h, dd // x, s_ % bs, dd % x] == k[tok, h, dd]
                assert vc[s_ // bs, h, dd, s_ % bs] == v[tok, h, dd]
    assert kc.count_nonzero() == (t - 1) * hkv * d                 # the skipped token wrote nothing
    slots = torch.arange(bs, bs + t)
    kc.zero_(); vc.zero_()
    orc.paged_cache_write(k, v, kc, vc, slots)
    kb, vb = orc.gather_pages(kc, vc, torch.arange(1, 1 + t // bs))
    assert torch.equal(kb, k) and torch.equal(vb, v)


@pytest.mark.parametrize("kv,top,step_at_1", [("fp8", 448.0, 0.125), ("fp8_e5m2", 57344.0, 0.25)])
def test_paged_cache_write_fp8_codes(kv, top, step_at_1):
    """value / scale saturated to the format's largest finite number, nearest-even: exact values, a tie, the
    saturation and the byte codes of 1.0 (0x38 in e4m3, 0x3C in e5m2) fixed by the formats themselves."""
    f8 = torch.float8_e4m3fn if kv == "fp8" else torch.float8_e5m2
    vals = torch.tensor([1.0, -2.0, 1.0 + step_at_1 / 2, 1e9, -1e9, 0.0, 3.0, 0.5])
    k = (vals * 0.5).view(8, 1, 1).expand(8, 1, 16).contiguous()       # scale 0.5: stored value = vals
    kc = torch.zeros(1, 1, 1, 8, 16, dtype=torch.uint8); vc = torch.zeros(1, 1, 16, 8, dtype=torch.uint8)
    orc.paged_cache_write(k, k, kc, vc, torch.arange(8), kv, 0.5, 0.5)
    got = kc.view(f8).float()[0, 0, 0, :, 0]
    assert got.tolist() == [1.0, -2.0, 1.0, top, -top, 0.0, 3.0, 0.5]     # the tie goes to the even code
    assert int(kc[0, 0, 0, 0, 0]) == (0x38 if kv == "fp8" else 0x3C)
    assert torch.equal(vc.view(f8).float()[0, 0, 0, :], got)


def test_rotary_new_tokens_q_only_leaves_key_and_preserves_norm():
    g = torch.Generator().manual_seed(2)
    table = orc.build_cos_sin_table(512, 32, 10000.0)
    q = torch.randn(9, 4, 32, generator=g, dtype=torch.float64); k = torch.randn(9, 2, 32, generator=g, dtype=torch.float64)
    pos = torch.randint(0, 512, (9,), generator=g)
    q1, k1 = orc.rotary_new_tokens(pos, q, k, table, q_only=True, compute_dtype=torch.float64)
    assert k1 is k
    assert torch.allclose(q1.norm(dim=-1), q.norm(dim=-1), atol=1e-12)
    q2, k2 = orc.rotary_new_tokens(pos, q, k, table, q_only=False, compute_dtype=torch.float64)
    # relative-position property: <R(p)q, R(p)k> = <q, k>
    assert torch.allclose((q2[:, :2] * k2).sum(-1), (q[:, :2] * k).sum(-1), atol=1e-10)


def test_reposition_blocks_equals_rotation_of_the_unrotated_keys():
    """With an exact (float64) table, un-rotating from `from` and rotating to `to` must give the keys
    one gets by rotating the never-rotated keys at `to` directly -- and must leave norms alone."""
    g = torch.Generator().manual_seed(4)
    hkv, d, bs, x, nb = 2, 32, 8, 8, 5
    table = orc.build_cos_sin_table(256, d, 10000.0, dtype=torch.float64, math_dtype=torch.float64)
    raw = torch.randn(bs, hkv, d, generator=g, dtype=torch.float64)                     # un-rotated keys of one block
    stored = orc.rotate_at(raw, 40 + torch.arange(bs), table)                            # as cached: local positions 40..
    kc = torch.zeros(nb, hkv, d // x, bs, x, dtype=torch.float64); vc = torch.randn(nb, hkv, d, bs, generator=g, dtype=torch.float64)
    kc[1] = stored.reshape(bs, hkv, d // x, x).permute(1, 2, 0, 3)
    v_old = vc[1].clone()
    orc.reposition_blocks(kc, vc, [(3, 1, 40, 113)], table, compute_dtype=torch.float64)
    got = kc[3].permute(2, 0, 1, 3).reshape(bs, hkv, d)
    want = orc.rotate_at(raw, 113 + torch.arange(bs), table)
    assert torch.allclose(got, want, atol=1e-9)
    assert torch.allclose(got.norm(dim=-1), raw.norm(dim=-1), atol=1e-9)
    assert torch.equal(vc[3], v_old) and torch.equal(kc[1].permute(2, 0, 1, 3).reshape(bs, hkv, d), stored)


def test_reference_known_answers_from_the_golden_file():
    """tests/golden/reference_known_answers.json holds what the reference's own unit tests assert about the metadata
    path (inputs and expected outputs, with the lines they come from): the host function and the oracle's
    restatement must both reproduce them."""
    import json
    import os
    from lazy_amd.core.sched import metadata as host
    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")) as f:
        kat = json.load(f)
    expand = lambda v: [v["repeat"]] * v["times"] if isinstance(v, dict) else v
    for case in kat["metadata_for_lazy_attention"]:
        want = (case["q_offset"], case["q_mask"])
        args = (case["document_lens"], case["document_lens_padded"], case["block_size"])
        assert host.metadata_for_lazy_attention(*args) == want, case["cite"]
        assert tuple(list(map(int, x)) for x in orc.metadata_for_lazy_attention(*args)) == want, case["cite"]
    for case in kat["metadata_for_mepic"]:
        args = (case["document_lens"], case["document_lens_padded"], case["block_size"])
        assert host.metadata_for_mepic(*args) == (case["q_offset"], case["q_mask"]), case["cite"]
    for case in kat["max_rotation_offset"]:
        assert host.max_rotation_offset(expand(case["document_lens"]), expand(case["document_lens_padded"])) == case["expected"], case["cite"]
    for case in kat["packed_block_table"]:
        packed = (case["block"] << 32) | (case["q_offset"] << 16) | case["q_mask"]
        assert (packed >> 32) & 0xFFFFFFFF == case["unpacked_block"] and (packed >> 16) & 0xFFFF == case["unpacked_q_offset"]
