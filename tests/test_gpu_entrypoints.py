"""GPU parity of the entry points the attention backend calls
(``chunked_prefill_paged_decode`` of both variants): a mixed batch of prefill requests
and q_len==1 requests, checked against the CPU oracle."""
import pytest
import torch

from oracle import deferred_rope as orc
from lazy_amd import workloads as wl
from lazy_amd.attention.old_ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode as entry_unrotated
from lazy_amd.attention.ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode as entry_block_uniform

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _mixed(variant, dtype, d, seed=41):
    w = wl.make_workload("mixed", dtype=dtype, hq=8, hkv=2, d=d, theta=500000.0, block_size=16,
                         doc_lens=[40, 16, 33, 70, 5], requests=[[3, 1, 0], [2], [0, 2, 3, 1], [4, 0]],
                         q_lens=[70, 1, 9, 1], variant=variant, seed=seed)
    # the attention backend writes the new tokens into the paged cache before the call
    # (backends/triton_attn.py:100-109); the q_len==1 kernels read them from there
    x = w.k_cache.shape[4]
    for b in range(4):
        qs, qe = int(w.b_start_loc[b]), int(w.b_start_loc[b + 1])
        ctx = int(w.b_seq_len[b]) - (qe - qs)
        for t in range(qe - qs):
            n = ctx + t
            pb = int(w.block_table[b, n // 16]); o_ = n % 16
            w.k_cache[pb, :, :, o_, :] = w.k[qs + t].view(2, d // x, x)
            w.v_cache[pb, :, :, o_] = w.v[qs + t]
    return w


def _expected(w, lazy=None):
    ref = torch.full_like(w.q, 5.0)
    orc.prefix_prefill(w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                       w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode,
                       rotate_new_k=w.rotate_new_k, is_lazy=lazy, skip_decode=True, out=ref)
    orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                     w.cos_sin_cache, w.q_mask, q_offset=w.q_offset, is_lazy=lazy,
                     pos_mode=orc.POS_NATURAL if w.pos_mode != orc.POS_BLOCK_UNIFORM else w.pos_mode, out=ref)
    return ref


@pytest.mark.parametrize("dtype,d,tol", [(torch.float32, 64, 1e-5), (torch.bfloat16, 128, 2e-2)])
def test_entry_unrotated_cache_mixed_batch(dtype, d, tol):
    print(f"case: entry old_ops {dtype}", flush=True)
    w = _mixed("natural", dtype, d)
    ref = _expected(w)
    g = w.to(DEV)
    out = torch.full_like(g.q, 5.0)
    entry_unrotated(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                    g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=d ** -0.5, rotary_dim=d,
                    cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err < tol, err


@pytest.mark.parametrize("dtype,d,tol", [(torch.float32, 64, 1e-5), (torch.bfloat16, 128, 2e-2)])
def test_entry_block_uniform_mixed_batch_with_packed_table(dtype, d, tol):
    print(f"case: entry ops {dtype}", flush=True)
    w = _mixed("block_uniform", dtype, d)
    lazy = torch.tensor([True, True, False, False])
    ref = _expected(w, lazy)
    g = w.to(DEV)
    out = torch.full_like(g.q, 5.0)
    packed = (g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()
    entry_block_uniform(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc,
                        g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=d ** -0.5,
                        rotary_dim=d, cos_sin_cache=g.cos_sin_cache, is_lazy=lazy.to(DEV), q_offset=None,
                        q_mask=None, packed_block_table=packed)
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err < tol, err


@pytest.mark.parametrize("block_size", [32, 16])
@pytest.mark.parametrize("head_size", [128, 96, 24])
@pytest.mark.parametrize("queries_per_kv", [1, 8, 64])
def test_reference_kernel_test_grid(head_size, queries_per_kv, block_size):
    """The grid of the reference's own kernel test (tests/kernels/test_prefix_prefill.py:37-48, 85-93, with
    vLLM's NUM_HEADS = 64, NUM_QUERIES_PER_KV = 1 / 8 / 64, HEAD_SIZES = 128 / 96 / 24, float16, pages of 32
    tokens, ten requests the last of which has one new token), lengths cut so that the CPU oracle takes
    well under a second, through both entry points of the un-rotated-cache variant; pages of 16 added."""
    import random
    from lazy_amd.attention.old_ops.prefix_prefill import context_attention_fwd
    print(f"case: reference grid head {head_size} group {queries_per_kv} page {block_size}", flush=True)
    r = random.Random(0)
    q_lens = [r.randint(16, 128) for _ in range(10)]
    q_lens[-1] = 1
    docs = [r.randint(16, 256) for _ in range(10)]
    d, hkv = head_size, 64 // queries_per_kv
    w = wl.make_workload("refgrid", dtype=torch.float16, hq=64, hkv=hkv, d=d, theta=10000.0, block_size=block_size,
                         doc_lens=docs, requests=[[i] for i in range(10)], q_lens=q_lens, variant="natural", seed=0)
    # the decode request's token is in the cache when the backend calls (backends/triton_attn.py:100-109)
    x = w.k_cache.shape[4]
    qs = int(w.b_start_loc[9]); n = int(w.b_seq_len[9]) - 1
    pb = int(w.block_table[9, n // block_size]); o_ = n % block_size
    w.k_cache[pb, :, :, o_, :] = w.k[qs].view(hkv, d // x, x)
    w.v_cache[pb, :, :, o_] = w.v[qs]
    prefill_only = torch.full_like(w.q, 5.0)
    orc.prefix_prefill(w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                       w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode, rotate_new_k=w.rotate_new_k,
                       out=prefill_only)
    both = _expected(w)
    g = w.to(DEV)
    out = torch.full_like(g.q, 5.0)
    context_attention_fwd(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                          g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, rotary_dim=d,
                          cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
    err = (out.cpu().float() - prefill_only.float()).abs().max().item()
    assert err < 5e-3, err
    # the scale is passed, as the backend does: this entry point's default is 1/sqrt(number of heads), like the
    # reference's (old_ops/chunked_prefill_paged_decode.py:311-312)
    out = torch.full_like(g.q, 5.0)
    entry_unrotated(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                    g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=d ** -0.5, rotary_dim=d,
                    cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
    err = (out.cpu().float() - both.float()).abs().max().item()
    assert err < 5e-3, err


def test_tables_made_under_inference_mode():
    """In serving the cos/sin table is an inference tensor (the model runner works under
    torch.inference_mode() and converts the table there, rotary_embedding.py:79-82): such a tensor has no
    edit counter.  Both entry points of the un-rotated-cache variant, which re-lay the table out once and
    cache the copy, take it -- inside and outside inference mode, repeatedly."""
    from lazy_amd.attention.old_ops.prefix_prefill import context_attention_fwd
    print("case: inference-mode table", flush=True)
    w = _mixed("offset", torch.bfloat16, 128, seed=43)
    ref = _expected(w)
    prefill_only = torch.full_like(w.q, 5.0)
    orc.prefix_prefill(w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                       w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode, rotate_new_k=w.rotate_new_k,
                       out=prefill_only)
    g = w.to(DEV)
    with torch.inference_mode():
        table = g.cos_sin_cache.float().to(torch.bfloat16)
        assert table.is_inference()
        for _ in range(2):
            out = torch.full_like(g.q, 5.0)
            context_attention_fwd(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc,
                                  g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, rotary_dim=128,
                                  cos_sin_cache=table, q_mask=g.q_mask, q_offset=g.q_offset, is_mepic=False)
            err = (out.cpu().float() - prefill_only.float()).abs().max().item()
            assert err < 2e-2, err
    out = torch.full_like(g.q, 5.0)
    entry_unrotated(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                    g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=128 ** -0.5, rotary_dim=128,
                    cos_sin_cache=table, q_mask=g.q_mask, q_offset=g.q_offset, is_mepic=False)
    # (the q_len==1 rows of this variant are rotated at their natural positions, old_ops/chunked...:204-213)
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err < 2e-2, err


def _call(entry, variant, g, out, packed=None, lazy=None, block_table=None):
    bt = g.block_table if block_table is None else block_table
    if variant == "natural":
        entry(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, bt, g.b_start_loc, g.b_seq_len,
              g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=128 ** -0.5, rotary_dim=128,
              cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
    else:
        entry(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, bt, g.b_start_loc, g.b_seq_len, g.max_seq_len,
              g.max_query_len, g.k_scale, g.v_scale, sm_scale=128 ** -0.5, rotary_dim=128,
              cos_sin_cache=g.cos_sin_cache, is_lazy=lazy, q_offset=g.q_offset, q_mask=g.q_mask,
              packed_block_table=packed)         # all three tables, as backends/triton_attn.py:137-185 passes them


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
def test_repeat_calls_on_the_same_buffers_follow_their_contents(variant):
    """A serving loop calls with the same buffers at the same addresses and new contents.  The entry points
    remember the validated call (addresses, shapes, strides, scalars) and skip straight to the launch: the
    second result must be that of the NEW contents, and the call must have been served from memory."""
    from lazy_amd.attention import _launch
    print(f"case: repeat calls {variant}", flush=True)
    entry = entry_unrotated if variant == "natural" else entry_block_uniform
    lazy_host = torch.tensor([True, True, False, False]) if variant == "block_uniform" else None
    first, second = _mixed(variant, torch.bfloat16, 128, seed=51), _mixed(variant, torch.bfloat16, 128, seed=52)
    g = first.to(DEV)
    lazy = lazy_host.to(DEV) if lazy_host is not None else None
    pack = lambda w: (w.block_table.long() << 32) | (w.q_offset.long() << 16) | w.q_mask.long()
    packed = pack(g) if variant == "block_uniform" else None
    out = torch.full_like(g.q, 5.0)
    _launch.forget_calls()
    _call(entry, variant, g, out, packed, lazy)
    assert (out.cpu().float() - _expected(first, lazy_host).float()).abs().max().item() < 2e-2
    assert len(_launch._calls) == 1
    for name in ("q", "k", "v", "k_cache", "v_cache", "block_table", "q_mask", "q_offset"):
        if getattr(g, name) is not None:
            getattr(g, name).copy_(getattr(second, name))
    if packed is not None:
        packed.copy_(pack(second))
    out.fill_(5.0)
    _call(entry, variant, g, out, packed, lazy)
    assert len(_launch._calls) == 1
    assert (out.cpu().float() - _expected(second, lazy_host).float()).abs().max().item() < 2e-2
    # an edit of the cos/sin table is seen (the kernels read a re-laid-out copy of it)
    other = wl.cos_sin_table(second.cos_sin_cache.shape[0], 128, 10000.0, torch.bfloat16)
    g.cos_sin_cache.copy_(other)
    second.cos_sin_cache.copy_(other)
    out.fill_(5.0)
    _call(entry, variant, g, out, packed, lazy)
    assert (out.cpu().float() - _expected(second, lazy_host).float()).abs().max().item() < 2e-2
    # a table that must be converted (int64 here) is converted on every call, so its new contents are seen too
    wide = g.block_table.long()
    out.fill_(5.0)
    _call(entry, variant, g, out, packed, lazy, block_table=wide)
    assert (out.cpu().float() - _expected(second, lazy_host).float()).abs().max().item() < 2e-2
    if variant == "natural":
        wide.copy_(first.block_table)
        for name in ("q", "k", "v", "k_cache", "v_cache", "q_mask"):
            getattr(g, name).copy_(getattr(first, name))
        first.cos_sin_cache.copy_(other)
        out.fill_(5.0)
        _call(entry, variant, g, out, packed, lazy, block_table=wide)
        assert (out.cpu().float() - _expected(first, lazy_host).float()).abs().max().item() < 2e-2


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
def test_single_request_with_many_new_tokens_needs_no_single_token_launch(variant):
    """One request with more than one new token: the q_len==1 launches have no row to work on and are left out
    (the reference's second kernel finds nothing to do there: old_ops/chunked_prefill_paged_decode.py:396-442);
    the output is the prefill kernel's."""
    from lazy_amd.attention import _launch
    print(f"case: single request {variant}", flush=True)
    d = 128
    w = wl.make_workload("single", dtype=torch.bfloat16, hq=8, hkv=2, d=d, theta=500000.0, block_size=16,
                         doc_lens=[40, 16, 33], requests=[[2, 0, 1]], q_lens=[21], variant=variant, seed=5)
    lazy = torch.tensor([True]) if variant == "block_uniform" else None
    ref = torch.full_like(w.q, 5.0)
    orc.prefix_prefill(w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                       w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode,
                       rotate_new_k=w.rotate_new_k, is_lazy=lazy, skip_decode=True, out=ref)
    g = w.to(DEV)
    out = torch.full_like(g.q, 5.0)
    _launch.forget_calls()
    if variant == "natural":
        entry_unrotated(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                        g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=d ** -0.5, rotary_dim=d,
                        cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
    else:
        entry_block_uniform(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc,
                            g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=d ** -0.5,
                            rotary_dim=d, cos_sin_cache=g.cos_sin_cache, is_lazy=lazy.to(DEV), q_offset=g.q_offset,
                            q_mask=g.q_mask)
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err < 2e-2, err
    (entry,) = _launch._calls.values()
    assert len(entry[1]) == 1 and not entry[1][0].decode


def _sub_batch_call(entry, variant, g, w, b, out, packed, lazy, clone=False):
    """The first ``b`` requests of the batch as views of its buffers (or as fresh copies of those views)."""
    ntok = int(w.b_start_loc[b])
    f = (lambda t: None if t is None else t.clone()) if clone else (lambda t: t)
    q_lens = (w.b_start_loc[1:b + 1] - w.b_start_loc[:b])
    args = (f(g.q[:ntok]), f(g.k[:ntok]), f(g.v[:ntok]), out[:ntok], "auto", g.k_cache, g.v_cache, f(g.block_table[:b]),
            f(g.b_start_loc[:b + 1]), f(g.b_seq_len[:b]), int(w.b_seq_len[:b].max()), int(q_lens.max()),
            g.k_scale, g.v_scale)
    kw = dict(sm_scale=128 ** -0.5, rotary_dim=128, cos_sin_cache=g.cos_sin_cache, q_mask=f(g.q_mask[:b]))
    if variant == "natural":
        entry(*args, **kw)
    else:
        entry(*args, is_lazy=None if lazy is None else f(lazy[:b]), q_offset=f(g.q_offset[:b]),
              packed_block_table=None if packed is None else f(packed[:b]), **kw)


@pytest.mark.parametrize("variant,lazy_given", [("natural", False), ("block_uniform", True), ("block_uniform", False)])
def test_views_of_persistent_buffers_reuse_the_call_made_for_other_counts(variant, lazy_given):
    """An engine step passes views ``buf[:n]`` of persistent buffers, with a new ``n``, ``max_seq_len`` and
    ``max_query_len`` every step (backends/triton_attn.py:146-187).  Those counts are not part of the remembered
    call's key: the call made for one step serves the next, with its counts set anew.  Results must equal those of
    calls validated from scratch (fresh copies of the same views, which share no address with the buffers), and
    rows past the step's tokens must stay untouched.  Without ``is_lazy`` the entry point owns an all-false one sized
    by the batch: such a call is tied to its batch size."""
    from lazy_amd.attention import _launch
    print(f"case: views of persistent buffers {variant} lazy_given={lazy_given}", flush=True)
    entry = entry_unrotated if variant == "natural" else entry_block_uniform
    w = _mixed(variant, torch.bfloat16, 128, seed=61)
    g = w.to(DEV)
    lazy = torch.tensor([True, True, False, True]).to(DEV) if lazy_given else None
    packed = ((g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()) if variant == "block_uniform" else None
    steps = (2, 3, 4, 2, 1, 4)
    want = {}
    for b in set(steps):
        o = torch.full_like(g.q, 5.0)
        _sub_batch_call(entry, variant, g, w, b, o, packed, lazy, clone=True)
        want[b] = o
    _launch.forget_calls()
    out = torch.full_like(g.q, 5.0)
    for b in steps:
        out.fill_(5.0)
        _sub_batch_call(entry, variant, g, w, b, out, packed, lazy)
        assert torch.equal(out, want[b]), b
        assert bool((out[int(w.b_start_loc[b]):] == 5.0).all())
    # one remembered call for the steps with several requests (made again at every change of the batch size when it
    # owns batch-sized tensors), one for the single request (no q_len == 1 launch there)
    assert len(_launch._calls) == 2


def _block_uniform_call(g, out, lazy, packed=None, **kw):
    entry_block_uniform(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc,
                        g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale,
                        sm_scale=g.q.shape[-1] ** -0.5, rotary_dim=g.q.shape[-1], cos_sin_cache=g.cos_sin_cache,
                        is_lazy=lazy, q_offset=None if packed is not None else g.q_offset,
                        q_mask=None if packed is not None else g.q_mask, packed_block_table=packed, **kw)


@pytest.mark.parametrize("use_packed", [True, False])
def test_ignore_q_mask_switch_drops_the_pad_counts_of_the_single_token_rows(monkeypatch, use_packed):
    """LAZY_DECODE_IGNORE_Q_MASK (ops/chunked_prefill_paged_decode.py:146,218; ops/models/llama_v1.py:161-162):
    the q_len == 1 rows see every slot of every page, the prefill rows keep their masks."""
    print(f"case: LAZY_DECODE_IGNORE_Q_MASK packed={use_packed}", flush=True)
    w = _mixed("block_uniform", torch.bfloat16, 128)
    lazy = torch.tensor([True, True, True, True])
    ref = torch.full_like(w.q, 5.0)
    orc.prefix_prefill(w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                       w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode, rotate_new_k=w.rotate_new_k,
                       is_lazy=lazy, skip_decode=True, out=ref)
    masked = ref.clone()
    orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len, w.cos_sin_cache,
                     None, q_offset=w.q_offset, is_lazy=lazy, pos_mode=w.pos_mode, out=ref)
    orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len, w.cos_sin_cache,
                     w.q_mask, q_offset=w.q_offset, is_lazy=lazy, pos_mode=w.pos_mode, out=masked)
    assert (ref.float() - masked.float()).abs().max().item() > 5e-2      # the switch changes these rows
    g = w.to(DEV)
    packed = ((g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()) if use_packed else None
    for value, want in (("1", ref), ("off", masked)):
        monkeypatch.setenv("LAZY_DECODE_IGNORE_Q_MASK", value)
        out = torch.full_like(g.q, 5.0)
        _block_uniform_call(g, out, lazy.to(DEV), packed)
        err = (out.cpu().float() - want.float()).abs().max().item()
        assert err < 2e-2, (value, err)


def test_computed_cos_sin_takes_its_frequencies_from_rope_meta_not_from_the_layers_bf16_buffer(monkeypatch):
    """LAZY_DECODE_COMPUTE_COS_SIN: the reference passes the layer's bfloat16 ``inv_freq`` as ``freqs`` and its kernel
    never reads it (ops/models/llama_v1.py:127-133 derives the frequencies from ``rope_meta``)."""
    print("case: LAZY_DECODE_COMPUTE_COS_SIN with a bf16 freqs buffer", flush=True)
    w = _mixed("block_uniform", torch.bfloat16, 128)
    lazy = torch.tensor([True, True, False, True])
    ref = _expected(w, lazy)
    g = w.to(DEV)
    inv = (500000.0 ** (-torch.arange(0, 128, 2, dtype=torch.float32) / 128)).to(torch.bfloat16).to(DEV)
    meta = dict(ROPE_TYPE=0, BASE=500000.0, SCALING_FACTOR=1.0, LOW_FACTOR=1.0, HIGH_FACTOR=1.0,
                ORIG_MAX_POSITION=8192, PI_VALUE=3.141592653589793)
    monkeypatch.setenv("LAZY_DECODE_COMPUTE_COS_SIN", "1")
    packed = (g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()
    for _ in range(2):                                   # the second call is the remembered one
        out = torch.full_like(g.q, 5.0)
        _block_uniform_call(g, out, lazy.to(DEV), packed, freqs=inv, rope_meta=meta)
        err = (out.cpu().float() - ref.float()).abs().max().item()
        assert err < 2e-2, err
    # another rope_meta is another call
    out2 = torch.full_like(g.q, 5.0)
    _block_uniform_call(g, out2, lazy.to(DEV), packed, freqs=inv, rope_meta=dict(meta, BASE=10000.0))
    assert (out2.float() - out.float()).abs().max().item() > 1e-2


def test_packed_table_with_operands_the_streaming_kernel_does_not_take():
    """A query view that is not 16-byte aligned: only the library's own predicate sees that, and the call must then
    run the generic kernel on un-packed tables instead of failing."""
    print("case: packed table + misaligned query view", flush=True)
    w = _mixed("block_uniform", torch.bfloat16, 128)
    lazy = torch.tensor([True, False, True, True])
    ref = _expected(w, lazy)
    g = w.to(DEV)
    buf = torch.zeros(g.q.shape[0], g.q.shape[1], 128 + 4, dtype=g.q.dtype, device=DEV)
    buf[:, :, 4:] = g.q
    import dataclasses
    gv = dataclasses.replace(g, q=buf[:, :, 4:])
    assert gv.q.data_ptr() % 16 == 8
    packed = (g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()
    out = torch.full_like(g.q, 5.0)
    with pytest.warns(RuntimeWarning, match="fp32 fallback kernel"):
        _block_uniform_call(gv, out, lazy.to(DEV), packed)
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err < 2e-2, err
