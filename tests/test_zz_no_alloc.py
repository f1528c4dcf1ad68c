"""The prefill entry point that allocates nothing (``lazyattn_prefix_prefill_static_scratch``): split-KV partials in
the library's static per-GPU buffer instead of a caller's workspace.  Same kernels as ``lazyattn_prefix_prefill``,
so the outputs must be the same bits -- on two calls in a row, the second with a smaller input (the buffer still
holds the first call's partials then)."""
import ctypes

import pytest
import torch

from lazy_amd import _ffi, workloads as wl
from lazy_amd.attention.old_ops.prefix_prefill import context_attention_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _plan(g, o, num_splits):
    return context_attention_fwd(
        g.q, g.k, g.v, o, g.kv_cache_dtype, g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
        g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, cos_sin_cache=g.cos_sin_cache, rotary_dim=g.q.shape[-1],
        q_mask=g.q_mask, q_offset=g.q_offset, is_mepic=g.pos_mode == _ffi.POS_NATURAL, _num_splits=num_splits,
        _return_plan=True)


def test_static_scratch_entry_matches_workspace_entry_twice_second_call_smaller():
    print("case: no-alloc prefill entry, config 2 then a ragged batch", flush=True)
    lib = _ffi.lib()
    assert lib.lazyattn_static_scratch_bytes() == 32 << 20
    big = wl.config(2, variant="offset").to(DEV)
    small = wl.make_workload("ragged", dtype=torch.bfloat16, hq=32, hkv=8, d=128, theta=500000.0, block_size=16,
                             doc_lens=[100, 16, 333, 70, 5, 250], requests=[[3, 1, 0], [2], [0, 2, 3, 1, 5], [4], []],
                             q_lens=[70, 1, 9, 33, 130], variant="offset", seed=31).to(DEV)
    for g, ns in ((big, 0), (small, 3)):
        ref = torch.full_like(g.q, 5.0)
        plan = _plan(g, ref, ns)
        assert lib.lazyattn_prefill_workspace_bytes(ctypes.byref(plan.params)) > 0      # the split path is taken
        plan.run()
        got = torch.full_like(g.q, 5.0)
        plan2 = _plan(g, got, ns)
        plan2.params.workspace = None                                                    # nothing handed over
        plan2.params.workspace_bytes = 0
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.lazyattn_prefix_prefill_static_scratch(ctypes.byref(plan2.params), stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert torch.equal(got, ref)
        assert not torch.all(got == 5.0)


def test_static_scratch_entry_rejects_calls_beyond_its_buffer():
    print("case: no-alloc prefill entry, too large", flush=True)
    lib = _ffi.lib()
    g = wl.config(3).to(DEV)                       # 1 024 tokens x 32 heads: 8.65 MB of partials per split
    o = torch.full_like(g.q, 5.0)
    plan = _plan(g, o, 4)
    need = lib.lazyattn_prefill_workspace_bytes(ctypes.byref(plan.params))
    assert need > lib.lazyattn_static_scratch_bytes()
    rc = lib.lazyattn_prefix_prefill_static_scratch(ctypes.byref(plan.params), torch.cuda.current_stream().cuda_stream)
    assert rc == -7 and b"static buffer" in lib.lazyattn_error_string(rc)
    torch.cuda.synchronize()
    assert torch.all(o == 5.0)


def test_static_scratch_entry_allocates_nothing_and_replays_from_a_captured_graph():
    """Capture is what the entry point is for: after ``lazyattn_static_scratch_prepare()`` (outside the capture) a
    call inside a stream capture must record, replay with the right result every time, and leave the amount of
    free device memory where it was."""
    print("case: no-alloc prefill entry under stream capture", flush=True)
    lib = _ffi.lib()
    g = wl.config(2, shrink=2).to(DEV)
    ref = torch.full_like(g.q, 5.0)
    _plan(g, ref, 0).run()
    got = torch.full_like(g.q, 5.0)
    plan = _plan(g, got, 0)
    assert lib.lazyattn_prefill_workspace_bytes(ctypes.byref(plan.params)) > 0
    plan.params.workspace = None
    plan.params.workspace_bytes = 0
    assert lib.lazyattn_static_scratch_prepare() == 0
    # one eager call first: kernel attributes of this shape are set, nothing is left to do but launches
    assert lib.lazyattn_prefix_prefill_static_scratch(ctypes.byref(plan.params), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    free0 = torch.cuda.mem_get_info()[0]
    assert lib.lazyattn_prefix_prefill_static_scratch(ctypes.byref(plan.params), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.lazyattn_prefix_prefill_static_scratch(ctypes.byref(plan.params), side.cuda_stream)
    assert rc == 0, rc
    for step in range(3):
        got.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, ref), step
        torch.zeros(1 << 20, device=DEV).sum().item()          # unrelated eager work between the replays
