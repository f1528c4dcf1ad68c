"""The prefill call and the q_len == 1 call recorded into a HIP graph (through torch's capture) and replayed:
serving loops replay captured steps, and the library must neither allocate nor synchronise inside a call.
Every replay is checked against an eager call on the same inputs, with eager work and synchronisations
between the replays."""
import pytest
import torch

from lazy_amd import _ffi, workloads as wl
from opcall import run_op

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _workload(variant):
    return wl.make_workload("graph", dtype=torch.bfloat16, hq=32, hkv=8, d=128, theta=500000.0, block_size=16,
                            doc_lens=[200, 48, 333, 70], requests=[[3, 1, 0], [2, 0], [1]], q_lens=[40, 1, 70],
                            variant=variant, seed=12).to(DEV)


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
def test_prefill_call_replays_from_a_graph(variant):
    print(f"case: graph replay {variant}", flush=True)
    w = _workload(variant)
    out = torch.zeros_like(w.q)
    run_op(w, num_splits=3, out=out)                 # warm-up: packed table, workspace and kernel attributes exist now
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            run_op(w, num_splits=3, out=out)
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(4):
        # new queries and new-token keys each step, written in place like a serving loop does
        w.q.copy_(torch.randn(w.q.shape, generator=gen, device=DEV).to(w.q.dtype))
        w.k.copy_(torch.randn(w.k.shape, generator=gen, device=DEV).to(w.k.dtype))
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = run_op(w, num_splits=3)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), (step, (got.float() - eager.float()).abs().max().item())


def test_mixed_batch_entry_point_replays_from_a_graph():
    """``chunked_prefill_paged_decode`` on a batch with prefill rows and q_len == 1 rows: four launches (prefill main,
    prefill merge, q_len == 1 main, its merge) in one captured graph."""
    print("case: graph replay of the mixed-batch entry point", flush=True)
    import test_gpu_entrypoints as ep
    w = ep._mixed("natural", torch.bfloat16, 128)
    ref = ep._expected(w)
    g = w.to(DEV)
    out = torch.full_like(g.q, 5.0)

    def call():
        ep.entry_unrotated(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                           g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale, sm_scale=128 ** -0.5, rotary_dim=128,
                           cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
    call()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call()
    for step in range(3):
        out.fill_(5.0)
        graph.replay()
        torch.cuda.synchronize()
        err = (out.cpu().float() - ref.float()).abs().max().item()
        assert err < 2e-2, (step, err)
        torch.zeros(1 << 20, device=DEV).sum().item()          # unrelated eager work between the replays
