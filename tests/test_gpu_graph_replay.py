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


def test_replay_with_other_lengths_cuts_the_batch_anew():
    """The lengths live on the device and the batch is cut into work items there: a captured call replayed after
    the lengths were rewritten in place (same buffers, same host-side maxima) must give what a fresh call gives on
    the new lengths -- and what the oracle gives."""
    print("case: graph replay with rewritten lengths", flush=True)
    from opcall import run_oracle
    import dataclasses
    wc = wl.make_workload("graph", dtype=torch.bfloat16, hq=32, hkv=8, d=128, theta=500000.0, block_size=16,
                          doc_lens=[512, 256, 1024, 128], requests=[[0, 2, 1], [3, 1], [2, 0, 3, 1], [1]],
                          q_lens=[96, 40, 64, 56], variant="natural", seed=5)
    w = wc.to(DEV)
    out = torch.zeros_like(w.q)
    run_op(w, out=out)                                # warm-up (AUTO: splits chosen per request on the device)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            run_op(w, out=out)
    ctx0 = (wc.b_seq_len - (wc.b_start_loc[1:] - wc.b_start_loc[:-1])).tolist()
    # the same 256 tokens divided otherwise, over contexts cut back to other whole pages (each request keeps a
    # prefix of its pages; no new token count exceeds the captured call's longest)
    for step, (q_lens, cut) in enumerate((([96, 40, 64, 56], [0, 0, 0, 0]), ([16, 96, 80, 64], [512, 128, 1040, 0]),
                                          ([1, 95, 96, 64], [1280, 0, 48, 128]), ([64, 64, 64, 64], [256, 256, 256, 128]))):
        ctx = [c - d for c, d in zip(ctx0, cut)]
        assert all(c >= 0 for c in ctx) and sum(q_lens) == w.q.shape[0] and max(q_lens) <= w.max_query_len
        starts = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=wc.b_start_loc.dtype)
        seqs = torch.tensor([c + q for c, q in zip(ctx, q_lens)], dtype=wc.b_seq_len.dtype)
        w.b_start_loc.copy_(starts.to(DEV))
        w.b_seq_len.copy_(seqs.to(DEV))
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = run_op(w)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), (step, (got.float() - eager.float()).abs().max().item())
        ref = run_oracle(dataclasses.replace(wc, b_start_loc=starts, b_seq_len=seqs))
        err = (got.cpu().float() - ref.float()).abs().max().item()
        assert err < 2e-2, (step, err)
