#!/usr/bin/env python3
"""Benchmark of the deferred-RoPE prefix-prefill operator on one MI355X.

A step is one call of the operator (rotate cached K per page, QK^T, online softmax, PV,
split-KV merge) on a synthetic batch that is already resident in HBM.  The default
workload is the north-star configuration: Llama-3-8B geometry, bf16, 10 x 512-token
shuffled documents, 128 query tokens.  Prints one JSON line.

    python bench.py [--steps K] [--warmup W] [--config 2|3|4|5] [--num-splits S] [--no-cpu]
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "lazy-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
# HBM bytes one launch of the dominant kernel moves, from hardware counters (rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, each scaled by what the same counter reads for a 256 MiB copy; summary under profiles/).
# Counters cannot be read from inside this script, so the figure is the committed measurement of the
# named workload; workloads without one report null.
MEASURED_TRAFFIC_BYTES = {"c2_8b_bf16_10x512_q128": 43_300_000, "c3_8b_bf16_pool64x256_16req_x20_q64": 242_200_000,
                          "c4_8b_bf16_64x1024_q256": 441_100_000, "c5_8b_fp8kv_8req_32x512_q128": 335_000_000,
                          "d1_8b_bf16_decode_32req_20x256": 679_600_000}
PEAK_HBM_GBS = 8000.0


def make_plan(g, num_splits, phases):
    """The call as a re-usable plan, through the operator of the workload's position mode."""
    import torch
    from lazy_amd import _ffi
    from lazy_amd.attention.old_ops.prefix_prefill import context_attention_fwd as fwd_unrotated
    from lazy_amd.attention.ops.prefix_prefill import context_attention_fwd as fwd_block_uniform
    o = torch.zeros_like(g.q)
    args = (g.q, g.k, g.v, o, g.kv_cache_dtype, g.k_cache, g.v_cache, g.block_table, g.b_start_loc,
            g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale)
    kw = dict(cos_sin_cache=g.cos_sin_cache, rotary_dim=g.q.shape[-1], q_mask=g.q_mask, q_offset=g.q_offset,
              _num_splits=num_splits, _phases=phases, _return_plan=True)
    if g.pos_mode == _ffi.POS_BLOCK_UNIFORM:
        plan = fwd_block_uniform(*args, is_lazy=g.is_lazy, **kw)
    else:
        plan = fwd_unrotated(*args, is_mepic=g.pos_mode == _ffi.POS_NATURAL, **kw)
    return plan, o


def host_us_per_call(g, calls=1000, chunk=100):
    """Host time of one call of the backend's entry point (``chunked_prefill_paged_decode``: the prefill launch,
    its merge and the q_len==1 launch) on fixed buffers, in microseconds: ``calls`` calls in chunks the GPU is
    drained between, so no enqueue ever waits for queue space.  Returns (entry point, its launches alone)."""
    import torch
    from lazy_amd import _ffi
    from lazy_amd.attention import _launch
    from lazy_amd.attention.old_ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode as unrotated
    from lazy_amd.attention.ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode as block_uniform
    o = torch.zeros_like(g.q)
    args = (g.q, g.k, g.v, o, g.kv_cache_dtype, g.k_cache, g.v_cache, g.block_table, g.b_start_loc,
            g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale)
    kw = dict(cos_sin_cache=g.cos_sin_cache, rotary_dim=g.q.shape[-1], q_mask=g.q_mask, q_offset=g.q_offset)
    if g.pos_mode == _ffi.POS_BLOCK_UNIFORM:
        call = lambda: block_uniform(*args, is_lazy=g.is_lazy, **kw)
    else:
        call = lambda: unrotated(*args, is_mepic=g.pos_mode == _ffi.POS_NATURAL, **kw)
    call()
    plans = next(reversed(_launch._calls.values()))[1]       # the launches that call was reduced to
    stream = torch.cuda.current_stream().cuda_stream
    raw = lambda: [p._entry(p.params, stream) for p in plans]
    res = []
    for fn in (call, raw):
        for _ in range(chunk):
            fn()
        spent = 0.0
        for _ in range(calls // chunk):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(chunk):
                fn()
            spent += time.perf_counter() - t0
        torch.cuda.synchronize()
        res.append(spent / (calls // chunk * chunk) * 1e6)
    return res


def time_calls(plan, n):
    """ms per call over n back-to-back launches, HIP events on the launch stream."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(n):
        plan.run()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / n


COLD_BYTES = 320 << 20       # distinct K/V the cold-cache loop goes round: more than the 256 MB last-level cache


def cold_plans(g, num_splits, phases):
    """The same call on enough distinct copies of the paged K/V cache that no launch finds its keys and
    values in L2 or the last-level cache (a served model's layers each own a cache)."""
    import dataclasses
    set_bytes = g.k_cache.numel() * g.k_cache.element_size() + g.v_cache.numel() * g.v_cache.element_size()
    n = max(2, -(-COLD_BYTES // set_bytes) + 1)
    plans = []
    for _ in range(n):
        gi = dataclasses.replace(g, k_cache=g.k_cache.clone(), v_cache=g.v_cache.clone())
        plans.append(make_plan(gi, num_splits, phases)[0])
    return plans, set_bytes


def time_round_robin(plans, n):
    """ms per call over n back-to-back launches that go round the plans."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(n):
        plans[i % len(plans)].run()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / n


def cpu_baseline(w, reps):
    """The float32 PyTorch-eager statement of the same op on the host cores."""
    import torch
    from oracle import deferred_rope as orc

    def once():
        t = time.perf_counter()
        orc.prefix_prefill(w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc,
                           w.b_seq_len, w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode,
                           rotate_new_k=w.rotate_new_k, kv_cache_dtype=w.kv_cache_dtype,
                           k_scale=w.k_scale, v_scale=w.v_scale)
        return time.perf_counter() - t
    once()
    if reps is None:                     # about ten seconds of host work, at least five calls
        reps = max(5, min(1000, int(10.0 / max(min(once(), once()), 1e-4))))
    return statistics.median(once() for _ in range(reps)), reps


def bench_decode(a):
    """The q_len==1 path: 32 requests x 5 120 context keys, one new token each.  HBM-bound: value and
    roofline are bytes of K/V (each read once) per second."""
    import torch
    from lazy_amd import _ffi, workloads as wl
    from lazy_amd.attention import _launch
    from lazy_amd.model_executor.rope import cos_sin as rope_cs
    bu = a.variant == "block_uniform"
    w = wl.decode_config(variant="block_uniform" if bu else "natural")
    g = w.to("cuda:0")
    o = torch.zeros_like(g.q)
    # --compute-cos-sin: the kernel forms cos/sin from the inverse frequencies instead of reading the table;
    # --packed-table: it walks the int64 table [block:32 | q_offset:16 | q_mask:16] instead of three int32 tables
    freqs = rope_cs.rope_freqs(dict(ROPE_TYPE=0, BASE=500000.0), g.q.shape[-1], "cuda:0") if a.compute_cos_sin else None
    packed = ((g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()) if a.packed_table else None

    def plan(phases):
        return _launch.launch_prefill(
            q=g.q, k=g.k, v=g.v, o=o, kv_cache_dtype="auto", k_cache=g.k_cache, v_cache=g.v_cache,
            b_loc=g.block_table, b_start_loc=g.b_start_loc, b_seq_len=g.b_seq_len, max_input_len=1,
            max_seq_len=g.max_seq_len, k_scale=g.k_scale, v_scale=g.v_scale, alibi_slopes=None,
            sliding_window=0, sm_scale=g.q.shape[-1] ** -0.5, skip_decode=False, cos_sin_cache=g.cos_sin_cache,
            rotary_dim=g.q.shape[-1], is_neox_style=True, is_lazy=None, q_offset=g.q_offset if bu else None, q_mask=g.q_mask,
            pos_mode=_ffi.POS_BLOCK_UNIFORM if bu else _ffi.POS_NATURAL, rotate_new_k=not bu, decode=True,
            num_splits=a.num_splits, phases=phases, packed_block_table=packed, rope_freqs=freqs, _return_plan=True)
    full, main_only = plan(_ffi.PHASE_ALL), plan(_ffi.PHASE_MAIN)
    for _ in range(a.warmup):
        full.run()
    torch.cuda.synchronize()
    ms = time_calls(full, a.steps)
    for _ in range(a.warmup):
        main_only.run()
    torch.cuda.synchronize()
    main_ms = statistics.median([time_calls(main_only, max(a.steps // 4, 10)) for _ in range(7)])
    full.run()
    torch.cuda.synchronize()
    gbs = w.bytes / (ms * 1e-3) / 1e9
    main_gbs = w.bytes / (main_ms * 1e-3) / 1e9
    out = {
        "metric": "fused-rotary paged decode (q_len==1): K/V GB/s, 8B geometry, 32 requests x 5K context",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w.name, "hq": 32, "hkv": 8, "head_dim": 128, "page": 16,
                   "requests": int(w.b_seq_len.numel()), "keys_per_request": int(w.b_seq_len[0]),
                   "mb_per_call": round(w.bytes / 1e6, 2), "positions": a.variant if bu else "natural",
                   "cos_sin": "computed" if a.compute_cos_sin else "table", "packed_table": bool(a.packed_table)},
        "roofline": {"bound": "hbm", "achieved": round(main_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(main_gbs / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(w.name),
                     "traffic_unit": "HBM bytes per launch", "kernel": "paged_decode_kernel",
                     "kernel_ms": round(main_ms, 5)},
    }
    if not a.no_cpu:
        from oracle import deferred_rope as orc
        torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        ws = wl.decode_config(nreq=4)
        ts = []
        for _ in range(3):
            t = time.perf_counter()
            orc.paged_decode(ws.q, ws.k_cache, ws.v_cache, ws.block_table, ws.b_start_loc, ws.b_seq_len,
                             ws.cos_sin_cache, ws.q_mask, pos_mode=orc.POS_NATURAL)
            ts.append(time.perf_counter() - t)
        sec = statistics.median(ts)
        out["cpu_baseline"] = {"value": round(ws.bytes / sec / 1e9, 3), "unit": "GB/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{ws.name}: 3 calls of 4 requests, median {sec * 1e3:.1f} ms/call"}
    print(json.dumps(out))


def bench_rope_write(a):
    """The step before the attention call for a prefill chunk of 8 192 new tokens, 8B geometry, bf16:
    Q rotated in place, un-rotated K and V scattered into 16-token pages.  One launch."""
    import torch
    from lazy_amd import workloads as wl
    from lazy_amd.model_executor.layers import rotary_embedding as rope
    T, hq, hkv, d, bs = 8192, 32, 8, 128, 16
    gen = torch.Generator().manual_seed(4)
    table = wl.cos_sin_table(T + bs, d, 500000.0, torch.bfloat16).cuda()
    q = torch.randn(T, hq, d, generator=gen).to(torch.bfloat16).cuda()
    k = torch.randn(T, hkv, d, generator=gen).to(torch.bfloat16).cuda()
    v = torch.randn(T, hkv, d, generator=gen).to(torch.bfloat16).cuda()
    pos = torch.arange(T, device="cuda")
    nb = T // bs + 4
    blocks = torch.randperm(nb, generator=gen)[:T // bs]
    slots = (blocks[:, None] * bs + torch.arange(bs)[None, :]).flatten().cuda()     # whole pages, shuffled blocks
    kc = torch.zeros(nb, hkv, d // 8, bs, 8, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros(nb, hkv, d, bs, device="cuda", dtype=torch.bfloat16)

    class Plan:
        def run(self):
            rope.rotate_and_write(pos, q, k, v, d, table, rotate_query=True, rotate_key=False, key_cache=kc,
                                  value_cache=vc, slot_mapping=slots)
    plan = Plan()
    for _ in range(a.warmup):
        plan.run()
    torch.cuda.synchronize()
    ms = time_calls(plan, a.steps)
    nbytes = T * (2 * hq + 4 * hkv) * d * 2            # Q read + written, K and V read, both caches written
    gbs = nbytes / (ms * 1e-3) / 1e9
    out = {
        "metric": "Q rotary + paged-cache write of new tokens: GB/s, 8B geometry, 8192 tokens",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "w1_8b_bf16_rope_write_8192tok", "hq": hq, "hkv": hkv, "head_dim": d, "page": bs,
                   "tokens": T, "mb_per_call": round(nbytes / 1e6, 2)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel": "rope_cache_write_kernel",
                     "kernel_ms": round(ms, 5)},
    }
    if not a.no_cpu:
        from oracle import deferred_rope as orc
        torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        Ts = 1024
        qc, kcpu, vcpu = q[:Ts].cpu(), k[:Ts].cpu(), v[:Ts].cpu()
        kcc, vcc, tc, sc = kc.cpu(), vc.cpu(), table.cpu(), slots[:Ts].cpu()
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            orc.rotary_new_tokens(pos[:Ts].cpu(), qc, kcpu, tc, q_only=True)
            orc.paged_cache_write(kcpu, vcpu, kcc, vcc, sc)
            ts.append(time.perf_counter() - t0)
        sec = statistics.median(ts)
        out["cpu_baseline"] = {"value": round(nbytes * Ts / T / sec / 1e9, 3), "unit": "GB/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"first {Ts} of the {T} tokens, 3 calls, median {sec * 1e3:.1f} ms"}
    print(json.dumps(out))


def bench_reposition(a):
    """Copy-on-write re-positioning of shared blocks (the per-block loop of the reference's block-attention
    model runner): 2 048 blocks of one layer copied to new blocks, their keys moved from one rotation
    position to another.  One launch."""
    import torch
    from lazy_amd import workloads as wl
    from lazy_amd.block_attn import utils as ba
    n, hkv, d, bs = 2048, 8, 128, 16
    gen = torch.Generator().manual_seed(6)
    nb = 2 * n
    kc = torch.randn(nb, hkv, d // 8, bs, 8, generator=gen).to(torch.bfloat16).cuda()
    vc = torch.randn(nb, hkv, d, bs, generator=gen).to(torch.bfloat16).cuda()
    table = wl.cos_sin_table(n * bs + 4096 + bs, d, 500000.0, torch.bfloat16).cuda()
    perm = torch.randperm(n, generator=gen)
    items = torch.stack([n + torch.arange(n), perm, perm * bs % 4096, torch.arange(n) * bs], 1).int()
    items_dev = items.cuda()

    class Plan:
        def run(self):
            ba.reposition_blocks(kc, vc, items_dev, table)
    plan = Plan()
    for _ in range(a.warmup):
        plan.run()
    torch.cuda.synchronize()
    ms = time_calls(plan, a.steps)
    nbytes = n * hkv * d * bs * 2 * 2 * 2              # K and V of every block, read and written
    gbs = nbytes / (ms * 1e-3) / 1e9
    out = {
        "metric": "block re-positioning (copy + un-rotate + rotate): GB/s read+written, 8B geometry, 2048 blocks",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "r1_8b_bf16_reposition_2048blocks", "hkv": hkv, "head_dim": d, "page": bs,
                   "blocks": n, "mb_per_call": round(nbytes / 1e6, 2)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "kernel": "block_reposition_kernel",
                     "kernel_ms": round(ms, 5)},
    }
    if not a.no_cpu:
        from oracle import deferred_rope as orc
        torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        ns = 256
        kcc, vcc, tc = kc.cpu(), vc.cpu(), table.cpu()
        sample = [tuple(int(x) for x in row) for row in items[:ns]]
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            orc.reposition_blocks(kcc, vcc, sample, tc)
            ts.append(time.perf_counter() - t0)
        sec = statistics.median(ts)
        out["cpu_baseline"] = {"value": round(nbytes * ns / n / sec / 1e9, 3), "unit": "GB/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"first {ns} of the {n} blocks, 3 calls, median {sec * 1e3:.1f} ms"}
    print(json.dumps(out))


def bench_layer_step(a):
    """What one engine step asks of this library for a prefill chunk, layer by layer (the call contract of the
    reference's backend, lazy_attn/lazy/attention/backends/triton_attn.py:96-187, without the model around it):
    per layer, rotary embedding of the new tokens' queries + write of their un-rotated K and V into that layer's
    own paged cache (one launch), then ``chunked_prefill_paged_decode`` on that cache.  32 layers, persistent
    buffers, the north-star shape (one request: 10 x 512 cached tokens in shuffled order, 128 new ones)."""
    import torch
    from lazy_amd import workloads as wl
    from lazy_amd.attention.old_ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode
    from lazy_amd.model_executor.layers import rotary_embedding as rope
    layers = a.layers
    w = wl.config(2)
    g = w.to("cuda:0")
    d, bs = g.q.shape[-1], g.v_cache.shape[3]
    ql, ctx = int(w.max_query_len), int(w.b_seq_len[0] - w.max_query_len)
    caches = [(g.k_cache.clone(), g.v_cache.clone()) for _ in range(layers)]
    positions = ctx + torch.arange(ql, device="cuda:0")
    m = torch.arange(ql, device="cuda:0")
    slots = (g.block_table[0, ctx // bs + m // bs].long() * bs + m % bs)
    q_src, out = g.q.clone(), torch.zeros_like(g.q)
    q = g.q

    def step():
        for kc, vc in caches:
            rope.rotate_and_write(positions, q, g.k, g.v, d, g.cos_sin_cache, rotate_query=True, rotate_key=False,
                                  key_cache=kc, value_cache=vc, slot_mapping=slots)
            chunked_prefill_paged_decode(q, g.k, g.v, out, "auto", kc, vc, g.block_table, g.b_start_loc,
                                         g.b_seq_len, g.max_seq_len, g.max_query_len, g.k_scale, g.v_scale,
                                         cos_sin_cache=g.cos_sin_cache, rotary_dim=d, q_mask=g.q_mask, is_mepic=True)
    for _ in range(max(a.warmup, 10)):
        step()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    host = []
    start.record()
    for _ in range(a.steps):
        step()
    end.record()
    end.synchronize()
    gpu_us = start.elapsed_time(end) * 1e3 / (a.steps * layers)
    for _ in range(20):                      # host side alone: the queue is empty when a step starts
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step()
        host.append((time.perf_counter() - t0) * 1e6 / layers)
    torch.cuda.synchronize()
    host_us = statistics.median(host)
    tflops = w.flops / (gpu_us * 1e-6) / 1e12
    set_mb = (g.k_cache.numel() * g.k_cache.element_size() + g.v_cache.numel() * g.v_cache.element_size()) / 1e6
    print(json.dumps({
        "metric": "deferred-RoPE prefill layer step (rotary + cache write, then attention): TFLOP/s of the attention "
                  "work per layer time, 8B geometry, 5K context, every layer on its own cache",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(gpu_us * layers * 1e-3, 5), "us_per_layer": round(gpu_us, 2),
        "host_us_per_layer": round(host_us, 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "l1_8b_bf16_layer_step_10x512_q128", "layers": layers, "hq": 32, "hkv": 8,
                   "head_dim": d, "page": bs, "ctx_keys": ctx, "query_tokens": ql,
                   "cache_mb_per_layer": round(set_mb, 1), "launches_per_layer": 3},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "kernel": "rope_cache_write_kernel + prefill_mfma_kernel + prefill_combine_kernel"},
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, choices=[2, 3, 4, 5])
    ap.add_argument("--num-splits", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--min-warmup", type=int, default=300,
                    help="floor on the untimed warm-up calls, whatever --warmup says (profiler runs lower it)")
    ap.add_argument("--no-host-timing", action="store_true",
                    help="skip the 1 100 entry-point calls that measure host_us_per_call (profiler runs)")
    ap.add_argument("--path", choices=["prefill", "decode", "rope_write", "reposition", "layer_step"], default="prefill",
                    help="prefill: the headline prefix-prefill call (default); decode: the q_len==1 kernel; "
                         "rope_write: Q rotary + paged-cache write of the new tokens; reposition: copy-on-write block "
                         "re-positioning (all three HBM-bound); layer_step: per layer the cache write and the attention "
                         "call on that layer's own cache, as an engine step issues them")
    ap.add_argument("--layers", type=int, default=32, help="layer_step: number of layers (each owns a K/V cache)")
    ap.add_argument("--no-cold", action="store_true",
                    help="skip the cold-cache figures (the call going round distinct copies of the K/V cache)")
    ap.add_argument("--variant", choices=["natural", "offset", "block_uniform"], default="natural",
                    help="how a cached key's rotation position is derived: its index (default), the page's q_offset "
                         "(per-block offsets of the un-rotated cache), or one rotation per page of a cache rotated at "
                         "document-local positions")
    ap.add_argument("--compute-cos-sin", action="store_true", help="decode path: cos/sin computed in the kernel")
    ap.add_argument("--packed-table", action="store_true", help="decode path: the kernel walks the packed int64 table")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 256 MiB device-to-device copy (known traffic, for scaling profiler counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: the operator has no multi-GPU path "
              "(kv-heads / requests shard without any exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from lazy_amd import _ffi, workloads as wl
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    _ffi.lib()
    torch.cuda.set_device(0)
    if a.path == "decode":
        return bench_decode(a)
    if a.path == "rope_write":
        return bench_rope_write(a)
    if a.path == "reposition":
        return bench_reposition(a)
    if a.path == "layer_step":
        return bench_layer_step(a)
    w = wl.config(a.config, variant=a.variant)
    g = w.to("cuda:0")
    plan, o = make_plan(g, a.num_splits, _ffi.PHASE_ALL)
    main_only, _ = make_plan(g, a.num_splits, _ffi.PHASE_MAIN)

    # The first hundreds of launches of a process run up to 10-40 % slow (clocks, caches, code upload): whatever
    # --warmup says, at least --min-warmup untimed calls come first, and the dominant kernel is timed as the
    # median of 7 runs of at least 50 launches (the discipline of the reference's own kernel benchmark,
    # benchmarks/bench_rope_cos_sin.py:451-461,514-522).  The K timed steps of the whole call stay exactly K.
    MIN_WARMUP, MIN_MAIN_LAUNCHES = a.min_warmup, 50
    for _ in range(max(a.warmup, MIN_WARMUP)):
        plan.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms = time_calls(plan, a.steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    # the dominant kernel alone (no merge launch), same stream, same events
    for _ in range(max(a.warmup, MIN_WARMUP)):
        main_only.run()
    torch.cuda.synchronize()
    reps = [time_calls(main_only, max(a.steps // 4, MIN_MAIN_LAUNCHES)) for _ in range(7)]
    main_ms = statistics.median(reps)
    plan.run()
    torch.cuda.synchronize()
    cold = None
    if not a.no_cold:
        # the same call when K/V come from HBM: round-robin over copies of the cache that together exceed the
        # last-level cache; the headline figures above re-use one cache, which stays in L2 / last-level cache
        cp, set_bytes = cold_plans(g, a.num_splits, _ffi.PHASE_ALL)
        cm, _ = cold_plans(g, a.num_splits, _ffi.PHASE_MAIN)
        n_cold = max(a.steps, 4 * len(cp))
        for pl in (cp, cm):
            time_round_robin(pl, 2 * len(pl))
        cold = {"ms_per_call_cold": round(statistics.median(time_round_robin(cp, n_cold) for _ in range(5)), 5),
                "kernel_ms_cold": round(statistics.median(time_round_robin(cm, n_cold) for _ in range(5)), 5),
                "cold_cache_sets": len(cp), "cold_set_mb": round(set_bytes / 1e6, 1)}
        del cp, cm
    if a.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    tflops = w.flops / (ms * 1e-3) / 1e12
    main_tflops = w.flops / (main_ms * 1e-3) / 1e12
    out = {
        "metric": "deferred-RoPE prefix-prefill TFLOP/s (8B geometry, 5K context); ms/call and MFMA fraction alongside",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 5), "ms_per_call": round(ms, 5), "wall_ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": w.name, "hq": 32, "hkv": 8, "head_dim": 128, "page": 16,
                   "requests": int(w.b_seq_len.numel()), "ctx_keys": int(w.b_seq_len[0] - w.max_query_len),
                   "query_tokens": int(w.max_query_len), "kv_cache": w.kv_cache_dtype, "positions": a.variant,
                   "gflop_per_call": round(w.flops / 1e9, 3), "mb_per_call": round(w.bytes / 1e6, 2)},
        "roofline": {"bound": "mfma", "achieved": round(main_tflops, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(main_tflops / PEAK_BF16_TFLOPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(w.name), "traffic_unit": "HBM bytes per launch",
                     "kernel": "prefill_mfma_kernel", "kernel_ms": round(main_ms, 5),
                     # algorithmic bytes over kernel time; the repeats find their inputs in L2/MALL, so this is
                     # an operand rate, not a measurement of HBM traffic (that is `traffic`)
                     "operand_gbs_algorithmic_cache_warm": round(w.bytes / (main_ms * 1e-3) / 1e9, 1)},
    }
    if cold is not None:
        out.update(cold)
        out["tflops_cold"] = round(w.flops / (cold["ms_per_call_cold"] * 1e-3) / 1e12, 2)
    if not a.no_host_timing:
        entry_us, launches_us = host_us_per_call(g)
        out["host_us_per_call"] = round(entry_us, 1)            # entry point, repeat call on fixed buffers
        out["host_us_in_hip_launches"] = round(launches_us, 1)  # of which: the C calls (four kernel launches)
    if not a.no_cpu:
        torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        wc = w if a.config in (2, 3) else wl.config(a.config, shrink=8)
        sec, reps_cpu = cpu_baseline(wc, None)
        out["cpu_baseline"] = {"value": round(wc.flops / sec / 1e12, 4), "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{wc.name}: {reps_cpu} full calls, median {sec * 1e3:.1f} ms/call"
                                         + ("" if wc is w else " (1/8 of the documents)")}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
