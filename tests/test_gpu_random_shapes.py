"""Randomised ragged batches through the operators against the CPU oracle: document lengths, request
composition, new-token counts, GQA group, split count, position mode and cache type are drawn from a
seeded generator (the reference's own tests sweep fixed grids, tests/kernels/test_prefix_prefill.py:27-60;
the draws here reach the corners in between: documents shorter than a page, requests with no context,
one-token requests next to long ones, tiles that end inside a page)."""
import os
import random

import pytest
import torch

from lazy_amd import _ffi, workloads as wl
from opcall import run_op, run_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"
# LAZYATTN_RANDOM_CASES=N widens both sweeps to N draws (the default keeps the suite short)
N_PREFILL = int(os.environ.get("LAZYATTN_RANDOM_CASES", 64))
N_DECODE = int(os.environ.get("LAZYATTN_RANDOM_CASES", 24))


def _excess(got, ref, dtype):
    """Largest |got - ref| beyond one unit in the last place of ref: both are rounded to the operand type, and
    a row that sees a handful of keys can have outputs above 4, where one bf16 step is 2^-5."""
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    return ((got.float() - ref.float()).abs() - ulp * ref.float().abs()).clamp(min=0).max().item()


def _draw(seed):
    r = random.Random(seed)
    hkv = r.choice([1, 2, 4, 8])
    group = r.choice([1, 2, 4, 8])
    n_docs = r.randint(1, 7)
    doc_lens = [r.choice([1, 5, 15, 16, 17, 31, 48, 63, 64, 65, 100, 129, 200, 333]) for _ in range(n_docs)]
    n_req = r.randint(1, 5)
    requests = []
    for _ in range(n_req):
        k = r.randint(0, min(4, n_docs))
        requests.append(r.sample(range(n_docs), k))
    q_lens = [r.choice([1, 2, 7, 31, 32, 33, 64, 70, 129]) for _ in range(n_req)]
    variant = r.choice(["natural", "offset", "block_uniform"])
    kv = r.choice(["auto", "auto", "fp8"])
    nsplit = r.choice([0, 1, 2, 3, 5])
    kernel = r.choice([_ffi.KERNEL_MFMA4, _ffi.KERNEL_MFMA8, _ffi.KERNEL_AUTO])
    dtype = r.choice([torch.bfloat16, torch.bfloat16, torch.float16])
    window = r.choice([0, 0, 7, 50, 300])
    d = r.choice([128, 128, 64])
    page = r.choice([16, 16, 32])
    if r.random() < 0.25:
        d = r.choice([96, 80, 48, 112])     # padded to 128 inside the matrix kernel
    return dict(page=page, dtype=dtype, window=window, d=d, hq=hkv * group, hkv=hkv, doc_lens=doc_lens, requests=requests, q_lens=q_lens, variant=variant,
                kv=kv, nsplit=nsplit, kernel=kernel)


@pytest.mark.parametrize("seed", range(N_PREFILL))
def test_random_ragged_batch(seed):
    c = _draw(1000 + seed)
    print(f"case: random batch seed={seed} {c}", flush=True)
    w = wl.make_workload("rand", dtype=c["dtype"], hq=c["hq"], hkv=c["hkv"], d=c["d"], theta=500000.0, block_size=c["page"],
                         doc_lens=c["doc_lens"], requests=c["requests"], q_lens=c["q_lens"], variant=c["variant"],
                         kv_cache_dtype=c["kv"], seed=seed)
    lazy = None
    if c["variant"] == "block_uniform":
        lazy = torch.tensor([(seed + b) % 3 != 0 for b in range(len(c["q_lens"]))])
    ref = run_oracle(w, sliding_window=c["window"], **({"is_lazy": lazy} if lazy is not None else {}))
    got = run_op(w.to(DEV), kernel=c["kernel"], num_splits=c["nsplit"], sliding_window=c["window"] or None,
                 is_lazy=None if lazy is None else lazy.to(DEV)).cpu()
    assert torch.isfinite(got.float()).all()
    err = _excess(got, ref, c["dtype"])
    assert err < (5e-2 if c["kv"] == "fp8" else 2e-2 if c["dtype"] == torch.bfloat16 else 5e-3), err


@pytest.mark.parametrize("seed", range(N_DECODE))
def test_random_decode_batch(seed):
    """The q_len == 1 rows through the decode launch: every key, the new token included, sits in the paged
    cache when the call is made; requests with more than one new token must be left alone."""
    from oracle import deferred_rope as orc
    import test_gpu_decode as dec
    r = random.Random(5000 + seed)
    hkv = r.choice([1, 2, 8])
    group = r.choice([1, 2, 4, 8, 16])
    variant = r.choice(["natural", "block_uniform"])
    kv = r.choice(["auto", "auto", "fp8"])
    q_lens = tuple(r.choice([1, 1, 1, 3]) for _ in range(5))
    nsplit = r.choice([0, 1, 2, 5, 9])
    page = r.choice([16, 16, 32])
    d = r.choice([128, 128, 64, 96, 80, 48])
    if r.random() < 0.2:
        group = r.choice([24, 40, 64])        # above 16: several head blocks per kv head
    print(f"case: random decode seed={seed} hkv={hkv} group={group} {variant} kv={kv} q_lens={q_lens} nsplit={nsplit} "
          f"page={page} d={d}", flush=True)
    w = dec._decode_batch(variant, hq=hkv * group, hkv=hkv, q_lens=q_lens, seed=seed, kv=kv, bs=page, d=d)
    lazy = torch.tensor([(seed + b) % 4 != 0 for b in range(5)]) if variant == "block_uniform" else None
    ref = dec._oracle(w, lazy)
    got = dec._run(w, lazy=lazy, num_splits=nsplit)
    assert torch.isfinite(got.float()).all()
    err = (got.float() - ref.float()).abs().max().item()
    assert err < (5e-2 if kv == "fp8" else 2e-2), err
