"""GPU parity of the geometry-agnostic HIP kernel against the CPU oracle, through the
Python operator (which goes through the C ABI).  Tolerances: 1e-5 for float32 operands,
2e-2 for bf16, 5e-2 with an fp8 cache (max abs error on N(0,1) inputs)."""
import pytest
import torch

from lazy_amd import _ffi, workloads as wl
from opcall import run_op, run_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 5e-3}


def _small(variant, dtype=torch.float32, d=64, bs=16, kv="auto", seed=21):
    return wl.make_workload("small", dtype=dtype, hq=8, hkv=2, d=d, theta=500000.0, block_size=bs,
                            doc_lens=[40, 16, 33, 70, 5], requests=[[3, 1, 0], [2], [0, 2, 3, 1], [4]],
                            q_lens=[70, 1, 9, 33], variant=variant, kv_cache_dtype=kv, seed=seed)


def test_config1_fp32_plumbing():
    print("case: config 1 fp32 generic", flush=True)
    w = wl.config(1)
    ref = run_oracle(w)
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC).cpu()
    assert got.shape == (64, 32, 64)
    err = (got - ref).abs().max().item()
    assert err < 1e-5, err


@pytest.mark.parametrize("variant", ["natural", "offset", "block_uniform"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_generic_variants(variant, dtype):
    print(f"case: generic {variant} {dtype}", flush=True)
    w = _small(variant, dtype)
    ref = run_oracle(w).float()
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC).cpu().float()
    err = (got - ref).abs().max().item()
    assert err < TOL[dtype], err


@pytest.mark.parametrize("d,bs", [(32, 8), (128, 16), (96, 32), (256, 16)])
def test_generic_geometries(d, bs):
    print(f"case: generic d={d} bs={bs}", flush=True)
    w = _small("offset", torch.float32, d=d, bs=bs)
    ref = run_oracle(w)
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC).cpu()
    err = (got - ref).abs().max().item()
    assert err < 1e-5, err


def test_generic_sliding_window_skip_decode_and_int64_index():
    print("case: generic sliding/skip/int64", flush=True)
    w = _small("natural")
    ref = run_oracle(w, sliding_window=37, skip_decode=True, out=torch.full_like(w.q, 3.0))
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC, sliding_window=37, skip_decode=True,
                 out=torch.full_like(w.q, 3.0).to(DEV), index_dtype=torch.int64).cpu()
    assert torch.all(got[70] == 3.0)                       # q_len == 1 request untouched
    err = (got - ref).abs().max().item()
    assert err < 1e-5, err


def test_generic_vanilla_requests():
    print("case: generic vanilla", flush=True)
    w = _small("block_uniform")
    lazy = torch.tensor([True, False, False, True])
    ref = run_oracle(w, is_lazy=lazy)
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC, is_lazy=lazy.to(DEV)).cpu()
    err = (got - ref).abs().max().item()
    assert err < 1e-5, err


@pytest.mark.parametrize("kv", ["fp8", "fp8_e5m2"])
def test_generic_fp8_cache(kv):
    print(f"case: generic {kv}", flush=True)
    w = _small("natural", torch.bfloat16, d=128, kv="fp8")
    if kv == "fp8_e5m2":           # reinterpret the same bytes as e5m2: still a valid cache
        w.kv_cache_dtype = kv
        w.k_cache &= 0x7B          # keep exponents below inf/NaN
        w.v_cache &= 0x7B
        w.k_scale = torch.tensor(2.0 ** -12); w.v_scale = torch.tensor(2.0 ** -12)
    ref = run_oracle(w).float()
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC).cpu().float()
    err = (got - ref).abs().max().item()
    assert err < 5e-2, err


def test_pad_slots_may_hold_nan():
    print("case: generic NaN pad", flush=True)
    w = _small("offset")
    ref = run_oracle(w)
    bs = 16
    for b in range(4):
        for j in range(w.block_table.shape[1]):
            m = int(w.q_mask[b, j])
            if m:
                pb = int(w.block_table[b, j])
                w.k_cache[pb, :, :, bs - m:, :] = float("nan")
                w.v_cache[pb, :, :, bs - m:] = float("nan")
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC).cpu()
    err = (got - ref).abs().max().item()
    assert err < 1e-5, err


def test_no_context_request():
    print("case: generic no context", flush=True)
    w = wl.make_workload("nocontext", dtype=torch.float32, hq=4, hkv=2, d=64, theta=10000.0,
                         block_size=16, doc_lens=[16], requests=[[], [0]], q_lens=[40, 3],
                         variant="natural", seed=2)
    ref = run_oracle(w)
    got = run_op(w.to(DEV), kernel=_ffi.KERNEL_GENERIC).cpu()
    err = (got - ref).abs().max().item()
    assert err < 1e-5, err


def test_cos_sin_builder_matches_closed_form():
    from lazy_amd.model_executor.rope.cos_sin import build_cos_sin_cache, ROPE_LLAMA3
    from oracle import deferred_rope as orc
    print("case: cos/sin builder", flush=True)
    for meta, l3 in [(None, None),
                     (dict(ROPE_TYPE=ROPE_LLAMA3, SCALING_FACTOR=8.0, LOW_FACTOR=1.0, HIGH_FACTOR=4.0,
                           ORIG_MAX_POSITION=8192),
                      dict(scaling_factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                           orig_max_position=8192))]:
        got = build_cos_sin_cache(66000, 128, meta, base=500000.0, dtype=torch.float32).cpu()
        ref = orc.build_cos_sin_table(66000, 128, 500000.0, llama3=l3, dtype=torch.float64,
                                      math_dtype=torch.float64)
        err = (got.double() - ref).abs().max().item()
    assert err < 1e-7, err
    got = build_cos_sin_cache(4096, 64, None, base=10000.0, dtype=torch.bfloat16).cpu()
    ref = orc.build_cos_sin_table(4096, 64, 10000.0, dtype=torch.float64, math_dtype=torch.float64)
    want = ref.float().to(torch.bfloat16)
    # bf16 rounding of the same fp32 value; a last-place difference of the device's double
    # cos/sin can flip a tie, so allow one bf16 ulp on a vanishing fraction of entries
    assert (got.float() - want.float()).abs().max().item() <= 2.0 ** -8
    assert (got != want).float().mean().item() < 1e-3
