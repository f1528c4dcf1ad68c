"""GPU parity of the fused "rotary embedding of the new tokens + paged-cache write" launch
(``lazyattn_rope_and_cache_write``) against the CPU restatement, through the Python functions
that mirror the reference's call sites (``rotary_embedding.py:67-94``,
``backends/triton_attn.py:100-109``)."""
import pytest
import torch

from oracle import deferred_rope as orc
from lazy_amd.model_executor.layers import rotary_embedding as rope

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(dtype, d, hq, hkv, t, *, fp8=False, seed=3, bs=16):
    g = torch.Generator().manual_seed(seed)
    table = orc.build_cos_sin_table(4096, d, 500000.0).to(dtype)
    q = torch.randn(t, hq, d, generator=g).to(dtype)
    k = torch.randn(t, hkv, d, generator=g).to(dtype)
    v = torch.randn(t, hkv, d, generator=g).to(dtype)
    pos = torch.randint(0, 4096, (t,), generator=g)
    nb = (t + bs - 1) // bs + 3
    slots = torch.randperm(nb * bs, generator=g)[:t]
    slots[t // 3] = -1                                            # a padded token: not written
    x = 16 if fp8 else 16 // q.element_size()
    cdt = torch.uint8 if fp8 else dtype
    kc = torch.zeros(nb, hkv, d // x, bs, x, dtype=cdt)
    vc = torch.zeros(nb, hkv, d, bs, dtype=cdt)
    return table, q, k, v, pos, slots, kc, vc


def _tol(dtype):
    return 1e-5 if dtype == torch.float32 else 2e-2


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float32, 64), (torch.float16, 128)])
@pytest.mark.parametrize("q_only", [True, False])
def test_fused_rotate_and_write(dtype, d, q_only):
    print(f"case: rope+write {dtype} d={d} q_only={q_only}", flush=True)
    table, q, k, v, pos, slots, kc, vc = _case(dtype, d, 8, 2, 75)
    q_ref, k_ref = orc.rotary_new_tokens(pos, q, k, table, q_only=q_only)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    orc.paged_cache_write(k_ref, v, kc_ref, vc_ref, slots)
    qg, kg, vg, kcg, vcg = (a.to(DEV) for a in (q, k, v, kc, vc))
    rope.rotate_and_write(pos.to(DEV), qg, kg, vg, d, table.to(DEV), rotate_query=True, rotate_key=not q_only,
                          key_cache=kcg, value_cache=vcg, slot_mapping=slots.to(DEV))
    tol = _tol(dtype)
    assert (qg.cpu().float() - q_ref.float()).abs().max() < tol
    assert (kg.cpu().float() - k_ref.float()).abs().max() < tol
    assert (kcg.cpu().float() - kc_ref.float()).abs().max() < tol
    assert torch.equal(vcg.cpu(), vc_ref)                         # V is moved, not computed: bit-exact
    if q_only:
        assert torch.equal(kg.cpu(), k) and torch.equal(kcg.cpu(), kc_ref)


def test_reference_call_sites_separately():
    """rotary_embedding(positions, query, None, ...) then write_to_paged_cache(...), as the reference does."""
    print("case: rope then write, two calls", flush=True)
    dtype, d = torch.bfloat16, 128
    table, q, k, v, pos, slots, kc, vc = _case(dtype, d, 32, 8, 130, seed=5)
    q_ref, _ = orc.rotary_new_tokens(pos, q, k, table, q_only=True)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    orc.paged_cache_write(k, v, kc_ref, vc_ref, slots)
    qg, kg, vg, kcg, vcg = (a.to(DEV) for a in (q, k, v, kc, vc))
    q2 = qg.view(130, 32 * d)                                      # the model hands [T, H*D]
    out_q, out_k = rope.forward(pos.to(DEV), q2, kg.view(130, 8 * d), d, table.to(DEV), q_only=True)
    assert out_q.data_ptr() == q2.data_ptr()
    rope.write_to_paged_cache(kg, vg, kcg, vcg, slots.to(DEV), "auto", None, None)
    assert (qg.cpu().float() - q_ref.float()).abs().max() < 2e-2
    assert torch.equal(kg.cpu(), k)
    assert torch.equal(kcg.cpu(), kc_ref) and torch.equal(vcg.cpu(), vc_ref)


@pytest.mark.parametrize("kv,top,f8", [("fp8", 448.0, torch.float8_e4m3fn), ("fp8_e5m2", 57344.0, torch.float8_e5m2)])
def test_fp8_quantise_on_write(kv, top, f8):
    print(f"case: {kv} cache write", flush=True)
    dtype, d = torch.bfloat16, 128
    table, q, k, v, pos, slots, kc, vc = _case(dtype, d, 8, 2, 64, fp8=True, seed=9)
    k = k * 3.0
    ks, vs = float(k.abs().max() / (top * 2.0)), float(v.abs().max() / top)       # K saturates on purpose
    kc_ref, vc_ref = kc.clone(), vc.clone()
    orc.paged_cache_write(k, v, kc_ref, vc_ref, slots, kv, ks, vs)
    kg, vg, kcg, vcg = (a.to(DEV) for a in (k, v, kc, vc))
    rope.write_to_paged_cache(kg, vg, kcg, vcg, slots.to(DEV), kv, ks, vs)
    a = kcg.cpu().view(f8).float()
    assert torch.isfinite(a).all() and a.abs().max() == top
    # byte work: the kernel divides by the scale like the writer it replaces, so every code is the same
    assert torch.equal(kcg.cpu(), kc_ref)
    assert torch.equal(vcg.cpu(), vc_ref)


def test_written_cache_feeds_the_attention_oracle_layout():
    """The write is the inverse of the page gather the attention kernels read with."""
    print("case: write/gather round trip", flush=True)
    dtype, d = torch.bfloat16, 128
    table, q, k, v, pos, slots, kc, vc = _case(dtype, d, 8, 2, 48, seed=11)
    slots = torch.arange(16, 64)                                   # blocks 1..3, in order
    kg, vg, kcg, vcg = (a.to(DEV) for a in (k, v, kc, vc))
    rope.write_to_paged_cache(kg, vg, kcg, vcg, slots.to(DEV), "auto", None, None)
    kb, vb = orc.gather_pages(kcg.cpu(), vcg.cpu(), torch.tensor([1, 2, 3]))
    assert torch.equal(kb, k) and torch.equal(vb, v)


@pytest.mark.parametrize("bs", [16, 32])
@pytest.mark.parametrize("dtype,fp8", [(torch.bfloat16, False), (torch.float32, False), (torch.bfloat16, True)])
def test_page_ordered_runs_and_broken_runs(dtype, fp8, bs):
    """A prefill chunk is written page by page (whole 16-token runs land in 16 aligned slots of one page, in
    order); runs broken by a skipped token or ending short take the per-token route."""
    print(f"case: page-ordered slots {dtype} fp8={fp8} page={bs}", flush=True)
    d, t = 64 if dtype == torch.float32 else 128, 70
    table, q, k, v, pos, slots, kc, vc = _case(dtype, d, 4, 2, t, fp8=fp8, seed=21, bs=bs)
    nb = kc.shape[0]
    pages = torch.randperm(nb)[:5]
    slots = (pages[:, None] * bs + torch.arange(bs)[None, :]).flatten()[:t].clone()
    slots[37] = -1                                                # breaks the third run
    ks, vs = (0.02, 0.01) if fp8 else (1.0, 1.0)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    orc.paged_cache_write(k, v, kc_ref, vc_ref, slots, "fp8" if fp8 else "auto", ks, vs)
    kg, vg, kcg, vcg = (a.to(DEV) for a in (k, v, kc, vc))
    rope.write_to_paged_cache(kg, vg, kcg, vcg, slots.to(DEV), "fp8" if fp8 else "auto", ks, vs)
    assert torch.equal(kcg.cpu(), kc_ref) and torch.equal(vcg.cpu(), vc_ref)      # bytes: exact, fp8 included


@pytest.mark.parametrize("kv,f8", [("fp8", torch.float8_e4m3fn), ("fp8_e5m2", torch.float8_e5m2)])
def test_fp8_write_passes_nan_through_and_rejects_narrow_chunks(kv, f8):
    """A NaN key or value stays a NaN code (the clamp before the conversion propagates it); an fp8 cache whose
    innermost K axis is narrower than one 8-byte chunk is refused instead of spilling into the next slot."""
    print(f"case: {kv} NaN / x=4", flush=True)
    table, q, k, v, pos, slots, kc, vc = _case(torch.bfloat16, 128, 4, 2, 40, fp8=True, seed=13)
    k[5, 1, 17] = float("nan")
    v[7, 0, 3] = float("nan")
    kc_ref, vc_ref = kc.clone(), vc.clone()
    orc.paged_cache_write(k, v, kc_ref, vc_ref, slots, kv, 0.03, 0.02)
    kg, vg, kcg, vcg = (a.to(DEV) for a in (k, v, kc, vc))
    rope.write_to_paged_cache(kg, vg, kcg, vcg, slots.to(DEV), kv, 0.03, 0.02)
    for got, ref in ((kcg.cpu(), kc_ref), (vcg.cpu(), vc_ref)):
        nan = ref.view(f8).float().isnan()
        assert nan.sum() == 1 and torch.equal(got.view(f8).float().isnan(), nan)     # (a NaN has several codes)
        assert torch.equal(got[~nan], ref[~nan])
    kc4 = torch.zeros(kc.shape[0], 2, 32, 16, 4, dtype=torch.uint8, device=DEV)
    with pytest.raises(NotImplementedError):
        rope.write_to_paged_cache(kg, vg, kc4, vcg, slots.to(DEV), kv, 0.03, 0.02)
