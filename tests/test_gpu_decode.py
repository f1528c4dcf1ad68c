"""GPU parity of the q_len==1 kernel with the rotation fused in (``lazyattn_paged_decode_rotary``,
reached through ``chunked_prefill_paged_decode`` of both variants) against the CPU oracle.

Shapes follow the reference's own decode callers: every key, the new token included, is in the
paged cache when the call is made (``backends/triton_attn.py:100-109``)."""
import pytest
import torch

from oracle import deferred_rope as orc
from lazy_amd import _ffi, workloads as wl
from lazy_amd.attention import _launch
from lazy_amd.attention.old_ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode as entry_unrotated
from lazy_amd.attention.ops.chunked_prefill_paged_decode import chunked_prefill_paged_decode as entry_block_uniform

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _decode_batch(variant, *, hq=8, hkv=2, q_lens=(1, 1, 1, 1, 1), table_f32=False, seed=77, kv="auto",
                  dtype=torch.bfloat16, d=128, bs=16):
    """Ragged documents (pads at document ends), requests of 1 to 9 documents, one new token each
    (or more: such requests must be skipped)."""
    w = wl.make_workload("decode", dtype=dtype, hq=hq, hkv=hkv, d=d, theta=500000.0, block_size=bs,
                         doc_lens=[40, 16, 33, 70, 5, 128, 97],
                         requests=[[3, 1, 0], [2], [0, 2, 3, 1, 5, 6, 4, 5, 6], [4, 0], [6, 5, 3]],
                         q_lens=list(q_lens), variant=variant, seed=seed, kv_cache_dtype=kv)
    if table_f32:
        w.cos_sin_cache = w.cos_sin_cache.float()
    x = w.k_cache.shape[4]
    fp8 = "fp8" in kv

    def to_cache(t, scale):
        # a cache write saturates: a new token may exceed the range the scale was chosen for
        return (t.float() / scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8) if fp8 else t
    for b in range(len(q_lens)):
        qs, qe = int(w.b_start_loc[b]), int(w.b_start_loc[b + 1])
        ctx = int(w.b_seq_len[b]) - (qe - qs)
        for t in range(qe - qs):
            n = ctx + t
            pb = int(w.block_table[b, n // bs]); o_ = n % bs
            w.k_cache[pb, :, :, o_, :] = to_cache(w.k[qs + t], w.k_scale).view(hkv, d // x, x)
            w.v_cache[pb, :, :, o_] = to_cache(w.v[qs + t], w.v_scale)
    return w


def _oracle(w, lazy=None, sliding_window=0):
    ref = torch.full_like(w.q, 5.0)
    orc.paged_decode(w.q, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
                     w.cos_sin_cache, w.q_mask, q_offset=w.q_offset, is_lazy=lazy,
                     kv_cache_dtype=w.kv_cache_dtype, k_scale=w.k_scale, v_scale=w.v_scale, sliding_window=sliding_window,
                     pos_mode=orc.POS_NATURAL if w.pos_mode != orc.POS_BLOCK_UNIFORM else w.pos_mode, out=ref)
    return ref


def _run(w, *, lazy=None, num_splits=0, kernel=_ffi.KERNEL_AUTO, sliding_window=0, packed=False, freqs=None):
    """The q_len==1 launch the entry points make, with the slicing and kernel choice exposed.  packed: the
    kernel is given the int64 table [block:32 | q_offset:16 | q_mask:16] and none of the three int32 tables'
    contents (they are overwritten with junk); freqs: cos/sin computed in the kernel, no table."""
    g = w.to(DEV)
    out = torch.full_like(g.q, 5.0)
    bu = w.pos_mode == orc.POS_BLOCK_UNIFORM
    pk = None
    if packed:
        pk = (g.block_table.long() << 32) | (g.q_offset.long() << 16) | g.q_mask.long()
        g.block_table = torch.full_like(g.block_table, 1 << 20)
        g.q_offset = torch.full_like(g.q_offset, 12345)
        g.q_mask = torch.full_like(g.q_mask, 15)
    fr = None
    if freqs is not None:
        fr = freqs.to(DEV)
        g.cos_sin_cache = None
    _launch.launch_prefill(
        q=g.q, k=g.k, v=g.v, o=out, kv_cache_dtype=w.kv_cache_dtype, k_cache=g.k_cache, v_cache=g.v_cache,
        b_loc=g.block_table, b_start_loc=g.b_start_loc, b_seq_len=g.b_seq_len, max_input_len=1,
        max_seq_len=g.max_seq_len, k_scale=g.k_scale, v_scale=g.v_scale, alibi_slopes=None, sliding_window=sliding_window,
        sm_scale=g.q.shape[-1] ** -0.5, skip_decode=False, cos_sin_cache=g.cos_sin_cache, rotary_dim=g.q.shape[-1],
        is_neox_style=True, is_lazy=None if lazy is None else lazy.to(DEV),
        q_offset=g.q_offset if bu else None, q_mask=g.q_mask,
        pos_mode=_ffi.POS_BLOCK_UNIFORM if bu else _ffi.POS_NATURAL, rotate_new_k=not bu, decode=True,
        kernel=kernel, num_splits=num_splits, packed_block_table=pk, rope_freqs=fr)
    return out.cpu()


def _err(a, b):
    return (a.float() - b.float()).abs().max().item()


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("nsplit", [0, 1, 3, 7, 8, 9, 33, 64])      # the merge loads 8 or 32 slices at a time
def test_decode_ragged(variant, nsplit):
    print(f"case: decode ragged {variant} nsplit={nsplit}", flush=True)
    w = _decode_batch(variant)
    ref = _oracle(w)
    got = _run(w, num_splits=nsplit)
    assert _err(got, ref) < 2e-2, _err(got, ref)


def test_decode_matches_generic_kernel():
    print("case: decode fast vs generic kernel", flush=True)
    w = _decode_batch("natural")
    a = _run(w, num_splits=2)
    b = _run(w, kernel=_ffi.KERNEL_GENERIC)
    assert _err(a, b) < 2e-2, _err(a, b)


def test_decode_skips_longer_requests_and_leaves_their_rows():
    print("case: decode skips q_len>1", flush=True)
    w = _decode_batch("natural", q_lens=(1, 4, 1, 2, 1))
    ref = _oracle(w)
    got = _run(w, num_splits=3)
    assert _err(got, ref) < 2e-2, _err(got, ref)
    qs = int(w.b_start_loc[1])
    assert torch.all(got[qs:qs + 4] == 5.0)                      # old_ops/chunked_prefill_paged_decode.py:72-79


def test_decode_vanilla_requests_and_fp32_table():
    print("case: decode is_lazy mix, fp32 table", flush=True)
    w = _decode_batch("block_uniform", table_f32=True)
    lazy = torch.tensor([True, False, True, False, True])
    ref = _oracle(w, lazy)
    got = _run(w, lazy=lazy, num_splits=2)
    assert _err(got, ref) < 2e-2, _err(got, ref)


@pytest.mark.parametrize("hq,hkv", [(4, 4), (16, 2), (32, 2), (3, 1), (28, 4), (24, 2), (64, 1), (40, 2), (34, 2)])
def test_decode_group_sizes(hq, hkv):
    print(f"case: decode group {hq // hkv}", flush=True)
    w = _decode_batch("natural", hq=hq, hkv=hkv)
    ref = _oracle(w)
    for nsplit in (0, 1, 3):
        got = _run(w, num_splits=nsplit, kernel=_ffi.KERNEL_MFMA)      # groups above 16: blocks of 16 heads
        assert _err(got, ref) < 2e-2, (nsplit, _err(got, ref))


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("dtype,kv,d", [(torch.bfloat16, "auto", 128), (torch.float16, "fp8", 128), (torch.bfloat16, "auto", 64)])
def test_decode_pages_of_32_slots(variant, dtype, kv, d):
    """Cache pages of 32 slots (the page size of the reference's kernel test, tests/kernels/test_prefix_prefill.py:86):
    read as two parts of 16; pads at the end of a document span parts."""
    print(f"case: decode pages of 32 {variant} {dtype} kv={kv} d={d}", flush=True)
    w = _decode_batch(variant, dtype=dtype, kv=kv, d=d, bs=32)
    lazy = torch.tensor([True, False, True, True, True]) if variant == "block_uniform" else None
    ref = _oracle(w, lazy)
    for nsplit in (0, 1, 3):
        got = _run(w, lazy=lazy, num_splits=nsplit, kernel=_ffi.KERNEL_MFMA)
        assert _err(got, ref) < (5e-2 if kv == "fp8" else 2e-2), (nsplit, _err(got, ref))
    ref = _oracle(w, lazy, sliding_window=20)
    got = _run(w, lazy=lazy, sliding_window=20, kernel=_ffi.KERNEL_MFMA)
    assert _err(got, ref) < (5e-2 if kv == "fp8" else 2e-2), _err(got, ref)


@pytest.mark.parametrize("d", [96, 80, 112, 48, 16])
@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("dtype,kv,page", [(torch.bfloat16, "auto", 16), (torch.float16, "auto", 32), (torch.bfloat16, "fp8", 16)])
def test_decode_head_sizes_padded_to_128(d, variant, dtype, kv, page):
    """Head sizes that are multiples of 16 below 128 run the 128-wide kernel with the lane's chunks, the query and
    the V rows zero-padded; forcing the fast kernel fails if it does not take them."""
    print(f"case: decode head size {d} {variant} {dtype} kv={kv} page={page}", flush=True)
    w = _decode_batch(variant, dtype=dtype, kv=kv, d=d, bs=page, seed=d)
    lazy = torch.tensor([True, False, True, True, True]) if variant == "block_uniform" else None
    for window in (0, 20):
        ref = _oracle(w, lazy, sliding_window=window)
        for nsplit in (0, 1, 3):
            got = _run(w, lazy=lazy, num_splits=nsplit, sliding_window=window, kernel=_ffi.KERNEL_MFMA)
            assert _err(got, ref) < (5e-2 if kv == "fp8" else 2e-2), (window, nsplit, _err(got, ref))


@pytest.mark.parametrize("d,page", [(128, 16), (64, 32), (96, 16)])
@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decode_fp8_e5m2_cache(d, page, variant, dtype):
    """kv_cache_dtype "fp8_e5m2" (ops/chunked_prefill_paged_decode.py:123-124) on the fast kernel: the e4m3 bytes of
    the batch read as e5m2, exponents kept below inf/NaN; outputs reach 14, so one unit in the last place is allowed."""
    print(f"case: decode fp8_e5m2 d={d} page={page} {variant} {dtype}", flush=True)
    w = _decode_batch(variant, dtype=dtype, kv="fp8", d=d, bs=page, seed=d)
    w.kv_cache_dtype = "fp8_e5m2"
    w.k_cache &= 0x7B
    w.v_cache &= 0x7B
    w.k_scale = torch.tensor(2.0 ** -12)
    w.v_scale = torch.tensor(2.0 ** -12)
    lazy = torch.tensor([True, False, True, True, True]) if variant == "block_uniform" else None
    ref = _oracle(w, lazy).float()
    for nsplit in (0, 1, 3):
        got = _run(w, lazy=lazy, num_splits=nsplit, kernel=_ffi.KERNEL_MFMA).float()
        e = ((got.cpu() - ref).abs() - 2.0 ** -7 * ref.abs()).clamp(min=0).max().item()
        assert e < 5e-2, (nsplit, e)


@pytest.mark.parametrize("variant,table_f32", [("natural", False), ("block_uniform", True)])
def test_decode_fp8_cache(variant, table_f32):
    print(f"case: decode fp8 {variant} table_f32={table_f32}", flush=True)
    w = _decode_batch(variant, kv="fp8", table_f32=table_f32)
    ref = _oracle(w)
    got = _run(w, num_splits=3)
    assert _err(got, ref) < 5e-2, _err(got, ref)
    same = _run(w, kernel=_ffi.KERNEL_GENERIC)
    assert _err(got, same) < 2e-2, _err(got, same)


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("kv", ["auto", "fp8"])
def test_decode_float16_operands(variant, kv):
    print(f"case: decode float16 {variant} kv={kv}", flush=True)
    w = _decode_batch(variant, kv=kv, dtype=torch.float16)
    ref = _oracle(w)
    for nsplit in (1, 3):
        got = _run(w, num_splits=nsplit)
        assert got.dtype == torch.float16
        assert _err(got, ref) < (5e-2 if kv == "fp8" else 5e-3), (nsplit, _err(got, ref))
    same = _run(w, kernel=_ffi.KERNEL_GENERIC)
    assert _err(got, same) < (2e-2 if kv == "fp8" else 5e-3), _err(got, same)


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("window", [3, 20, 100, 4096])
def test_decode_sliding_window(variant, window):
    print(f"case: decode sliding window {window} {variant}", flush=True)
    w = _decode_batch(variant)
    ref = _oracle(w, sliding_window=window)
    for nsplit in (1, 3):
        got = _run(w, num_splits=nsplit, sliding_window=window)
        assert _err(got, ref) < 2e-2, (nsplit, _err(got, ref))
    same = _run(w, kernel=_ffi.KERNEL_GENERIC, sliding_window=window)
    assert _err(got, same) < 2e-2, _err(got, same)


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("dtype,kv", [(torch.bfloat16, "auto"), (torch.float16, "auto"), (torch.bfloat16, "fp8")])
def test_decode_head_dim_64(variant, dtype, kv):
    print(f"case: decode head_dim 64 {variant} {dtype} kv={kv}", flush=True)
    w = _decode_batch(variant, hq=16, hkv=4, kv=kv, dtype=dtype, d=64)
    ref = _oracle(w)
    tol = 5e-2 if kv == "fp8" else (2e-2 if dtype == torch.bfloat16 else 5e-3)
    for nsplit in (1, 3):
        got = _run(w, num_splits=nsplit)
        assert _err(got, ref) < tol, (nsplit, _err(got, ref))
    same = _run(w, kernel=_ffi.KERNEL_GENERIC)
    assert _err(got, same) < 2e-2, _err(got, same)


def test_decode_pad_slots_may_hold_nan():
    print("case: decode NaN pad", flush=True)
    w = _decode_batch("natural")
    ref = _oracle(w)
    for b in range(5):
        for j in range(w.block_table.shape[1]):
            m = int(w.q_mask[b, j])
            if m:
                pb = int(w.block_table[b, j])
                w.k_cache[pb, :, :, 16 - m:, :] = float("nan")
                w.v_cache[pb, :, :, 16 - m:] = float("nan")
    got = _run(w, num_splits=2)
    assert _err(got, ref) < 2e-2, _err(got, ref)


def test_decode_entry_points_long_context():
    """Both entry points at a serving-like size: 8 requests x 2 K keys, Llama-3-8B geometry."""
    print("case: decode entry points 8 x 2K", flush=True)
    g0 = torch.Generator().manual_seed(3)
    for variant, entry in (("natural", entry_unrotated), ("block_uniform", entry_block_uniform)):
        reqs = [torch.randperm(16, generator=g0)[:8].tolist() for _ in range(8)]
        w = wl.make_workload("dec8", dtype=torch.bfloat16, **wl.LLAMA_8B, block_size=16, doc_lens=[250] * 16,
                             requests=reqs, q_lens=[1] * 8, variant=variant, seed=9)
        x = w.k_cache.shape[4]
        for b in range(8):
            qs = int(w.b_start_loc[b]); n = int(w.b_seq_len[b]) - 1
            pb = int(w.block_table[b, n // 16])
            w.k_cache[pb, :, :, n % 16, :] = w.k[qs].view(8, 128 // x, x)
            w.v_cache[pb, :, :, n % 16] = w.v[qs]
        ref = _oracle(w)
        g = w.to(DEV)
        out = torch.full_like(g.q, 5.0)
        if variant == "natural":
            entry(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                  g.max_seq_len, 1, g.k_scale, g.v_scale, sm_scale=128 ** -0.5, rotary_dim=128,
                  cos_sin_cache=g.cos_sin_cache, q_mask=g.q_mask)
        else:
            entry(g.q, g.k, g.v, out, "auto", g.k_cache, g.v_cache, g.block_table, g.b_start_loc, g.b_seq_len,
                  g.max_seq_len, 1, g.k_scale, g.v_scale, sm_scale=128 ** -0.5, rotary_dim=128,
                  cos_sin_cache=g.cos_sin_cache, is_lazy=g.is_lazy, q_offset=g.q_offset, q_mask=g.q_mask)
        assert _err(out.cpu(), ref) < 2e-2, (variant, _err(out.cpu(), ref))


def _with_zero_offsets(w):
    """Entries of the offset table set to 0 where the reference's page walk then keeps the previous page's rotation:
    the second and later pages of documents (rotated like their first page)."""
    qo = w.q_offset.clone()
    for b in range(qo.shape[0]):
        row = qo[b].tolist()
        for j in range(1, len(row)):
            if row[j] == row[j - 1] and row[j] > 1 and j % 3:
                qo[b, j] = 0
        # (row[] keeps the original values, so runs longer than two pages get several zeros)
    assert (qo != w.q_offset).any()
    return qo


@pytest.mark.parametrize("nsplit", [1, 5])
@pytest.mark.parametrize("kernel,dtype,d", [(_ffi.KERNEL_AUTO, torch.bfloat16, 128), (_ffi.KERNEL_GENERIC, torch.float32, 64)])
def test_decode_zero_offset_keeps_previous_rotation(kernel, dtype, d, nsplit):
    """ops/models/llama_v1.py:207-262: the query is re-rotated only when a page's offset differs from the previous
    page's, and an offset of 0 does nothing -- such a page is rotated like the one before it.  With the page axis
    cut into slices a slice may start on such a page and has to look back for the offset in force."""
    print(f"case: decode offset-0 carry kernel={kernel} {dtype} nsplit={nsplit}", flush=True)
    w = _decode_batch("block_uniform", dtype=dtype, d=d)
    same = _oracle(w)
    w.q_offset = _with_zero_offsets(w)
    ref = _oracle(w)
    assert _err(ref, same) < 1e-6                      # zeros inside a document change nothing ...
    got = _run(w, num_splits=nsplit, kernel=kernel)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert _err(got, ref) < tol, _err(got, ref)
    w.q_offset[:, 0] = 0                              # ... and before the first non-zero entry there is no rotation
    ref0 = _oracle(w)
    assert _err(ref0, ref) > 1e-3
    got = _run(w, num_splits=nsplit, kernel=kernel)
    assert _err(got, ref0) < tol, _err(got, ref0)


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("bs", [16, 32])
def test_decode_reads_the_packed_table(variant, bs):
    """The int64 table of ops/models/llama_v1.py:157-160 read in place (one 8-byte entry per page): same result as
    with the three int32 tables, which hold junk here."""
    print(f"case: decode packed table {variant} page={bs}", flush=True)
    w = _decode_batch(variant, bs=bs)
    if variant == "block_uniform":
        w.q_offset = _with_zero_offsets(w)
    ref = _oracle(w)
    for nsplit in (1, 4):
        got = _run(w, num_splits=nsplit, packed=True)
        assert _err(got, ref) < 2e-2, (nsplit, _err(got, ref))


@pytest.mark.parametrize("variant", ["natural", "block_uniform"])
@pytest.mark.parametrize("llama3", [False, True])
@pytest.mark.parametrize("dtype,d,kv", [(torch.bfloat16, 128, "auto"), (torch.float16, 64, "auto"), (torch.bfloat16, 96, "fp8")])
def test_decode_computed_cos_sin(variant, llama3, dtype, d, kv):
    """cos/sin computed in the kernel from the inverse frequencies (rope_freqs / rope_cos_sin_from_freqs,
    model_executor/rope/cos_sin.py:24-66; the reference's COMPUTE_COS_SIN switch) against the oracle reading a
    table built in float64: plain and Llama-3-smoothed frequencies."""
    from lazy_amd.model_executor.rope import cos_sin as rope_cs
    print(f"case: decode computed cos/sin {variant} llama3={llama3} {dtype} d={d} kv={kv}", flush=True)
    l3 = dict(scaling_factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, orig_max_position=8192) if llama3 else None
    w = wl.make_workload("cdec", dtype=dtype, hq=8, hkv=2, d=d, theta=500000.0, block_size=16,
                         doc_lens=[40, 16, 333, 700, 5, 128, 97], requests=[[3, 1, 0], [2], [0, 2, 3, 1, 5, 6, 4, 5, 6], [4, 0]],
                         q_lens=[1, 1, 1, 1], variant=variant, seed=5, kv_cache_dtype=kv, llama3=l3)
    x = w.k_cache.shape[4]
    for b in range(4):
        n = int(w.b_seq_len[b]) - 1
        pb = int(w.block_table[b, n // 16]); qs = int(w.b_start_loc[b])
        enc = (lambda t, sc: (t.float() / sc).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)) if kv == "fp8" else (lambda t, sc: t)
        w.k_cache[pb, :, :, n % 16, :] = enc(w.k[qs], w.k_scale).view(2, d // x, x)
        w.v_cache[pb, :, :, n % 16] = enc(w.v[qs], w.v_scale)
    ref = _oracle(w)
    meta = dict(ROPE_TYPE=1, BASE=500000.0, SCALING_FACTOR=8.0, LOW_FACTOR=1.0, HIGH_FACTOR=4.0, ORIG_MAX_POSITION=8192) \
        if llama3 else dict(ROPE_TYPE=0, BASE=500000.0)
    freqs = rope_cs.rope_freqs(meta, d, DEV)
    tol = 5e-2 if kv == "fp8" else (5e-3 if dtype == torch.float16 else 2e-2)
    for nsplit in (1, 3):
        got = _run(w, num_splits=nsplit, freqs=freqs)
        assert _err(got, ref) < tol, (nsplit, _err(got, ref))


def test_computed_cos_sin_at_long_positions():
    """Positions in the tens of thousands (the long-context configuration reaches 65 791): the angle is reduced to one
    revolution from an exact product, so the computed values agree with a float64 table to the table's own rounding."""
    from lazy_amd.model_executor.rope import cos_sin as rope_cs
    print("case: decode computed cos/sin, positions to 66K", flush=True)
    w = wl.make_workload("cdecl", dtype=torch.bfloat16, hq=8, hkv=2, d=128, theta=500000.0, block_size=16,
                         doc_lens=[16] * 8, requests=[[0, 1, 2, 3, 4, 5, 6, 7]], q_lens=[1], variant="block_uniform", seed=6)
    n = int(w.b_seq_len[0]) - 1
    pb = int(w.block_table[0, n // 16])
    w.k_cache[pb, :, :, n % 16, :] = w.k[0].view(2, 16, 8)
    w.v_cache[pb, :, :, n % 16] = w.v[0]
    # the eight documents are moved far out: offsets 65 000 + 100 i (+1 for the bias), table to match
    for i in range(8):
        w.q_offset[0, i] = 65001 + 100 * i
    w.cos_sin_cache = orc.build_cos_sin_table(66000, 128, 500000.0).to(torch.bfloat16)      # float64 angles
    ref = _oracle(w)
    got = _run(w, freqs=rope_cs.rope_freqs(dict(ROPE_TYPE=0, BASE=500000.0), 128, DEV))
    assert _err(got, ref) < 2e-2, _err(got, ref)
