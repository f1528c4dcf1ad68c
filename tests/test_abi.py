"""The C-ABI library loads and exports every symbol include/lazyattn.h declares, and the
host-side checks of the operators raise what the reference raises.  No GPU needed."""
import ctypes
import os
import re

import pytest
import torch

from lazy_amd import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "lazyattn.h")).read()
    return sorted(set(re.findall(r"\b(lazyattn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _ffi.lib()
    names = _declared()
    assert set(names) == set(_ffi.EXPORTS)
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.lazyattn_abi_version() == 3
    assert lib.lazyattn_error_string(-4).decode().startswith("request not supported")


def test_struct_layout_matches_header(tmp_path):
    """Compile the header with gcc and compare sizeof/offsetof with the ctypes mirror."""
    import subprocess
    fields = [n for n, _ in _ffi.PrefillParams._fields_]
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "lazyattn.h"\nint main(void){\n'
        + 'printf("%zu\\n", sizeof(lazyattn_prefill_params));\n'
        + "".join(f'printf("%zu\\n", offsetof(lazyattn_prefill_params, {f}));\n' for f in fields)
        + "return 0;}\n")
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    out = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert out[0] == ctypes.sizeof(_ffi.PrefillParams)
    assert out[1:] == [getattr(_ffi.PrefillParams, f).offset for f in fields]


def test_null_and_shape_errors_without_gpu():
    lib = _ffi.lib()
    p = _ffi.PrefillParams()
    assert lib.lazyattn_prefix_prefill(ctypes.byref(p), None) == -1
    assert lib.lazyattn_prefix_prefill(None, None) == -1
    assert lib.lazyattn_build_cos_sin_cache(None, 0, 8, 4, 8, 1e4, 0, 1.0, 1.0, 1.0, 8192, None) == -1
    assert lib.lazyattn_build_cos_sin_cache(1, 0, 8, 4, 7, 1e4, 0, 1.0, 1.0, 1.0, 8192, None) == -2


def _args(dtype=torch.float32, cache_dtype=None):
    q = torch.zeros(4, 4, 64, dtype=dtype); k = torch.zeros(4, 2, 64, dtype=dtype); v = k.clone()
    cd = cache_dtype or dtype
    kc = torch.zeros(8, 2, 16, 16, 4, dtype=cd); vc = torch.zeros(8, 2, 64, 16, dtype=cd)
    bt = torch.zeros(1, 4, dtype=torch.int32)
    return [q, k, v, torch.zeros_like(q), "auto", kc, vc, bt, torch.tensor([0, 4]), torch.tensor([20]),
            20, 4, torch.tensor(1.0), torch.tensor(1.0)]


def test_reference_error_behaviour():
    from lazy_amd.attention.old_ops.prefix_prefill import context_attention_fwd as f_old
    from lazy_amd.attention.ops.prefix_prefill import context_attention_fwd as f_new
    tab = torch.zeros(64, 64)
    a = _args()
    with pytest.raises(NotImplementedError):                   # ops/prefix_prefill.py:673-674
        f_old(*a, alibi_slopes=torch.zeros(4), cos_sin_cache=tab, rotary_dim=64)
    a = _args(); a[4] = "fp8"
    with pytest.raises(AssertionError):                        # ops/prefix_prefill.py:637-639
        f_old(*a, cos_sin_cache=tab, rotary_dim=64)
    a = _args(cache_dtype=torch.uint8); a[4] = "fp8_e3m4"
    with pytest.raises(ValueError, match="Unsupported FP8"):   # ops/prefix_prefill.py:646
        f_new(*a, cos_sin_cache=tab, rotary_dim=64, is_lazy=torch.ones(1, dtype=torch.bool),
              q_offset=torch.zeros(1, 4, dtype=torch.int32))
    a = _args(cache_dtype=torch.uint8)
    with pytest.raises(ValueError, match="auto"):              # ops/prefix_prefill.py:651-654
        f_old(*a, cos_sin_cache=tab, rotary_dim=64)
    a = _args(); a[8] = torch.tensor([0, 4, 8])
    with pytest.raises(AssertionError):                        # ops/prefix_prefill.py:667
        f_old(*a, cos_sin_cache=tab, rotary_dim=64)
    a = _args(); a[2] = torch.zeros(4, 2, 32)
    with pytest.raises(AssertionError):                        # ops/prefix_prefill.py:657-658
        f_old(*a, cos_sin_cache=tab, rotary_dim=64)
    with pytest.raises(RuntimeError, match="GPU only"):        # no CPU path
        f_old(*_args(), cos_sin_cache=tab, rotary_dim=64)


def test_metadata_producer_known_answer():
    from lazy_amd.core.sched.metadata import (metadata_for_lazy_attention, metadata_for_mepic,
                                              max_rotation_offset)
    # lazy_attn/tests/core/test_scheduler.py:49-61
    assert metadata_for_lazy_attention([6, 15, 8, 2], [8, 16, 8, 8], 8) == (
        [10, 16, 16, 31, 39, 1], [2, 0, 1, 0, 6, 0])
    assert metadata_for_mepic([6, 15, 8, 2], [8, 16, 8, 8], 8) == ([0] * 6, [2, 0, 1, 0, 6, 0])
    # lazy_attn/tests/core/test_rotation_offset_bound.py:47-75
    assert max_rotation_offset([1024] * 64, [1024] * 64) == 1024 * 63 + 1
    assert max_rotation_offset([1] * 8, [16] * 8) == 8 * 15 + 7 + 1
    for lens in ([6], [16, 16], [6, 15, 8, 2], [1] * 5, [4096, 17], [100] * 32):
        padded = [((n + 15) // 16) * 16 for n in lens]
        assert max_rotation_offset(lens, padded) == max(metadata_for_lazy_attention(lens, padded, 16)[0])


def test_unpack_block_table_layout():
    from lazy_amd.attention.ops.chunked_prefill_paged_decode import unpack_block_table
    packed = torch.tensor([[(6 << 32) | (0xFFFF << 16) | 3, (123456 << 32) | (1 << 16)]], dtype=torch.int64)
    blk, off, msk = unpack_block_table(packed)
    assert blk.tolist() == [[6, 123456]] and off.tolist() == [[0xFFFF, 1]] and msk.tolist() == [[3, 0]]
    # lazy_attn/tests/worker/test_q_offset_range.py:71-79: one past the limit carries into the block
    over = (6 << 32) | ((0xFFFF + 1) << 16)
    blk, off, _ = unpack_block_table(torch.tensor([[over]], dtype=torch.int64))
    assert blk.item() == 7 and off.item() == 0


def test_table_version_of_inference_tensors():
    """A table made under torch.inference_mode() has no edit counter (reading it raises): the cache of
    re-laid-out tables keys such a table on its address and shape only."""
    with torch.inference_mode():
        t = torch.zeros(32, 16).to(torch.bfloat16)
    assert t.is_inference() and _ffi.table_version(t) is None
    u = torch.zeros(32, 16)
    v0 = _ffi.table_version(u)
    u.add_(1)
    assert _ffi.table_version(u) == v0 + 1


@pytest.mark.parametrize("compiled", [True, False])
def test_remembered_calls_keying_and_invalidation(compiled, monkeypatch):
    """Host logic of the entry points' call memory: the key tells apart views of one buffer that differ in shape,
    strides or dtype; a remembered call is dropped when the cos/sin table it was made for has been edited in place,
    and all of them when the re-laid-out tables are invalidated by hand.  Both forms of the key: the compiled
    helper (csrc/host/callkey.cpp) and the Python tuple used when it is not built."""
    from lazy_amd.attention import _launch
    if compiled:
        assert _launch._tensor_key is not None, "lazy_amd/_lib/_callkey.so is not built (python lazy-attention_amd/build.py)"
    else:
        monkeypatch.setattr(_launch, "_tensor_key", None)
    base = torch.zeros(8, 16)
    scalar = torch.tensor(3.0)                            # zero-dimensional
    assert _launch.call_key("t", (base, None, scalar), ()) == _launch.call_key("t", (base, None, scalar), ())
    assert _launch.call_key("t", (base, None), ()) != _launch.call_key("t", (None, base), ())
    assert _launch.call_key("t", (base,), ()) != _launch.call_key("t", (base[1:],), ())             # other address
    assert _launch.call_key("t", (base[:4], base), ()) != _launch.call_key("t", (base, base[:4]), ())
    # the first dimension of chosen tensors left open (views [:n] of one buffer share a key)
    assert _launch.call_key("t", (base[:4], base), (), 0b01) == _launch.call_key("t", (base[:6], base), (), 0b01)
    assert _launch.call_key("t", (base[:4], base), (), 0b10) != _launch.call_key("t", (base[:6], base), (), 0b10)
    assert _launch.call_key("t", (base[:, :4],), (), 0b1) != _launch.call_key("t", (base[:, :6],), (), 0b1)
    assert _launch.call_key("t", (base[:4],), (), 0b1) != _launch.call_key("t", (base[:4],), (), 0)
    with torch.inference_mode():
        inf = torch.zeros(8, 16)
    assert _launch.call_key("t", (inf,), ()) == _launch.call_key("t", (inf,), ())
    with pytest.raises((TypeError, AttributeError)):
        _launch.call_key("t", (1.0,), ())
    k0 = _launch.call_key("t", (base, None), (1, 2.0, None))
    assert k0 == _launch.call_key("t", (base, None), (1, 2.0, None))
    assert k0 != _launch.call_key("t", (base.t(), None), (1, 2.0, None))            # same address, other strides
    assert k0 != _launch.call_key("t", (base[:4], None), (1, 2.0, None))            # same address, other shape
    assert k0 != _launch.call_key("t", (base.view(torch.int32), None), (1, 2.0, None))
    assert k0 != _launch.call_key("t", (base, None), (1, 2.5, None))
    assert k0 != _launch.call_key("u", (base, None), (1, 2.0, None))

    class Plan:                                       # stands in for a validated call
        repeatable = True
        count_sized = False
        def detached(self): return self
    _launch.forget_calls()
    table = torch.ones(4, 16)
    _launch.remember(k0, (Plan(),), table)
    assert _launch.recall(k0, table) is not None
    table.mul_(2.0)                                   # in-place edit: the plans point at a copy of the old contents
    assert _launch.recall(k0, table) is None and len(_launch._calls) == 0
    unrepeatable = Plan(); unrepeatable.repeatable = False
    _launch.remember(k0, (Plan(), unrepeatable), table)
    assert len(_launch._calls) == 0                   # a call with a converted operand is validated every time
    _launch.remember(k0, (Plan(),), table)
    _ffi.invalidate_packed_tables()
    assert len(_launch._calls) == 0
    # counts left out of the key are written into the remembered plans; a plan whose workspace is too small for
    # them is dropped; a plan that owns batch-sized tensors only serves the batch it was made for
    class Sized(Plan):
        def __init__(self): self.seen, self.fits = None, True
        def resize(self, *counts): self.seen = counts; return self.fits
    sp = Sized()
    _launch.remember(k0, (sp,), None, (4, 80, 100, 70))
    assert _launch.recall(k0, None, (4, 80, 100, 70)) is not None and sp.seen is None        # same counts: nothing to set
    assert _launch.recall(k0, None, (2, 71, 90, 70)) is not None and sp.seen == (2, 71, 90, 70)
    sp.fits = False
    assert _launch.recall(k0, None, (3, 80, 95, 70)) is None and len(_launch._calls) == 0
    sp.fits, sp.count_sized = True, True
    _launch.remember(k0, (sp,), None, (4, 80, 100, 70), bound=(4, 4))
    assert _launch.recall(k0, None, (2, 71, 90, 70), bound=(2, 2)) is None and len(_launch._calls) == 1
    assert _launch.recall(k0, None, (4, 71, 90, 70), bound=(4, 4)) is not None
    _launch.forget_calls()
    for i in range(_launch._CALLS_MAX + 5):           # bounded: the oldest entries leave
        _launch.remember(("k", i), (Plan(),), None)
    assert len(_launch._calls) == _launch._CALLS_MAX and _launch.recall(("k", 0), None) is None
    _launch.forget_calls()


def test_fast_division_is_exact(tmp_path):
    """csrc/fastdiv.hpp (the kernel prologue's divisions by launch-time constants): the multiply-high form equals
    n / d for divisors from 1 to 2^32 - 1 and numerators over the whole 32-bit range, edges included."""
    import subprocess
    src = tmp_path / "fd.cpp"
    src.write_text('''
#include "fastdiv.hpp"
#include <cstdio>
int main() {
    using lazyattn::FastDiv;
    unsigned long long bad = 0;
    const uint32_t ds[] = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 1000, 4096,
                           65535, 65536, 65537, 1000003, 0x7fffffffu, 0x80000000u, 0xfffffffeu, 0xffffffffu};
    for (uint32_t d : ds) {
        const FastDiv f(d);
        for (uint64_t i = 0; i < 400000; ++i) {
            uint32_t n = (uint32_t)(i * 2654435761ull + i * i);
            if (i < 100000) n = (uint32_t)i;
            if (i > 300000) n = 0xffffffffu - (uint32_t)(i - 300000);
            const uint32_t q = f.quot(n);
            if (q != n / d || f.rem(n, q) != n % d) ++bad;
        }
    }
    printf("%llu\\n", bad);
    return bad != 0;
}
''')
    exe = tmp_path / "fd"
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "lazy-attention_amd", "csrc"), str(src), "-o", str(exe)])
    assert subprocess.check_output([str(exe)]).split()[0] == b"0"


def test_env_switches_take_the_reference_truthy_values(monkeypatch):
    """lazy_attn/lazy/utils/variants.py:63-68: only 1 / true / yes / on (any case, stripped) switch something on."""
    from lazy_amd.attention.ops.chunked_prefill_paged_decode import _env_flag
    for value, want in (("1", True), (" True ", True), ("YES", True), ("on", True), ("0", False), ("false", False),
                        ("off", False), ("", False), ("2", False)):
        monkeypatch.setenv("NO_LAZY", value)
        assert _env_flag("NO_LAZY") is want, value
    monkeypatch.delenv("NO_LAZY")
    assert _env_flag("NO_LAZY") is False


def _fake_params(dtype=_ffi.BF16, head_dim=128, block_size=16, tokens=128, seq=5248, kernel=_ffi.KERNEL_AUTO):
    """A parameter block with made-up (aligned, never dereferenced) addresses, for the host-side queries."""
    p = _ffi.PrefillParams()
    for i, n in enumerate(("q", "k", "v", "o", "k_cache", "v_cache", "block_table", "b_start_loc", "b_seq_len",
                           "cos_sin_cache")):
        setattr(p, n, 0x10000 * (i + 1))
    p.batch, p.num_q_heads, p.num_kv_heads, p.head_dim, p.rotary_dim = 1, 32, 8, head_dim, head_dim
    p.block_size, p.x = block_size, 8 if dtype != _ffi.F32 else 4
    p.dtype = p.cache_dtype = p.table_dtype = dtype
    p.index_bits, p.max_q_len, p.num_tokens, p.max_seq_len, p.kernel = 32, tokens, tokens, seq, kernel
    for n, st in (("q_stride", (32 * head_dim, head_dim, 1)), ("o_stride", (32 * head_dim, head_dim, 1)),
                  ("k_stride", (8 * head_dim, head_dim, 1)), ("v_stride", (8 * head_dim, head_dim, 1)),
                  ("kc_stride", (8 * head_dim * block_size, head_dim * block_size, block_size * p.x, p.x, 1)),
                  ("vc_stride", (8 * head_dim * block_size, head_dim * block_size, block_size, 1))):
        getattr(p, n)[:] = st
    p.bt_stride[:] = (512, 1)
    p.table_stride = head_dim
    return p


def test_kernel_query_names_the_kernel_and_the_reason_for_the_fallback():
    lib = _ffi.lib()
    splits, why = ctypes.c_int32(0), ctypes.c_char_p()
    p = _fake_params()
    k = lib.lazyattn_prefill_kernel_for(ctypes.byref(p), ctypes.byref(splits), ctypes.byref(why))
    assert k in (_ffi.KERNEL_MFMA4, _ffi.KERNEL_MFMA8) and splits.value >= 1 and why.value is None
    p = _fake_params(dtype=_ffi.F32)
    assert lib.lazyattn_prefill_kernel_for(ctypes.byref(p), None, ctypes.byref(why)) == _ffi.KERNEL_GENERIC
    assert b"bfloat16" in why.value
    p = _fake_params(head_dim=136)
    assert lib.lazyattn_prefill_kernel_for(ctypes.byref(p), None, ctypes.byref(why)) == _ffi.KERNEL_GENERIC
    assert b"head size" in why.value
    p = _fake_params(block_size=8)
    assert lib.lazyattn_prefill_kernel_for(ctypes.byref(p), None, ctypes.byref(why)) == _ffi.KERNEL_GENERIC
    assert b"pages" in why.value
    p = _fake_params(block_size=8, kernel=_ffi.KERNEL_MFMA)         # asked for, not available: what the call returns
    assert lib.lazyattn_prefill_kernel_for(ctypes.byref(p), None, ctypes.byref(why)) == _ffi.E_UNSUPPORTED
    p = _fake_params(); p.q = 0x10008
    assert lib.lazyattn_prefill_kernel_for(ctypes.byref(p), None, ctypes.byref(why)) == _ffi.KERNEL_GENERIC
    assert b"aligned" in why.value
    assert lib.lazyattn_prefill_kernel_for(None, None, None) == -1


def test_launch_shape_queries_for_batches():
    """What the host decides for a call with several requests, asked without a GPU (the CU count falls back to 256):
    the splits of a batch are left to the device (0) unless the caller fixes them; every batch needs a workspace
    (the device may split any request), sized for at most three rounds of the chip's compute units -- 96 work items per
    kv head, 4 or 8 waves of 32 partial rows of 128 halves + 2 floats each -- plus one 16-byte record per request; a
    caller's split count is sized by the bound on the batch's m-tiles; batches beyond 256 requests get one split count
    from the host, within a quarter of a GB."""
    lib = _ffi.lib()
    splits, why = ctypes.c_int32(-1), ctypes.c_char_p()
    row = 128 * 2 + 8

    def ask(batch, tokens, max_q, seq, num_splits=0, skip=0):
        p = _fake_params(tokens=tokens, seq=seq)
        p.batch, p.max_q_len, p.num_splits, p.skip_decode = batch, max_q, num_splits, skip
        k = lib.lazyattn_prefill_kernel_for(ctypes.byref(p), ctypes.byref(splits), ctypes.byref(why))
        return k, splits.value, lib.lazyattn_prefill_workspace_bytes(ctypes.byref(p))

    for batch, tokens, max_q in ((16, 1024, 64), (3, 384, 128), (8, 1024, 128), (6, 777, 400), (200, 328, 128)):
        k, s, ws = ask(batch, tokens, max_q, 5248)
        nw = 4 if k == _ffi.KERNEL_MFMA4 else 8
        assert k in (_ffi.KERNEL_MFMA4, _ffi.KERNEL_MFMA8) and s == 0, (batch, k, s)
        table = (batch * 16 + 255) // 256 * 256
        assert table < ws <= table + 8 * 96 * nw * 32 * row, (batch, ws)
        assert (ws - table) % (8 * nw * 32 * row) == 0
        k3, s3, ws3 = ask(batch, tokens, max_q, 5248, num_splits=3)
        assert s3 == 3 and ws3 > table
    # one request: the host's split count, a workspace only when it is split
    k, s, ws = ask(1, 128, 128, 5248)
    assert s >= 2 and ws == 8 * (128 // 32 * 4 // (4 if k == _ffi.KERNEL_MFMA4 else 8)) * s * (4 if k == _ffi.KERNEL_MFMA4 else 8) * 32 * row
    k, s, ws = ask(1, 128, 128, 5248, num_splits=1)
    assert s == 1 and ws == 0
    # a large serving batch: one split count for all, and a bounded workspace
    k, s, ws = ask(600, 728, 128, 5248, skip=1)
    assert s >= 1 and ws <= (256 << 20) + 600 * 16 + 256
