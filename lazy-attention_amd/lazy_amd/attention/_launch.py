"""Host side shared by the two operator variants: the reference's argument checks
(``lazy_attn/lazy/attention/ops/prefix_prefill.py:627-676``,
``old_ops/prefix_prefill.py:437-486``) and the hand-off to the C ABI."""
from __future__ import annotations

import ctypes
import warnings
from collections import OrderedDict
from typing import Optional

import torch

from .. import _ffi

# Repeat calls (a serving loop with fixed buffers, a benchmark) skip validation and the filling of the C struct:
# the entry points keep the plans of their most recent distinct calls, keyed on every tensor's address, shape,
# strides and dtype plus the scalar arguments.  A plan is a pure function of that key -- it holds no reference to
# the caller's tensors except the cos/sin table -- unless making it had to convert an operand (int64 tables, a host-side scale, a 0/1
# ``is_lazy``), whose copy depends on the operand's contents: such calls are validated every time.
# The backend's entry points (``chunked_prefill_paged_decode``) leave the counts that change from one engine step to
# the next out of the key -- the first dimension of the per-token and per-request tensors (views ``buf[:n]`` of
# persistent buffers share an address), ``max_seq_len``, ``max_query_len`` -- and write them into the remembered
# structs before the launch (``PrefillPlan.resize``): they are four fields there, and nothing else in a plan depends
# on them.  A plan that owns a tensor sized by such a count is bound to the counts it was made for.
_calls: "OrderedDict" = OrderedDict()
_CALLS_MAX = 256                            # (one per layer and kind of step of a served model)


def _load_tensor_key():
    """The compiled form of the per-tensor part of the key (csrc/host/callkey.cpp), or None when it is not built."""
    import importlib.util
    import os
    path = os.path.join(os.path.dirname(_ffi._LIB_PATH), "_callkey.so")
    if not os.path.exists(path):
        return None
    try:
        spec = importlib.util.spec_from_file_location("_callkey", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        return mod.tensor_key
    except (ImportError, OSError):
        return None


_tensor_key = _load_tensor_key()


def call_key(tag, tensors, scalars, open_dim0: int = 0):
    """``open_dim0``: bit i set = the first dimension of ``tensors[i]`` is not part of the key."""
    if _tensor_key is not None:
        return (tag, scalars, _tensor_key(tensors, open_dim0))      # 0.2 us for fifteen tensors; the tuple below takes 6
    return (tag, scalars, tuple([None if t is None else
                                 (t.data_ptr(), t.shape[1:] if (open_dim0 >> i) & 1 else t.shape, t.stride(), t.dtype)
                                 for i, t in enumerate(tensors)]))


def recall(key, table, counts=None, bound=None):
    """The plans remembered for this call, or None.  ``table`` is the caller's cos/sin table: its edit counter
    is compared because the plans point at a re-laid-out copy of it.  ``counts`` = (batch, num_tokens, max_seq_len,
    max_q_len) of this call when the key leaves them open: the plans are set to them (None when their workspace
    is too small for these counts).  ``bound``: what a plan that owns count-sized tensors must have been made for."""
    hit = _calls.get(key)
    if hit is None:
        return None
    if hit[0] != (None if table is None else _ffi.table_version(table)):
        del _calls[key]
        return None
    if hit[3] is not None and hit[3] != bound:
        return None
    if counts is not None and hit[4] != counts:
        for p in hit[1]:
            if not p.resize(*counts):
                del _calls[key]
                return None
        hit[4] = counts
    _calls.move_to_end(key)
    return hit[1]


def remember(key, plans, table, counts=None, bound=None) -> None:
    if not all(p.repeatable for p in plans):
        return
    while len(_calls) >= _CALLS_MAX:
        _calls.popitem(last=False)
    # (the entry holds the cos/sin table as well: the plans point at a re-laid-out copy of its contents, and while
    # the table lives its address cannot pass to another table that would then be taken for it)
    _calls[key] = [None if table is None else _ffi.table_version(table), tuple(p.detached() for p in plans), table,
                   bound if any(p.count_sized for p in plans) else None, counts]


def run_plans(plans) -> None:
    stream = torch._C._cuda_getCurrentRawStream(plans[0].device.index)
    for p in plans:
        p.run(stream)


def forget_calls() -> None:
    _calls.clear()


_ffi.on_workspace_growth(forget_calls)      # remembered plans point into the old buffer


_warned_generic = set()


def _warn_generic(reason: str) -> None:
    """Once per reason: a 16-bit call that the matrix-core kernels do not take runs the fp32 kernel, some hundred
    times slower, and nothing else would tell."""
    if reason in _warned_generic:
        return
    _warned_generic.add(reason)
    warnings.warn("lazy_amd: this prefix-prefill call runs the fp32 fallback kernel (about 100x slower than the "
                  f"matrix-core kernels): {reason}", RuntimeWarning, stacklevel=4)


def _cache_code(kv_cache_dtype: str, k_cache: torch.Tensor, v_cache: torch.Tensor, q_dtype) -> int:
    # ops/prefix_prefill.py:637-654
    if "fp8" in kv_cache_dtype:
        assert k_cache.dtype == torch.uint8
        assert v_cache.dtype == torch.uint8
        if kv_cache_dtype in ("fp8", "fp8_e4m3"):
            return _ffi.FP8_E4M3
        if kv_cache_dtype == "fp8_e5m2":
            return _ffi.FP8_E5M2
        raise ValueError("Unsupported FP8 dtype:", kv_cache_dtype)
    if k_cache.dtype == torch.uint8 or v_cache.dtype == torch.uint8:
        raise ValueError("kv_cache_dtype='auto' unsupported for FP8 KV Cache prefill kernel")
    if k_cache.dtype != q_dtype or v_cache.dtype != q_dtype:
        raise TypeError(f"cache dtype {k_cache.dtype} does not match query dtype {q_dtype}")
    return _ffi.dtype_code(q_dtype)


def _i32(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None or t.dtype == torch.int32:
        return t
    return t.to(torch.int32)


def _require_gpu(*tensors) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError("lazy_amd operators run on the GPU only (got a tensor on "
                           f"'{dev}'); there is no CPU path")
    for t in tensors:
        if t is not None and t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} vs {t.device}")
    return dev


def launch_prefill(*, q, k, v, o, kv_cache_dtype, k_cache, v_cache, b_loc, b_start_loc, b_seq_len,
                   max_input_len, max_seq_len=0, k_scale, v_scale, alibi_slopes, sliding_window, sm_scale,
                   skip_decode, cos_sin_cache, rotary_dim, is_neox_style, is_lazy, q_offset, q_mask,
                   pos_mode: int, rotate_new_k: bool, fp32_rotary: bool = False,
                   kernel: int = _ffi.KERNEL_AUTO, num_splits: int = 0,
                   phases: int = _ffi.PHASE_ALL, decode: bool = False, packed_block_table=None, rope_freqs=None,
                   _return_plan: bool = False):
    lib = _ffi.lib()
    cache_code = _cache_code(kv_cache_dtype, k_cache, v_cache, q.dtype)
    if not decode:
        Lq, Lk, Lv = q.shape[-1], k.shape[-1], v.shape[-1]
        assert Lq == Lk and Lk == Lv                                   # ops/prefix_prefill.py:657-658
    else:
        Lq = q.shape[-1]
    if sm_scale is None:
        sm_scale = 1.0 / (Lq ** 0.5)
    batch = b_seq_len.shape[0]
    assert batch + 1 == len(b_start_loc)                               # ops/prefix_prefill.py:667
    if sliding_window is None or sliding_window <= 0:
        sliding_window = 0
    if alibi_slopes is not None:
        raise NotImplementedError("Alibi slopes are not implemented for prefix prefill")
    if not is_neox_style:
        raise NotImplementedError("only NeoX-style rotary embedding is supported")
    dev = _require_gpu(q, k, v, o, k_cache, v_cache, b_loc, b_start_loc, b_seq_len,
                       cos_sin_cache, q_offset, q_mask, is_lazy, packed_block_table, rope_freqs)
    if rotary_dim is None:
        rotary_dim = cos_sin_cache.shape[-1] if cos_sin_cache is not None else Lq
    if rope_freqs is not None:
        # q_len == 1 rows with cos/sin computed from the inverse frequencies: the table is not read
        assert decode and rope_freqs.dtype == torch.float32 and rope_freqs.is_contiguous()
        assert rope_freqs.numel() * 2 == rotary_dim
    elif cos_sin_cache is None:
        raise ValueError("cos_sin_cache is required")
    if packed_block_table is not None:
        assert decode and packed_block_table.dtype == torch.int64
    given = (b_seq_len, is_lazy, k_scale, v_scale, b_loc, q_offset, q_mask)
    if b_start_loc.dtype != b_seq_len.dtype:
        b_seq_len = b_seq_len.to(b_start_loc.dtype)
    if b_start_loc.dtype not in (torch.int32, torch.int64):
        raise TypeError("b_start_loc / b_seq_len must be int32 or int64")
    if is_lazy is not None and is_lazy.dtype != torch.bool and is_lazy.dtype != torch.uint8:
        is_lazy = is_lazy != 0
    if cache_code in (_ffi.FP8_E4M3, _ffi.FP8_E5M2):
        k_scale = k_scale.to(device=dev, dtype=torch.float32) if (
            k_scale.device != dev or k_scale.dtype != torch.float32) else k_scale
        v_scale = v_scale.to(device=dev, dtype=torch.float32) if (
            v_scale.device != dev or v_scale.dtype != torch.float32) else v_scale
    else:
        k_scale = v_scale = None
    b_loc, q_offset, q_mask = _i32(b_loc), _i32(q_offset), _i32(q_mask)
    if cache_code not in (_ffi.FP8_E4M3, _ffi.FP8_E5M2):
        given = given[:2] + (None, None) + given[4:]
    repeatable = all(a is b for a, b in zip(given, (b_seq_len, is_lazy, k_scale, v_scale, b_loc, q_offset, q_mask)))
    packed = None
    if not decode and q.dtype in (torch.bfloat16, torch.float16) and pos_mode != _ffi.POS_BLOCK_UNIFORM:
        packed = _ffi.packed_cos_sin(cos_sin_cache)      # built once per table
    p = _ffi.fill_params(
        q=q, k=k, v=v, o=o, k_cache=k_cache, v_cache=v_cache, block_table=b_loc,
        b_start_loc=b_start_loc, b_seq_len=b_seq_len, cos_sin_cache=cos_sin_cache,
        k_scale=k_scale, v_scale=v_scale, q_offset=q_offset, q_mask=q_mask,
        is_lazy=is_lazy, cache_code=cache_code, max_q_len=max_input_len, rotary_dim=rotary_dim,
        sliding_window=sliding_window, sm_scale=sm_scale, pos_mode=pos_mode,
        rotate_new_k=rotate_new_k, skip_decode=skip_decode, fp32_rotary=fp32_rotary,
        kernel=kernel, num_splits=num_splits, phases=phases, max_seq_len=max_seq_len, packed_table=packed,
        packed_block_table=packed_block_table, rope_freqs=rope_freqs)
    if not decode and kernel == _ffi.KERNEL_AUTO and q.dtype in (torch.bfloat16, torch.float16):
        why = ctypes.c_char_p()
        if lib.lazyattn_prefill_kernel_for(p, None, ctypes.byref(why)) == _ffi.KERNEL_GENERIC and why.value:
            _warn_generic(why.value.decode())
    plan = PrefillPlan(p, dev, decode, keep=(q, k, v, o, k_cache, v_cache, b_loc, b_start_loc, b_seq_len,
                                            cos_sin_cache, q_offset, q_mask, is_lazy, k_scale, v_scale,
                                            packed_block_table, rope_freqs), own=(packed,), repeatable=repeatable)
    if _return_plan:
        return plan
    plan.run()


class PrefillPlan:
    """A validated call: the filled C struct plus references that keep its tensors alive.
    ``run()`` enqueues it on torch's current stream; calling it again repeats the call
    on the same operands (a serving loop re-uses the plan while shapes stay fixed)."""

    def __init__(self, params, device, decode, keep, own=(), repeatable=False):
        self.params, self.device, self.decode, self._keep, self._own = params, device, decode, keep, own
        self.repeatable = repeatable        # no operand had to be converted: the struct depends on the key alone
        self.count_sized = False            # owns tensors sized by the batch (made by the entry point for this call)
        self._lib = _ffi.lib()
        self._entry = self._lib.lazyattn_paged_decode_rotary if decode else self._lib.lazyattn_prefix_prefill
        self._ws = None
        nbytes = (self._lib.lazyattn_paged_decode_workspace_bytes(params) if decode
                  else self._lib.lazyattn_prefill_workspace_bytes(params))
        self._ws = _ffi.workspace(device, nbytes, "decode" if decode else "prefill")
        if self._ws is not None:
            params.workspace = self._ws.data_ptr()
            params.workspace_bytes = self._ws.numel()

    def run(self, stream: Optional[int] = None) -> None:
        if stream is None:
            stream = torch._C._cuda_getCurrentRawStream(self.device.index)
        rc = self._entry(self.params, stream)
        if rc:
            _ffi.check(rc, "lazyattn_paged_decode_rotary" if self.decode else "lazyattn_prefix_prefill")

    def kernel(self):
        """(LAZYATTN_KERNEL_* the call resolves to or a negative error code, key-axis splits, why the fp32 kernel if
        it is the one) -- what ``run()`` will launch."""
        if self.decode:
            return self._lib.lazyattn_paged_decode_kernel_for(self.params), 0, None
        splits, why = ctypes.c_int32(0), ctypes.c_char_p()
        k = self._lib.lazyattn_prefill_kernel_for(self.params, ctypes.byref(splits), ctypes.byref(why))
        return k, splits.value, why.value.decode() if why.value else None

    def resize(self, batch: int, num_tokens: int, max_seq_len: int, max_q_len: int) -> bool:
        """Set the counts of the call (the struct's only fields that depend on the first dimension of the per-token
        and per-request tensors, and the two host-side maxima).  False: the plan's workspace is too small for them."""
        pr = self.params
        pr.batch, pr.num_tokens, pr.max_seq_len = batch, num_tokens, int(max_seq_len or 0)
        if not self.decode:
            pr.max_q_len = max_q_len
        need = (self._lib.lazyattn_paged_decode_workspace_bytes(pr) if self.decode
                else self._lib.lazyattn_prefill_workspace_bytes(pr))
        return need <= (self._ws.numel() if self._ws is not None else 0)

    def also_keep(self, *tensors) -> None:
        """Tensors the entry point made for this call whose contents do not depend on the caller's (an all-false
        ``is_lazy``, a zero ``q_offset``): they live as long as the plan, and being sized by the batch they bind a
        remembered plan to the batch it was made for."""
        self._own = self._own + tensors
        self.count_sized = self.count_sized or len(tensors) > 0

    def detached(self) -> "PrefillPlan":
        """The same call without references to the caller's tensors (what the entry points remember)."""
        twin = object.__new__(PrefillPlan)
        twin.__dict__.update(self.__dict__)
        twin._keep = ()
        return twin

    def run_static_scratch(self) -> None:
        """The same prefill call through the entry point that allocates nothing: the split-KV partials go to
        the library's static per-GPU buffer instead of this plan's workspace."""
        assert not self.decode
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _ffi.check(self._lib.lazyattn_prefix_prefill_static_scratch(self.params, stream),
                   "lazyattn_prefix_prefill_static_scratch")
