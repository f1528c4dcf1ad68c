"""ctypes binding of liblazyattn.so (the C ABI declared in include/lazyattn.h).

The library is loaded from ``lazy_amd/_lib``; if it is missing the import of any
operator raises -- there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os
from collections import OrderedDict
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib", "liblazyattn.so")
_lib = None

F32, BF16, F16, FP8_E4M3, FP8_E5M2 = 0, 1, 2, 3, 4
POS_NATURAL, POS_OFFSET, POS_BLOCK_UNIFORM = 0, 1, 2
KERNEL_AUTO, KERNEL_GENERIC, KERNEL_MFMA, KERNEL_MFMA4, KERNEL_MFMA8 = 0, 1, 2, 3, 4
PHASE_MAIN, PHASE_COMBINE, PHASE_ALL = 1, 2, 3

E_UNSUPPORTED = -4
ERRORS = {-1: "NULL", -2: "SHAPE", -3: "DTYPE", -4: "UNSUPPORTED", -5: "WORKSPACE", -6: "LAUNCH", -7: "SCRATCH_LIMIT"}
EXPORTS = ("lazyattn_prefill_workspace_bytes", "lazyattn_prefix_prefill", "lazyattn_prefix_prefill_static_scratch",
           "lazyattn_static_scratch_bytes", "lazyattn_paged_decode_workspace_bytes",
           "lazyattn_paged_decode_rotary", "lazyattn_build_cos_sin_cache",
           "lazyattn_pack_cos_sin_cache", "lazyattn_rope_and_cache_write", "lazyattn_build_rotation_metadata", "lazyattn_reposition_blocks", "lazyattn_pack_block_table",
           "lazyattn_static_scratch_prepare", "lazyattn_prefill_kernel_for", "lazyattn_paged_decode_kernel_for",
           "lazyattn_error_string", "lazyattn_abi_version")

_DTYPE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}


class PrefillParams(C.Structure):
    _fields_ = (
        [(n, C.c_void_p) for n in ("q", "k", "v", "o", "k_cache", "v_cache", "block_table",
                                   "q_offset", "q_mask", "is_lazy", "b_start_loc", "b_seq_len",
                                   "cos_sin_cache", "cos_sin_packed", "k_scale", "v_scale", "workspace")]
        + [("workspace_bytes", C.c_int64),
           ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3),
           ("v_stride", C.c_int64 * 3), ("o_stride", C.c_int64 * 3),
           ("kc_stride", C.c_int64 * 5), ("vc_stride", C.c_int64 * 4),
           ("bt_stride", C.c_int64 * 2), ("qo_stride", C.c_int64 * 2), ("qm_stride", C.c_int64 * 2),
           ("table_stride", C.c_int64)]
        + [(n, C.c_int32) for n in ("batch", "num_q_heads", "num_kv_heads", "head_dim", "block_size",
                                    "x", "max_q_len", "rotary_dim", "sliding_window", "dtype",
                                    "cache_dtype", "table_dtype", "index_bits", "pos_mode",
                                    "rotate_new_k", "skip_decode", "fp32_rotary", "kernel",
                                    "num_splits", "phases")]
        + [("sm_scale", C.c_float), ("num_tokens", C.c_int32), ("max_seq_len", C.c_int32),
           ("packed_rows", C.c_int32),
           ("packed_block_table", C.c_void_p), ("pbt_stride", C.c_int64 * 2), ("rope_freqs", C.c_void_p)])


class RopeWriteParams(C.Structure):
    _fields_ = (
        [(n, C.c_void_p) for n in ("q", "k", "v", "k_cache", "v_cache", "slot_mapping", "positions",
                                   "cos_sin_cache", "k_scale", "v_scale")]
        + [("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
           ("kc_stride", C.c_int64 * 5), ("vc_stride", C.c_int64 * 4), ("table_stride", C.c_int64)]
        + [(n, C.c_int32) for n in ("num_tokens", "num_q_heads", "num_kv_heads", "head_dim", "rotary_dim",
                                    "block_size", "x", "dtype", "cache_dtype", "table_dtype", "rotate_q",
                                    "rotate_k", "pos_bits", "slot_bits")])


class RepositionParams(C.Structure):
    _fields_ = ([(n, C.c_void_p) for n in ("k_cache", "v_cache", "items", "cos_sin_cache")]
                + [("kc_stride", C.c_int64 * 5), ("vc_stride", C.c_int64 * 4), ("table_stride", C.c_int64)]
                + [(n, C.c_int32) for n in ("num_items", "num_kv_heads", "head_dim", "block_size", "x", "dtype",
                                            "table_dtype")])


def lib() -> C.CDLL:
    """Load the HIP library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python lazy-attention_amd/build.py` "
                "(there is no non-HIP path)")
        L = C.CDLL(_LIB_PATH)
        L.lazyattn_prefill_workspace_bytes.restype = C.c_size_t
        L.lazyattn_prefill_workspace_bytes.argtypes = [C.POINTER(PrefillParams)]
        L.lazyattn_paged_decode_workspace_bytes.restype = C.c_size_t
        L.lazyattn_paged_decode_workspace_bytes.argtypes = [C.POINTER(PrefillParams)]
        L.lazyattn_static_scratch_bytes.restype = C.c_size_t
        L.lazyattn_static_scratch_bytes.argtypes = []
        L.lazyattn_static_scratch_prepare.restype = C.c_int
        L.lazyattn_static_scratch_prepare.argtypes = []
        L.lazyattn_prefill_kernel_for.restype = C.c_int
        L.lazyattn_prefill_kernel_for.argtypes = [C.POINTER(PrefillParams), C.POINTER(C.c_int32), C.POINTER(C.c_char_p)]
        L.lazyattn_paged_decode_kernel_for.restype = C.c_int
        L.lazyattn_paged_decode_kernel_for.argtypes = [C.POINTER(PrefillParams)]
        for name in ("lazyattn_prefix_prefill", "lazyattn_prefix_prefill_static_scratch", "lazyattn_paged_decode_rotary"):
            fn = getattr(L, name)
            fn.restype = C.c_int
            fn.argtypes = [C.POINTER(PrefillParams), C.c_void_p]
        L.lazyattn_build_cos_sin_cache.restype = C.c_int
        L.lazyattn_build_cos_sin_cache.argtypes = [
            C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.c_double, C.c_int32,
            C.c_double, C.c_double, C.c_double, C.c_int32, C.c_void_p]
        L.lazyattn_pack_cos_sin_cache.restype = C.c_int
        L.lazyattn_pack_cos_sin_cache.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32,
                                                  C.c_int32, C.c_void_p]
        L.lazyattn_rope_and_cache_write.restype = C.c_int
        L.lazyattn_rope_and_cache_write.argtypes = [C.POINTER(RopeWriteParams), C.c_void_p]
        L.lazyattn_build_rotation_metadata.restype = C.c_int
        L.lazyattn_build_rotation_metadata.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                                       C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
        L.lazyattn_reposition_blocks.restype = C.c_int
        L.lazyattn_reposition_blocks.argtypes = [C.POINTER(RepositionParams), C.c_void_p]
        L.lazyattn_pack_block_table.restype = C.c_int
        L.lazyattn_pack_block_table.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int32,
                                                C.c_int32, C.c_void_p, C.c_int64, C.c_void_p]
        L.lazyattn_error_string.restype = C.c_char_p
        L.lazyattn_error_string.argtypes = [C.c_int]
        L.lazyattn_abi_version.restype = C.c_int
        _lib = L
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().lazyattn_error_string(rc).decode()
        if rc == -4:
            raise NotImplementedError(f"{what}: {msg}")
        raise RuntimeError(f"{what}: {msg} (code {rc})")


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE[dt]
    except KeyError:
        raise TypeError(f"unsupported tensor dtype {dt}") from None


_workspaces: dict = {}
_growth_hooks: list = []


def on_workspace_growth(fn) -> None:
    """``fn()`` runs whenever something a remembered call may point at goes away: a workspace replaced by a larger
    one, the re-laid-out tables dropped by ``invalidate_packed_tables()``."""
    _growth_hooks.append(fn)


def workspace(device: torch.device, nbytes: int, kind: str = "prefill") -> Optional[torch.Tensor]:
    """Per-device scratch for split-KV partials, grown on demand and kept; one per kind of call."""
    if nbytes <= 0:
        return None
    key = (device.type, device.index, kind)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            for fn in _growth_hooks:
                fn()
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


_packed_tables: "OrderedDict" = OrderedDict()
_PACKED_TABLES_MAX = 8


def table_version(table: torch.Tensor) -> Optional[int]:
    """torch's in-place edit counter of the table, or None for a tensor made under
    ``torch.inference_mode()`` (those carry no counter and reading it raises)."""
    return None if table.is_inference() else table._version


def invalidate_packed_tables() -> None:
    """Drop every re-laid-out copy, and every remembered call that points at one.  Needed only after writing in
    place to a table that was created under ``torch.inference_mode()``: such an edit cannot be seen from here (other
    tables are re-packed on their own)."""
    _packed_tables.clear()
    for fn in _growth_hooks:
        fn()


def packed_cos_sin(table: torch.Tensor) -> Optional[torch.Tensor]:
    """The table in the gather-friendly layout, built once per table (and again if the
    caller writes to it) by the library's pack kernel.  The few most recently used tables are kept."""
    if table.dim() != 2 or table.shape[1] % 16 or table.stride(1) != 1:
        return None
    key = (table.data_ptr(), tuple(table.shape), table.stride(0), table.dtype, table.device)
    version = table_version(table)
    hit = _packed_tables.get(key)
    if hit is not None and hit[0] == version:
        _packed_tables.move_to_end(key)
        return hit[1]
    while len(_packed_tables) >= _PACKED_TABLES_MAX:
        _packed_tables.popitem(last=False)
    packed = torch.empty(table.shape[0] * table.shape[1], dtype=table.dtype, device=table.device)
    rc = lib().lazyattn_pack_cos_sin_cache(table.data_ptr(), packed.data_ptr(), dtype_code(table.dtype),
                                           table.stride(0), table.shape[0], table.shape[1],
                                           torch.cuda.current_stream(table.device).cuda_stream)
    check(rc, "lazyattn_pack_cos_sin_cache")
    # the entry holds the table too: while it is cached its address cannot be handed to another tensor
    _packed_tables[key] = (version, packed, table)
    return packed


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def fill_params(*, q, k, v, o, k_cache, v_cache, block_table, b_start_loc, b_seq_len,
                cos_sin_cache, k_scale, v_scale, q_offset, q_mask, is_lazy, cache_code: int,
                max_q_len: int, rotary_dim: int, sliding_window: int, sm_scale: float,
                pos_mode: int, rotate_new_k: bool, skip_decode: bool, fp32_rotary: bool = False,
                kernel: int = KERNEL_AUTO, num_splits: int = 0, phases: int = PHASE_ALL,
                max_seq_len: int = 0, packed_table=None, packed_block_table=None, rope_freqs=None) -> PrefillParams:
    p = PrefillParams()
    p.q, p.k, p.v, p.o = _ptr(q), _ptr(k), _ptr(v), _ptr(o)
    p.k_cache, p.v_cache = _ptr(k_cache), _ptr(v_cache)
    p.block_table, p.q_offset, p.q_mask, p.is_lazy = _ptr(block_table), _ptr(q_offset), _ptr(q_mask), _ptr(is_lazy)
    p.b_start_loc, p.b_seq_len = _ptr(b_start_loc), _ptr(b_seq_len)
    p.cos_sin_cache, p.k_scale, p.v_scale = _ptr(cos_sin_cache), _ptr(k_scale), _ptr(v_scale)
    if packed_table is not None:
        p.cos_sin_packed = packed_table.data_ptr()
        p.packed_rows = cos_sin_cache.shape[0]
    p.q_stride[:] = q.stride()
    p.k_stride[:] = k.stride() if k is not None else (0, 0, 0)
    p.v_stride[:] = v.stride() if v is not None else (0, 0, 0)
    p.o_stride[:] = o.stride()
    p.kc_stride[:] = k_cache.stride()
    p.vc_stride[:] = v_cache.stride()
    p.bt_stride[:] = block_table.stride()
    p.qo_stride[:] = q_offset.stride() if q_offset is not None else (0, 0)
    p.qm_stride[:] = q_mask.stride() if q_mask is not None else (0, 0)
    p.table_stride = cos_sin_cache.stride(0) if cos_sin_cache is not None else 0
    if packed_block_table is not None:
        p.packed_block_table = packed_block_table.data_ptr()
        p.pbt_stride[:] = packed_block_table.stride()
    p.rope_freqs = _ptr(rope_freqs)
    p.batch = b_seq_len.shape[0]
    p.num_q_heads, p.head_dim = q.shape[1], q.shape[2]
    p.num_kv_heads = k_cache.shape[1]
    p.block_size, p.x = v_cache.shape[3], k_cache.shape[4]
    p.max_q_len = int(max_q_len)
    p.rotary_dim = int(rotary_dim)
    p.sliding_window = int(sliding_window)
    p.dtype = dtype_code(q.dtype)
    p.cache_dtype = cache_code
    p.table_dtype = dtype_code(cos_sin_cache.dtype) if cos_sin_cache is not None else p.dtype
    p.index_bits = 64 if b_start_loc.dtype == torch.int64 else 32
    p.pos_mode = pos_mode
    p.rotate_new_k = int(rotate_new_k)
    p.skip_decode = int(skip_decode)
    p.fp32_rotary = int(fp32_rotary)
    p.kernel = kernel
    p.num_splits = num_splits
    p.phases = phases
    p.sm_scale = float(sm_scale)
    p.num_tokens = o.shape[0]
    p.max_seq_len = int(max_seq_len or 0)
    return p
