"""Rotary embedding of the new tokens and the paged-cache write, on the GPU library.

Counterparts, for the attention path, of
``lazy_attn/lazy/model_executor/layers/rotary_embedding.py:40-94`` (``forward_native`` /
``forward_cuda``: query only when the cache holds un-rotated keys, query and key otherwise) and
of the cache write the backend does right before the attention call
(``lazy_attn/lazy/attention/backends/triton_attn.py:100-109``,
``PagedAttention.write_to_paged_cache``).  ``rotate_and_write`` does both in one launch.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ... import _ffi


def _cache_code(kv_cache_dtype: str, dtype: torch.dtype) -> int:
    if kv_cache_dtype in ("fp8", "fp8_e4m3"):
        return _ffi.FP8_E4M3
    if kv_cache_dtype == "fp8_e5m2":
        return _ffi.FP8_E5M2
    if kv_cache_dtype == "auto":
        return _ffi.dtype_code(dtype)
    raise NotImplementedError(f"kv_cache_dtype {kv_cache_dtype!r} is not supported by the cache write")


def _as_heads(t: torch.Tensor, head_size: int) -> torch.Tensor:
    return t if t.dim() == 3 else t.view(t.shape[0], -1, head_size)


def rotate_and_write(positions: Optional[torch.Tensor], query: Optional[torch.Tensor], key: torch.Tensor,
                     value: Optional[torch.Tensor], head_size: int, cos_sin_cache: Optional[torch.Tensor], *,
                     rotate_query: bool, rotate_key: bool, key_cache: Optional[torch.Tensor] = None,
                     value_cache: Optional[torch.Tensor] = None, slot_mapping: Optional[torch.Tensor] = None,
                     kv_cache_dtype: str = "auto", k_scale=None, v_scale=None, rotary_dim: Optional[int] = None,
                     is_neox_style: bool = True) -> None:
    """In place: ``query`` / ``key`` ``[T, H*D]`` or ``[T, H, D]`` rotated at ``positions``; ``key`` (as
    left) and ``value`` scattered to ``slot_mapping`` in the paged caches when those are given."""
    if not is_neox_style:
        raise NotImplementedError("only NeoX-style rotary embedding is supported")
    dev = key.device
    if dev.type != "cuda":
        raise RuntimeError("rotate_and_write runs on the GPU only; there is no CPU path")
    p = _ffi.RopeWriteParams()
    k3 = _as_heads(key, head_size)
    keep = [k3]
    p.k = k3.data_ptr()
    p.k_stride[:] = k3.stride()
    p.num_tokens, p.num_kv_heads, p.head_dim = k3.shape[0], k3.shape[1], head_size
    p.dtype = _ffi.dtype_code(key.dtype)
    if query is not None:
        q3 = _as_heads(query, head_size)
        keep.append(q3)
        p.q = q3.data_ptr()
        p.q_stride[:] = q3.stride()
        p.num_q_heads = q3.shape[1]
    p.rotate_q, p.rotate_k = int(rotate_query and query is not None), int(rotate_key)
    if p.rotate_q or p.rotate_k:
        if cos_sin_cache.dtype not in (key.dtype, torch.float32):
            cos_sin_cache = cos_sin_cache.to(key.dtype)         # rotary_embedding.py:79-82
        positions = positions.flatten()
        keep += [cos_sin_cache, positions]
        p.positions = positions.data_ptr()
        p.pos_bits = 64 if positions.dtype == torch.int64 else 32
        p.cos_sin_cache = cos_sin_cache.data_ptr()
        p.table_stride = cos_sin_cache.stride(0)
        p.table_dtype = _ffi.dtype_code(cos_sin_cache.dtype)
        p.rotary_dim = int(rotary_dim or cos_sin_cache.shape[-1])
    else:
        p.table_dtype = p.dtype
        p.rotary_dim = int(rotary_dim or head_size)
    p.pos_bits = p.pos_bits or 64
    if key_cache is not None and slot_mapping is not None:
        v3 = _as_heads(value, head_size)
        code = _cache_code(kv_cache_dtype, key.dtype)
        keep += [v3, key_cache, value_cache, slot_mapping]
        p.v = v3.data_ptr()
        p.v_stride[:] = v3.stride()
        p.k_cache, p.v_cache = key_cache.data_ptr(), value_cache.data_ptr()
        p.kc_stride[:] = key_cache.stride()
        p.vc_stride[:] = value_cache.stride()
        p.block_size, p.x = value_cache.shape[3], key_cache.shape[4]
        p.slot_mapping = slot_mapping.data_ptr()
        p.slot_bits = 64 if slot_mapping.dtype == torch.int64 else 32
        p.cache_dtype = code
        if code in (_ffi.FP8_E4M3, _ffi.FP8_E5M2):
            ks = torch.as_tensor(k_scale, dtype=torch.float32, device=dev).reshape(1)
            vs = torch.as_tensor(v_scale, dtype=torch.float32, device=dev).reshape(1)
            keep += [ks, vs]
            p.k_scale, p.v_scale = ks.data_ptr(), vs.data_ptr()
    else:
        p.cache_dtype = p.dtype
    _ffi.check(_ffi.lib().lazyattn_rope_and_cache_write(p, torch.cuda.current_stream(dev).cuda_stream),
               "lazyattn_rope_and_cache_write")


def rotary_embedding(positions: torch.Tensor, query: torch.Tensor, key: Optional[torch.Tensor], head_size: int,
                     cos_sin_cache: torch.Tensor, is_neox: bool = True) -> None:
    """The op ``forward_cuda`` calls (``rotary_embedding.py:90-93``): in place; ``key=None`` rotates
    the query only."""
    if key is None:
        q3 = _as_heads(query, head_size)
        # the library takes K as its mandatory operand: hand it the query's heads under that name
        rotate_and_write(positions, None, q3, None, head_size, cos_sin_cache, rotate_query=False,
                         rotate_key=True, is_neox_style=is_neox)
    else:
        rotate_and_write(positions, query, key, None, head_size, cos_sin_cache, rotate_query=True,
                         rotate_key=True, is_neox_style=is_neox)


def forward(positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor, head_size: int,
            cos_sin_cache: torch.Tensor, *, q_only: bool, offsets: Optional[torch.Tensor] = None,
            is_neox_style: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """``_LazyRotaryMixin.forward_cuda`` (``rotary_embedding.py:67-94``): ``q_only`` is the reference's
    process-wide ``USE_MEPIC_Q_ONLY_ROTARY``."""
    if offsets is not None:
        positions = positions + offsets
    rotary_embedding(positions, query, None if q_only else key, head_size, cos_sin_cache, is_neox_style)
    return query, key


def write_to_paged_cache(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                         slot_mapping: torch.Tensor, kv_cache_dtype: str, k_scale, v_scale) -> None:
    """``PagedAttention.write_to_paged_cache`` as the backend calls it (``backends/triton_attn.py:100-109``)."""
    head_size = value_cache.shape[2]
    rotate_and_write(None, None, key, value, head_size, None, rotate_query=False, rotate_key=False,
                     key_cache=key_cache, value_cache=value_cache, slot_mapping=slot_mapping.flatten(),
                     kv_cache_dtype=kv_cache_dtype, k_scale=k_scale, v_scale=v_scale)
