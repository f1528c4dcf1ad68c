"""Re-positioning of cached document blocks on the GPU library.

Counterpart of ``block_attn_vllm/utils.py:48-95`` (``place_paged_block_keys``, ``copy_paged_block``)
and of the loop that calls them per layer and per block (``block_attn_vllm/gpu_model_runner.py:94-106``):
``reposition_blocks`` does all blocks of one layer in one launch.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import torch

from .. import _ffi


def reposition_blocks(key_cache: torch.Tensor, value_cache: torch.Tensor,
                      items, cos_sin_cache: torch.Tensor) -> None:
    """``items``: sequence of ``(new_id, old_id, from_start, to_start)`` (the reference's ``cow_blocks``) or an
    int32 device tensor ``[n, 4]``.  Block ``old_id`` is copied to ``new_id`` (K and V) and the copy's keys
    are moved from rotation positions ``from_start + slot`` to ``to_start + slot``."""
    dev = key_cache.device
    if dev.type != "cuda":
        raise RuntimeError("reposition_blocks runs on the GPU only; there is no CPU path")
    if not torch.is_tensor(items):
        items = torch.tensor(list(items), dtype=torch.int32).reshape(-1, 4).to(dev)
    if items.numel() == 0:
        return
    items = items.to(device=dev, dtype=torch.int32).contiguous()
    if cos_sin_cache.dtype not in (key_cache.dtype, torch.float32):
        cos_sin_cache = cos_sin_cache.to(key_cache.dtype)
    p = _ffi.RepositionParams()
    p.k_cache, p.v_cache = key_cache.data_ptr(), value_cache.data_ptr()
    p.items, p.cos_sin_cache = items.data_ptr(), cos_sin_cache.data_ptr()
    p.kc_stride[:] = key_cache.stride()
    p.vc_stride[:] = value_cache.stride()
    p.table_stride = cos_sin_cache.stride(0)
    p.num_items = items.shape[0]
    p.num_kv_heads, p.head_dim, p.block_size = value_cache.shape[1], value_cache.shape[2], value_cache.shape[3]
    p.x = key_cache.shape[4]
    p.dtype, p.table_dtype = _ffi.dtype_code(key_cache.dtype), _ffi.dtype_code(cos_sin_cache.dtype)
    _ffi.check(_ffi.lib().lazyattn_reposition_blocks(p, torch.cuda.current_stream(dev).cuda_stream),
               "lazyattn_reposition_blocks")


def place_paged_block_keys(key_cache: torch.Tensor, value_cache: torch.Tensor, block_id: int,
                           cos_sin_cache: torch.Tensor, from_start: int, to_start: int) -> None:
    """One block, in place (``utils.py:48-88``; the value cache is passed because the library call covers both)."""
    reposition_blocks(key_cache, value_cache, [(block_id, block_id, from_start, to_start)], cos_sin_cache)
