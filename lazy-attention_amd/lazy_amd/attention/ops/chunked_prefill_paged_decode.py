"""Entry point the attention backend calls, block-uniform ("lazy") variant.

Drop-in for ``lazy_attn/lazy/attention/ops/chunked_prefill_paged_decode.py:36-234``:
``context_attention_fwd`` for requests with more than one new token (``:79-106``), then
the q_len==1 kernel for the rest (``:162-221``).  The reference's q_len==1 kernel reads a
packed int64 table ``[block:32 | q_offset:16 | q_mask:16]``; here the un-packed
``block_table`` / ``q_offset`` / ``q_mask`` the caller also passes are used, and a packed
table is unpacked only when they are absent.  The ``NO_LAZY`` switch (``:66-67``) is the
``NO_LAZY`` environment variable, read per call like the reference does.
"""
from __future__ import annotations

import os

import torch

from .. import _launch
from ... import _ffi
from .prefix_prefill import context_attention_fwd


def unpack_block_table(packed: torch.Tensor):
    """[block:32 | q_offset:16 | q_mask:16] -> (block, q_offset, q_mask) int32
    (``ops/models/llama_v1.py:157-160``)."""
    blk = (packed >> 32).to(torch.int32)
    off = ((packed >> 16) & 0xFFFF).to(torch.int32)
    msk = (packed & 0xFFFF).to(torch.int32)
    return blk, off, msk


def chunked_prefill_paged_decode(query, key, value, output, kv_cache_dtype, key_cache, value_cache,
                                 block_table, query_start_loc, seq_lens, max_seq_len, max_query_len,
                                 k_scale, v_scale, alibi_slopes=None, sliding_window=None,
                                 sm_scale=None, rotary_dim=None, freqs=None, cos_sin_cache=None,
                                 rope_meta=None, is_neox_style=True, is_lazy=None, lazy_variant=None,
                                 q_offset=None, q_mask=None, packed_block_table=None):
    if os.environ.get("NO_LAZY", "0") not in ("", "0") and is_lazy is not None:
        is_lazy.fill_(False)                             # ops/chunked...:66-67
    if sm_scale is None:
        sm_scale = 1.0 / (query.shape[1] ** 0.5)         # sic: ops/chunked...:71-72
    if sliding_window is None or sliding_window <= 0:
        sliding_window = 0
    if (q_offset is None or q_mask is None) and packed_block_table is not None:
        _, off, msk = unpack_block_table(packed_block_table)
        q_offset = off if q_offset is None else q_offset
        q_mask = msk if q_mask is None else q_mask
    if max_query_len > 1:
        context_attention_fwd(
            q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
            v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
            max_seq_len=max_seq_len, max_input_len=max_query_len, k_scale=k_scale, v_scale=v_scale,
            alibi_slopes=alibi_slopes, sliding_window=sliding_window, sm_scale=sm_scale,
            skip_decode=True, rotary_dim=rotary_dim, cos_sin_cache=cos_sin_cache,
            is_neox_style=is_neox_style, is_lazy=is_lazy, q_offset=q_offset, q_mask=q_mask)
    if is_lazy is None:
        is_lazy = torch.zeros(seq_lens.shape[0], dtype=torch.bool, device=query.device)
    if q_offset is None:
        q_offset = torch.zeros_like(block_table, dtype=torch.int32)
    _launch.launch_prefill(
        q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
        v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
        max_input_len=1, max_seq_len=max_seq_len, k_scale=k_scale, v_scale=v_scale, alibi_slopes=alibi_slopes,
        sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=False,
        cos_sin_cache=cos_sin_cache, rotary_dim=rotary_dim, is_neox_style=is_neox_style,
        is_lazy=is_lazy, q_offset=q_offset, q_mask=q_mask, pos_mode=_ffi.POS_BLOCK_UNIFORM,
        rotate_new_k=False, decode=True)
