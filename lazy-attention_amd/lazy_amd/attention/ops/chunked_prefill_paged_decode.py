"""Entry point the attention backend calls, block-uniform ("lazy") variant.

Drop-in for ``lazy_attn/lazy/attention/ops/chunked_prefill_paged_decode.py:36-234``:
``context_attention_fwd`` for requests with more than one new token (``:79-106``), then
the q_len==1 kernel for the rest (``:162-221``).  Like the reference's, the q_len==1 kernel
walks the packed int64 table ``[block:32 | q_offset:16 | q_mask:16]`` when one is passed
(``:162-164``); the prefill kernel reads the un-packed ``q_offset`` / ``q_mask``
(``ops/prefix_prefill.py:180-182``), which are unpacked from it only if the caller did not
pass them.  Switches, read per call like the reference does (``utils/variants.py``):
``NO_LAZY`` (``:66-67``) and ``LAZY_DECODE_COMPUTE_COS_SIN`` (``:146-151``: cos/sin of the
q_len==1 kernel computed from the inverse frequencies -- ``freqs`` if given, else formed
from ``rope_meta`` -- instead of read from ``cos_sin_cache``).
"""
from __future__ import annotations

import os

import torch

from .. import _launch
from ... import _ffi
from ...model_executor.rope import cos_sin as _rope
from .prefix_prefill import context_attention_fwd


def _env_flag(name: str) -> bool:
    return os.environ.get(name, "0") not in ("", "0")


def _streaming_decode_covers(query, value_cache) -> bool:
    """What the kernel that reads the packed table / computes cos and sin takes: 16-bit operands, head sizes
    that are multiples of 16 up to 128, pages of 16 or 32 slots.  Anything else runs the generic kernel on the
    un-packed tables and the cos/sin table."""
    return (query.dtype in (torch.bfloat16, torch.float16) and query.shape[2] % 16 == 0 and query.shape[2] <= 128
            and value_cache.shape[3] in (16, 32))


def unpack_block_table(packed: torch.Tensor):
    """[block:32 | q_offset:16 | q_mask:16] -> (block, q_offset, q_mask) int32
    (``ops/models/llama_v1.py:157-160``)."""
    blk = (packed >> 32).to(torch.int32)
    off = ((packed >> 16) & 0xFFFF).to(torch.int32)
    msk = (packed & 0xFFFF).to(torch.int32)
    return blk, off, msk


# tensors of the key whose first dimension is a token or request count: query, key, value, output, block_table,
# query_start_loc, seq_lens, is_lazy, q_offset, q_mask, packed_block_table (positions in the tuple below)
_OPEN_DIM0 = sum(1 << i for i in (0, 1, 2, 3, 6, 7, 8, 14, 15, 16, 17))


def chunked_prefill_paged_decode(query, key, value, output, kv_cache_dtype, key_cache, value_cache,
                                 block_table, query_start_loc, seq_lens, max_seq_len, max_query_len,
                                 k_scale, v_scale, alibi_slopes=None, sliding_window=None,
                                 sm_scale=None, rotary_dim=None, freqs=None, cos_sin_cache=None,
                                 rope_meta=None, is_neox_style=True, is_lazy=None, lazy_variant=None,
                                 q_offset=None, q_mask=None, packed_block_table=None):
    if _env_flag("NO_LAZY") and is_lazy is not None:
        is_lazy.fill_(False)                             # ops/chunked...:66-67
    compute = _env_flag("LAZY_DECODE_COMPUTE_COS_SIN")   # ops/chunked...:146-151
    # the counts that change from step to step are not part of the key: views [:n] of persistent buffers find the
    # call made for another n, and its structs are set to this call's counts
    max_seq_len, max_query_len = int(max_seq_len or 0), int(max_query_len)      # (plain numbers from here on)
    batch, single = seq_lens.shape[0], seq_lens.shape[0] == 1
    counts = (batch, output.shape[0], max_seq_len, max_query_len)
    bound = (batch, block_table.shape[0])                # what a plan that owns batch-sized tensors stays tied to
    sig = _launch.call_key(
        "block-uniform", (query, key, value, output, key_cache, value_cache, block_table, query_start_loc, seq_lens,
                          k_scale, v_scale, alibi_slopes, freqs, cos_sin_cache, is_lazy, q_offset, q_mask,
                          packed_block_table),
        (kv_cache_dtype, sliding_window, sm_scale, rotary_dim, is_neox_style, compute, max_query_len > 1, single),
        _OPEN_DIM0)
    if query_start_loc.shape[0] == batch + 1:            # (anything else goes to the checks below)
        plans = _launch.recall(sig, cos_sin_cache, counts, bound)
        if plans is not None:
            return _launch.run_plans(plans)
    plans, pure = [], True
    if sm_scale is None:
        sm_scale = 1.0 / (query.shape[1] ** 0.5)         # sic: ops/chunked...:71-72
    if sliding_window is None or sliding_window <= 0:
        sliding_window = 0
    if max_query_len > 1:
        pq_offset, pq_mask = q_offset, q_mask
        if (q_offset is None or q_mask is None) and packed_block_table is not None:
            _, off, msk = unpack_block_table(packed_block_table)
            pq_offset = off if q_offset is None else q_offset
            pq_mask = msk if q_mask is None else q_mask
            pure = False                                 # copies of the table's contents
        plans.append(context_attention_fwd(
            q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
            v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
            max_seq_len=max_seq_len, max_input_len=max_query_len, k_scale=k_scale, v_scale=v_scale,
            alibi_slopes=alibi_slopes, sliding_window=sliding_window, sm_scale=sm_scale,
            skip_decode=True, rotary_dim=rotary_dim, cos_sin_cache=cos_sin_cache,
            is_neox_style=is_neox_style, is_lazy=is_lazy, q_offset=pq_offset, q_mask=pq_mask, _return_plan=True))
    if plans and single:
        # the only request has more than one new token: the q_len == 1 launches would find no row of theirs
        _launch.run_plans(plans)
        if pure:
            _launch.remember(sig, plans, cos_sin_cache, counts, bound)
        return
    made = ()
    if is_lazy is None:
        is_lazy = torch.zeros(seq_lens.shape[0], dtype=torch.bool, device=query.device)
        made = (is_lazy,)
    streaming = _streaming_decode_covers(query, value_cache)
    packed = packed_block_table if streaming else None
    if packed is None:
        if (q_offset is None or q_mask is None) and packed_block_table is not None:
            _, off, msk = unpack_block_table(packed_block_table)
            q_offset = off if q_offset is None else q_offset
            q_mask = msk if q_mask is None else q_mask
            pure = False
        if q_offset is None:
            q_offset = torch.zeros_like(block_table, dtype=torch.int32)
            made += (q_offset,)
    rope_freqs = None
    if streaming and compute:
        if freqs is not None:
            rope_freqs = freqs
        else:
            rope_freqs = _rope.rope_freqs(rope_meta, query.shape[2], query.device)
            pure = False                                 # rope_meta is not part of the key
    plans.append(_launch.launch_prefill(
        q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
        v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
        max_input_len=1, max_seq_len=max_seq_len, k_scale=k_scale, v_scale=v_scale, alibi_slopes=alibi_slopes,
        sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=False,
        cos_sin_cache=cos_sin_cache, rotary_dim=rotary_dim, is_neox_style=is_neox_style,
        is_lazy=is_lazy, q_offset=q_offset, q_mask=q_mask, pos_mode=_ffi.POS_BLOCK_UNIFORM,
        rotate_new_k=False, decode=True, packed_block_table=packed, rope_freqs=rope_freqs, _return_plan=True))
    plans[-1].also_keep(*made)
    _launch.run_plans(plans)
    if pure:
        _launch.remember(sig, plans, cos_sin_cache, counts, bound)
