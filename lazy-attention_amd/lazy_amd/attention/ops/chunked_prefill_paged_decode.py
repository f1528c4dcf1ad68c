"""Entry point the attention backend calls, block-uniform ("lazy") variant.

Drop-in for ``lazy_attn/lazy/attention/ops/chunked_prefill_paged_decode.py:36-234``:
``context_attention_fwd`` for requests with more than one new token (``:79-106``), then
the q_len==1 kernel for the rest (``:162-221``).  Like the reference's, the q_len==1 kernel
walks the packed int64 table ``[block:32 | q_offset:16 | q_mask:16]`` when one is passed
(``:162-164``); the prefill kernel reads the un-packed ``q_offset`` / ``q_mask``
(``ops/prefix_prefill.py:180-182``), which are unpacked from it only if the caller did not
pass them.  Switches, read per call like the reference does (``utils/variants.py:63-68,124-137``, truthy values
1 / true / yes / on): ``NO_LAZY`` (``:66-67``); ``LAZY_DECODE_COMPUTE_COS_SIN`` (``:146-151``: cos/sin of the
q_len==1 kernel computed from inverse frequencies formed from ``rope_meta`` instead of read from
``cos_sin_cache``; ``freqs`` -- the layer's bfloat16 ``inv_freq`` buffer -- is accepted and, as in the reference's
kernel, not read: ``ops/models/llama_v1.py:127-133``); ``LAZY_DECODE_IGNORE_Q_MASK`` (``:146,218``: the q_len==1
rows treat every pad count as zero, ``ops/models/llama_v1.py:161-162``).  ``LAZY_FORCE_SPLIT_DECODE`` (``:145,162-163``)
picks between two Triton kernels with the same results; one kernel serves both here, so it has nothing to select.
"""
from __future__ import annotations

import os

import torch

from .. import _launch
from ... import _ffi
from ...model_executor.rope import cos_sin as _rope
from .prefix_prefill import context_attention_fwd


_TRUTHY = ("1", "true", "yes", "on")


def _env_flag(name: str) -> bool:
    value = os.environ.get(name)                         # utils/variants.py:63-68
    return value is not None and value.strip().lower() in _TRUTHY


def _meta_key(rope_meta):
    return None if rope_meta is None else tuple(sorted((k, float(v)) for k, v in rope_meta.items()))


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
    ignore_q_mask = _env_flag("LAZY_DECODE_IGNORE_Q_MASK")   # ops/chunked...:146,218
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
        (kv_cache_dtype, sliding_window, sm_scale, rotary_dim, is_neox_style, compute, ignore_q_mask,
         _meta_key(rope_meta) if compute else None, max_query_len > 1, single),
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
    if ignore_q_mask and packed is not None:
        packed = packed & ~0xFFFF                        # a copy of the table's contents without the mask field
        pure = False
    if packed is None:
        if (q_offset is None or q_mask is None) and packed_block_table is not None:
            _, off, msk = unpack_block_table(packed_block_table)
            q_offset = off if q_offset is None else q_offset
            q_mask = msk if q_mask is None else q_mask
            pure = False
        if q_offset is None:
            q_offset = torch.zeros_like(block_table, dtype=torch.int32)
            made += (q_offset,)
    if ignore_q_mask:
        # the q_len == 1 rows see every slot of every page (ops/models/llama_v1.py:161-162); the prefill rows above
        # kept their masks, as in the reference
        q_mask = None
    rope_freqs = None
    if streaming and compute:
        # float32 frequencies from rope_meta (kept per parameter set; rope_meta is part of the call's key)
        rope_freqs = _rope.rope_freqs(rope_meta, query.shape[2], query.device)
    def decode_plan(packed, rope_freqs, q_offset, q_mask):
        return _launch.launch_prefill(
            q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
            v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
            max_input_len=1, max_seq_len=max_seq_len, k_scale=k_scale, v_scale=v_scale, alibi_slopes=alibi_slopes,
            sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=False,
            cos_sin_cache=cos_sin_cache, rotary_dim=rotary_dim, is_neox_style=is_neox_style,
            is_lazy=is_lazy, q_offset=q_offset, q_mask=q_mask, pos_mode=_ffi.POS_BLOCK_UNIFORM,
            rotate_new_k=False, decode=True, packed_block_table=packed, rope_freqs=rope_freqs, _return_plan=True)
    plan = decode_plan(packed, rope_freqs, q_offset, q_mask)
    if (packed is not None or rope_freqs is not None) and plan.kernel()[0] == _ffi.E_UNSUPPORTED:
        # what the streaming kernel does not take after all (alignment, strides: only the library's own predicate
        # sees those) goes to the generic kernel, on the un-packed tables and the cos/sin table
        if packed is not None:
            _, off, msk = unpack_block_table(packed)
            q_offset = off if q_offset is None else q_offset
            q_mask = None if ignore_q_mask else (msk if q_mask is None else q_mask)
            pure = False
        plan = decode_plan(None, None, q_offset, q_mask)
    plans.append(plan)
    plans[-1].also_keep(*made)
    _launch.run_plans(plans)
    if pure:
        _launch.remember(sig, plans, cos_sin_cache, counts, bound)
