"""Entry point the attention backend calls, un-rotated-cache variant.

Drop-in for ``lazy_attn/lazy/attention/old_ops/chunked_prefill_paged_decode.py:283-454``:
requests with more than one new token go through ``context_attention_fwd`` with
``skip_decode=True`` (``:324-351``); requests with exactly one are handled by the
fused-rotary q_len==1 kernel (``:396-442``).  The reference raises
``NotImplementedError`` when vLLM's ROCm custom paged-attention op would be selected
(``:380-386``); that op does not exist here, so nothing is refused.
"""
from __future__ import annotations

from .. import _launch
from ... import _ffi
from .prefix_prefill import context_attention_fwd


# tensors of the key whose first dimension is a token or request count: query, key, value, output, block_table,
# query_start_loc, seq_lens, q_offset, q_mask (positions in the tuple below)
_OPEN_DIM0 = sum(1 << i for i in (0, 1, 2, 3, 6, 7, 8, 13, 14))


def chunked_prefill_paged_decode(query, key, value, output, kv_cache_dtype, key_cache, value_cache,
                                 block_table, query_start_loc, seq_lens, max_seq_len, max_query_len,
                                 k_scale, v_scale, alibi_slopes=None, sliding_window=None,
                                 sm_scale=None, rotary_dim=None, cos_sin_cache=None,
                                 is_neox_style=True, q_offset=None, q_mask=None,
                                 is_mepic: bool = True, force_fp32_rotary: bool = False):
    # the counts that change from step to step are not part of the key: views [:n] of persistent buffers find the
    # call made for another n, and its structs are set to this call's counts
    max_seq_len, max_query_len = int(max_seq_len or 0), int(max_query_len)      # (plain numbers from here on)
    batch, single = seq_lens.shape[0], seq_lens.shape[0] == 1
    counts = (batch, output.shape[0], max_seq_len, max_query_len)
    sig = _launch.call_key(
        "un-rotated", (query, key, value, output, key_cache, value_cache, block_table, query_start_loc, seq_lens,
                       k_scale, v_scale, alibi_slopes, cos_sin_cache, q_offset, q_mask),
        (kv_cache_dtype, sliding_window, sm_scale, rotary_dim, is_neox_style, is_mepic, force_fp32_rotary,
         max_query_len > 1, single), _OPEN_DIM0)
    if query_start_loc.shape[0] == batch + 1:            # (anything else goes to the checks below)
        plans = _launch.recall(sig, cos_sin_cache, counts)
        if plans is not None:
            return _launch.run_plans(plans)
    plans = []
    if sm_scale is None:
        sm_scale = 1.0 / (query.shape[1] ** 0.5)        # sic: old_ops/chunked...:311-312
    if sliding_window is None or sliding_window <= 0:
        sliding_window = 0
    if max_query_len > 1:
        plans.append(context_attention_fwd(
            q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
            v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
            max_seq_len=max_seq_len, max_input_len=max_query_len, k_scale=k_scale, v_scale=v_scale,
            alibi_slopes=alibi_slopes, sliding_window=sliding_window, sm_scale=sm_scale,
            skip_decode=True, rotary_dim=rotary_dim, cos_sin_cache=cos_sin_cache,
            is_neox_style=is_neox_style, q_mask=q_mask, q_offset=q_offset, is_mepic=is_mepic,
            force_fp32_rotary=force_fp32_rotary, _return_plan=True))
    if plans and single:
        # the only request has more than one new token: the q_len == 1 launches would find no row of theirs
        _launch.run_plans(plans)
        _launch.remember(sig, plans, cos_sin_cache, counts)
        return
    plans.append(_launch.launch_prefill(
        q=query, k=key, v=value, o=output, kv_cache_dtype=kv_cache_dtype, k_cache=key_cache,
        v_cache=value_cache, b_loc=block_table, b_start_loc=query_start_loc, b_seq_len=seq_lens,
        max_input_len=1, max_seq_len=max_seq_len, k_scale=k_scale, v_scale=v_scale, alibi_slopes=alibi_slopes,
        sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=False,
        cos_sin_cache=cos_sin_cache, rotary_dim=rotary_dim, is_neox_style=is_neox_style,
        is_lazy=None, q_offset=None, q_mask=q_mask, pos_mode=_ffi.POS_NATURAL, rotate_new_k=True,
        fp32_rotary=force_fp32_rotary, decode=True, _return_plan=True))
    _launch.run_plans(plans)
    _launch.remember(sig, plans, cos_sin_cache, counts)
