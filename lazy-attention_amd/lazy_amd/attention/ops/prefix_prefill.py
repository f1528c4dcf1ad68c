"""Prefix-prefill attention with a block-uniform rotation of cached keys.

Drop-in for ``lazy_attn/lazy/attention/ops/prefix_prefill.py:599-744``
(``context_attention_fwd``).  Requests with ``is_lazy[b]`` set: every page of cached K
(stored rotated at its document-local position) is rotated forward by ``q_offset-1``
(``:180-190``), pad slots are masked through ``q_mask`` (``:267-271``), new-token K is
used as given (``:341-354``).  Other requests take the un-rotated branch (``:398-592``).
``is_lazy=None`` means no request is lazy (plain paged prefix-prefill).
"""
from __future__ import annotations

import torch

from .. import _launch
from ... import _ffi


def context_attention_fwd(q, k, v, o, kv_cache_dtype: str, k_cache, v_cache, b_loc, b_start_loc,
                          b_seq_len, max_seq_len, max_input_len, k_scale: torch.Tensor,
                          v_scale: torch.Tensor, alibi_slopes=None, sliding_window=None,
                          sm_scale=None, skip_decode=False, cos_sin_cache=None, rotary_dim=None,
                          is_neox_style=True, is_lazy=None, q_offset=None, q_mask=None, *,
                          _kernel: int = _ffi.KERNEL_AUTO, _num_splits: int = 0,
                          _phases: int = _ffi.PHASE_ALL, _return_plan: bool = False):
    sig = None
    if not _return_plan:
        sig = _launch.call_key(
            "block-uniform prefill", (q, k, v, o, k_cache, v_cache, b_loc, b_start_loc, b_seq_len, k_scale, v_scale,
                                      alibi_slopes, cos_sin_cache, is_lazy, q_offset, q_mask),
            (kv_cache_dtype, max_seq_len, max_input_len, sliding_window, sm_scale, skip_decode, rotary_dim,
             is_neox_style, _kernel, _num_splits, _phases))
        plans = _launch.recall(sig, cos_sin_cache)
        if plans is not None:
            return _launch.run_plans(plans)
    made, given_table = (), cos_sin_cache
    with torch.inference_mode():                         # ops/prefix_prefill.py:599
        if is_lazy is None:
            is_lazy = torch.zeros(b_seq_len.shape[0], dtype=torch.bool, device=q.device)
            made = (is_lazy,)
            if cos_sin_cache is None:
                half = q.shape[-1] // 2                      # one row: cos 1, sin 0
                cos_sin_cache = torch.cat([q.new_ones(half), q.new_zeros(half)])[None]
                rotary_dim = q.shape[-1]
                made += (cos_sin_cache,)
            if q_offset is None:
                q_offset = torch.zeros_like(b_loc, dtype=torch.int32)
                made += (q_offset,)
        elif q_offset is None:
            raise ValueError("q_offset is required when is_lazy is given")
        plan = _launch.launch_prefill(
            q=q, k=k, v=v, o=o, kv_cache_dtype=kv_cache_dtype, k_cache=k_cache, v_cache=v_cache,
            b_loc=b_loc, b_start_loc=b_start_loc, b_seq_len=b_seq_len, max_input_len=max_input_len,
            max_seq_len=max_seq_len, k_scale=k_scale, v_scale=v_scale, alibi_slopes=alibi_slopes,
            sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=skip_decode, cos_sin_cache=cos_sin_cache,
            rotary_dim=rotary_dim, is_neox_style=is_neox_style, is_lazy=is_lazy, q_offset=q_offset,
            q_mask=q_mask, pos_mode=_ffi.POS_BLOCK_UNIFORM, rotate_new_k=False, kernel=_kernel,
            num_splits=_num_splits, phases=_phases, _return_plan=True)
    plan.also_keep(*made)        # constants made here: they live with the plan
    if _return_plan:
        return plan
    plan.run()
    _launch.remember(sig, (plan,), given_table)
