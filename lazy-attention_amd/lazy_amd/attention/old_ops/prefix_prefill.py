"""Prefix-prefill attention over an UN-ROTATED paged K cache.

Drop-in for ``lazy_attn/lazy/attention/old_ops/prefix_prefill.py:410-555``
(``context_attention_fwd``): same positional and keyword arguments, output written in
place into ``o``, returns ``None``.  Cached keys are rotated at load time -- at their
logical index when ``is_mepic`` (``:183-184``), else at ``q_offset-1+slot`` per page
(``:186-191``) -- new-token keys at ``ctx_len+m`` (``:342-362``); ``q`` arrives rotated.
"""
from __future__ import annotations

import torch

from .. import _launch
from ... import _ffi


def context_attention_fwd(q, k, v, o, kv_cache_dtype: str, k_cache, v_cache, b_loc, b_start_loc,
                          b_seq_len, max_seq_len, max_input_len, k_scale: torch.Tensor,
                          v_scale: torch.Tensor, alibi_slopes=None, sliding_window=None,
                          sm_scale=None, skip_decode=False, cos_sin_cache=None, rotary_dim=None,
                          is_neox_style=True, q_mask=None, q_offset=None, is_mepic: bool = True,
                          force_fp32_rotary: bool = False, *, _kernel: int = _ffi.KERNEL_AUTO,
                          _num_splits: int = 0, _phases: int = _ffi.PHASE_ALL, _return_plan: bool = False):
    sig = None
    if not _return_plan:
        sig = _launch.call_key(
            "un-rotated prefill", (q, k, v, o, k_cache, v_cache, b_loc, b_start_loc, b_seq_len, k_scale, v_scale,
                                   alibi_slopes, cos_sin_cache, q_mask, q_offset),
            (kv_cache_dtype, max_seq_len, max_input_len, sliding_window, sm_scale, skip_decode, rotary_dim,
             is_neox_style, is_mepic, force_fp32_rotary, _kernel, _num_splits, _phases))
        plans = _launch.recall(sig, cos_sin_cache)
        if plans is not None:
            return _launch.run_plans(plans)
    if not is_mepic and q_offset is None:
        raise ValueError("q_offset is required when is_mepic is False")
    with torch.inference_mode():                         # old_ops/prefix_prefill.py:410
        plan = _launch.launch_prefill(
            q=q, k=k, v=v, o=o, kv_cache_dtype=kv_cache_dtype, k_cache=k_cache, v_cache=v_cache,
            b_loc=b_loc, b_start_loc=b_start_loc, b_seq_len=b_seq_len, max_input_len=max_input_len,
            max_seq_len=max_seq_len, k_scale=k_scale, v_scale=v_scale, alibi_slopes=alibi_slopes,
            sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=skip_decode, cos_sin_cache=cos_sin_cache,
            rotary_dim=rotary_dim, is_neox_style=is_neox_style, is_lazy=None,
            q_offset=None if is_mepic else q_offset, q_mask=q_mask,
            pos_mode=_ffi.POS_NATURAL if is_mepic else _ffi.POS_OFFSET, rotate_new_k=True,
            fp32_rotary=force_fp32_rotary, kernel=_kernel, num_splits=_num_splits, phases=_phases,
            _return_plan=True)
    if _return_plan:
        return plan
    plan.run()
    _launch.remember(sig, (plan,), cos_sin_cache)
