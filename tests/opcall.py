"""Helpers shared by the GPU tests: run the operator / the oracle on a Workload."""
import torch

from oracle import deferred_rope as orc
from lazy_amd import _ffi
from lazy_amd.attention.old_ops.prefix_prefill import context_attention_fwd as fwd_unrotated
from lazy_amd.attention.ops.prefix_prefill import context_attention_fwd as fwd_block_uniform


def run_op(w, *, kernel=_ffi.KERNEL_AUTO, num_splits=0, sliding_window=None, skip_decode=False,
           is_lazy=None, out=None, sm_scale=None, index_dtype=None):
    """w: Workload already on the GPU.  Returns o (a new tensor unless ``out`` is given)."""
    o = out if out is not None else torch.zeros_like(w.q)
    bsl, bsq = w.b_start_loc, w.b_seq_len
    if index_dtype is not None:
        bsl, bsq = bsl.to(index_dtype), bsq.to(index_dtype)
    common = (w.q, w.k, w.v, o, w.kv_cache_dtype, w.k_cache, w.v_cache, w.block_table, bsl, bsq,
              w.max_seq_len, w.max_query_len, w.k_scale, w.v_scale)
    kw = dict(sliding_window=sliding_window, sm_scale=sm_scale, skip_decode=skip_decode,
              cos_sin_cache=w.cos_sin_cache, rotary_dim=w.q.shape[-1], _kernel=kernel,
              _num_splits=num_splits)
    if w.pos_mode == orc.POS_BLOCK_UNIFORM:
        fwd_block_uniform(*common, is_lazy=w.is_lazy if is_lazy is None else is_lazy,
                          q_offset=w.q_offset, q_mask=w.q_mask, **kw)
    else:
        fwd_unrotated(*common, q_mask=w.q_mask, q_offset=w.q_offset,
                      is_mepic=w.pos_mode == orc.POS_NATURAL, **kw)
    return o


def run_oracle(w, **kw):
    """w: Workload on the CPU."""
    return orc.prefix_prefill(
        w.q, w.k, w.v, w.k_cache, w.v_cache, w.block_table, w.b_start_loc, w.b_seq_len,
        w.cos_sin_cache, w.q_offset, w.q_mask, pos_mode=w.pos_mode, rotate_new_k=w.rotate_new_k,
        kv_cache_dtype=w.kv_cache_dtype, k_scale=w.k_scale, v_scale=w.v_scale, **kw)
