"""ctypes binding of the C restatement (oracle/prefix_prefill_ref.c) for the tests."""
import ctypes as C
import math

import torch


class RefParams(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("q", "k", "v", "o", "k_cache", "v_cache", "b_loc", "q_offset", "q_mask",
                 "is_lazy", "b_start_loc", "b_seq_len", "table")] + [
        ("sq", C.c_int64 * 3), ("sk", C.c_int64 * 3), ("sv", C.c_int64 * 3), ("so", C.c_int64 * 3),
        ("skc", C.c_int64 * 5), ("svc", C.c_int64 * 4), ("sbl", C.c_int64 * 2),
        ("batch", C.c_int32), ("hq", C.c_int32), ("hkv", C.c_int32), ("d", C.c_int32),
        ("bs", C.c_int32), ("x", C.c_int32), ("rotary_dim", C.c_int32),
        ("pos_mode", C.c_int32), ("rotate_new_k", C.c_int32), ("sliding_window", C.c_int32),
        ("skip_decode", C.c_int32), ("sm_scale", C.c_float)]


def run_c_ref(lib, w, *, sliding_window=0, skip_decode=False, is_lazy=None, sm_scale=None):
    """Run the C restatement on a Workload (float copies of every operand)."""
    assert "fp8" not in w.kv_cache_dtype
    f = lambda t: t.float().contiguous()
    q, k, v = f(w.q), f(w.k), f(w.v)
    kc, vc, tab = f(w.k_cache), f(w.v_cache), f(w.cos_sin_cache)
    o = torch.zeros_like(q)
    bl = w.block_table.to(torch.int32).contiguous()
    qo = w.q_offset.to(torch.int32).contiguous()
    qm = w.q_mask.to(torch.int32).contiguous()
    lazy = (w.is_lazy if is_lazy is None else is_lazy).to(torch.int32).contiguous()
    bsl = w.b_start_loc.to(torch.int64).contiguous()
    bsq = w.b_seq_len.to(torch.int64).contiguous()
    p = RefParams()
    for name, t in dict(q=q, k=k, v=v, o=o, k_cache=kc, v_cache=vc, b_loc=bl, q_offset=qo,
                        q_mask=qm, is_lazy=lazy, b_start_loc=bsl, b_seq_len=bsq, table=tab).items():
        setattr(p, name, t.data_ptr())
    p.sq[:] = q.stride(); p.sk[:] = k.stride(); p.sv[:] = v.stride(); p.so[:] = o.stride()
    p.skc[:] = kc.stride(); p.svc[:] = vc.stride(); p.sbl[:] = bl.stride()
    p.batch = bsq.numel(); p.hq = q.shape[1]; p.hkv = k.shape[1]; p.d = q.shape[2]
    p.bs = vc.shape[3]; p.x = kc.shape[4]; p.rotary_dim = tab.shape[1]
    p.pos_mode = w.pos_mode; p.rotate_new_k = int(w.rotate_new_k)
    p.sliding_window = sliding_window; p.skip_decode = int(skip_decode)
    p.sm_scale = sm_scale if sm_scale is not None else 1.0 / math.sqrt(q.shape[2])
    lib.ref_prefix_prefill.argtypes = [C.POINTER(RefParams)]
    assert lib.ref_prefix_prefill(C.byref(p)) == 0
    return o
