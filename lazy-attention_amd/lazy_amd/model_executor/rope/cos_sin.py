"""cos/sin table builder for the rotary kernels (device side).

Counterpart of ``lazy_attn/lazy/model_executor/rope/cos_sin.py``: the reference keeps the
formula as Triton device functions (``rope_freqs`` ``:24-59``, ``rope_cos_sin_from_freqs``
``:62-66``) and reads the table a third-party layer built; here one HIP kernel builds the
table in the layout the attention kernels read: row ``p`` =
``[cos(p*inv[0..R/2)) | sin(p*inv[0..R/2))]``.
"""
from __future__ import annotations

import math

import torch

from ... import _ffi

ROPE_DEFAULT: int = 0
ROPE_LLAMA3: int = 1


def rope_meta_from_layer(rotary_emb) -> dict:
    """RoPE parameters of a rotary layer (``cos_sin.py:94-124``): same keys."""
    base = float(getattr(rotary_emb, "base", 10000.0))
    if all(hasattr(rotary_emb, a) for a in ("scaling_factor", "low_freq_factor",
                                            "high_freq_factor", "orig_max_position")):
        return dict(ROPE_TYPE=ROPE_LLAMA3, BASE=base,
                    SCALING_FACTOR=float(rotary_emb.scaling_factor),
                    LOW_FACTOR=float(rotary_emb.low_freq_factor),
                    HIGH_FACTOR=float(rotary_emb.high_freq_factor),
                    ORIG_MAX_POSITION=int(rotary_emb.orig_max_position), PI_VALUE=math.pi)
    return dict(ROPE_TYPE=ROPE_DEFAULT, BASE=base, SCALING_FACTOR=1.0, LOW_FACTOR=1.0,
                HIGH_FACTOR=1.0, ORIG_MAX_POSITION=8192, PI_VALUE=math.pi)


def build_cos_sin_cache(max_position: int, rotary_dim: int, rope_meta: dict | None = None, *,
                        base: float | None = None, dtype: torch.dtype = torch.bfloat16,
                        device="cuda") -> torch.Tensor:
    """Build ``[max_position, rotary_dim]`` on ``device`` with the HIP kernel."""
    meta = dict(ROPE_TYPE=ROPE_DEFAULT, BASE=10000.0, SCALING_FACTOR=1.0, LOW_FACTOR=1.0,
                HIGH_FACTOR=1.0, ORIG_MAX_POSITION=8192)
    if rope_meta:
        meta.update(rope_meta)
    if base is not None:
        meta["BASE"] = float(base)
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("build_cos_sin_cache runs on the GPU only")
    out = torch.empty(max_position, rotary_dim, dtype=dtype, device=device)
    rc = _ffi.lib().lazyattn_build_cos_sin_cache(
        out.data_ptr(), _ffi.dtype_code(dtype), out.stride(0), max_position, rotary_dim,
        float(meta["BASE"]), int(meta["ROPE_TYPE"]), float(meta["SCALING_FACTOR"]),
        float(meta["LOW_FACTOR"]), float(meta["HIGH_FACTOR"]), int(meta["ORIG_MAX_POSITION"]),
        torch.cuda.current_stream(device).cuda_stream)
    _ffi.check(rc, "lazyattn_build_cos_sin_cache")
    return out


_freq_cache: dict = {}


def rope_freqs(rope_meta: dict | None, head_size: int, device="cuda") -> torch.Tensor:
    """``[head_size/2]`` float32 inverse frequencies (radians per position) on ``device``: what the
    reference's ``rope_freqs`` evaluates inside its kernel (``cos_sin.py:24-59``), formed once on the
    host in float64 and kept per (parameters, device).  ``inv[i] = BASE^(-2i/D)``; Llama-3: unchanged
    where the wavelength is below ``orig/high``, divided by the factor above ``orig/low``, blended in
    between."""
    meta = dict(ROPE_TYPE=ROPE_DEFAULT, BASE=10000.0, SCALING_FACTOR=1.0, LOW_FACTOR=1.0,
                HIGH_FACTOR=1.0, ORIG_MAX_POSITION=8192)
    if rope_meta:
        meta.update(rope_meta)
    device = torch.device(device)
    key = (int(meta["ROPE_TYPE"]), float(meta["BASE"]), float(meta["SCALING_FACTOR"]), float(meta["LOW_FACTOR"]),
           float(meta["HIGH_FACTOR"]), int(meta["ORIG_MAX_POSITION"]), int(head_size), device)
    hit = _freq_cache.get(key)
    if hit is not None:
        return hit
    i = torch.arange(head_size // 2, dtype=torch.float64)
    inv = float(meta["BASE"]) ** (-2.0 * i / head_size)
    if int(meta["ROPE_TYPE"]) == ROPE_LLAMA3:
        orig, low, high = float(meta["ORIG_MAX_POSITION"]), float(meta["LOW_FACTOR"]), float(meta["HIGH_FACTOR"])
        factor = float(meta["SCALING_FACTOR"])
        wavelen = 2.0 * math.pi / inv
        smooth = (orig / wavelen - low) / (high - low)
        blended = (1.0 - smooth) * inv / factor + smooth * inv
        inv = torch.where(wavelen < orig / high, inv, torch.where(wavelen > orig / low, inv / factor, blended))
    out = inv.to(torch.float32).to(device)
    _freq_cache[key] = out
    return out
