"""CPU oracle for deferred-RoPE prefix-prefill attention.  TEST INFRASTRUCTURE ONLY.

This module is a checker: a PyTorch-eager restatement, on the CPU, of what the
reference's Triton kernels compute for the prefix-prefill path.  Only the test
suite, the smoke check and the benchmark's ``cpu_baseline`` leg may import it.
The shipped operator never calls anything in here; it fails loudly when its HIP
library is missing.

Every function cites the reference lines it restates (paths relative to the
reference checkout):

* the un-rotated-cache ("mepic") kernel
  ``lazy_attn/lazy/attention/old_ops/prefix_prefill.py:95-407``
* the block-uniform ("lazy") kernel and its un-rotated vanilla branch
  ``lazy_attn/lazy/attention/ops/prefix_prefill.py:95-592``
* the q_len==1 fused-rotary kernel
  ``lazy_attn/lazy/attention/old_ops/chunked_prefill_paged_decode.py:68-280``
* the cos/sin formula ``lazy_attn/lazy/model_executor/rope/cos_sin.py:24-66,127-148``
  (table layout: vLLM 0.9.2 ``RotaryEmbedding._compute_cos_sin_cache``, a
  third-party dependency that is not vendored: row p = [cos(p*inv) | sin(p*inv)],
  ``inv[i] = base**(-2i/rotary_dim)``)
* the metadata producer ``lazy_attn/lazy/core/sched/scheduler.py:758-787`` and
  ``lazy_attn/lazy/utils/rotation.py:20-37``

Parity status of each function (what pins it without running the reference):

* ``metadata_for_lazy_attention`` / ``max_rotation_offset``: the reference's
  known-answer vectors (``tests/core/test_scheduler.py:49-50``) and closed form
  (``tests/core/test_rotation_offset_bound.py:18-75``).
* ``build_cos_sin_table`` / ``llama3_inv_freq``: closed form in float64,
  ``T[0] = [1..1, 0..0]``, ``cos^2+sin^2 = 1``, angle addition.
* ``prefix_prefill`` (all position modes) and ``paged_decode``: a float64
  brute-force triple loop on tiny shapes, the C restatement in this folder
  (independent loop structure: page-by-page online softmax), equality with
  ``torch.nn.functional.scaled_dot_product_attention`` on pre-rotated keys (the
  construction of the reference's own kernel test,
  ``tests/kernels/test_prefix_prefill.py:107-134,238-289,364``), the
  relative-position identity, page-permutation invariance and pad truncation.
* The reference holds no stored numeric vectors for the attention kernels, and
  its Triton code was not run (no vLLM, no GPU in the build container), so the
  bit-level behaviour of the Triton kernels (bf16 rounding order, tl.exp) is
  parity unpinned; the stated tolerances are against this float32 restatement.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

POS_NATURAL = 0        # p = logical index n                       (old_ops:183-184)
POS_OFFSET = 1         # p = q_offset-1+o, or n when q_offset == 0  (old_ops:186-191)
POS_BLOCK_UNIFORM = 2  # p = q_offset-1 or 0, same for the page     (ops:180-186)

SLIDING_FILL = -10000.0  # old_ops:282-284, ops:290-292


# --------------------------------------------------------------------------
# RoPE tables (rope/cos_sin.py:24-66,127-148; vLLM _compute_cos_sin_cache)
# --------------------------------------------------------------------------
def plain_inv_freq(rotary_dim: int, base: float, dtype=torch.float64) -> torch.Tensor:
    """inv[i] = base**(-2i/rotary_dim), i in [0, rotary_dim/2)  (cos_sin.py:41-43)."""
    idx = torch.arange(0, rotary_dim, 2, dtype=dtype)
    return 1.0 / (torch.tensor(base, dtype=dtype) ** (idx / rotary_dim))


def llama3_inv_freq(rotary_dim: int, base: float, scaling_factor: float,
                    low_freq_factor: float, high_freq_factor: float,
                    orig_max_position: int, dtype=torch.float64) -> torch.Tensor:
    """Llama-3 wavelength-dependent smoothing of inv_freq (cos_sin.py:44-58,135-146)."""
    inv = plain_inv_freq(rotary_dim, base, dtype)
    wave_len = 2 * math.pi / inv
    low_wl = orig_max_position / low_freq_factor
    high_wl = orig_max_position / high_freq_factor
    smooth = (orig_max_position / wave_len - low_freq_factor) / (
        high_freq_factor - low_freq_factor)
    return torch.where(
        wave_len < high_wl, inv,
        torch.where(wave_len > low_wl, inv / scaling_factor,
                    (1 - smooth) * inv / scaling_factor + smooth * inv))


def build_cos_sin_table(max_position: int, rotary_dim: int, base: float,
                        llama3: Optional[dict] = None,
                        dtype: torch.dtype = torch.float32,
                        math_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """[max_position, rotary_dim] table, row p = [cos(p*inv) | sin(p*inv)].

    ``math_dtype`` float32 follows the third-party builder (fp32 outer product,
    fp32 cos/sin, then a cast to the model dtype); float64 is the closed form.
    """
    if llama3 is None:
        inv = plain_inv_freq(rotary_dim, base, math_dtype)
    else:
        inv = llama3_inv_freq(rotary_dim, base, llama3["scaling_factor"],
                              llama3["low_freq_factor"], llama3["high_freq_factor"],
                              llama3["orig_max_position"], math_dtype)
    t = torch.arange(max_position, dtype=math_dtype)
    ang = torch.outer(t, inv)
    return torch.cat([ang.cos(), ang.sin()], dim=-1).to(dtype)


def neox_rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x: [..., D]; cos/sin: broadcastable [..., D/2]   (old_ops:256-257)."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1)


def rotate_at(x: torch.Tensor, positions: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Rotate x[n, H, D] at integer positions[n] using rows of ``table``."""
    half = table.shape[-1] // 2
    rows = table[positions.long()].to(x.dtype)
    return neox_rotate(x, rows[:, None, :half], rows[:, None, half:])


# --------------------------------------------------------------------------
# Metadata (scheduler.py:758-787, rotation.py:20-37)
# --------------------------------------------------------------------------
def metadata_for_lazy_attention(document_lens: Sequence[int],
                                document_lens_padded: Sequence[int],
                                block_size: int):
    """q_offset / q_mask lists, one entry per document page plus one for the query."""
    num_blocks = sum(document_lens_padded) // block_size + 1
    q_offset = [0] * num_blocks
    q_mask = [0] * num_blocks
    pads = [p - t for t, p in zip(document_lens, document_lens_padded)]
    rot = sum(pads)
    cursor = 0
    for true_len, padded, pad in zip(document_lens, document_lens_padded, pads):
        nblk = padded // block_size
        for j in range(cursor, cursor + nblk):
            q_offset[j] = rot + 1
        cursor += nblk
        q_mask[cursor - 1] = pad
        rot += true_len
    q_offset[cursor] = 1
    return q_offset, q_mask


def metadata_for_mepic(document_lens, document_lens_padded, block_size):
    """scheduler.py:784-787: offsets all zero, same pad mask."""
    q_offset, q_mask = metadata_for_lazy_attention(document_lens, document_lens_padded, block_size)
    return [0] * len(q_offset), q_mask


def max_rotation_offset(document_lens, document_lens_padded) -> int:
    """rotation.py:20-37."""
    if not document_lens:
        return 0
    pad = sum(p - t for t, p in zip(document_lens, document_lens_padded))
    return pad + sum(document_lens[:-1]) + 1


# --------------------------------------------------------------------------
# Paged cache access
# --------------------------------------------------------------------------
def _dequant(cache: torch.Tensor, kv_cache_dtype: str, scale, q_dtype) -> torch.Tensor:
    """fp8 -> float(x)*scale -> q dtype (old_ops:239-244,304-307); else identity."""
    if "fp8" in kv_cache_dtype:
        assert cache.dtype == torch.uint8
        if kv_cache_dtype in ("fp8", "fp8_e4m3"):
            cache = cache.view(torch.float8_e4m3fn)
        elif kv_cache_dtype == "fp8_e5m2":
            cache = cache.view(torch.float8_e5m2)
        else:
            raise ValueError("Unsupported FP8 dtype:", kv_cache_dtype)
        return (cache.to(torch.float32) * float(scale)).to(q_dtype)
    return cache


def gather_pages(k_cache, v_cache, blocks: torch.Tensor):
    """K[NB,Hkv,D/x,BS,x], V[NB,Hkv,D,BS] -> K,V [len(blocks)*BS, Hkv, D]
    (index math of old_ops:172-181,196-199)."""
    nb, hkv, dx, bs, x = k_cache.shape
    kb = k_cache[blocks.long()]                       # [P,Hkv,D/x,BS,x]
    kb = kb.permute(0, 3, 1, 2, 4).reshape(-1, hkv, dx * x)
    vb = v_cache[blocks.long()]                       # [P,Hkv,D,BS]
    vb = vb.permute(0, 3, 1, 2).reshape(-1, hkv, v_cache.shape[2])
    return kb, vb


def _attend(q, keys, vals, mask, fill_mask, sm_scale, group, cdt):
    """q [Tq,Hq,D]; keys/vals [Tk,Hkv,D]; mask [Tq,Tk] True = -inf;
    fill_mask [Tq,Tk] True = SLIDING_FILL.  Returns [Tq,Hq,D] in cdt."""
    tq, hq, d = q.shape
    hkv = keys.shape[1]
    out = torch.empty(tq, hq, d, dtype=cdt)
    for g in range(hkv):                              # per kv head: bounds the score tensor
        qg = q[:, g * group:(g + 1) * group, :].to(cdt)          # [Tq,G,D]
        s = torch.einsum("tgd,nd->gtn", qg, keys[:, g, :].to(cdt)) * sm_scale
        if fill_mask is not None:
            s = torch.where(fill_mask[None], torch.full_like(s, SLIDING_FILL), s)
        s = s.masked_fill(mask[None], float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, g * group:(g + 1) * group, :] = torch.einsum(
            "gtn,nd->tgd", p, vals[:, g, :].to(cdt))
    return out


def prefix_prefill(q, k, v, k_cache, v_cache, block_table, b_start_loc, b_seq_len,
                   cos_sin_cache, q_offset=None, q_mask=None, *,
                   pos_mode: int = POS_NATURAL, rotate_new_k: bool = True,
                   is_lazy=None, kv_cache_dtype: str = "auto",
                   k_scale=1.0, v_scale=1.0, sm_scale: Optional[float] = None,
                   sliding_window: int = 0, skip_decode: bool = False,
                   out: Optional[torch.Tensor] = None,
                   compute_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Deferred-RoPE prefix-prefill attention, eager.

    Modes (what selects them in the reference):
      pos_mode=POS_NATURAL, rotate_new_k=True    old_ops kernel, is_mepic=True
      pos_mode=POS_OFFSET,  rotate_new_k=True    old_ops kernel, is_mepic=False
      pos_mode=POS_BLOCK_UNIFORM, rotate_new_k=False   ops kernel, is_lazy[b] set;
          requests with is_lazy[b] == 0 take the vanilla branch: no rotation,
          no pad mask (ops:398-592).
    ``q`` is already rotated by the caller.  Rows the reference does not write
    (q_len==1 under skip_decode) keep the value they have in ``out``.
    """
    cdt = compute_dtype
    hq, d = q.shape[1], q.shape[2]
    hkv = k.shape[1]
    group = hq // hkv
    bs = v_cache.shape[3]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    table = cos_sin_cache.to(cdt) if cos_sin_cache is not None else None
    half = d // 2
    kc = _dequant(k_cache, kv_cache_dtype, k_scale, q.dtype)
    vc = _dequant(v_cache, kv_cache_dtype, v_scale, q.dtype)
    o = out if out is not None else torch.zeros(q.shape[0], hq, d, dtype=q.dtype)
    batch = b_seq_len.shape[0]
    for b in range(batch):
        qs = int(b_start_loc[b]); qe = int(b_start_loc[b + 1])
        q_len = qe - qs
        ctx_len = int(b_seq_len[b]) - q_len
        if q_len <= 0 or (skip_decode and q_len == 1):
            continue
        lazy_b = True if is_lazy is None else bool(is_lazy[b])
        npages = (ctx_len + bs - 1) // bs
        blocks = block_table[b, :npages]
        kg, vg = gather_pages(kc, vc, blocks)                       # [npages*bs,Hkv,D]
        kg = kg[:ctx_len].to(cdt); vg = vg[:ctx_len].to(cdt)
        n = torch.arange(ctx_len)
        page = n // bs
        slot = n % bs
        valid = torch.ones(ctx_len, dtype=torch.bool)
        rotate_ctx = True
        if pos_mode == POS_BLOCK_UNIFORM and not lazy_b:
            rotate_ctx = False                                      # vanilla branch
        else:
            if q_mask is not None:
                qm = q_mask[b, :npages].long()[page]
                valid = slot < (bs - qm)                            # old_ops:165-167,262-263
            if pos_mode == POS_NATURAL:
                pos = n
            else:
                qo = q_offset[b, :npages].long()[page]
                if pos_mode == POS_OFFSET:
                    pos = torch.where(qo != 0, qo - 1 + slot, n)
                else:
                    pos = torch.where(qo != 0, qo - 1, torch.zeros_like(qo))
        if rotate_ctx and ctx_len > 0:
            rows = table[pos]
            kg = neox_rotate(kg, rows[:, None, :half], rows[:, None, half:])
        # masked slots may hold anything (NaN included): they never reach the math
        kg = torch.where(valid[:, None, None], kg, torch.zeros_like(kg))
        vg = torch.where(valid[:, None, None], vg, torch.zeros_like(vg))
        kn = k[qs:qe].to(cdt); vn = v[qs:qe].to(cdt)
        if rotate_new_k and not (pos_mode == POS_BLOCK_UNIFORM and not lazy_b):
            rows = table[ctx_len + torch.arange(q_len)]             # old_ops:342-362
            kn = neox_rotate(kn, rows[:, None, :half], rows[:, None, half:])
        keys = torch.cat([kg, kn], dim=0)
        vals = torch.cat([vg, vn], dim=0)
        t = torch.arange(q_len)
        mask_ctx = (~valid)[None, :].expand(q_len, ctx_len)
        mask_new = t[None, :] > t[:, None]                          # old_ops:371-372
        mask = torch.cat([mask_ctx, mask_new], dim=1)
        fill = None
        if sliding_window and sliding_window > 0:
            f_ctx = ((ctx_len + t)[:, None] - n[None, :]) >= sliding_window
            f_new = (t[:, None] - t[None, :]) >= sliding_window
            fill = torch.cat([f_ctx, f_new], dim=1)
        o[qs:qe] = _attend(q[qs:qe], keys, vals, mask, fill, sm_scale, group, cdt).to(o.dtype)
    return o


def paged_decode(q, k_cache, v_cache, block_table, query_start_loc, seq_lens,
                 cos_sin_cache, q_mask=None, *, q_offset=None, is_lazy=None,
                 pos_mode: int = POS_NATURAL, kv_cache_dtype="auto",
                 k_scale=1.0, v_scale=1.0, sm_scale=None, sliding_window: int = 0,
                 out=None, compute_dtype=torch.float32):
    """q_len==1 rows: all seq_len keys come from the paged cache (the new token was
    written there by the caller); requests with q_len>1 are skipped.

    pos_mode=POS_NATURAL: un-rotated cache, key n rotated at n
      (old_ops/chunked_prefill_paged_decode.py:68-280).
    pos_mode=POS_BLOCK_UNIFORM: the reference de-rotates Q by q_offset-1 once per distinct
      offset (ops/models/llama_v1.py:231-262); rotating the page's keys forward by the same
      angle gives the same scores, which is how it is stated here.  An offset of 0 keeps the
      previous page's rotation.  Requests with is_lazy[b]==0 are not rotated and ignore q_mask."""
    cdt = compute_dtype
    hq, d = q.shape[1], q.shape[2]
    hkv = k_cache.shape[1]
    group = hq // hkv
    bs = v_cache.shape[3]
    half = d // 2
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    table = cos_sin_cache.to(cdt)
    kc = _dequant(k_cache, kv_cache_dtype, k_scale, q.dtype)
    vc = _dequant(v_cache, kv_cache_dtype, v_scale, q.dtype)
    o = out if out is not None else torch.zeros(q.shape[0], hq, d, dtype=q.dtype)
    for b in range(seq_lens.shape[0]):
        qs = int(query_start_loc[b]); qe = int(query_start_loc[b + 1])
        if qe - qs != 1:
            continue
        seq_len = int(seq_lens[b])
        npages = (seq_len + bs - 1) // bs
        kg, vg = gather_pages(kc, vc, block_table[b, :npages])
        kg = kg[:seq_len].to(cdt); vg = vg[:seq_len].to(cdt)
        n = torch.arange(seq_len)
        lazy_b = True if is_lazy is None else bool(is_lazy[b])
        vanilla = pos_mode == POS_BLOCK_UNIFORM and not lazy_b
        valid = torch.ones(seq_len, dtype=torch.bool)
        if q_mask is not None and not vanilla:
            valid = (n % bs) < (bs - q_mask[b, :npages].long()[n // bs])
        if not vanilla:
            if pos_mode == POS_NATURAL:
                pos = n
            else:
                # A page whose offset is 0 keeps the rotation of the page before it (the kernel only acts
                # when the value changes and does nothing for 0: `prev_rot_offset`, llama_v1.py:231-262);
                # before the first non-zero entry there is no rotation.  1 is "rotation by 0".
                carried = []
                last = 0
                for v in q_offset[b, :npages].tolist():
                    last = v if v != 0 else last
                    carried.append(last)
                qo = torch.tensor(carried, dtype=torch.long)[n // bs]
                pos = torch.where(qo != 0, qo - 1, torch.zeros_like(qo))
            rows = table[pos]
            kg = neox_rotate(kg, rows[:, None, :half], rows[:, None, half:])
        kg = torch.where(valid[:, None, None], kg, torch.zeros_like(kg))
        vg = torch.where(valid[:, None, None], vg, torch.zeros_like(vg))
        fill = None
        if sliding_window and sliding_window > 0:
            fill = (((seq_len - 1) - n) >= sliding_window)[None, :]
        o[qs:qe] = _attend(q[qs:qe], kg, vg, (~valid)[None, :], fill, sm_scale, group, cdt).to(o.dtype)
    return o


# --------------------------------------------------------------------------
# The step before the attention call: rotary embedding of the new tokens and the
# paged-cache write (rotary_embedding.py:40-94; backends/triton_attn.py:100-109).
# The two third-party ops behind them (vLLM rotary_embedding / reshape_and_cache) are absent
# from the reference tree: their published layouts are restated; the write is pinned by the
# round trip through gather_pages (the inverse index map the attention oracle reads with).
# --------------------------------------------------------------------------
def rotary_new_tokens(positions, query, key, table, *, q_only: bool, compute_dtype=torch.float32):
    """NeoX rotary of query [T,Hq,D] (and key [T,Hkv,D] unless q_only) at positions[t];
    returns new tensors in the inputs' dtypes (rotary_embedding.py:40-65 arithmetic, one rounding)."""
    tab = table.to(compute_dtype)
    q = rotate_at(query.to(compute_dtype), positions, tab).to(query.dtype)
    k = key if q_only else rotate_at(key.to(compute_dtype), positions, tab).to(key.dtype)
    return q, k


def paged_cache_write(key, value, k_cache, v_cache, slot_mapping, kv_cache_dtype="auto", k_scale=1.0, v_scale=1.0):
    """In place: token t -> slot_mapping[t] = block*BS + offset (negative: skipped);
    K[block, h, d // x, offset, d % x] = key[t, h, d]; V[block, h, d, offset] = value[t, h, d];
    fp8 caches (uint8 storage) hold (value / scale) saturated to +-448 as e4m3, or to +-57344 as e5m2."""
    nb, hkv, dx, bs, x = k_cache.shape
    fp8 = "fp8" in kv_cache_dtype

    def enc(t, scale):
        if not fp8:
            return t.to(k_cache.dtype)
        if kv_cache_dtype == "fp8_e5m2":
            return (t.float() / float(scale)).clamp(-57344.0, 57344.0).to(torch.float8_e5m2).view(torch.uint8)
        return (t.float() / float(scale)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    for t in range(key.shape[0]):
        slot = int(slot_mapping[t])
        if slot < 0:
            continue
        blk, off = slot // bs, slot % bs
        k_cache[blk, :, :, off, :] = enc(key[t], k_scale).view(hkv, dx, x)
        v_cache[blk, :, :, off] = enc(value[t], v_scale)


# --------------------------------------------------------------------------
# Block re-positioning (block_attn_vllm/utils.py:48-95): copy a paged block, un-rotate its keys
# from from_start+slot to position 0, rotate them to to_start+slot.  Two explicit steps.
# --------------------------------------------------------------------------
def reposition_blocks(k_cache, v_cache, items, table, compute_dtype=torch.float32):
    """In place on the caches; items = [(new_id, old_id, from_start, to_start)]."""
    nb, hkv, dx, bs, x = k_cache.shape
    d = dx * x
    half = d // 2
    tab = table.to(compute_dtype)
    src_k = {old: k_cache[old].clone() for _, old, _, _ in items}
    src_v = {old: v_cache[old].clone() for _, old, _, _ in items}
    for new_id, old_id, from_start, to_start in items:
        k = src_k[old_id].permute(0, 2, 1, 3).reshape(hkv, bs, d).to(compute_dtype)      # [Hkv, BS, D]
        o = torch.arange(bs)
        rf, rt = tab[from_start + o], tab[to_start + o]
        k = neox_rotate(k, rf[None, :, :half], -rf[None, :, half:])                  # R(-from)  utils.py:84
        k = neox_rotate(k, rt[None, :, :half], rt[None, :, half:])                   # R(+to)    utils.py:86
        k_cache[new_id] = k.to(k_cache.dtype).reshape(hkv, bs, dx, x).permute(0, 2, 1, 3)
        v_cache[new_id] = src_v[old_id]


# --------------------------------------------------------------------------
# Brute force (independent of everything above except the table rows):
# scalar loops in Python floats.  Tiny shapes only.
# --------------------------------------------------------------------------
def brute_force_prefix_prefill(q, k, v, k_cache, v_cache, block_table, b_start_loc,
                               b_seq_len, table, q_offset, q_mask, *, pos_mode,
                               rotate_new_k, is_lazy=None, sm_scale=None,
                               sliding_window=0):
    """Triple loop following the numbered restatement: for each (request, head, row)
    build the list of (score, value-vector) over valid context keys and visible new
    keys, then a two-pass softmax.  Python floats (double)."""
    tq_all, hq, d = q.shape
    hkv = k.shape[1]
    group = hq // hkv
    bs = v_cache.shape[3]
    x = k_cache.shape[4]
    half = d // 2
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    tab = table.double().tolist()
    qL = q.double().tolist(); kL = k.double().tolist(); vL = v.double().tolist()
    kcL = k_cache.double().tolist(); vcL = v_cache.double().tolist()
    out = torch.zeros(tq_all, hq, d, dtype=torch.float64)

    def rot(vec, p):
        c = tab[p][:half]; s = tab[p][half:2 * half]
        r = [0.0] * d
        for i in range(half):
            r[i] = vec[i] * c[i] - vec[i + half] * s[i]
            r[i + half] = vec[i] * s[i] + vec[i + half] * c[i]
        return r

    for b in range(len(b_seq_len)):
        qs = int(b_start_loc[b]); q_len = int(b_start_loc[b + 1]) - qs
        ctx_len = int(b_seq_len[b]) - q_len
        lazy_b = True if is_lazy is None else bool(is_lazy[b])
        vanilla = pos_mode == POS_BLOCK_UNIFORM and not lazy_b
        for h in range(hq):
            g = h // group
            for t in range(q_len):
                scores = []; vecs = []
                for n in range(ctx_len):
                    j, o_ = divmod(n, bs)
                    pb = int(block_table[b][j])
                    if not vanilla and q_mask is not None and o_ >= bs - int(q_mask[b][j]):
                        continue
                    kv = [kcL[pb][g][dd // x][o_][dd % x] for dd in range(d)]
                    vv = [vcL[pb][g][dd][o_] for dd in range(d)]
                    if not vanilla:
                        if pos_mode == POS_NATURAL:
                            p = n
                        else:
                            qo = int(q_offset[b][j])
                            if pos_mode == POS_OFFSET:
                                p = qo - 1 + o_ if qo != 0 else n
                            else:
                                p = qo - 1 if qo != 0 else 0
                        kv = rot(kv, p)
                    s = sm_scale * sum(a * c for a, c in zip(qL[qs + t][h], kv))
                    if sliding_window > 0 and (ctx_len + t) - n >= sliding_window:
                        s = SLIDING_FILL
                    scores.append(s); vecs.append(vv)
                for m in range(t + 1):
                    kv = kL[qs + m][g]
                    if rotate_new_k and not vanilla:
                        kv = rot(kv, ctx_len + m)
                    s = sm_scale * sum(a * c for a, c in zip(qL[qs + t][h], kv))
                    if sliding_window > 0 and t - m >= sliding_window:
                        s = SLIDING_FILL
                    scores.append(s); vecs.append(vL[qs + m][g])
                mx = max(scores)
                w = [math.exp(s - mx) for s in scores]
                z = sum(w)
                for dd in range(d):
                    out[qs + t, h, dd] = sum(wi * vi[dd] for wi, vi in zip(w, vecs)) / z
    return out
