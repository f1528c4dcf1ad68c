"""Seeded synthetic workloads for the deferred-RoPE prefix-prefill operator.

Everything is generated on the CPU in float32 and then cast, so a CPU checker and
the GPU operator see identical values.  The construction follows the reference's
kernel test (``lazy_attn/tests/kernels/test_prefix_prefill.py:82-197``: paged cache
filled through a permuted block table, K cache ``[NB,Hkv,D/x,BS,x]``, V cache
``[NB,Hkv,D,BS]``) and its metadata producer
(``lazy_attn/lazy/core/sched/scheduler.py:758-781``), extended with a pool of cached
documents that requests reference in shuffled slot orders.

Three cache/rotation conventions ("variants"):

``natural``        K cached un-rotated, key n rotated at position n
                   (``old_ops/prefix_prefill.py:183-184``), new-token K rotated in
                   the operator.
``offset``         K cached un-rotated, each page carries its own position base
                   ``q_offset-1`` (``old_ops/prefix_prefill.py:186-191``): documents are
                   compacted, i.e. document d starts at total_padding + sum of the true
                   lengths before it.
``block_uniform``  K cached rotated at its document-local position; the operator adds
                   one rotation per page, ``q_offset-1`` (``ops/prefix_prefill.py:180-190``);
                   new-token K arrives rotated.  Same effective key positions as ``offset``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch

POS_NATURAL, POS_OFFSET, POS_BLOCK_UNIFORM = 0, 1, 2
_VARIANT = {"natural": POS_NATURAL, "offset": POS_OFFSET, "block_uniform": POS_BLOCK_UNIFORM}


def cos_sin_table(max_position: int, rotary_dim: int, base: float,
                  dtype: torch.dtype, llama3: Optional[dict] = None) -> torch.Tensor:
    """Host builder used only for synthetic inputs (float32 math, like the layer's
    own table; the operator-side builder lives in model_executor/rope)."""
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    inv = 1.0 / (base ** (idx / rotary_dim))
    if llama3 is not None:
        wl = 2 * math.pi / inv
        low_wl = llama3["orig_max_position"] / llama3["low_freq_factor"]
        high_wl = llama3["orig_max_position"] / llama3["high_freq_factor"]
        smooth = (llama3["orig_max_position"] / wl - llama3["low_freq_factor"]) / (
            llama3["high_freq_factor"] - llama3["low_freq_factor"])
        inv = torch.where(wl < high_wl, inv,
                          torch.where(wl > low_wl, inv / llama3["scaling_factor"],
                                      (1 - smooth) * inv / llama3["scaling_factor"] + smooth * inv))
    ang = torch.outer(torch.arange(max_position, dtype=torch.float32), inv)
    return torch.cat([ang.cos(), ang.sin()], dim=-1).to(dtype)


def _rotate(x: torch.Tensor, pos: torch.Tensor, table_f32: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    rows = table_f32[pos.long()]
    c, s = rows[:, None, :half], rows[:, None, half:]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1)


@dataclass
class Workload:
    name: str
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    block_table: torch.Tensor
    b_start_loc: torch.Tensor
    b_seq_len: torch.Tensor
    cos_sin_cache: torch.Tensor
    q_offset: torch.Tensor
    q_mask: torch.Tensor
    is_lazy: torch.Tensor
    k_scale: torch.Tensor
    v_scale: torch.Tensor
    kv_cache_dtype: str
    pos_mode: int
    rotate_new_k: bool
    max_query_len: int
    max_seq_len: int
    flops: float
    bytes: float
    # per request: un-rotated logical context K/V [ctx,Hkv,D] f32, effective key
    # positions [ctx], validity [ctx], un-rotated q and new k (f32) -- only when keep_aux
    aux: List[dict] = field(default_factory=list)

    def tensors(self):
        return ["q", "k", "v", "k_cache", "v_cache", "block_table", "b_start_loc",
                "b_seq_len", "cos_sin_cache", "q_offset", "q_mask", "is_lazy",
                "k_scale", "v_scale"]

    def to(self, device) -> "Workload":
        kw = {n: getattr(self, n).to(device) for n in self.tensors()}
        rest = {n: getattr(self, n) for n in self.__dataclass_fields__ if n not in kw}
        return Workload(**kw, **rest)


def make_workload(name: str, *, dtype: torch.dtype, hq: int, hkv: int, d: int,
                  theta: float, block_size: int, doc_lens: Sequence[int],
                  requests: Sequence[Sequence[int]], q_lens: Sequence[int],
                  variant: str = "natural", kv_cache_dtype: str = "auto",
                  seed: int = 0, spare_blocks: int = 4, keep_aux: bool = False,
                  llama3: Optional[dict] = None, value_scale: float = 1.0) -> Workload:
    """Build one batch.  ``doc_lens`` are the TRUE lengths of the pooled documents
    (each is right-padded to a whole number of pages, like the engine does);
    ``requests[b]`` lists pool document ids in slot order; ``q_lens[b]`` new tokens."""
    gen = torch.Generator().manual_seed(seed)
    bs = block_size
    pos_mode = _VARIANT[variant]
    fp8 = "fp8" in kv_cache_dtype
    elem = {torch.float32: 4, torch.bfloat16: 2, torch.float16: 2}[dtype]
    x = 16 if fp8 else 16 // elem
    padded = [((L + bs - 1) // bs) * bs for L in doc_lens]
    doc_pages = [p // bs for p in padded]
    ctx_lens = [sum(padded[i] for i in r) for r in requests]
    new_pages = [(ql + bs - 1) // bs for ql in q_lens]
    nb = sum(doc_pages) + sum(new_pages) + spare_blocks
    perm = torch.randperm(nb, generator=gen)
    # rows for every request position and (rotated-cache variant) every document-local position
    max_pos = max(max(c + ql for c, ql in zip(ctx_lens, q_lens)), max(padded)) + bs
    table = cos_sin_table(max_pos, d, theta, dtype, llama3)
    table_f32 = table.float()

    cache_dtype = torch.float32 if fp8 else dtype
    k_pages = torch.zeros(nb, bs, hkv, d, dtype=cache_dtype)
    v_pages = torch.zeros(nb, bs, hkv, d, dtype=cache_dtype)
    doc_blocks = []
    doc_k = []
    doc_v = []
    cur = 0
    for L, P in zip(doc_lens, doc_pages):
        blocks = perm[cur:cur + P]
        cur += P
        doc_blocks.append(blocks)
        # pad slots hold ordinary values too (they are real pad-token K/V in the engine)
        ku = torch.randn(P * bs, hkv, d, generator=gen) * value_scale
        vu = torch.randn(P * bs, hkv, d, generator=gen) * value_scale
        kc = ku
        if pos_mode == POS_BLOCK_UNIFORM:
            kc = _rotate(ku, torch.arange(P * bs), table_f32)   # cached at document-local position
        k_pages[blocks] = kc.view(P, bs, hkv, d).to(cache_dtype)
        v_pages[blocks] = vu.view(P, bs, hkv, d).to(cache_dtype)
        if keep_aux:
            doc_k.append(ku.to(dtype).float() if not fp8 else ku)
            doc_v.append(vu.to(dtype).float() if not fp8 else vu)

    k_scale = torch.tensor(1.0, dtype=torch.float32)
    v_scale = torch.tensor(1.0, dtype=torch.float32)
    if fp8:
        k_scale = (k_pages.abs().max() / 448.0).to(torch.float32)
        v_scale = (v_pages.abs().max() / 448.0).to(torch.float32)
        k_pages = (k_pages / k_scale).to(torch.float8_e4m3fn)
        v_pages = (v_pages / v_scale).to(torch.float8_e4m3fn)
    k_cache = k_pages.view(nb, bs, hkv, d // x, x).permute(0, 2, 3, 1, 4).contiguous()
    v_cache = v_pages.permute(0, 2, 3, 1).contiguous()
    if fp8:
        k_cache = k_cache.view(torch.uint8)
        v_cache = v_cache.view(torch.uint8)
    del k_pages, v_pages

    batch = len(requests)
    nbmax = max(sum(doc_pages[i] for i in r) + npg for r, npg in zip(requests, new_pages)) + 1
    block_table = torch.zeros(batch, nbmax, dtype=torch.int32)
    q_offset = torch.zeros(batch, nbmax, dtype=torch.int32)
    q_mask = torch.zeros(batch, nbmax, dtype=torch.int32)
    total_q = sum(q_lens)
    q = torch.empty(total_q, hq, d, dtype=torch.float32)
    k = torch.empty(total_q, hkv, d, dtype=torch.float32)
    v = torch.empty(total_q, hkv, d, dtype=torch.float32)
    b_start = [0]
    aux = []
    flops = 0.0
    for b, (r, ql) in enumerate(zip(requests, q_lens)):
        ctx = ctx_lens[b]
        pages = torch.cat([doc_blocks[i] for i in r]) if len(r) else torch.zeros(0, dtype=torch.long)
        npg = pages.numel()
        block_table[b, :npg] = pages.to(torch.int32)
        block_table[b, npg:npg + new_pages[b]] = perm[cur:cur + new_pages[b]].to(torch.int32)
        cur += new_pages[b]
        true = [doc_lens[i] for i in r]
        pad = [padded[i] for i in r]
        total_pad = sum(p - t for t, p in zip(true, pad))
        # per-document rotation base (compacted layout) and pad mask: scheduler.py:758-781
        bases = []
        rot = total_pad
        cursor = 0
        eff_pos = torch.empty(ctx, dtype=torch.long)
        valid = torch.ones(ctx, dtype=torch.bool)
        tok = 0
        for t_len, p_len in zip(true, pad):
            nblk = p_len // bs
            bases.append(rot)
            if pos_mode == POS_BLOCK_UNIFORM:
                q_offset[b, cursor:cursor + nblk] = rot + 1
            elif pos_mode == POS_OFFSET:
                q_offset[b, cursor:cursor + nblk] = (rot + 1 + bs * torch.arange(nblk)).to(torch.int32)
            q_mask[b, cursor + nblk - 1] = p_len - t_len
            if pos_mode == POS_NATURAL:
                eff_pos[tok:tok + p_len] = tok + torch.arange(p_len)
            else:
                eff_pos[tok:tok + p_len] = rot + torch.arange(p_len)
            valid[tok + t_len:tok + p_len] = False
            cursor += nblk
            tok += p_len
            rot += t_len
        if pos_mode != POS_NATURAL:
            q_offset[b, cursor] = 1
        qu = torch.randn(ql, hq, d, generator=gen) * value_scale
        knu = torch.randn(ql, hkv, d, generator=gen) * value_scale
        vn = torch.randn(ql, hkv, d, generator=gen) * value_scale
        qpos = ctx + torch.arange(ql)
        s = b_start[-1]
        q[s:s + ql] = _rotate(qu, qpos, table_f32)               # caller rotates Q (test:121-127)
        k[s:s + ql] = _rotate(knu, qpos, table_f32) if pos_mode == POS_BLOCK_UNIFORM else knu
        v[s:s + ql] = vn
        b_start.append(s + ql)
        flops += 4.0 * hq * d * ql * (ctx + (ql + 1) / 2.0)
        if keep_aux:
            aux.append(dict(
                k_ctx=torch.cat([doc_k[i] for i in r]) if len(r) else torch.zeros(0, hkv, d),
                v_ctx=torch.cat([doc_v[i] for i in r]) if len(r) else torch.zeros(0, hkv, d),
                eff_pos=eff_pos, valid=valid, q_pos=qpos,
                k_new_unrot=knu.to(dtype).float(), ctx_len=ctx))
    e_kv = 1 if fp8 else elem
    nbytes = (sum(ctx_lens) * hkv * d * 2 * e_kv + 2 * total_q * hq * d * elem +
              2 * total_q * hkv * d * elem + 3 * 4 * sum(c // bs for c in ctx_lens))
    return Workload(
        name=name, q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), k_cache=k_cache, v_cache=v_cache,
        block_table=block_table, b_start_loc=torch.tensor(b_start, dtype=torch.int32),
        b_seq_len=torch.tensor([c + ql for c, ql in zip(ctx_lens, q_lens)], dtype=torch.int32),
        cos_sin_cache=table, q_offset=q_offset, q_mask=q_mask,
        is_lazy=torch.ones(batch, dtype=torch.bool), k_scale=k_scale, v_scale=v_scale,
        kv_cache_dtype=kv_cache_dtype, pos_mode=pos_mode,
        rotate_new_k=pos_mode != POS_BLOCK_UNIFORM, max_query_len=max(q_lens),
        max_seq_len=max(c + ql for c, ql in zip(ctx_lens, q_lens)),
        flops=flops, bytes=float(nbytes), aux=aux)


LLAMA_1B = dict(hq=32, hkv=8, d=64, theta=500000.0)
LLAMA_8B = dict(hq=32, hkv=8, d=128, theta=500000.0)


def config(index: int, *, variant: str = "natural", keep_aux: bool = False,
           shrink: int = 1) -> Workload:
    """The five benchmark configurations.  Seed = 1000 + index.  ``shrink`` divides the
    number of documents / requests for quick parity runs (1 = full size)."""
    seed = 1000 + index
    g = torch.Generator().manual_seed(seed)
    if index == 1:
        return make_workload("c1_plumbing_fp32_1b_4x128_q64", dtype=torch.float32, **LLAMA_1B,
                             block_size=16, doc_lens=[128] * 4,
                             requests=[torch.randperm(4, generator=g).tolist()], q_lens=[64],
                             variant=variant, seed=seed, spare_blocks=28, keep_aux=keep_aux)
    if index == 2:
        nd = max(10 // shrink, 1)
        return make_workload("c2_8b_bf16_10x512_q128", dtype=torch.bfloat16, **LLAMA_8B,
                             block_size=16, doc_lens=[512] * nd,
                             requests=[torch.randperm(nd, generator=g).tolist()], q_lens=[128],
                             variant=variant, seed=seed, keep_aux=keep_aux)
    if index == 3:
        nreq = max(16 // shrink, 1)
        reqs = [torch.randperm(64, generator=g)[:20].tolist() for _ in range(nreq)]
        return make_workload("c3_8b_bf16_pool64x256_16req_x20_q64", dtype=torch.bfloat16, **LLAMA_8B,
                             block_size=16, doc_lens=[256] * 64, requests=reqs,
                             q_lens=[64] * nreq, variant=variant, seed=seed, keep_aux=keep_aux)
    if index == 4:
        nd = max(64 // shrink, 1)
        return make_workload("c4_8b_bf16_64x1024_q256", dtype=torch.bfloat16, **LLAMA_8B,
                             block_size=16, doc_lens=[1024] * nd,
                             requests=[torch.randperm(nd, generator=g).tolist()], q_lens=[256],
                             variant=variant, seed=seed, keep_aux=keep_aux)
    if index == 5:
        nreq = max(8 // shrink, 1)
        ndoc = max(32 // shrink, 1)
        doc_lens = [512] * (nreq * ndoc)
        reqs = [(b * ndoc + torch.randperm(ndoc, generator=g)).tolist() for b in range(nreq)]
        return make_workload("c5_8b_fp8kv_8req_32x512_q128", dtype=torch.bfloat16, **LLAMA_8B,
                             block_size=16, doc_lens=doc_lens, requests=reqs,
                             q_lens=[128] * nreq, variant=variant, kv_cache_dtype="fp8",
                             seed=seed, keep_aux=keep_aux)
    raise ValueError(f"no such config: {index}")


def decode_config(*, variant: str = "natural", nreq: int = 32, ndoc: int = 20, doc_len: int = 256) -> Workload:
    """q_len == 1 batch for the fused-rotary decode kernel: ``nreq`` requests, each over its own
    ``ndoc`` documents of ``doc_len`` tokens in shuffled slot order (no sharing between requests, so
    every K/V byte comes from HBM once), Llama-3-8B geometry, bf16.  The new token of every request is
    already in the paged cache, as the attention backend leaves it (backends/triton_attn.py:100-109)."""
    seed = 2000 + nreq
    g = torch.Generator().manual_seed(seed)
    reqs = [[b * ndoc + i for i in torch.randperm(ndoc, generator=g).tolist()] for b in range(nreq)]
    w = make_workload(f"d1_8b_bf16_decode_{nreq}req_{ndoc}x{doc_len}", dtype=torch.bfloat16, **LLAMA_8B,
                      block_size=16, doc_lens=[doc_len] * (nreq * ndoc), requests=reqs, q_lens=[1] * nreq,
                      variant=variant, seed=seed)
    hkv, d = LLAMA_8B["hkv"], LLAMA_8B["d"]
    x = w.k_cache.shape[4]
    bs = w.v_cache.shape[3]
    for b in range(nreq):
        qs = int(w.b_start_loc[b]); n = int(w.b_seq_len[b]) - 1
        pb = int(w.block_table[b, n // bs])
        w.k_cache[pb, :, :, n % bs, :] = w.k[qs].view(hkv, d // x, x)
        w.v_cache[pb, :, :, n % bs] = w.v[qs]
    keys = int(w.b_seq_len.sum())
    w.bytes = float(keys * hkv * d * 2 * 2 + 2 * w.q.numel() * 2)      # K + V once, Q in, O out
    w.flops = float(4 * LLAMA_8B["hq"] * d * keys)
    return w
