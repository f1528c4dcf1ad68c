"""Rotation metadata of a request: ``q_offset`` / ``q_mask`` per page.

Same arithmetic as ``lazy_attn/lazy/core/sched/scheduler.py:758-787`` and
``lazy_attn/lazy/utils/rotation.py:15-37``, taking the document lengths directly
instead of a request object.
"""
from __future__ import annotations

from typing import Sequence

MAX_PACKED_Q_OFFSET = 0xFFFF


def metadata_for_lazy_attention(document_lens: Sequence[int], document_lens_padded: Sequence[int],
                                block_size: int) -> tuple[list[int], list[int]]:
    n_pages = sum(document_lens_padded) // block_size + 1      # + the query page
    q_offset = [0] * n_pages
    q_mask = [0] * n_pages
    shift = sum(document_lens_padded) - sum(document_lens)     # all padding, up front
    page = 0
    for true_len, padded_len in zip(document_lens, document_lens_padded):
        pages = padded_len // block_size
        q_offset[page:page + pages] = [shift + 1] * pages      # +1: 0 stays "no offset"
        page += pages
        q_mask[page - 1] = padded_len - true_len
        shift += true_len
    q_offset[page] = 1                                          # query page: global orientation
    return q_offset, q_mask


def metadata_for_mepic(document_lens, document_lens_padded, block_size):
    q_offset, q_mask = metadata_for_lazy_attention(document_lens, document_lens_padded, block_size)
    return [0] * len(q_offset), q_mask


def max_rotation_offset(document_lens: Sequence[int], document_lens_padded: Sequence[int]) -> int:
    if not document_lens:
        return 0
    return (sum(document_lens_padded) - sum(document_lens)) + sum(document_lens[:-1]) + 1


def build_rotation_metadata_device(document_lens, document_lens_padded, block_size: int, q_offset, q_mask, *,
                                   mepic: bool = False, max_offset=None) -> None:
    """Batch form on the GPU: ``document_lens[b]`` / ``document_lens_padded[b]`` are request b's lists
    (or, with ``doc_start`` semantics, already-flattened int32 device tensors passed as a 3-tuple
    ``(lens, padded, doc_start)`` in ``document_lens``).  Fills the int32 device buffers ``q_offset`` and
    ``q_mask`` ``[batch, row_len]`` in place -- what ``_refresh_lazy_metadata_buffers``
    (``lazy_attn/lazy/worker/gpu_model_runner.py:193-239``) does with a host loop and two copies."""
    import torch
    from ... import _ffi
    dev = q_offset.device
    if dev.type != "cuda":
        raise RuntimeError("build_rotation_metadata_device writes GPU buffers; there is no CPU path")
    if isinstance(document_lens, tuple):
        lens, padded, start = document_lens
    else:
        flat, flat_p, start_l = [], [], [0]
        for a, b in zip(document_lens, document_lens_padded):
            if len(a) != len(b):
                raise ValueError("document_lens and document_lens_padded differ in length")
            flat += list(a); flat_p += list(b); start_l.append(len(flat))
        need = max((sum(b) // block_size + 1 for b in document_lens_padded), default=1)
        if need > q_offset.shape[1]:
            raise ValueError(f"a request needs {need} pages, the buffers hold {q_offset.shape[1]}")
        host = torch.tensor(flat + flat_p + start_l, dtype=torch.int32).pin_memory()
        both = host.to(dev, non_blocking=True)                       # one small copy
        n = len(flat)
        lens, padded, start = both[:n], both[n:2 * n], both[2 * n:]
    batch = start.numel() - 1
    assert q_offset.dtype == torch.int32 and q_mask.dtype == torch.int32
    assert q_offset.shape == q_mask.shape and q_offset.stride() == q_mask.stride() and q_offset.stride(1) == 1
    assert batch <= q_offset.shape[0]
    rc = _ffi.lib().lazyattn_build_rotation_metadata(
        lens.data_ptr(), padded.data_ptr(), start.data_ptr(), batch, block_size, int(mepic), q_offset.data_ptr(),
        q_mask.data_ptr(), q_offset.stride(0), q_offset.shape[1], None if max_offset is None else max_offset.data_ptr(),
        torch.cuda.current_stream(dev).cuda_stream)
    _ffi.check(rc, "lazyattn_build_rotation_metadata")


def pack_block_table_device(block_table, q_offset, q_mask, packed, rows=None) -> None:
    """``packed[r, j] = block << 32 | q_offset << 16 | q_mask`` on the GPU for ``rows`` (an int32 device tensor or a
    list; ``None`` = every row of ``packed``): ``_rebuild_packed_block_table``
    (``lazy_attn/lazy/worker/gpu_model_runner.py:296-340``), full or delta, in one launch."""
    import torch
    from ... import _ffi
    dev = packed.device
    if dev.type != "cuda":
        raise RuntimeError("pack_block_table_device writes a GPU buffer; there is no CPU path")
    assert block_table.dtype == torch.int32 and q_offset.dtype == torch.int32 and q_mask.dtype == torch.int32
    assert packed.dtype == torch.int64 and q_offset.stride() == q_mask.stride()
    assert block_table.stride(1) == 1 and q_offset.stride(1) == 1 and packed.stride(1) == 1
    row_len = min(packed.shape[1], block_table.shape[1], q_offset.shape[1])
    if rows is not None and not torch.is_tensor(rows):
        rows = torch.tensor(list(rows), dtype=torch.int32, device=dev)
    n_rows = packed.shape[0] if rows is None else rows.numel()
    rc = _ffi.lib().lazyattn_pack_block_table(
        block_table.data_ptr(), block_table.stride(0), q_offset.data_ptr(), q_mask.data_ptr(), q_offset.stride(0),
        None if rows is None else rows.data_ptr(), n_rows, row_len, packed.data_ptr(), packed.stride(0),
        torch.cuda.current_stream(dev).cuda_stream)
    _ffi.check(rc, "lazyattn_pack_block_table")
