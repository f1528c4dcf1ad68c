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
