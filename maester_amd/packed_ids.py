"""position_ids / document_ids of packed rows (host side of the input contract).

Counterpart of ``PackedSFTDataset._generate_position_ids`` / ``_generate_document_ids``
(maester/sft/packed_dataset.py:138-185) and of the id part of ``packed_collate_fn``
(maester/sft/dataset.py:198-220).  ``boundaries`` are ``(conv_id, start, length)`` triples.
"""
from __future__ import annotations

from typing import Iterable, Sequence, Tuple

import torch

Boundary = Tuple[int, int, int]


def generate_position_ids(boundaries: Iterable[Boundary], seq_len: int) -> torch.Tensor:
    """Positions restart at 0 at every boundary; tokens outside any boundary (padding) get 0."""
    position_ids = torch.zeros(seq_len, dtype=torch.long)
    for _conv_id, start, length in boundaries:
        end = min(start + length, seq_len)
        if end > start:
            position_ids[start:end] = torch.arange(end - start)
    return position_ids


def generate_document_ids(boundaries: Iterable[Boundary], seq_len: int) -> torch.Tensor:
    """The i-th boundary gets id i; padding gets -1 (an ordinary id for the mask: padding tokens
    attend causally among themselves)."""
    document_ids = torch.full((seq_len,), -1, dtype=torch.long)
    for doc_id, (_conv_id, start, length) in enumerate(boundaries):
        end = min(start + length, seq_len)
        if end > start:
            document_ids[start:end] = doc_id
    return document_ids


def packed_collate_ids(rows: Sequence[Sequence[Boundary]], seq_len: int):
    """Stack per-row ids into int64 ``[B,S]`` tensors: ``(position_ids, document_ids)``."""
    pos = torch.stack([generate_position_ids(b, seq_len) for b in rows])
    doc = torch.stack([generate_document_ids(b, seq_len) for b in rows])
    return pos, doc
