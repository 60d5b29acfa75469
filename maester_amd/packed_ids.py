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


def boundaries_to_tensors(rows: Sequence[Sequence[Boundary]], device=None):
    """``(starts, lengths, counts)``: int32 ``[B, max_docs]`` (zero padded), ``[B, max_docs]``, ``[B]`` --
    the form the device-side generator takes (what a dataloader would ship instead of two ``[B,S]``
    int64 id tensors)."""
    n = max((len(r) for r in rows), default=0)
    starts = torch.zeros(len(rows), max(n, 1), dtype=torch.int32)
    lengths = torch.zeros(len(rows), max(n, 1), dtype=torch.int32)
    for b, row in enumerate(rows):
        for i, (_conv_id, start, length) in enumerate(row):
            starts[b, i], lengths[b, i] = int(start), int(length)
    counts = torch.tensor([len(r) for r in rows], dtype=torch.int32)
    return tuple(t.to(device) if device is not None else t for t in (starts, lengths, counts))


def device_packed_ids(starts: torch.Tensor, lengths: torch.Tensor, counts: torch.Tensor, seq_len: int):
    """``(position_ids, document_ids)``, int64 ``[B,S]``, built on the GPU from the rows' boundaries
    (same result as ``packed_collate_ids``; maester/sft/packed_dataset.py:138-185)."""
    from ctypes import c_void_p

    from . import _lib
    _lib.require_gpu(starts, "device_packed_ids")
    if starts.shape != lengths.shape or starts.dim() != 2 or counts.shape != (starts.shape[0],):
        raise ValueError(f"starts {tuple(starts.shape)}, lengths {tuple(lengths.shape)}, counts {tuple(counts.shape)}: "
                         "expected [B,N], [B,N], [B]")
    starts, lengths, counts = (t.to(torch.int32).contiguous() for t in (starts, lengths, counts))
    dev = starts.device
    B, N = starts.shape
    pos = torch.empty(B, seq_len, dtype=torch.int64, device=dev)
    doc = torch.empty(B, seq_len, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().ma_packed_ids_build(_lib.ptr(starts), _lib.ptr(lengths), _lib.ptr(counts), B, N, int(seq_len),
                                           _lib.ptr(pos), _lib.ptr(doc), _lib.current_stream(dev))
    _lib.check(rc)
    return pos, doc
