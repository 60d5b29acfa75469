"""position_ids / document_ids of a packed row, restated.  Test infrastructure only.

Follows maester/sft/packed_dataset.py:138-185 (``_generate_position_ids``,
``_generate_document_ids``): boundaries are (conv_id, start, length) triples; positions count from
0 inside each boundary and are 0 elsewhere; document ids are the enumerate index of the boundary and
-1 elsewhere (padding); both int64, clipped to ``seq_len``.  Batches are a plain ``torch.stack``
(maester/sft/dataset.py:198-220).
"""
from __future__ import annotations

import torch


def position_ids(boundaries, seq_len: int) -> torch.Tensor:
    out = torch.zeros(seq_len, dtype=torch.long)
    for _conv, start, length in boundaries:
        end = min(start + length, seq_len)
        for p in range(start, end):
            out[p] = p - start
    return out


def document_ids(boundaries, seq_len: int) -> torch.Tensor:
    out = torch.full((seq_len,), -1, dtype=torch.long)
    for doc, (_conv, start, length) in enumerate(boundaries):
        end = min(start + length, seq_len)
        for p in range(start, end):
            out[p] = doc
    return out
