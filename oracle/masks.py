"""Mask predicates of the Gemma packed-SFT path, restated.  Test infrastructure only.

Follows maester/models/gemma/model.py:203-256:
  causal_mask (203-204)              q >= kv
  sliding_window_causal (206-207)    (q >= kv) & (q - kv <= W)      -- W inclusive
  make_document_mask_wrapper (216-256)  doc[b,q] == doc[b,kv] & base; ``None`` ids -> base
Padding id -1 is an ordinary id (it equals itself).  The head index is ignored.
"""
from __future__ import annotations

import numpy as np
import torch


def allowed(document_ids, b: int, q: int, kv: int, causal: bool = True, window: int | None = None) -> bool:
    """Scalar predicate, the form the reference's truth-table tests call."""
    ok = True
    if causal:
        ok = ok and (q >= kv)
    if window is not None:
        ok = ok and (q >= kv) and (q - kv <= window)
    if document_ids is not None:
        ok = ok and bool(document_ids[b][q] == document_ids[b][kv])
    return bool(ok)


def dense_mask_np(document_ids, B: int, S: int, causal: bool = True, window: int | None = None) -> np.ndarray:
    """Dense bool [B, S, S] (what torch ``create_mask`` materialises, model.py:259-272)."""
    q = np.arange(S)[:, None]
    kv = np.arange(S)[None, :]
    base = np.ones((S, S), dtype=bool)
    if causal:
        base &= q >= kv
    if window is not None:
        base &= (q >= kv) & (q - kv <= window)
    out = np.broadcast_to(base, (B, S, S)).copy()
    if document_ids is not None:
        ids = np.asarray(document_ids).astype(np.int64)
        out &= ids[:, :, None] == ids[:, None, :]
    return out


def dense_mask(document_ids, B: int, S: int, causal: bool = True, window: int | None = None,
               device="cpu") -> torch.Tensor:
    """Dense bool torch mask [B, 1, S, S]."""
    q = torch.arange(S, device=device)[:, None]
    kv = torch.arange(S, device=device)[None, :]
    base = torch.ones(S, S, dtype=torch.bool, device=device)
    if causal:
        base &= q >= kv
    if window is not None:
        base &= (q >= kv) & (q - kv <= window)
    out = base[None].expand(B, S, S).clone()
    if document_ids is not None:
        ids = document_ids.to(device=device, dtype=torch.long)
        out &= ids[:, :, None] == ids[:, None, :]
    return out[:, None]


def make_mask_mod(document_ids, causal: bool = True, window: int | None = None):
    """A torch FlexAttention ``mask_mod`` with the restated predicate (for torch's own
    ``create_block_mask`` / ``flex_attention``); counterpart of model.py:216-256."""
    ids = None if document_ids is None else document_ids.detach().to(torch.long)

    def mod(b, h, q_idx, kv_idx):
        ok = q_idx >= kv_idx if causal else (q_idx == q_idx)
        if window is not None:
            ok = ok & (q_idx >= kv_idx) & (q_idx - kv_idx <= window)
        if ids is not None:
            ok = ok & (ids[b, q_idx] == ids[b, kv_idx])
        return ok

    return mod
