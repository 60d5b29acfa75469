"""CPU oracle of the fused linear + cross-entropy loss.  TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Restates, in numpy fp64, what ``linear_cross_entropy(hidden.flatten(0, 1), embedder_weight, labels.flatten(0, 1))``
computes at its call site (maester/models/gemma/model.py:762-769) and what the reference's materialising path
computes (train.py:258-259: ``F.cross_entropy(pred.flatten(0, 1).float(), labels.flatten(0, 1))``):

    x = e @ c.T;   lse_i = log sum_j exp(x_ij);   nll_i = lse_i - x_{i, t_i}
    loss = sum_i nll_i / #{i : t_i != ignore_index}      (rows with t_i == ignore_index dropped)
    dx_ij = (softmax(x_i)_j - [j == t_i]) / count;   de = dx @ c;   dc = dx.T @ e

The loss itself lives in a third-party dependency that is absent from the reference tree and from this image:
cut-cross-entropy 25.9.3 (git b7a02791, uv.lock:206-208).  Its published algorithm is this formula, evaluated
blockwise, with one documented approximation in the backward (blocks of the softmax below 2^-12 are skipped).
Pinned in ``tests/test_oracle_linear_ce.py`` against ``torch.nn.functional.cross_entropy`` (the routine the
reference's other path calls, including ``ignore_index`` as tests/test_packed_sft.py:300-310 uses it), against
scipy's ``logsumexp``, closed forms (uniform logits give log V; a dominant logit gives ~0), the zero row sum of the
gradient, and central finite differences of the loss.  The gradient filter of cut-cross-entropy is not restated:
that part of its behaviour is "parity unpinned".
"""
from __future__ import annotations

import numpy as np


def round_bf16(a: np.ndarray) -> np.ndarray:
    """Round fp32 values to the nearest bf16 (ties to even), returned as fp32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def linear_cross_entropy(e, c, targets, ignore_index=-100, softcap=None, reduction="mean", logits_bf16=False):
    """Returns ``dict(loss, lse, nll, de, dc, count)`` in fp64.

    ``logits_bf16`` rounds the logits to bf16 before the softmax, which is what the reference's materialising path
    does for a bf16 model (the GEMM's output dtype); the gradient is then the gradient with respect to the rounded
    logits carried through the GEMMs unchanged."""
    e64, c64 = np.asarray(e, dtype=np.float64), np.asarray(c, dtype=np.float64)
    t = np.asarray(targets, dtype=np.int64)
    n, vocab = e64.shape[0], c64.shape[0]
    x = e64 @ c64.T
    if logits_bf16:
        x = round_bf16(x.astype(np.float32)).astype(np.float64)
    if softcap:
        th = np.tanh(x / softcap)
        x, dcap = softcap * th, 1.0 - th * th
    else:
        dcap = 1.0
    counts = (t != ignore_index) & (t >= 0) & (t < vocab)
    m = x.max(axis=1, keepdims=True)
    lse = (m + np.log(np.exp(x - m).sum(axis=1, keepdims=True)))[:, 0]
    picked = x[np.arange(n), np.where(counts, t, 0)]
    nll = np.where(counts, lse - picked, 0.0)
    count = int(counts.sum())
    if reduction == "mean":
        scale = 1.0 / count if count else float("nan")
    elif reduction == "sum":
        scale = 1.0
    else:
        raise ValueError(reduction)
    loss = nll.sum() * scale
    dx = np.exp(x - lse[:, None])
    dx[np.arange(n), np.where(counts, t, 0)] -= 1.0
    dx = dx * counts[:, None] * (scale if count else 0.0) * dcap
    return dict(loss=loss, lse=lse, nll=nll, de=dx @ c64, dc=dx.T @ e64, dx=dx, count=count)
