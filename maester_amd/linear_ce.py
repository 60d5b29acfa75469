"""Fused linear + cross-entropy loss: the model's last step, without the [tokens, vocab] logits.

Counterpart of ``linear_cross_entropy(hidden_states.flatten(0, 1), embedder_weight, labels.flatten(0, 1),
impl=LinearCrossEntropyImpl.CCE)`` as ``GemmaTextModel.forward`` calls it (maester/models/gemma/model.py:762-769;
cut-cross-entropy 25.9.3, whose defaults apply: ``ignore_index=-100``, ``reduction="mean"`` over the tokens that
count, no soft cap, no shift), and of the materialising path it replaces, ``F.cross_entropy(pred.flatten(0, 1).float(),
labels.flatten(0, 1))`` (train.py:258-259).

Gemma's vocabulary is 262 208 wide: at 32 768 tokens the logits would be 17 GB in bf16 and their fp32 copy and
gradients several times that.  Here the tokens are taken a block of rows at a time: a library GEMM forms the block's
logits, one HIP kernel (``ma_ce_rows``) turns them in place into ``(softmax - onehot) / count`` while it writes the
rows' loss terms, and two more library GEMMs fold the block into ``d hidden`` and ``d weight``; the gradients are
complete when the forward returns, and the backward only scales them by the incoming gradient.  Like the reference's
loss, rows whose label is ``ignore_index`` are dropped before any GEMM (packed SFT masks the prompt tokens, often more
than half of a batch); finding them costs the one host synchronisation of the call.

Two properties differ from cut-cross-entropy by design: its backward skips blocks of the softmax whose entries are all
below 2^-12 (a bounded approximation; this gradient is the exact one, rounded to the activation dtype before the
gradient GEMMs as theirs is), and the logits of a block pass through the activation dtype between the GEMM and the
softmax, as they do in the reference's materialising path.
"""
from __future__ import annotations

import torch

from . import _lib

REDUCTIONS = ("mean", "sum")


def default_chunk_rows(vocab: int, elt: int, rows: int) -> int:
    """Rows per block: about 4 GiB of logits, a multiple of 256."""
    n = -(-(1 << 32) // (vocab * elt * 256)) * 256
    return max(1, min(n, rows))


def ce_rows(logits: torch.Tensor, targets: torch.Tensor, ignore_index: int = -100, softcap: float | None = None,
            grad_scale: torch.Tensor | None = None, write_grad: bool = True, lse: torch.Tensor | None = None,
            nll: torch.Tensor | None = None):
    """Runs the cross-entropy kernel on ``logits`` ``[rows, vocab]`` (rows may be strided) in place.

    Returns ``(lse, nll)`` fp32 ``[rows]`` (written into the given tensors when they are passed); with
    ``write_grad`` the logits are replaced by their gradient."""
    _lib.require_gpu(logits, "ce_rows")
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise ValueError("logits must be [rows, vocab] with unit stride along the vocabulary")
    rows, vocab = logits.shape
    if targets.shape != (rows,) or targets.dtype != torch.int64:
        raise ValueError("targets must be int64 [rows]")
    targets = targets.contiguous()
    for name, t in (("lse", lse), ("nll", nll)):
        if t is not None and (t.shape != (rows,) or t.dtype != torch.float32 or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous fp32 [rows] tensor")
    lse = torch.empty(rows, dtype=torch.float32, device=logits.device) if lse is None else lse
    nll = torch.empty(rows, dtype=torch.float32, device=logits.device) if nll is None else nll
    with torch.cuda.device(logits.device):
        rc = _lib.lib().ma_ce_rows(_lib.ptr(logits), logits.stride(0), _lib.ptr(targets), rows, vocab, int(ignore_index),
                                  float(softcap or 0.0), _lib.ptr(grad_scale), _lib.ptr(lse), _lib.ptr(nll),
                                  1 if write_grad else 0, _lib.dtype_code(logits.dtype), _lib.current_stream(logits.device))
    _lib.check(rc)
    return lse, nll


def transpose(x: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
    """``x.t().contiguous()`` of a contiguous 2-d tensor (bf16 or fp32) with the library's tile kernel; with
    ``dtype=torch.bfloat16`` an fp32 ``x`` is rounded on the way."""
    _lib.require_gpu(x, "transpose")
    if x.dim() != 2 or not x.is_contiguous():
        raise ValueError("transpose needs a contiguous 2-d tensor")
    dtype = x.dtype if dtype is None else dtype
    out = torch.empty(x.shape[1], x.shape[0], dtype=dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ma_transpose(_lib.ptr(x), _lib.ptr(out), x.shape[0], x.shape[1], _lib.dtype_code(x.dtype),
                                    _lib.dtype_code(dtype), _lib.current_stream(x.device))
    _lib.check(rc)
    return out


def _valid_count(targets, ignore_index, vocab):
    stats = torch.empty(2, dtype=torch.float32, device=targets.device)
    with torch.cuda.device(targets.device):
        rc = _lib.lib().ma_ce_valid_count(_lib.ptr(targets), targets.numel(), int(ignore_index), vocab, _lib.ptr(stats),
                                         _lib.current_stream(targets.device))
    _lib.check(rc)
    return stats


def _loss_reduce(nll, scale):
    loss = torch.empty((), dtype=torch.float32, device=nll.device)
    with torch.cuda.device(nll.device):
        rc = _lib.lib().ma_ce_loss_reduce(_lib.ptr(nll), nll.numel(), _lib.ptr(scale), _lib.ptr(loss),
                                         _lib.current_stream(nll.device))
    _lib.check(rc)
    return loss


def linear_ce_forward(e, c, targets, ignore_index=-100, softcap=None, reduction="mean", chunk_rows=None,
                      filter_ignored=True, need_de=True, need_dc=True):
    """Loss and gradients in one sweep over the tokens.

    ``e`` ``[N, K]``, ``c`` ``[V, K]`` (same dtype, bf16 or fp32), ``targets`` int64 ``[N]``.  Returns
    ``(loss fp32 scalar, de [N, K] or None, dc [V, K] or None)``; the gradients are those of ``loss``."""
    _lib.require_gpu(e, "linear_cross_entropy")
    if reduction not in REDUCTIONS:
        raise ValueError(f"reduction must be one of {REDUCTIONS}, got {reduction!r}")
    if e.dim() != 2 or c.dim() != 2 or e.shape[1] != c.shape[1]:
        raise ValueError(f"e {tuple(e.shape)} and c {tuple(c.shape)} must be [N, K] and [V, K]")
    if e.dtype != c.dtype or e.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("e and c must share a dtype, bf16 or fp32")
    n_all, k = e.shape
    vocab = c.shape[0]
    if targets.shape != (n_all,) or targets.dtype != torch.int64:
        raise ValueError("targets must be int64 [N]")
    if n_all == 0:
        raise ValueError("no tokens")
    e, c, targets = e.detach().contiguous(), c.detach().contiguous(), targets.contiguous()
    dev = e.device

    stats = _valid_count(targets, ignore_index, vocab)
    scale = stats[1:] if reduction == "mean" else None
    keep = None
    if filter_ignored:
        keep = torch.nonzero(targets != ignore_index).squeeze(1)      # the call's one host synchronisation
        if keep.numel() == n_all:
            keep = None
    e_kept = e if keep is None else e.index_select(0, keep)
    t_kept = targets if keep is None else targets.index_select(0, keep)
    n = e_kept.shape[0]
    want_grad = need_de or need_dc
    de_kept = torch.empty_like(e_kept) if need_de else None
    dc = dc_t = None
    if n == 0:
        loss = _loss_reduce(torch.zeros(1, dtype=torch.float32, device=dev), scale)
        return (loss, torch.zeros_like(e) if need_de else None, torch.zeros_like(c) if need_dc else None)

    step = int(chunk_rows) if chunk_rows else default_chunk_rows(vocab, e.element_size(), n)
    step = max(1, min(step, n))
    block = torch.empty(step, vocab, dtype=e.dtype, device=dev)
    # both operands of the d hidden GEMM contiguous along the vocabulary: more than twice the library's rate
    c_t = transpose(c) if need_de else None
    mixed = {"out_dtype": torch.float32} if e.dtype != torch.float32 else {}
    nll = torch.empty(n, dtype=torch.float32, device=dev)
    lse = torch.empty(n, dtype=torch.float32, device=dev)
    for r0 in range(0, n, step):
        r1 = min(r0 + step, n)
        x = block[: r1 - r0]
        torch.mm(e_kept[r0:r1], c.t(), out=x)
        ce_rows(x, t_kept[r0:r1], ignore_index, softcap, scale, want_grad, lse=lse[r0:r1], nll=nll[r0:r1])
        if need_de:
            torch.mm(x, c_t.t(), out=de_kept[r0:r1])
        if need_dc:
            # d weight^T [K, V] = e^T . d logits: with the hidden states transposed (small) this is the operand
            # order the library runs fastest for these shapes (9.1 against 10.5 ms per 8192-row block)
            e_t = transpose(e_kept[r0:r1])
            if n <= step:
                dc_t = torch.mm(e_t, x)
            elif dc_t is None:               # several blocks: summed in fp32 by the GEMMs, rounded once at the end
                dc_t = torch.mm(e_t, x, **mixed)
            else:
                torch.addmm(dc_t, e_t, x, out=dc_t, **mixed)
    if need_dc:
        dc = transpose(dc_t, c.dtype)        # back to [V, K], rounded to the parameter's dtype on the way
    loss = _loss_reduce(nll, scale)
    de = de_kept
    if need_de and keep is not None:
        de = torch.zeros_like(e)
        de.index_copy_(0, keep, de_kept)
    return loss, de, dc


class _LinearCrossEntropyFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, e, c, targets, ignore_index, softcap, reduction, chunk_rows, filter_ignored):
        need_de, need_dc = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        loss, de, dc = linear_ce_forward(e, c, targets, ignore_index, softcap, reduction, chunk_rows, filter_ignored,
                                         need_de, need_dc)
        ctx.save_for_backward(*(t for t in (de, dc) if t is not None))
        ctx.has = (de is not None, dc is not None)
        return loss

    @staticmethod
    def backward(ctx, dloss):
        saved = list(ctx.saved_tensors)
        de = saved.pop(0) if ctx.has[0] else None
        dc = saved.pop(0) if ctx.has[1] else None
        return (de * dloss.to(de.dtype) if de is not None else None, dc * dloss.to(dc.dtype) if dc is not None else None,
                None, None, None, None, None, None)


def linear_cross_entropy(e: torch.Tensor, c: torch.Tensor, targets: torch.Tensor, ignore_index: int = -100,
                         softcap: float | None = None, reduction: str = "mean", chunk_rows: int | None = None,
                         filter_ignored: bool = True) -> torch.Tensor:
    """``cross_entropy(e @ c.T, targets)`` as an fp32 scalar, differentiable in ``e`` and ``c``.

    ``e`` ``[..., K]`` hidden states, ``c`` ``[V, K]`` classifier (Gemma: the tied embedding table), ``targets``
    int64 of the leading shape of ``e``.  ``reduction``: ``"mean"`` over the targets that are not ``ignore_index``
    (NaN when there is none, as torch gives) or ``"sum"``."""
    lead = e.shape[:-1]
    if targets.shape != lead:
        raise ValueError(f"targets shape {tuple(targets.shape)} != leading shape of e {tuple(lead)}")
    return _LinearCrossEntropyFn.apply(e.reshape(-1, e.shape[-1]), c, targets.reshape(-1), int(ignore_index),
                                       None if softcap is None else float(softcap), reduction, chunk_rows,
                                       bool(filter_ignored))
