"""Gemma's RMSNorm over the model dimension, with the residual add of the post-norms fused in.

Counterpart of ``RMSNorm`` (maester/models/gemma/model.py:135-175) as ``Gemma2DecoderLayer.forward``
uses it (model.py:488-508): ``rms_norm(x, w)`` for the norms that feed a GEMM
(``input_layernorm``, ``pre_feedforward_layernorm``) and ``rms_norm(x, w, residual=r)`` for
``r + post_norm(x)`` (``post_attention_layernorm``, ``post_feedforward_layernorm``).
"""
from __future__ import annotations

import torch
from torch import nn

from . import _lib


def _rows(x: torch.Tensor):
    dim = x.shape[-1]
    return x.numel() // dim, dim


def rmsnorm_forward(x, weight, residual=None, eps=1e-6, add_unit_offset=True, need_rstd=True):
    """Returns ``(out, rstd)``; ``out`` has the shape and dtype of ``x``."""
    _lib.require_gpu(x, "rmsnorm_forward")
    x = x.contiguous()
    rows, dim = _rows(x)
    w = weight.detach().float().contiguous()
    if w.shape != (dim,):
        raise ValueError(f"weight shape {tuple(w.shape)} != ({dim},)")
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("residual must have the shape and dtype of x")
        residual = residual.contiguous()
    out = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device) if need_rstd else None
    with torch.cuda.device(x.device):
        rc = _lib.lib().ma_rmsnorm_fwd(_lib.ptr(x), _lib.ptr(residual), _lib.ptr(w), _lib.ptr(out), _lib.ptr(rstd), rows, dim,
                                      float(eps), 1 if add_unit_offset else 0, _lib.dtype_code(x.dtype),
                                      _lib.current_stream(x.device))
    _lib.check(rc)
    return out, rstd


def rmsnorm_backward(x, weight, rstd, dout, add_unit_offset=True):
    """Returns ``(dx, dweight fp32)``."""
    x, dout = x.contiguous(), dout.contiguous()
    rows, dim = _rows(x)
    w = weight.detach().float().contiguous()
    L = _lib.lib()
    ws_bytes = L.ma_rmsnorm_bwd_workspace_bytes(rows, dim)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=x.device)
    dx = torch.empty_like(x)
    dw = torch.empty(dim, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.ma_rmsnorm_bwd(_lib.ptr(x), _lib.ptr(w), _lib.ptr(rstd), _lib.ptr(dout), _lib.ptr(dx), _lib.ptr(dw), _lib.ptr(ws),
                              ws_bytes, rows, dim, 1 if add_unit_offset else 0, _lib.dtype_code(x.dtype),
                              _lib.current_stream(x.device))
    _lib.check(rc)
    return dx, dw


class _RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, residual, eps, add_unit_offset):
        out, rstd = rmsnorm_forward(x, weight, residual, eps, add_unit_offset)
        ctx.save_for_backward(x, weight, rstd)
        ctx.unit, ctx.has_residual = add_unit_offset, residual is not None
        return out

    @staticmethod
    def backward(ctx, dout):
        x, weight, rstd = ctx.saved_tensors
        dx, dw = rmsnorm_backward(x, weight, rstd, dout, ctx.unit)
        return dx, dw.to(weight.dtype), (dout if ctx.has_residual else None), None, None


def rms_norm(x, weight, residual=None, eps: float = 1e-6, add_unit_offset: bool = True):
    """``x * rsqrt(mean(x^2) + eps) * (1 + weight)`` in fp32, cast to the dtype of ``x``; with
    ``residual`` the result is ``residual + that`` (differentiable in x, weight and residual)."""
    return _RMSNormFn.apply(x, weight, residual, float(eps), bool(add_unit_offset))


class RMSNorm(nn.Module):
    """Drop-in for maester's ``RMSNorm`` (same parameter, zeros-initialised, scale ``1 + weight``);
    ``forward(x, residual=None)`` adds the residual of a post-norm in the same pass."""

    def __init__(self, dim: int, eps: float = 1e-6, add_unit_offset: bool = True):
        super().__init__()
        self.eps = eps
        self.add_unit_offset = add_unit_offset
        self.weight = nn.Parameter(torch.zeros(dim))

    def forward(self, x, residual=None):
        return rms_norm(x, self.weight, residual, self.eps, self.add_unit_offset)

    def reset_parameters(self):
        nn.init.zeros_(self.weight)
