"""QK-RMSNorm + RoPE prologue of the Gemma attention, restated in torch (CPU).
Test infrastructure only.

Follows maester/models/gemma/model.py:
  precompute_freqs_cis (84-94): inv_freq = 1/(theta**(arange(0,D,2)[:D/2].float()/D)) / factor;
      angle = outer(arange(end), inv_freq).float(); table = polar(1, angle);
  apply_rotary_emb (97-106): half-split RoPE in fp32 (x1 = x[..., :D/2], x2 = x[..., D/2:]),
      out = [x1*c - x2*s, x1*s + x2*c], cast back to x's dtype;
  RMSNorm._compute_norm / forward (135-172): y = x.float() * rsqrt(mean(x^2) + eps) * (1 + w.float()),
      cast back to x's dtype; weight initialised to zeros (146);
  GemmaAttention.forward (366-372): norm(q), norm(k), then rope(q), rope(k); v untouched;
  GemmaTextModel.forward (680-687, 744-747): table rows gathered by position_ids, default arange(S).
"""
from __future__ import annotations

import torch


def rope_tables(head_dim: int, end: int, theta: float = 10000.0, rope_scaling_factor: float = 1.0):
    """(cos, sin), each [end, head_dim/2] fp32 -- the real and imaginary part of the reference's
    complex64 ``freqs_cis`` table, built with the same expression (model.py:84-94)."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: (head_dim // 2)].float() / head_dim))
    freqs = freqs / rope_scaling_factor
    t = torch.arange(end)
    ang = torch.outer(t, freqs).float()
    cis = torch.polar(torch.ones_like(ang), ang)       # complex64, as the reference stores it
    return cis.real.contiguous(), cis.imag.contiguous()


def rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, position_ids: torch.Tensor | None):
    """x [B,S,H,D]; cos/sin [P,D/2]; position_ids [B,S] int64 or None (-> arange)."""
    B, S, H, D = x.shape
    if position_ids is None:
        position_ids = torch.arange(S).unsqueeze(0).expand(B, S)
    c = cos[position_ids][:, :, None, :].to(torch.float64 if x.dtype == torch.float64 else torch.float32)
    s = sin[position_ids][:, :, None, :].to(c.dtype)
    xf = x.to(c.dtype)
    x1, x2 = xf[..., : D // 2], xf[..., D // 2:]
    out = torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1)
    return out.to(x.dtype)


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6, add_unit_offset: bool = True):
    """Gemma RMSNorm over the last dim, fp32 math (fp64 if x is fp64), cast back (model.py:155-172)."""
    if weight is None:
        return x
    wd = torch.float64 if x.dtype == torch.float64 else torch.float32
    xf = x.to(wd)
    normed = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    g = (1 + weight.to(wd)) if add_unit_offset else weight.to(wd)
    return (normed * g).to(x.dtype)


def prologue(xq, xk, q_w, k_w, cos, sin, position_ids, eps=1e-6, add_unit_offset=True, cast_between=True):
    """norm -> rope on q and k.  ``cast_between=True`` reproduces the reference's cast to the IO
    dtype after the norm (model.py:172) before RoPE re-upcasts (model.py:99); ``False`` keeps the
    intermediate in fp32 like a fused kernel does (differs by at most 1 ulp of the IO dtype)."""
    def one(x, w):
        if w is None:
            return rope_apply(x, cos, sin, position_ids)
        if cast_between:
            return rope_apply(rms_norm(x, w, eps, add_unit_offset), cos, sin, position_ids)
        y = rms_norm(x.float(), w, eps, add_unit_offset)
        return rope_apply(y, cos, sin, position_ids).to(x.dtype)
    return one(xq, q_w), one(xk, k_w)
