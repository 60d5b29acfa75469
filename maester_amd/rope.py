"""RoPE tables for the fused prologue.

Counterpart of ``precompute_freqs_cis`` (maester/models/gemma/model.py:84-94) and its registration
(model.py:588-623: ``end = 2 * max_seq_len``; local theta with factor 1, global theta with
``rope_scaling['factor']``).  The reference keeps one complex64 table; the kernel gathers rows of
its real and imaginary parts, kept as two fp32 tables built with the same torch expression so the
values are the reference's bit for bit.
"""
from __future__ import annotations

import torch


def precompute_rope_tables(head_dim: int, end: int, theta: float = 10000.0, rope_scaling_factor: float = 1.0,
                           device=None):
    """Returns ``(cos, sin)``, each fp32 ``[end, head_dim // 2]``."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: (head_dim // 2)].float() / head_dim))
    freqs = freqs / rope_scaling_factor
    t = torch.arange(end, device=freqs.device)
    freqs = torch.outer(t, freqs).float()
    cis = torch.polar(torch.ones_like(freqs), freqs)
    cos, sin = cis.real.contiguous(), cis.imag.contiguous()
    if device is not None:
        cos, sin = cos.to(device), sin.to(device)
    return cos, sin
