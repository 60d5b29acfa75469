"""Pins the prologue oracle: RoPE table and half-split rotation against the HF rotate_half form
(as maester tests/test_rope.py does), Gemma RMSNorm against transformers' Gemma3RMSNorm and
invariants."""
import math

import pytest
import torch

from oracle import prologue as P


def _rotate_half(x):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def test_rope_table_equals_polar_form():
    # model.py:84-94 builds polar(1, angle); cos/sin must be its real/imag parts bit for bit
    D, end, theta, factor = 256, 512, 1e6, 8.0
    freqs = 1.0 / (theta ** (torch.arange(0, D, 2)[: D // 2].float() / D)) / factor
    ang = torch.outer(torch.arange(end), freqs).float()
    cis = torch.polar(torch.ones_like(ang), ang)
    cos, sin = P.rope_tables(D, end, theta, factor)
    assert torch.equal(cos, cis.real) and torch.equal(sin, cis.imag)
    # ... and those are cos/sin of the angle (torch.polar and torch.cos differ by at most an ulp)
    assert torch.allclose(cos, torch.cos(ang), atol=2e-7, rtol=0) and torch.allclose(sin, torch.sin(ang), atol=2e-7, rtol=0)
    assert torch.allclose(cos.double(), torch.cos(ang.double()), atol=2e-7, rtol=0)
    assert cos.shape == (end, D // 2) and cos.dtype == torch.float32
    # closed form of a few entries
    assert abs(float(cos[3, 0]) - math.cos(3 / 8.0)) < 1e-6
    i = 5
    assert abs(float(sin[7, i]) - math.sin(7 * theta ** (-2 * i / D) / factor)) < 1e-6


def test_rope_matches_hf_rotate_half():
    # tests/test_rope.py:120-138: theta=5e5, D=128, S=512, atol 1e-5 vs HF LlamaRotaryEmbedding form
    torch.manual_seed(0)
    S, H, D, theta = 512, 4, 128, 500000.0
    x = torch.randn(1, S, H, D)
    cos, sin = P.rope_tables(D, S, theta)
    got = P.rope_apply(x, cos, sin, None)
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.int64).float() / D))
    ang = torch.arange(S).float()[:, None] * inv_freq[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    c, s = emb.cos()[None, :, None, :], emb.sin()[None, :, None, :]
    want = x * c + _rotate_half(x) * s
    assert torch.allclose(got, want, atol=1e-5)
    try:
        from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding, LlamaConfig
        cfg = LlamaConfig(hidden_size=H * D, num_attention_heads=H, max_position_embeddings=S, rope_theta=theta)
        if hasattr(cfg, "rope_parameters") and isinstance(getattr(cfg, "rope_parameters", None), dict):
            cfg.rope_parameters["rope_theta"] = theta
        rot = LlamaRotaryEmbedding(config=cfg)
        hc, hs = rot(x, torch.arange(S).unsqueeze(0))
        want2 = x * hc.unsqueeze(2) + _rotate_half(x) * hs.unsqueeze(2)
        assert torch.allclose(got, want2, atol=1e-5)
    except Exception as e:  # the closed HF form above already pins it
        pytest.skip(f"transformers LlamaRotaryEmbedding not constructible here: {e}")


def test_rope_invariants_and_positions():
    torch.manual_seed(1)
    B, S, H, D = 2, 40, 3, 64
    x = torch.randn(B, S, H, D, dtype=torch.float64)
    cos, sin = P.rope_tables(D, 64, 1e4)
    pos = torch.tensor([list(range(10)) + list(range(15)) + list(range(8)) + [0] * 7] * B)
    y = P.rope_apply(x, cos.double(), sin.double(), pos)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)        # rotations preserve norms
    zero = pos == 0
    assert torch.equal(y[zero], x[zero])                                     # position 0 is the identity
    # a token at position p inside its document equals the same vector at absolute position p
    y_abs = P.rope_apply(x, cos.double(), sin.double(), None)
    assert torch.allclose(y[:, 3], y_abs[:, 3]) and torch.allclose(y[0, 12], P.rope_apply(
        x[:, 12:13], cos.double(), sin.double(), torch.full((B, 1), 2))[0, 0])
    # pairing is half-split (i with i + D/2), not interleaved: rotate a one-hot vector
    e = torch.zeros(1, 1, 1, D, dtype=torch.float64); e[..., 0] = 1.0
    r = P.rope_apply(e, cos.double(), sin.double(), torch.tensor([[5]]))
    assert abs(float(r[0, 0, 0, 0]) - math.cos(5.0)) < 1e-6 and abs(float(r[0, 0, 0, D // 2]) - math.sin(5.0)) < 1e-6
    assert float(r[0, 0, 0, 1].abs()) == 0.0


def test_rms_norm_against_gemma3_and_invariants():
    torch.manual_seed(2)
    D = 256
    x = torch.randn(3, 7, 4, D) * 3.0
    w = torch.randn(D) * 0.1
    got = P.rms_norm(x, w, 1e-6)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * (1 + w)
    assert torch.allclose(got, want, atol=1e-6)
    try:
        from transformers.models.gemma3.modeling_gemma3 import Gemma3RMSNorm
        mod = Gemma3RMSNorm(D, eps=1e-6)
        with torch.no_grad():
            mod.weight.copy_(w)
        assert torch.allclose(got, mod(x), atol=1e-5, rtol=1e-5)
    except ImportError:
        pass
    unit = P.rms_norm(x, torch.zeros(D), 1e-6)                               # zero stored weight = unit scale
    assert torch.allclose(unit.pow(2).mean(-1), torch.ones(3, 7, 4), atol=1e-4)
    assert torch.allclose(P.rms_norm(7.0 * x, w, 0.0), P.rms_norm(x, w, 0.0), atol=1e-5)   # scale invariance
    assert P.rms_norm(x, None) is x
    xb = x.to(torch.bfloat16)
    assert P.rms_norm(xb, w).dtype == torch.bfloat16


def test_prologue_cast_points():
    torch.manual_seed(3)
    B, S, D = 1, 16, 64
    xq = torch.randn(B, S, 2, D).to(torch.bfloat16)
    xk = torch.randn(B, S, 1, D).to(torch.bfloat16)
    w = torch.randn(D) * 0.05
    cos, sin = P.rope_tables(D, S, 1e4)
    qa, ka = P.prologue(xq, xk, w, w, cos, sin, None, cast_between=True)
    qb, kb = P.prologue(xq, xk, w, w, cos, sin, None, cast_between=False)
    # one extra bf16 rounding: differences stay within a couple of bf16 ulps of the values
    assert float((qa.float() - qb.float()).abs().max()) <= 2 ** -6
    assert float((ka.float() - kb.float()).abs().max()) <= 2 ** -6
    qn, kn = P.prologue(xq, xk, None, None, cos, sin, None)
    assert torch.equal(qn, P.rope_apply(xq, cos, sin, None))
