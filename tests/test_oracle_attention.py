"""Pins the dense attention oracle against torch's eager FlexAttention (CPU), the reference's
known-answer test, fp64 brute-force loops, and gradcheck."""
import math

import torch

from conftest import max_abs
from oracle import attention as A
from oracle import masks


def test_matches_eager_flex_attention_gqa():
    torch.manual_seed(0)
    B, S, Hq, Hkv, D = 2, 256, 4, 2, 32
    q, k, v = torch.randn(B, S, Hq, D), torch.randn(B, S, Hkv, D), torch.randn(B, S, Hkv, D)
    ids = torch.zeros(B, S, dtype=torch.long)
    ids[0, 100:176] = 1; ids[0, 176:] = 2; ids[1, 30:] = 1
    for window in (None, 40):
        want = A.flex_attention_cpu(q, k, v, ids, D ** -0.5, True, window)
        got = A.dense_attention(q, k, v, ids, D ** -0.5, True, window)
        assert max_abs(got, want) < 1e-5


def test_reference_known_answer_boundary_inside_block():
    # tests/test_packed_sft.py:164-212: boundary at 176, q=k=1, v=-1 before / +1 after
    S, D, boundary = 256, 4, 176
    ids = torch.zeros((1, S), dtype=torch.long); ids[:, boundary:] = 1
    q = torch.ones(1, S, 1, D); k = torch.ones_like(q); v = torch.ones_like(q)
    v[:, :boundary] = -1
    out = A.dense_attention(q, k, v, ids, D ** -0.5)[0, :, 0]
    assert torch.allclose(out[:boundary], torch.full_like(out[:boundary], -1))
    assert torch.allclose(out[boundary:], torch.ones_like(out[boundary:]))


def test_block_mask_matches_dense_case():
    # tests/test_packed_sft.py:104-162: S=128, 4 docs of 32, H=2, D=8; atol 1e-5 / rtol 1e-4
    torch.manual_seed(1)
    S, H, D = 128, 2, 8
    ids = torch.zeros((1, S), dtype=torch.long)
    ids[:, 32:64] = 1; ids[:, 64:96] = 2; ids[:, 96:] = 3
    q, k, v = (torch.randn(1, S, H, D) for _ in range(3))
    want = A.flex_attention_cpu(q, k, v, ids, D ** -0.5)
    assert torch.allclose(A.dense_attention(q, k, v, ids, D ** -0.5), want, atol=1e-5, rtol=1e-4)


def test_fp64_brute_force_loops():
    torch.manual_seed(2)
    B, S, Hq, Hkv, D = 1, 24, 4, 2, 8
    q, k, v = (torch.randn(B, S, h, D, dtype=torch.float64) for h in (Hq, Hkv, Hkv))
    ids = torch.tensor([[0] * 7 + [1] * 9 + [-1] * 8])
    scale, W = 0.3, 4
    got, lse = A.dense_attention(q, k, v, ids, scale, True, W, compute_dtype=torch.float64, return_lse=True)
    G = Hq // Hkv
    for h in range(Hq):
        for qi in range(S):
            num = torch.zeros(D, dtype=torch.float64); den = 0.0
            for kv in range(S):
                if masks.allowed(ids, 0, qi, kv, True, W):
                    e = math.exp(scale * float(q[0, qi, h] @ k[0, kv, h // G]))
                    num += e * v[0, kv, h // G]; den += e
            assert torch.allclose(got[0, qi, h], num / den, atol=1e-12)
            assert abs(float(lse[0, h, qi]) - math.log(den)) < 1e-12


def test_backward_closed_form_and_gradcheck():
    torch.manual_seed(3)
    B, S, Hq, Hkv, D = 1, 12, 2, 1, 4
    q, k, v = (torch.randn(B, S, h, D, dtype=torch.float64) for h in (Hq, Hkv, Hkv))
    do = torch.randn(B, S, Hq, D, dtype=torch.float64)
    ids = torch.tensor([[0] * 5 + [1] * 7])
    scale = 0.5
    out, dq, dk, dv = A.dense_attention_fwd_bwd(q, k, v, do, ids, scale, compute_dtype=torch.float64)
    # closed form of torch/_higher_order_ops/flex_attention.py:825-993
    m = masks.dense_mask(ids, 1, S)[0, 0]
    dq2 = torch.zeros_like(dq); dk2 = torch.zeros_like(dk); dv2 = torch.zeros_like(dv)
    for h in range(Hq):
        s = (q[0, :, h] @ k[0, :, 0].t()) * scale
        p = torch.softmax(s.masked_fill(~m, float("-inf")), -1)
        delta = (out[0, :, h] * do[0, :, h]).sum(-1, keepdim=True)
        dp = do[0, :, h] @ v[0, :, 0].t()
        ds = p * (dp - delta)
        dv2[0, :, 0] += p.t() @ do[0, :, h]
        dq2[0, :, h] = scale * ds @ k[0, :, 0]
        dk2[0, :, 0] += scale * ds.t() @ q[0, :, h]
    assert max_abs(dq, dq2) < 1e-12 and max_abs(dk, dk2) < 1e-12 and max_abs(dv, dv2) < 1e-12

    def f(q_, k_, v_):
        return A.full_path(q_, k_, v_, None, None, torch.ones(64, D // 2, dtype=torch.float64),
                           torch.zeros(64, D // 2, dtype=torch.float64), None, ids, scale, compute_dtype=torch.float64)
    assert torch.autograd.gradcheck(f, (q.clone().requires_grad_(), k.clone().requires_grad_(),
                                        v.clone().requires_grad_()), atol=1e-6)


def test_eager_flex_backward_agrees():
    from torch.nn.attention.flex_attention import create_block_mask, flex_attention
    torch.manual_seed(4)
    B, S, Hq, Hkv, D = 1, 256, 2, 1, 16
    q, k, v = (torch.randn(B, S, h, D) for h in (Hq, Hkv, Hkv))
    do = torch.randn(B, S, Hq, D)
    ids = torch.zeros(B, S, dtype=torch.long); ids[:, 150:] = 1
    bm = create_block_mask(masks.make_mask_mod(ids), B, None, S, S, device="cpu")
    qt, kt, vt = (t.transpose(1, 2).detach().requires_grad_() for t in (q, k, v))
    o = flex_attention(qt, kt, vt, block_mask=bm, scale=D ** -0.5, enable_gqa=True)
    gq, gk, gv = torch.autograd.grad(o, (qt, kt, vt), do.transpose(1, 2))
    out, dq, dk, dv = A.dense_attention_fwd_bwd(q, k, v, do, ids, D ** -0.5)
    assert max_abs(out, o.transpose(1, 2)) < 1e-5
    assert max_abs(dq, gq.transpose(1, 2)) < 1e-4 and max_abs(dk, gk.transpose(1, 2)) < 1e-4
    assert max_abs(dv, gv.transpose(1, 2)) < 1e-4
