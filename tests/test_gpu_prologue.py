"""Fused QK-RMSNorm + RoPE prologue (HIP) vs the oracle, forward and backward."""
import pytest
import torch

from conftest import check_bf16, check_bf16_sum, max_abs, rel_l2
from maester_amd import qk_norm_rope, workloads
from maester_amd.attention import prologue_forward
from oracle import prologue as P

pytestmark = pytest.mark.gpu


def _mk(B, S, Hq, Hkv, D, dtype, seed=0, norm=True):
    g = torch.Generator().manual_seed(seed)
    xq = (torch.randn(B, S, Hq, D, generator=g) * 1.5).to(dtype)
    xk = (torch.randn(B, S, Hkv, D, generator=g) * 0.7).to(dtype)
    qw = torch.randn(D, generator=g) * 0.1 if norm else None
    kw = torch.randn(D, generator=g) * 0.1 if norm else None
    pos = torch.randint(0, 3 * S, (B, S), generator=g)
    cos, sin = P.rope_tables(D, 3 * S, 1e4)
    return xq, xk, qw, kw, cos, sin, pos


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("norm", [True, False])
def test_forward_fp32(gpu, D, norm):
    xq, xk, qw, kw, cos, sin, pos = _mk(2, 77, 6, 3, D, torch.float32, norm=norm)
    wq, wk = P.prologue(xq.double(), xk.double(), None if qw is None else qw.double(), None if kw is None else kw.double(),
                        cos.double(), sin.double(), pos)
    dev = lambda t: None if t is None else t.to(gpu)
    q, k, q_rstd, k_rstd = prologue_forward(dev(xq), dev(xk), dev(qw), dev(kw), dev(cos), dev(sin), dev(pos))
    assert max_abs(q.cpu(), wq) < 1e-5 and max_abs(k.cpu(), wk) < 1e-5          # fp32 tolerance
    if norm:
        want_r = torch.rsqrt(xq.double().pow(2).mean(-1) + 1e-6)
        assert max_abs(q_rstd.cpu(), want_r) < 1e-5


@pytest.mark.parametrize("D", [64, 128, 256])
def test_forward_bf16_and_strided_views(gpu, D):
    B, S, Hq, Hkv = 2, 130, 4, 2
    g = torch.Generator().manual_seed(1)
    qkv = torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16).to(gpu)
    xq, xk, xv = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)          # the views GemmaAttention holds
    xq = xq.view(B, S, Hq, D); xk = xk.view(B, S, Hkv, D)
    qw = (torch.randn(D, generator=g) * 0.1); kw = (torch.randn(D, generator=g) * 0.1)
    pos = torch.randint(0, S, (B, S), generator=g)
    cos, sin = P.rope_tables(D, S, 1e6)
    q, k, _, _ = prologue_forward(xq, xk, qw.to(gpu), kw.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu))
    wq, wk = P.prologue(xq.cpu(), xk.cpu(), qw, kw, cos, sin, pos, cast_between=False)
    # same fp32 math, one rounding to bf16: at most one bf16 ulp apart
    for got, want in ((q, wq), (k, wk)):
        err = (got.cpu().float() - want.float()).abs()
        assert bool((err <= want.float().abs() * 2 ** -7 + 1e-6).all())
    # against the reference's cast sequence (bf16 after the norm, then RoPE): tolerance of the path
    rq, rk = P.prologue(xq.cpu(), xk.cpu(), qw, kw, cos, sin, pos, cast_between=True)
    check_bf16(q, rq, "prologue q vs cast sequence")
    check_bf16(k, rk, "prologue k vs cast sequence")


def test_default_positions_and_unit_weight(gpu):
    xq, xk, _, _, cos, sin, _ = _mk(1, 64, 2, 1, 64, torch.float32)
    z = torch.zeros(64)
    q, k, _, _ = prologue_forward(xq.to(gpu), xk.to(gpu), z.to(gpu), z.to(gpu), cos.to(gpu), sin.to(gpu), None)
    wq, wk = P.prologue(xq, xk, z, z, cos, sin, None)
    assert max_abs(q.cpu(), wq) < 1e-5 and max_abs(k.cpu(), wk) < 1e-5
    # rotations preserve the norm; unit-weight RMSNorm output has mean square 1
    assert torch.allclose(q.cpu().pow(2).mean(-1), torch.ones(1, 64, 2), atol=1e-3)


@pytest.mark.parametrize("dtype,D,norm", [(torch.float32, 64, True), (torch.float32, 256, True),
                                          (torch.bfloat16, 256, True), (torch.bfloat16, 128, False)])
def test_backward(gpu, dtype, D, norm):
    B, S, Hq, Hkv = 2, 300, 4, 2
    xq, xk, qw, kw, cos, sin, pos = _mk(B, S, Hq, Hkv, D, dtype, seed=3, norm=norm)
    g = torch.Generator().manual_seed(5)
    gq = torch.randn(B, S, Hq, D, generator=g).to(dtype); gk = torch.randn(B, S, Hkv, D, generator=g).to(dtype)
    # oracle: autograd through the fp64 restatement
    ins = [xq.double().requires_grad_(), xk.double().requires_grad_()]
    ws = [qw.double().requires_grad_(), kw.double().requires_grad_()] if norm else [None, None]
    oq, ok = P.prologue(ins[0], ins[1], ws[0], ws[1], cos.double(), sin.double(), pos)
    grads = torch.autograd.grad([oq, ok], ins + ([w for w in ws] if norm else []), [gq.double(), gk.double()])
    dev = lambda t: None if t is None else t.to(gpu)
    hq, hk = dev(xq).requires_grad_(), dev(xk).requires_grad_()
    hqw = dev(qw).requires_grad_() if norm else None
    hkw = dev(kw).requires_grad_() if norm else None
    q, k = qk_norm_rope(hq, hk, hqw, hkw, dev(cos), dev(sin), dev(pos))
    got = torch.autograd.grad([q, k], [hq, hk] + ([hqw, hkw] if norm else []), [dev(gq), dev(gk)])
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    rtol = 1e-5 if dtype == torch.float32 else 1e-2
    for i, (a, b) in enumerate(zip(got, grads)):
        if dtype == torch.float32:
            assert max_abs(a.cpu(), b) <= tol * max(1.0, float(b.abs().max())), (max_abs(a.cpu(), b), float(b.abs().max()))
            assert rel_l2(a.cpu(), b) < rtol
        elif i < 2:       # activations' gradients: the bar of the path, element by element
            check_bf16(a, b, ("prologue bwd", D, norm, i))
        else:             # weight gradients are sums over B*S*H rows
            check_bf16_sum(a, b, B * S * (Hq if i == 2 else Hkv), ("prologue bwd weight", D, i))
    # run-to-run determinism of the weight-gradient reduction (no atomics)
    if norm:
        got2 = torch.autograd.grad(qk_norm_rope(hq, hk, hqw, hkw, dev(cos), dev(sin), dev(pos)), [hqw, hkw], [dev(gq), dev(gk)])
        assert torch.equal(got2[0], got[2]) and torch.equal(got2[1], got[3])


def test_full_size_c2_invariants(gpu):
    """At the benchmark shape: norm preservation under RoPE and agreement with the oracle on a slice."""
    wl = workloads.make("c2").to(gpu)
    q, k, q_rstd, _ = prologue_forward(wl.xq, wl.xk, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids)
    sl = slice(4000, 4200)
    wq, wk = P.prologue(wl.xq[:1, sl].cpu(), wl.xk[:1, sl].cpu(), wl.q_w.cpu(), wl.k_w.cpu(), wl.cos.cpu(), wl.sin.cpu(),
                        wl.position_ids[:1, sl].cpu(), cast_between=False)
    assert rel_l2(q[:1, sl].cpu(), wq) < 4e-3 and rel_l2(k[:1, sl].cpu(), wk) < 4e-3
    n = (wl.xq.float() * q_rstd[..., None] * (1 + wl.q_w.float())).norm(dim=-1)
    assert torch.allclose(q.float().norm(dim=-1), n, rtol=2e-2)
