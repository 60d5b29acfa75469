"""The decoder layer's sandwich RMSNorms (maester/models/gemma/model.py:135-172, 488-508) through the C
ABI, forward and backward, against the oracle's closed form (pinned in tests/test_oracle_prologue.py)."""
import pytest
import torch

from conftest import max_abs, rel_l2
from maester_amd import RMSNorm, rms_norm
from oracle import prologue as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


def _reference(x, w, residual):
    """The reference's sequence: norm in fp32, cast to the dtype of x, then `residual + hidden`."""
    y = P.rms_norm(x, w)
    return y if residual is None else residual + y


@pytest.mark.parametrize("dim", [64, 2560, 3840, 8192])
@pytest.mark.parametrize("with_residual", [False, True])
def test_forward_bit_exact_in_bf16_and_close_in_fp32(gpu, dim, with_residual):
    g = torch.Generator().manual_seed(dim)
    rows = 37
    w = 0.2 * torch.randn(dim, generator=g)
    for dtype in (torch.bfloat16, torch.float32):
        x = (3 * torch.randn(2, rows, dim, generator=g)).to(dtype)
        r = torch.randn(2, rows, dim, generator=g).to(dtype) if with_residual else None
        want = _reference(x, w, r)
        got = rms_norm(x.to(gpu), w.to(gpu), None if r is None else r.to(gpu))
        assert got.dtype == dtype and got.shape == x.shape
        if dtype == torch.float32:
            assert max_abs(got.cpu(), want) <= 1e-5 * max(1.0, float(want.abs().max()))
        else:
            # same fp32 math and the same two roundings: at most a last-bit tie of the norm output
            # differs (with a residual that is a bit of the norm output, not of the possibly smaller sum)
            diff = (got.cpu().float() - want.float()).abs()
            ulp = torch.maximum(want.float().abs(), P.rms_norm(x, w).float().abs()).clamp_min(1e-30) * 2.0 ** -7
            assert bool((diff <= ulp).all()) and float((diff > 0).float().mean()) < 0.01


@pytest.mark.parametrize("dim", [256, 2560])
@pytest.mark.parametrize("with_residual", [False, True])
def test_backward(gpu, dim, with_residual):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(3, 50, dim, generator=g)
    w = 0.2 * torch.randn(dim, generator=g)
    r = torch.randn(3, 50, dim, generator=g) if with_residual else None
    dy = torch.randn(3, 50, dim, generator=g)
    leaves = [t.clone().requires_grad_() for t in (x, w)] + ([r.clone().requires_grad_()] if with_residual else [])
    ref = P.rms_norm(leaves[0], leaves[1]) + (leaves[2] if with_residual else 0)
    want = torch.autograd.grad(ref, leaves, dy)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 1e-2)):
        hx = x.to(dtype).to(gpu).requires_grad_()
        hw = w.to(gpu).requires_grad_()
        hr = r.to(dtype).to(gpu).requires_grad_() if with_residual else None
        out = rms_norm(hx, hw, hr)
        got = torch.autograd.grad(out, [hx, hw] + ([hr] if with_residual else []), dy.to(dtype).to(gpu))
        for name, a, b in zip(("dx", "dw", "dresidual"), got, want):
            assert rel_l2(a.float().cpu(), b) <= tol, (dtype, name, rel_l2(a.float().cpu(), b))
        again = torch.autograd.grad(rms_norm(hx, hw, hr), [hx, hw], dy.to(dtype).to(gpu))
        assert torch.equal(again[0], got[0]) and torch.equal(again[1], got[1])      # no atomics: bit-identical reruns


def test_module_mirrors_the_reference_parameter(gpu):
    m = RMSNorm(128).to(gpu)
    assert dict(m.named_parameters()).keys() == {"weight"} and float(m.weight.abs().sum()) == 0.0   # zeros: scale 1 + w
    x = torch.randn(4, 128, device=gpu)
    y = m(x)
    assert max_abs((y.pow(2).mean(-1)).cpu(), torch.ones(4)) <= 1e-3
    assert torch.equal(m(x, residual=x), x + y)
