"""The fused linear + cross-entropy loss (maester/models/gemma/model.py:762-769, train.py:258-259) through the
C ABI against the fp64 oracle (pinned in tests/test_oracle_linear_ce.py).

Tolerances: fp32 logits 1e-5 (absolute, on values of order 1..10); bf16 2e-2 max-abs on the loss and 1e-2 rel-L2
on the gradients, against the oracle fed the same bf16-rounded logits."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import max_abs, rel_l2
from maester_amd import ce_rows, linear_cross_entropy
from maester_amd.linear_ce import transpose
from oracle import linear_ce as O

pytestmark = pytest.mark.gpu


def _targets(g, n, vocab, ignore_frac):
    t = torch.randint(0, vocab, (n,), generator=g)
    t[torch.rand(n, generator=g) < ignore_frac] = -100
    return t


@pytest.mark.parametrize("vocab", [5, 8, 1000, 1003, 4096 + 64, 262208])
@pytest.mark.parametrize("softcap", [None, 30.0])
def test_rows_kernel_fp32(gpu, vocab, softcap):
    # widths below one access, multiples of 8, ragged tails, Gemma's vocabulary
    g = torch.Generator().manual_seed(vocab)
    rows = 7 if vocab > 100000 else 19
    x = 4 * torch.randn(rows, vocab, generator=g)
    t = _targets(g, rows, vocab, 0.25)
    t[0], t[1] = vocab - 1, 0
    eye = np.eye(vocab, dtype=np.float64) if vocab <= 5000 else None
    scale = torch.tensor([0.125], device=gpu)
    xg = x.to(gpu)
    lse, nll = ce_rows(xg, t.to(gpu), softcap=softcap, grad_scale=scale)
    # oracle on the logits themselves: e = x, c = identity
    if eye is not None:
        want = O.linear_cross_entropy(x.numpy(), eye, t.numpy(), softcap=softcap, reduction="sum")
        want_lse, want_nll, want_dx = want["lse"], want["nll"], want["dx"] * 0.125
    else:
        xd = x.double()
        xd = softcap * torch.tanh(xd / softcap) if softcap else xd
        want_lse = torch.logsumexp(xd, 1).numpy()
        valid = (t != -100).numpy()
        want_nll = np.where(valid, want_lse - xd[torch.arange(rows), t.clamp_min(0)].numpy(), 0)
        p = torch.softmax(xd, 1)
        p[torch.arange(rows), t.clamp_min(0)] -= 1
        if softcap:
            p = p * (1 - torch.tanh(x.double() / softcap) ** 2)
        want_dx = (p * torch.tensor(valid)[:, None]).numpy() * 0.125
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 1e-5
    assert np.abs(nll.cpu().numpy() - want_nll).max() <= 1e-5
    assert np.abs(xg.cpu().numpy() - want_dx).max() <= 1e-6
    assert np.all(xg.cpu().numpy()[(t == -100).numpy()] == 0)


def test_rows_kernel_strided_rows_and_no_gradient(gpu):
    g = torch.Generator().manual_seed(1)
    buf = torch.full((11, 640), 7.0)
    x = torch.randn(11, 600, generator=g)
    buf[:, :600] = x
    t = _targets(g, 11, 600, 0.2)
    bg = buf.to(gpu)
    lse, nll = ce_rows(bg[:, :600], t.to(gpu), write_grad=False)
    assert torch.equal(bg.cpu(), buf)                       # untouched without write_grad
    want = torch.logsumexp(x.double(), 1)
    assert max_abs(lse.cpu(), want) <= 1e-5
    ce_rows(bg[:, :600], t.to(gpu))
    assert torch.all(bg[:, 600:].cpu() == 7.0)              # the padding between rows is not written
    assert float(bg[:, :600].sum(1).abs().max()) <= 1e-5    # rows of the gradient sum to zero


def test_rows_kernel_labels_out_of_range_do_not_count(gpu):
    x = torch.randn(4, 64)
    t = torch.tensor([3, 64, -5, -100])
    xg = x.to(gpu)
    _, nll = ce_rows(xg, t.to(gpu))
    assert float(nll[0]) > 0 and torch.all(nll[1:] == 0) and torch.all(xg[1:] == 0)


@pytest.mark.parametrize("vocab", [512, 262208, 300000, 1003])
def test_rows_kernel_bf16(gpu, vocab):
    # short rows, Gemma, longer than Gemma, a ragged width (element-wise path)
    g = torch.Generator().manual_seed(2)
    rows = 33
    x = (3 * torch.randn(rows, vocab, generator=g)).bfloat16()
    x[:, 100] += 9
    t = _targets(g, rows, vocab, 0.2)
    t[2] = 100
    xg = x.to(gpu)
    lse, nll = ce_rows(xg, t.to(gpu))
    xd = x.double()
    want_lse = torch.logsumexp(xd, 1)
    p = torch.softmax(xd, 1)
    valid = t != -100
    p[torch.arange(rows), t.clamp_min(0)] -= 1
    p = p * valid[:, None]
    assert max_abs(lse.cpu(), want_lse) <= 1e-5 * float(want_lse.abs().max())
    assert rel_l2(xg.cpu().float(), p) <= 4e-3             # one bf16 rounding per element
    assert max_abs(xg.cpu().float(), p) <= 2 ** -8


def _problem(g, n, k, vocab, dtype, ignore_frac=0.3):
    e = torch.randn(n, k, generator=g).to(dtype)
    c = (torch.randn(vocab, k, generator=g) / math.sqrt(k) * 3).to(dtype)
    return e, c, _targets(g, n, vocab, ignore_frac)


def _run(gpu, e, c, t, **kw):
    eg = e.to(gpu).requires_grad_()
    cg = c.to(gpu).requires_grad_()
    loss = linear_cross_entropy(eg, cg, t.to(gpu), **kw)
    loss.backward()
    return loss.detach().cpu(), eg.grad.cpu(), cg.grad.cpu()


@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("chunk_rows", [None, 64])
def test_loss_and_gradients_fp32(gpu, reduction, chunk_rows):
    g = torch.Generator().manual_seed(3)
    e, c, t = _problem(g, 300, 96, 1000, torch.float32)
    loss, de, dc = _run(gpu, e, c, t, reduction=reduction, chunk_rows=chunk_rows)
    want = O.linear_cross_entropy(e.numpy(), c.numpy(), t.numpy(), reduction=reduction)
    assert loss.dtype == torch.float32 and loss.shape == ()
    assert abs(float(loss) - want["loss"]) <= 1e-5 * max(1.0, abs(want["loss"]))
    assert rel_l2(de, torch.tensor(want["de"])) <= 1e-5 and rel_l2(dc, torch.tensor(want["dc"])) <= 1e-5
    assert torch.all(de[t == -100] == 0)


@pytest.mark.parametrize("shape", [(700, 256, 4096, None), (513, 128, 262208, 200), (64, 2560, 8192, None)])
def test_loss_and_gradients_bf16(gpu, shape):
    n, k, vocab, chunk = shape
    g = torch.Generator().manual_seed(n)
    e, c, t = _problem(g, n, k, vocab, torch.bfloat16)
    loss, de, dc = _run(gpu, e, c, t, chunk_rows=chunk)
    want = O.linear_cross_entropy(e.float().numpy(), c.float().numpy(), t.numpy(), logits_bf16=True)
    assert abs(float(loss) - want["loss"]) <= 2e-2
    assert de.dtype == torch.bfloat16 and dc.dtype == torch.bfloat16
    assert rel_l2(de.float(), torch.tensor(want["de"])) <= 1e-2
    assert rel_l2(dc.float(), torch.tensor(want["dc"])) <= 1e-2
    # against exact logits the loss moves by the rounding of the logits only
    exact = O.linear_cross_entropy(e.float().numpy(), c.float().numpy(), t.numpy())
    assert abs(float(loss) - exact["loss"]) <= 2e-2


def test_filtering_ignored_rows_changes_nothing(gpu):
    g = torch.Generator().manual_seed(5)
    e, c, t = _problem(g, 400, 64, 2048, torch.bfloat16, ignore_frac=0.6)
    a = _run(gpu, e, c, t, filter_ignored=True)
    b = _run(gpu, e, c, t, filter_ignored=False)
    assert abs(float(a[0]) - float(b[0])) <= 1e-6
    assert torch.equal(a[1], b[1])                          # per-row results do not depend on the other rows
    assert rel_l2(a[2].float(), b[2].float()) <= 4e-3       # dC: same terms, another GEMM shape


def test_incoming_gradient_scales_both_gradients(gpu):
    g = torch.Generator().manual_seed(6)
    e, c, t = _problem(g, 128, 64, 512, torch.float32)
    _, de, dc = _run(gpu, e, c, t)
    eg, cg = e.to(gpu).requires_grad_(), c.to(gpu).requires_grad_()
    (linear_cross_entropy(eg, cg, t.to(gpu)) / 4).backward()
    assert torch.allclose(eg.grad.cpu(), de / 4, rtol=1e-6, atol=0) and torch.allclose(cg.grad.cpu(), dc / 4, rtol=1e-6, atol=0)


def test_only_one_input_needs_a_gradient(gpu):
    g = torch.Generator().manual_seed(7)
    e, c, t = _problem(g, 128, 64, 512, torch.float32)
    _, de, dc = _run(gpu, e, c, t)
    eg = e.to(gpu).requires_grad_()
    linear_cross_entropy(eg, c.to(gpu), t.to(gpu)).backward()
    assert torch.equal(eg.grad.cpu(), de)
    with torch.no_grad():
        loss = linear_cross_entropy(e.to(gpu), c.to(gpu), t.to(gpu))
    assert abs(float(loss) - float(_run(gpu, e, c, t)[0])) == 0


def test_all_targets_ignored(gpu):
    g = torch.Generator().manual_seed(8)
    e, c, _ = _problem(g, 16, 32, 64, torch.float32)
    t = torch.full((16,), -100)
    loss, de, dc = _run(gpu, e, c, t)
    assert math.isnan(float(loss)) and torch.all(de == 0) and torch.all(dc == 0)      # torch's mean over nothing
    loss, de, dc = _run(gpu, e, c, t, reduction="sum")
    assert float(loss) == 0 and torch.all(de == 0)
    loss, de, dc = _run(gpu, e, c, t, filter_ignored=False)
    assert math.isnan(float(loss)) and torch.all(de == 0) and torch.all(dc == 0)


def test_leading_dimensions_and_argument_errors(gpu):
    g = torch.Generator().manual_seed(9)
    e, c, t = _problem(g, 6 * 50, 32, 200, torch.float32)
    flat = linear_cross_entropy(e.to(gpu), c.to(gpu), t.to(gpu))
    shaped = linear_cross_entropy(e.view(6, 50, 32).to(gpu), c.to(gpu), t.view(6, 50).to(gpu))   # [B, S, K], [B, S]
    assert float(flat) == float(shaped)
    with pytest.raises(ValueError):
        linear_cross_entropy(e.to(gpu), c.to(gpu), t[:-1].to(gpu))
    with pytest.raises(ValueError):
        linear_cross_entropy(e.to(gpu), c.to(gpu), t.to(gpu), reduction="none")
    with pytest.raises(ValueError):
        linear_cross_entropy(e.to(gpu), c.bfloat16().to(gpu), t.to(gpu))
    with pytest.raises(RuntimeError):
        linear_cross_entropy(e, c, t)                      # CPU tensors: no fallback


def test_gemma_width_against_the_materialising_path_on_the_gpu(gpu):
    # F.cross_entropy(pred.float(), labels) on the full bf16 logits (train.py:258-259) at the real vocabulary and
    # model width, with torch's own kernels as the library routine
    g = torch.Generator().manual_seed(10)
    n, k, vocab = 1024, 2560, 262208
    e, c, t = _problem(g, n, k, vocab, torch.bfloat16, ignore_frac=0.4)
    loss, de, dc = _run(gpu, e, c, t, chunk_rows=384)
    eg, cg = e.to(gpu).requires_grad_(), c.to(gpu).requires_grad_()
    ref = F.cross_entropy((eg @ cg.t()).float(), t.to(gpu))
    ref.backward()
    assert abs(float(loss) - float(ref)) <= 1e-3
    assert rel_l2(de.float(), eg.grad.cpu().float()) <= 1e-2
    assert rel_l2(dc.float(), cg.grad.cpu().float()) <= 1e-2


@pytest.mark.parametrize("shape", [(64, 64), (262208, 96), (130, 72), (77, 13), (1, 5)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_transpose(gpu, shape, dtype):
    x = torch.randn(*shape).to(dtype)
    assert torch.equal(transpose(x.to(gpu)).cpu(), x.t().contiguous())
    if dtype == torch.float32:                                 # rounded on the way, as torch's cast rounds
        assert torch.equal(transpose(x.to(gpu), torch.bfloat16).cpu(), x.t().contiguous().bfloat16())
    else:
        with pytest.raises(RuntimeError):
            transpose(x.to(gpu), torch.float32)


def test_rows_kernel_bf16_softcap(gpu):
    g = torch.Generator().manual_seed(11)
    rows, vocab, cap = 9, 256000, 30.0
    x = (12 * torch.randn(rows, vocab, generator=g)).bfloat16()
    t = _targets(g, rows, vocab, 0.2)
    xg = x.to(gpu)
    lse, nll = ce_rows(xg, t.to(gpu), softcap=cap)
    xd = cap * torch.tanh(x.double() / cap)
    p = torch.softmax(xd, 1)
    valid = t != -100
    p[torch.arange(rows), t.clamp_min(0)] -= 1
    p = p * valid[:, None] * (1 - torch.tanh(x.double() / cap) ** 2)
    assert max_abs(lse.cpu(), torch.logsumexp(xd, 1)) <= 1e-4
    want_nll = torch.where(valid, torch.logsumexp(xd, 1) - xd[torch.arange(rows), t.clamp_min(0)], torch.zeros(rows, dtype=torch.float64))
    assert max_abs(nll.cpu(), want_nll) <= 1e-4
    assert rel_l2(xg.cpu().float(), p) <= 4e-3
