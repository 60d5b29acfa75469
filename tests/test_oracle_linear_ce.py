"""Pins ``oracle.linear_ce`` against library routines, closed forms and finite differences (CPU)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from scipy.special import logsumexp

from oracle import linear_ce as O


def _case(n=37, k=24, v=53, seed=0, ignore_frac=0.3):
    g = np.random.default_rng(seed)
    e = g.standard_normal((n, k)).astype(np.float32)
    c = g.standard_normal((v, k)).astype(np.float32) * 0.7
    t = g.integers(0, v, n)
    t[g.random(n) < ignore_frac] = -100
    return e, c, t


@pytest.mark.parametrize("reduction", ["mean", "sum"])
def test_matches_torch_cross_entropy_and_its_autograd(reduction):
    # the routine the reference's materialising path calls (train.py:258-259), ignore_index as in
    # tests/test_packed_sft.py:300-310
    e, c, t = _case()
    te = torch.tensor(e, dtype=torch.float64, requires_grad=True)
    tc = torch.tensor(c, dtype=torch.float64, requires_grad=True)
    loss = F.cross_entropy(te @ tc.T, torch.tensor(t), ignore_index=-100, reduction=reduction)
    loss.backward()
    got = O.linear_cross_entropy(e, c, t, reduction=reduction)
    assert abs(got["loss"] - loss.item()) < 1e-12
    np.testing.assert_allclose(got["de"], te.grad.numpy(), atol=1e-13)
    np.testing.assert_allclose(got["dc"], tc.grad.numpy(), atol=1e-13)


def test_lse_matches_scipy():
    e, c, t = _case(seed=1)
    got = O.linear_cross_entropy(e, c, t)
    np.testing.assert_allclose(got["lse"], logsumexp(e.astype(np.float64) @ c.astype(np.float64).T, axis=1), atol=1e-12)


def test_closed_forms():
    # equal logits: every class has probability 1/V
    e = np.zeros((4, 8), np.float32)
    c = np.ones((50, 8), np.float32)
    t = np.array([0, 7, 49, 3])
    assert abs(O.linear_cross_entropy(e, c, t)["loss"] - np.log(50)) < 1e-12
    # one overwhelming logit on the label: loss ~ 0; on another class: loss ~ the gap
    e = np.eye(3, dtype=np.float32) * 40
    c = np.eye(3, dtype=np.float32)
    assert O.linear_cross_entropy(e, c, np.array([0, 1, 2]))["loss"] < 1e-15
    assert abs(O.linear_cross_entropy(e, c, np.array([1, 2, 0]))["loss"] - 40) < 1e-12


def test_gradient_rows_sum_to_zero_and_ignored_rows_vanish():
    e, c, t = _case(seed=2)
    got = O.linear_cross_entropy(e, c, t)
    np.testing.assert_allclose(got["dx"].sum(axis=1), 0, atol=1e-15)
    assert np.all(got["dx"][t == -100] == 0) and np.all(got["de"][t == -100] == 0)
    assert got["count"] == int((t != -100).sum())


@pytest.mark.parametrize("softcap", [None, 5.0])
def test_central_differences(softcap):
    e, c, t = _case(n=5, k=4, v=7, seed=3, ignore_frac=0.2)
    got = O.linear_cross_entropy(e, c, t, softcap=softcap)
    h = 1e-5
    e64, c64 = e.astype(np.float64), c.astype(np.float64)
    for arr, grad in ((e64, got["de"]), (c64, got["dc"])):
        for idx in [(0, 0), (2, 3), (4, 1)]:
            old = arr[idx]
            arr[idx] = old + h
            up = O.linear_cross_entropy(e64, c64, t, softcap=softcap)["loss"]
            arr[idx] = old - h
            dn = O.linear_cross_entropy(e64, c64, t, softcap=softcap)["loss"]
            arr[idx] = old
            assert abs((up - dn) / (2 * h) - grad[idx]) < 1e-8


def test_softcap_matches_torch():
    e, c, t = _case(seed=4)
    te = torch.tensor(e, dtype=torch.float64, requires_grad=True)
    tc = torch.tensor(c, dtype=torch.float64)
    loss = F.cross_entropy(3.0 * torch.tanh(te @ tc.T / 3.0), torch.tensor(t), ignore_index=-100)
    loss.backward()
    got = O.linear_cross_entropy(e, c, t, softcap=3.0)
    assert abs(got["loss"] - loss.item()) < 1e-12
    np.testing.assert_allclose(got["de"], te.grad.numpy(), atol=1e-13)


def test_all_ignored_is_nan_like_torch():
    e, c, _ = _case(n=3)
    t = np.full(3, -100)
    assert np.isnan(O.linear_cross_entropy(e, c, t)["loss"])
    assert torch.isnan(F.cross_entropy(torch.tensor(e) @ torch.tensor(c).T, torch.tensor(t)))
    assert O.linear_cross_entropy(e, c, t, reduction="sum")["loss"] == 0


def test_round_bf16_matches_torch():
    a = np.random.default_rng(5).standard_normal(4096).astype(np.float32) * 100
    np.testing.assert_array_equal(O.round_bf16(a), torch.tensor(a).bfloat16().float().numpy())
