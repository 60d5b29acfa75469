import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda", 0)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.double() - b.double()).abs().max())


# ---- the parity bar of the bf16 path ---------------------------------------------------------------
# Stated bar: max-abs <= 2e-2 and relative L2 <= 1e-2 against the reference evaluated in fp32.
# Outputs and log-sum-exps are held to the flat 2e-2.  Gradients reach magnitudes of 4..10 on N(0,1)
# inputs, where STORING the fp32 reference value in bf16 already costs up to half a unit in the last
# place: bf16 keeps 8 significant bits, so for 2^e <= |x| < 2^(e+1) the spacing is 2^(e-7) and the
# half-ulp 2^(e-8) (0.0156 for 4 <= |x| < 8, 0.031 from 8 on).  Gradients are held, element by element, to
#     |got - ref| <= 2e-2 + roundings * half_ulp_bf16(ref)
# where `roundings` is the number of times the compared value was stored in bf16 on its way: 1 for the
# attention backward (dq, dk, dv) and for the value gradient of the whole path, 2 for the query / key
# gradients of the whole path (the attention backward stores dq / dk, the prologue backward stores the
# result again).  An error of 0.1 on a small element fails this whatever the tensor's largest element is.
BF16_MAX_ABS, BF16_REL_L2 = 2e-2, 1e-2
PARITY_LOG = []          # one record per check of this session (written out by pytest_sessionfinish)


def bf16_half_ulp(x: torch.Tensor) -> torch.Tensor:
    """Half the spacing of bf16 at |x| (2^(floor(log2 |x|) - 8)); the smallest normal's for zero."""
    e = torch.floor(torch.log2(x.abs().double().clamp_min(2.0 ** -126)))
    return torch.exp2(e - 8)


def check_bf16(got: torch.Tensor, want: torch.Tensor, tag, flat: bool = False, roundings: int = 1) -> dict:
    """Asserts the bar above (``flat``: no half-ulp term) and returns / prints / records the raw numbers,
    among them how many elements exceed the flat 2e-2 and the smallest |ref| among those."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, (tag, tuple(got.shape), tuple(want.shape))
    err = (got - want).abs()
    lim = torch.full_like(err, BF16_MAX_ABS) if flat else BF16_MAX_ABS + roundings * bf16_half_ulp(want)
    over = err > BF16_MAX_ABS
    n_over = int(over.sum())
    rec = {"tag": str(tag), "max_abs": float(err.max()), "worst_over_limit": float((err / lim).max()),
           "rel_l2": float((got - want).norm() / want.norm().clamp_min(1e-30)), "max_ref": float(want.abs().max()),
           "roundings": 0 if flat else int(roundings), "elements": int(err.numel()), "over_flat_2e-2": n_over,
           "min_ref_over_flat": float(want.abs()[over].min()) if n_over else None}
    PARITY_LOG.append(rec)
    print(f"parity {rec['tag']}: max-abs {rec['max_abs']:.3e} (max |ref| {rec['max_ref']:.2f}), "
          f"worst err/limit {rec['worst_over_limit']:.3f}, rel-L2 {rec['rel_l2']:.3e}, "
          f"{n_over} of {rec['elements']} over flat 2e-2" + (f" (smallest |ref| among them {rec['min_ref_over_flat']:.2f})" if n_over else ""))
    assert bool(torch.isfinite(got).all()), tag
    assert rec["worst_over_limit"] <= 1.0, rec
    assert rec["rel_l2"] <= BF16_REL_L2, rec
    return rec


# Norm-weight gradients are sums over `rows` rows of products (gradient x normalised activation) whose
# factors went through bf16.  Every addend is within the elementwise bar e = 2e-2 + half_ulp of what the
# fp32 reference adds, and the addends' errors are independent roundings of either sign, so the error of
# the sum grows like a random walk: it is held to e(ref) * sqrt(rows) * BF16_SUM_SIGMAS / sqrt(3) (the
# standard deviation of `rows` errors uniform in +-e is e * sqrt(rows / 3)), and to the relative L2 bar.
BF16_SUM_SIGMAS = 1.0


def check_bf16_sum(got: torch.Tensor, want: torch.Tensor, rows: int, tag) -> dict:
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, (tag, tuple(got.shape), tuple(want.shape))
    err = (got - want).abs()
    lim = (BF16_MAX_ABS + bf16_half_ulp(want)) * (rows / 3.0) ** 0.5 * BF16_SUM_SIGMAS
    rec = {"tag": str(tag), "max_abs": float(err.max()), "worst_over_limit": float((err / lim).max()),
           "rel_l2": float((got - want).norm() / want.norm().clamp_min(1e-30)), "max_ref": float(want.abs().max()),
           "rows_summed": int(rows)}
    PARITY_LOG.append(rec)
    print(f"parity {rec['tag']}: sum over {rows} rows, max-abs {rec['max_abs']:.3e} (max |ref| {rec['max_ref']:.2f}), "
          f"worst err/limit {rec['worst_over_limit']:.3f}, rel-L2 {rec['rel_l2']:.3e}")
    assert bool(torch.isfinite(got).all()), tag
    assert rec["worst_over_limit"] <= 1.0, rec
    assert rec["rel_l2"] <= BF16_REL_L2, rec
    return rec


def pytest_sessionfinish(session, exitstatus):
    """Leaves the raw parity numbers of a GPU run where the run's other results go (if that folder exists)."""
    out = os.path.join(ROOT, "gpurun_out")
    if PARITY_LOG and os.path.isdir(out):
        import json
        with open(os.path.join(out, "parity_numbers.json"), "w") as f:
            json.dump(PARITY_LOG, f, indent=0)
