"""The error of the reference's own bf16 path, recorded beside this library's.

maester runs ``torch.compile(flex_attention)`` on bf16 activations (maester/models/gemma/model.py:384-396).
Both that path and the HIP kernels are compared here with the same fp32 oracle on the same bf16
inputs; the library must meet the bar of ``conftest.check_bf16``, the reference's numbers are
recorded next to it (printed, and kept with the run's other results) so that the bar can be read
against what the reference itself achieves in bf16."""
import json
import os

import pytest
import torch

from conftest import BF16_MAX_ABS, ROOT, bf16_half_ulp, check_bf16
from maester_amd import build_tile_map, workloads
from maester_amd.attention import attention_backward, attention_forward
from oracle import attention as A

pytestmark = pytest.mark.gpu


def _numbers(got, want, flat):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    lim = torch.full_like(err, BF16_MAX_ABS) if flat else BF16_MAX_ABS + bf16_half_ulp(want)
    over = err > BF16_MAX_ABS
    return {"max_abs": float(err.max()), "worst_over_limit": float((err / lim).max()),
            "rel_l2": float((got - want).norm() / want.norm()), "max_ref": float(want.abs().max()),
            "over_flat_2e-2": int(over.sum()), "min_ref_over_flat": float(want.abs()[over].min()) if bool(over.any()) else None}


@pytest.mark.parametrize("name,B,S", [("c2", 1, 2048), ("c3", 1, 2048), ("c5", 1, 2048)])
def test_library_and_reference_bf16_error_against_the_fp32_oracle(gpu, name, B, S):
    from torch.nn.attention.flex_attention import create_block_mask, flex_attention
    wl = workloads.make(name, B=B, S=S).to(gpu)
    sp = wl.spec
    q, k, v, do, doc, W = wl.xq, wl.xk, wl.xv, wl.dout, wl.document_ids, sp.window
    wo, wq, wk, wv = A.dense_attention_fwd_bwd(q, k, v, do, doc, wl.scale, True, W)       # fp32, on the GPU
    want = {"out": wo, "dq": wq, "dk": wk, "dv": wv}

    tm = build_tile_map(doc, sp.B, sp.S, True, W)
    out, lse = attention_forward(q, k, v, tm, doc, wl.scale, True, W)
    dq, dk, dv = attention_backward(q, k, v, out, do, lse, tm, doc, wl.scale, True, W)
    ours = {n: check_bf16(t, want[n], (name, "library", n), flat=(n == "out"))
            for n, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv))}

    record = {"workload": f"{sp.name} B={sp.B} S={sp.S}", "library": ours}
    try:      # the reference's kernel: Inductor's Triton template; recorded, not asserted
        def mod(b, h, qi, ki):
            ok = (doc[b, qi] == doc[b, ki]) & (qi >= ki)
            return ok & (qi - ki <= W) if W is not None else ok
        bm = create_block_mask(mod, sp.B, None, sp.S, sp.S, device=doc.device)
        Q, K_, V = (t.transpose(1, 2).detach().requires_grad_(True) for t in (q, k, v))
        fo = torch.compile(flex_attention)(Q, K_, V, block_mask=bm, scale=wl.scale, enable_gqa=sp.Hq != sp.Hkv)
        fq, fk, fv = torch.autograd.grad(fo, (Q, K_, V), do.transpose(1, 2))
        ref = {"out": fo.transpose(1, 2), "dq": fq.transpose(1, 2), "dk": fk.transpose(1, 2), "dv": fv.transpose(1, 2)}
        record["torch_compiled_flex_attention_bf16"] = {n: _numbers(t, want[n], n == "out") for n, t in ref.items()}
    except Exception as e:  # noqa: BLE001 - the template may not compile on a given box
        record["torch_compiled_flex_attention_bf16"] = {"skipped": f"{type(e).__name__}: {str(e)[:200]}"}
    print(json.dumps(record))
    dest = os.path.join(ROOT, "gpurun_out")
    if os.path.isdir(dest):
        with open(os.path.join(dest, f"reference_bf16_error_{name}.json"), "w") as f:
            json.dump(record, f, indent=1)
