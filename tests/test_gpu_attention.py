"""HIP attention (through the C ABI) vs the oracle.

Tolerances (the stated bar of the path): fp32 activations <= 1e-4 max-abs; bf16 activations
<= 2e-2 max-abs and <= 1e-2 relative L2 against the oracle evaluated in fp32 on the same
(bf16-rounded) inputs -- outputs and LSE flat, gradients element by element with the exact bf16 half-ulp
of the reference value, once per bf16 store on the compared path, on top (``conftest.check_bf16``)."""
import numpy as np
import pytest
import torch

from conftest import check_bf16, check_bf16_sum, max_abs, rel_l2
from maester_amd import build_tile_map, doc_masked_attention, packed_doc_attention, workloads
from maester_amd.attention import attention_backward, attention_forward, backward_workspace_bytes
from oracle import attention as A
from oracle import prologue as P

pytestmark = pytest.mark.gpu

FP32_MAX_ABS = 1e-4


def _ids(B, S, seed, kind="docs"):
    rng = np.random.default_rng(seed)
    if kind == "none":
        return None
    ids = np.zeros((B, S), dtype=np.int64)
    for b in range(B):
        cuts = np.sort(rng.integers(1, S, size=max(1, S // 150)))
        for c in cuts:
            ids[b, c:] += 1
    if kind == "padded":
        ids[:, S - S // 7:] = -1
    if kind == "recurring":          # ids that come back later in the row: the mask only asks for equality
        ids = ids % 3
    return torch.from_numpy(ids)


def _qkv(B, S, Hq, Hkv, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, D, generator=g).to(dtype)
    return mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)


def _check(got, want, dtype, tag, flat=False, roundings=1):
    if dtype == torch.float32:
        assert max_abs(got.cpu(), want) <= FP32_MAX_ABS, (tag, max_abs(got.cpu(), want))
    else:
        check_bf16(got, want, tag, flat=flat, roundings=roundings)


# ------------------------------------------------------------------ fp32 path ------------------
def test_c1_full_config_fp32(gpu):
    """Config 1 end to end (prologue + attention), fp32, forward only, <= 1e-4 max-abs."""
    wl = workloads.make("c1")
    want = A.full_path(wl.xq, wl.xk, wl.xv, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids, wl.document_ids, wl.scale,
                       compute_dtype=torch.float64)
    g = wl.to(gpu)
    out = packed_doc_attention(g.xq, g.xk, g.xv, g.q_w, g.k_w, g.cos, g.sin, g.position_ids, g.document_ids, g.scale)
    assert out.dtype == torch.float32 and out.shape == wl.xq.shape
    assert max_abs(out.cpu(), want) <= FP32_MAX_ABS
    # and against torch's own FlexAttention on the CPU, fed the oracle prologue
    q, k = P.prologue(wl.xq, wl.xk, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids)
    flex = A.flex_attention_cpu(q, k, wl.xv, wl.document_ids, wl.scale)
    assert max_abs(out.cpu(), flex) <= FP32_MAX_ABS


def test_reference_known_answers_fp32(gpu):
    # maester tests/test_packed_sft.py:164-212 -- boundary inside a 128-block, exact -1 / +1
    S, D, boundary = 256, 64, 176
    ids = torch.zeros((1, S), dtype=torch.long); ids[:, boundary:] = 1
    q = torch.ones(1, S, 1, D); k = torch.ones_like(q); v = torch.ones_like(q); v[:, :boundary] = -1
    out = doc_masked_attention(q.to(gpu), k.to(gpu), v.to(gpu), ids.to(gpu), D ** -0.5).cpu()[0, :, 0]
    assert torch.allclose(out[:boundary], torch.full_like(out[:boundary], -1))
    assert torch.allclose(out[boundary:], torch.ones_like(out[boundary:]))
    # tests/test_packed_sft.py:104-162 -- 4 docs of 32 in one block, vs dense softmax atol 1e-5 rtol 1e-4
    torch.manual_seed(0)
    ids = torch.zeros((1, 128), dtype=torch.long); ids[:, 32:64] = 1; ids[:, 64:96] = 2; ids[:, 96:] = 3
    q, k, v = (torch.randn(1, 128, 2, 64) for _ in range(3))
    got = doc_masked_attention(q.to(gpu), k.to(gpu), v.to(gpu), ids.to(gpu), 64 ** -0.5).cpu()
    assert torch.allclose(got, A.dense_attention(q, k, v, ids, 64 ** -0.5), atol=1e-5, rtol=1e-4)


@pytest.mark.parametrize("D,S,window,kind", [(64, 300, None, "docs"), (128, 513, 100, "padded"), (64, 256, 0, "none"),
                                             (256, 200, None, "docs")])
def test_fp32_forward_edge_cases(gpu, D, S, window, kind):
    B, Hq, Hkv = 2, 4, 2
    q, k, v, _ = _qkv(B, S, Hq, Hkv, D, torch.float32, 1)
    ids = _ids(B, S, 2, kind)
    want, wl = A.dense_attention(q, k, v, ids, 0.2, True, window, compute_dtype=torch.float64, return_lse=True)
    tm = build_tile_map(None if ids is None else ids.to(gpu), B, S, True, window, device=gpu)
    out, lse = attention_forward(q.to(gpu), k.to(gpu), v.to(gpu), tm, None if ids is None else ids.to(gpu), 0.2, True, window)
    assert max_abs(out.cpu(), want) <= FP32_MAX_ABS and max_abs(lse.cpu(), wl) <= FP32_MAX_ABS


@pytest.mark.parametrize("D", [64, 128])
def test_fp32_backward(gpu, D):
    B, S, Hq, Hkv = 1, 400, 4, 2
    q, k, v, do = _qkv(B, S, Hq, Hkv, D, torch.float32, 3)
    ids = _ids(B, S, 4)
    _, dq, dk, dv = A.dense_attention_fwd_bwd(q, k, v, do, ids, 0.15, True, 150, compute_dtype=torch.float64)
    hq, hk, hv = (t.to(gpu).requires_grad_() for t in (q, k, v))
    out = doc_masked_attention(hq, hk, hv, ids.to(gpu), 0.15, True, 150)
    gq, gk, gv = torch.autograd.grad(out, (hq, hk, hv), do.to(gpu))
    for a, b in ((gq, dq), (gk, dk), (gv, dv)):
        assert max_abs(a.cpu(), b) <= FP32_MAX_ABS


# ------------------------------------------------------------------ bf16 MFMA path -------------
BF16_CASES = [
    # name, B, S, Hq, Hkv, D, window, ids kind
    ("gemma4b_global_small", 2, 1024, 4, 2, 256, None, "docs"),
    ("gemma4b_local_small", 2, 1024, 4, 2, 256, 300, "docs"),
    ("llama_shape_small", 1, 1024, 8, 2, 128, None, "docs"),
    ("ragged_padded", 2, 777, 2, 1, 256, None, "padded"),
    ("ragged_window_d128", 1, 333, 4, 4, 128, 64, "docs"),
    ("no_ids_causal", 1, 640, 2, 1, 256, None, "none"),
    ("d64", 1, 512, 2, 2, 64, None, "docs"),
    ("tiny_one_tile", 1, 50, 2, 1, 128, None, "docs"),
    ("two_pairs_per_kv_head_d256", 1, 900, 8, 2, 256, None, "docs"),     # pair kernel, two pairs per kv head
    ("odd_group_d256", 1, 700, 3, 1, 256, 200, "docs"),                  # one-head kernel at D = 256
    ("mha_d256_padded", 1, 450, 2, 2, 256, None, "padded"),
    ("recurring_ids", 2, 1100, 4, 2, 256, None, "recurring"),
    ("recurring_ids_window_d128", 1, 1100, 4, 1, 128, 256, "recurring"),
]


@pytest.mark.parametrize("case", BF16_CASES, ids=[c[0] for c in BF16_CASES])
def test_bf16_forward(gpu, case):
    _, B, S, Hq, Hkv, D, window, kind = case
    q, k, v, _ = _qkv(B, S, Hq, Hkv, D, torch.bfloat16, 5)
    ids = _ids(B, S, 6, kind)
    scale = D ** -0.5
    want, wl = A.dense_attention(q, k, v, ids, scale, True, window, return_lse=True)
    gids = None if ids is None else ids.to(gpu)
    tm = build_tile_map(gids, B, S, True, window, device=gpu)
    out, lse = attention_forward(q.to(gpu), k.to(gpu), v.to(gpu), tm, gids, scale, True, window)
    assert out.dtype == torch.bfloat16
    _check(out, want, torch.bfloat16, (case[0], "out"), flat=True)
    assert max_abs(lse.cpu(), wl) <= 2e-2


@pytest.mark.parametrize("S", [1024, 777], ids=["whole_tiles", "ragged"])
def test_bf16_views_with_different_row_strides(gpu, S):
    """q, k, v, dO as views into wider buffers, each with a row stride of its own (what the fused qkv projection
    of model.py:358-364 hands over): bit-identical to the same call on packed copies.  S = 1024 takes the
    kernels' whole-tile loads, S = 777 the ones that go through a descriptor of the tile."""
    B, Hq, Hkv, D = 2, 4, 2, 256
    q, k, v, do = (t.to(gpu) for t in _qkv(B, S, Hq, Hkv, D, torch.bfloat16, 21))
    ids = _ids(B, S, 22, "docs").to(gpu)
    scale = D ** -0.5

    def wide(t, extra_heads, at):  # the tensor as heads [at, at + H) of a buffer with extra_heads more heads per row
        H = t.shape[2]
        buf = torch.full((B, S, H + extra_heads, D), float("nan"), dtype=t.dtype, device=gpu)
        buf[:, :, at:at + H] = t
        return buf[:, :, at:at + H]

    qv, kv, vv, dov = wide(q, 3, 1), wide(k, 1, 0), wide(v, 6, 4), wide(do, 2, 2)
    assert len({t.stride(1) for t in (qv, kv, vv, dov)}) == 4 and not any(t.is_contiguous() for t in (qv, kv, vv, dov))
    tm = build_tile_map(ids, B, S, True, None, device=gpu)
    out_a, lse_a = attention_forward(q, k, v, tm, ids, scale, True, None)
    out_b, lse_b = attention_forward(qv, kv, vv, tm, ids, scale, True, None)
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    grads_a = attention_backward(q, k, v, out_a, do, lse_a, tm, ids, scale, True, None)
    grads_b = attention_backward(qv, kv, vv, out_a, dov, lse_a, tm, ids, scale, True, None)
    for name, a, b in zip(("dq", "dk", "dv"), grads_a, grads_b):
        assert torch.equal(a, b), name
    want, _ = A.dense_attention(q.cpu(), k.cpu(), v.cpu(), ids.cpu(), scale, True, None, return_lse=True)
    _check(out_b, want, torch.bfloat16, ("views", S, "out"), flat=True)


@pytest.mark.parametrize("case", BF16_CASES, ids=[c[0] for c in BF16_CASES])
def test_bf16_backward(gpu, case):
    _, B, S, Hq, Hkv, D, window, kind = case
    q, k, v, do = _qkv(B, S, Hq, Hkv, D, torch.bfloat16, 7)
    ids = _ids(B, S, 8, kind)
    scale = D ** -0.5
    _, dq, dk, dv = A.dense_attention_fwd_bwd(q, k, v, do, ids, scale, True, window)
    gids = None if ids is None else ids.to(gpu)
    hq, hk, hv = (t.to(gpu).requires_grad_() for t in (q, k, v))
    out = doc_masked_attention(hq, hk, hv, gids, scale, True, window)
    gq, gk, gv = torch.autograd.grad(out, (hq, hk, hv), do.to(gpu))
    for name, a, b in (("dq", gq, dq), ("dk", gk, dk), ("dv", gv, dv)):
        _check(a, b, torch.bfloat16, (case[0], name))
    # dK/dV/dQ are produced without atomics: a second run is bit-identical
    out2 = doc_masked_attention(hq, hk, hv, gids, scale, True, window)
    g2 = torch.autograd.grad(out2, (hq, hk, hv), do.to(gpu))
    assert all(torch.equal(x, y) for x, y in zip(g2, (gq, gk, gv)))


def test_full_path_bf16_with_norm_weights(gpu):
    """Prologue + attention + both backward stages through PackedDocAttention, incl. dW of the norms."""
    wl = workloads.make("c2", B=1, S=1024)
    ins = [wl.xq.float().requires_grad_(), wl.xk.float().requires_grad_(), wl.xv.float().requires_grad_(),
           wl.q_w.clone().requires_grad_(), wl.k_w.clone().requires_grad_()]
    ref = A.full_path(ins[0], ins[1], ins[2], ins[3], ins[4], wl.cos, wl.sin, wl.position_ids, wl.document_ids, wl.scale)
    want = torch.autograd.grad(ref, ins, wl.dout.float())
    g = wl.to(gpu)
    hin = [g.xq.clone().requires_grad_(), g.xk.clone().requires_grad_(), g.xv.clone().requires_grad_(),
           g.q_w.clone().requires_grad_(), g.k_w.clone().requires_grad_()]
    out = packed_doc_attention(hin[0], hin[1], hin[2], hin[3], hin[4], g.cos, g.sin, g.position_ids, g.document_ids, g.scale)
    _check(out, ref.detach(), torch.bfloat16, "full path out", flat=True)
    got = torch.autograd.grad(out, hin, g.dout)
    for name, a, b in zip(("dxq", "dxk", "dxv"), got[:3], want[:3]):
        # (dq and dk are stored in bf16 by the attention backward and again by the prologue backward)
        _check(a, b, torch.bfloat16, "full path " + name, roundings=1 if name == "dxv" else 2)
    sp = wl.spec
    for name, a, b, heads in zip(("dq_w", "dk_w"), got[3:], want[3:], (sp.Hq, sp.Hkv)):
        check_bf16_sum(a, b, sp.B * sp.S * heads, "full path " + name)


@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_full_size_properties_and_slice(gpu, name):
    """At the benchmark shapes: one (row, kv head) slice against the oracle evaluated on the GPU, plus
    size-independent properties (constant V -> constant output, linearity in V, determinism)."""
    wl = workloads.make(name).to(gpu)
    sp = wl.spec
    q, k = wl.xq, wl.xk                                   # attention only: feed raw activations
    tm = build_tile_map(wl.document_ids, sp.B, sp.S, True, sp.window)
    out, lse = attention_forward(q, k, wl.xv, tm, wl.document_ids, wl.scale, True, sp.window)
    G = sp.Hq // sp.Hkv
    b, hk = sp.B - 1, sp.Hkv - 1
    want, wlse = A.dense_attention(q[b:b + 1, :, hk * G:(hk + 1) * G], k[b:b + 1, :, hk:hk + 1], wl.xv[b:b + 1, :, hk:hk + 1],
                                   wl.document_ids[b:b + 1], wl.scale, True, sp.window, return_lse=True)
    _check(out[b:b + 1, :, hk * G:(hk + 1) * G], want.cpu(), torch.bfloat16, (name, "out slice"), flat=True)
    assert max_abs(lse[b:b + 1, hk * G:(hk + 1) * G].cpu(), wlse.cpu()) <= 2e-2
    ones = torch.ones_like(wl.xv)
    o1, _ = attention_forward(q, k, ones, tm, wl.document_ids, wl.scale, True, sp.window)
    assert max_abs(o1.cpu(), torch.ones_like(o1).cpu()) <= 1e-2            # softmax rows sum to one
    o2, _ = attention_forward(q, k, wl.xv * 2, tm, wl.document_ids, wl.scale, True, sp.window)
    assert torch.equal(o2.float(), out.float() * 2)                        # exact: scaling V by 2 is exact in bf16
    o3, l3 = attention_forward(q, k, wl.xv, tm, wl.document_ids, wl.scale, True, sp.window)
    assert torch.equal(o3, out) and torch.equal(l3, lse)
    # first token of every document attends only to itself
    starts = (wl.position_ids == 0)
    for h in (0, sp.Hq - 1):
        assert torch.equal(out[:, :, h][starts], wl.xv[:, :, h // G][starts])


def _backward_both_ways(gpu, q, k, v, do, ids, scale, window):
    """(dq, dk, dv) with dS handed from the dK/dV kernel to the dQ kernel through a workspace that starts out full of
    NaNs (every block the dQ kernel reads must have been written by the dK/dV kernel), and with the dQ kernel
    recomputing S and dP."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    tm = build_tile_map(ids, B, S, True, window, device=gpu)
    out, lse = attention_forward(q, k, v, tm, ids, scale, True, window)
    ws = torch.full((backward_workspace_bytes(B, S, Hq, Hkv, D, q.dtype, True, tm),), 0xFF, dtype=torch.uint8, device=gpu)
    bufs = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), ws)
    handed = attention_backward(q, k, v, out, do, lse, tm, ids, scale, True, window, buffers=bufs)
    handed = tuple(t.clone() for t in handed)
    again = attention_backward(q, k, v, out, do, lse, tm, ids, scale, True, window, buffers=bufs)
    assert all(torch.equal(x, y) for x, y in zip(handed, again))
    recomputed = attention_backward(q, k, v, out, do, lse, tm, ids, scale, True, window, hand_over=False)
    return handed, recomputed


@pytest.mark.parametrize("case", BF16_CASES, ids=[c[0] for c in BF16_CASES])
def test_bf16_backward_ds_hand_over_and_recompute(gpu, case):
    _, B, S, Hq, Hkv, D, window, kind = case
    q, k, v, do = _qkv(B, S, Hq, Hkv, D, torch.bfloat16, 17)
    ids = _ids(B, S, 18, kind)
    scale = D ** -0.5
    _, dq, dk, dv = A.dense_attention_fwd_bwd(q, k, v, do, ids, scale, True, window)
    gids = None if ids is None else ids.to(gpu)
    handed, recomputed = _backward_both_ways(gpu, q.to(gpu), k.to(gpu), v.to(gpu), do.to(gpu), gids, scale, window)
    for got in (handed, recomputed):
        assert all(bool(torch.isfinite(t).all()) for t in got)
        for name, a, b in zip(("dq", "dk", "dv"), got, (dq, dk, dv)):
            _check(a, b, torch.bfloat16, (case[0], name))
    # the dK/dV kernel computes the same thing either way; delta comes from another kernel (another summation order)
    assert torch.equal(handed[2], recomputed[2])
    assert rel_l2(handed[1].float(), recomputed[1].float()) <= 2e-3


def test_ds_hand_over_random_geometries(gpu):
    """Sequence lengths, windows, id layouts, head dims and group sizes drawn at random: whatever block the dQ kernel
    reads from the NaN-filled workspace must have been written, and both ways of computing dQ must agree."""
    rng = np.random.default_rng(1234)
    for case in range(48):
        D = int(rng.choice([64, 128, 256]))
        Hkv = int(rng.choice([1, 2]))
        G = int(rng.choice([1, 2, 3, 4]))
        B = int(rng.choice([1, 2]))
        S = int(rng.integers(2, 1400))
        window = None if rng.random() < 0.4 else int(rng.integers(0, 700))
        kind = str(rng.choice(["docs", "padded", "none", "recurring"]))
        q, k, v, do = _qkv(B, S, Hkv * G, Hkv, D, torch.bfloat16, 100 + case)
        ids = _ids(B, S, 200 + case, kind)
        gids = None if ids is None else ids.to(gpu)
        handed, recomputed = _backward_both_ways(gpu, q.to(gpu), k.to(gpu), v.to(gpu), do.to(gpu), gids, D ** -0.5, window)
        what = (case, B, S, Hkv, G, D, window, kind)
        assert all(bool(torch.isfinite(t).all()) for t in handed), what
        assert torch.equal(handed[2], recomputed[2]), what
        for a, b in zip(handed[:2], recomputed[:2]):
            denom = float(b.float().norm())
            assert float((a.float() - b.float()).norm()) <= 4e-3 * denom + 1e-6, what


@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_full_size_ds_hand_over_reads_only_what_was_written(gpu, name):
    wl = workloads.make(name).to(gpu)
    sp = wl.spec
    handed, recomputed = _backward_both_ways(gpu, wl.xq, wl.xk, wl.xv, wl.dout, wl.document_ids, wl.scale, sp.window)
    assert all(bool(torch.isfinite(t).all()) for t in handed)
    assert torch.equal(handed[2], recomputed[2])
    assert rel_l2(handed[1].float(), recomputed[1].float()) <= 2e-3
    # both dQ kernels multiply a bf16 dS with K; they differ by the rounding of dS only where the two kernels'
    # fp32 sums of S and dP differ in the last bits
    assert rel_l2(handed[0].float(), recomputed[0].float()) <= 2e-3


@pytest.mark.parametrize("name", ["c2", "c3", "c4", "c4s", "c5"])
def test_full_size_backward_slices(gpu, name):
    """At the benchmark shapes: forward and backward of the whole batch through the C ABI, then two
    (row, kv head) slices of out / dq / dk / dv against the fp32 oracle evaluated on the GPU (the
    dense score matrix of one slice is all that fits)."""
    wl = workloads.make(name).to(gpu)
    sp = wl.spec
    q, k, v, do = wl.xq, wl.xk, wl.xv, wl.dout
    tm = build_tile_map(wl.document_ids, sp.B, sp.S, True, sp.window)
    out, lse = attention_forward(q, k, v, tm, wl.document_ids, wl.scale, True, sp.window)
    dq, dk, dv = attention_backward(q, k, v, out, do, lse, tm, wl.document_ids, wl.scale, True, sp.window)
    G = sp.Hq // sp.Hkv
    for b, hk in ((0, 0), (sp.B - 1, sp.Hkv - 1)):
        hs = slice(hk * G, (hk + 1) * G)
        ids = wl.document_ids[b:b + 1]
        wo, wq, wk, wv = A.dense_attention_fwd_bwd(q[b:b + 1, :, hs], k[b:b + 1, :, hk:hk + 1], v[b:b + 1, :, hk:hk + 1],
                                                   do[b:b + 1, :, hs], ids, wl.scale, True, sp.window)
        for what, got, want in (("out", out[b:b + 1, :, hs], wo), ("dq", dq[b:b + 1, :, hs], wq),
                                ("dk", dk[b:b + 1, :, hk:hk + 1], wk), ("dv", dv[b:b + 1, :, hk:hk + 1], wv)):
            _check(got.cpu(), want.cpu(), torch.bfloat16, (name, b, hk, what), flat=(what == "out"))
        del wo, wq, wk, wv
        torch.cuda.empty_cache()


@pytest.mark.parametrize("name", ["c2", "c3", "c4", "c5"])
def test_full_size_full_path(gpu, name):
    """The whole path at the benchmark shape -- QK-RMSNorm with the configuration's weights (none for the Llama-shaped
    configuration), RoPE with its theta over the per-document positions, attention, and the backward of all of it
    through ``PackedDocAttention`` -- against ``oracle.attention.full_path`` in fp32 on two (row, kv head) slices (the
    dense score matrix of one slice is what fits).  The norm-weight gradients sum over every row and head: they are
    checked on the loss restricted to a slice, which the library sees as an upstream gradient that is zero outside it."""
    wl = workloads.make(name).to(gpu)
    sp = wl.spec
    G = sp.Hq // sp.Hkv
    normed = wl.q_w is not None
    leaves = [t.clone().requires_grad_() for t in (wl.xq, wl.xk, wl.xv)]
    weights = [w.clone().requires_grad_() for w in (wl.q_w, wl.k_w)] if normed else [None, None]
    tm = build_tile_map(wl.document_ids, sp.B, sp.S, True, sp.window)
    out = packed_doc_attention(*leaves, *weights, wl.cos, wl.sin, wl.position_ids, wl.document_ids, wl.scale, True, sp.window,
                               tile_map=tm)
    dxq, dxk, dxv = torch.autograd.grad(out, leaves, wl.dout, retain_graph=True)
    for b, hk in ((0, 0), (sp.B - 1, sp.Hkv - 1)):
        hs = slice(hk * G, (hk + 1) * G)
        ins = [wl.xq[b:b + 1, :, hs].float().requires_grad_(), wl.xk[b:b + 1, :, hk:hk + 1].float().requires_grad_(),
               wl.xv[b:b + 1, :, hk:hk + 1].float().requires_grad_()]
        rw = [wl.q_w.clone().requires_grad_(), wl.k_w.clone().requires_grad_()] if normed else [None, None]
        ref = A.full_path(ins[0], ins[1], ins[2], rw[0], rw[1], wl.cos, wl.sin, wl.position_ids[b:b + 1],
                          wl.document_ids[b:b + 1], wl.scale, True, sp.window)
        want = torch.autograd.grad(ref, ins + (rw if normed else []), wl.dout[b:b + 1, :, hs].float())
        _check(out[b:b + 1, :, hs], ref.detach(), torch.bfloat16, (name, "full path", b, hk, "out"), flat=True)
        # dxq of the slice's heads depends on the slice alone; dxk / dxv of the kv head likewise (its G query heads are all in the slice)
        for what, got, exp in (("dxq", dxq[b:b + 1, :, hs], want[0]), ("dxk", dxk[b:b + 1, :, hk:hk + 1], want[1]),
                               ("dxv", dxv[b:b + 1, :, hk:hk + 1], want[2])):
            # (dq and dk are stored in bf16 by the attention backward and again by the prologue backward)
            _check(got, exp, torch.bfloat16, (name, "full path", b, hk, what), roundings=1 if what == "dxv" else 2)
        if normed:
            # norm-weight gradients of the loss restricted to this slice
            mask = torch.zeros_like(wl.dout)
            mask[b, :, hs] = wl.dout[b, :, hs]
            gq_w, gk_w = torch.autograd.grad(out, weights, mask, retain_graph=True)
            for what, got, exp, rows in (("dq_w", gq_w, want[3], sp.S * G), ("dk_w", gk_w, want[4], sp.S)):
                check_bf16_sum(got, exp, rows, (name, "full path", b, hk, what))
            del mask
        del ref, want, ins
        torch.cuda.empty_cache()


def test_saved_tensor_policies_give_identical_gradients(gpu):
    """Keeping everything, keeping only the attention output and LSE, or keeping nothing for the
    backward changes what is recomputed, not a bit of the result (the kernels are deterministic)."""
    from maester_amd.attention import SAVE_POLICIES
    wl = workloads.make("c2", B=2, S=1536).to(gpu)
    grads = {}
    for policy in SAVE_POLICIES:
        leaves = [t.clone().requires_grad_() for t in (wl.xq, wl.xk, wl.xv, wl.q_w, wl.k_w)]
        out = packed_doc_attention(*leaves, wl.cos, wl.sin, wl.position_ids, wl.document_ids, wl.scale, save=policy)
        grads[policy] = (out.detach(),) + torch.autograd.grad(out, leaves, wl.dout)
    for policy in SAVE_POLICIES[1:]:
        assert all(torch.equal(a, b) for a, b in zip(grads["all"], grads[policy])), policy
    with pytest.raises(ValueError):
        packed_doc_attention(wl.xq, wl.xk, wl.xv, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids, wl.document_ids, wl.scale, save="some")


@pytest.mark.parametrize("heads", [(4, 2), (3, 3)], ids=["pair", "single"])
def test_work_queues_give_the_same_results_and_reset_themselves(gpu, heads):
    """With work counters in the tile map the forward and dK/dV kernels run one workgroup per compute
    unit that pulls work items; without, one workgroup per item.  Same bits either way, and the
    counters are back at zero after every launch (so launches can follow one another)."""
    Hq, Hkv = heads
    B, S, D = 3, 1500, 128
    q, k, v, do = (t.to(gpu) for t in _qkv(B, S, Hq, Hkv, D, torch.bfloat16, 11))
    ids = _ids(B, S, 12, "docs").to(gpu)
    tm = build_tile_map(ids, B, S, True, None)
    assert tm.work_counters is not None and int(tm.work_counters.abs().sum()) == 0
    results = []
    for counters in (tm.work_counters, None, tm.work_counters):
        tm.work_counters = counters
        out, lse = attention_forward(q, k, v, tm, ids, D ** -0.5, True, None)
        grads = attention_backward(q, k, v, out, do, lse, tm, ids, D ** -0.5, True, None)
        results.append((out, lse) + tuple(grads))
        if counters is not None:
            assert int(counters.abs().sum()) == 0
    for other in results[1:]:
        assert all(torch.equal(x, y) for x, y in zip(results[0], other))


@pytest.mark.parametrize("heads", [(2, 1), (4, 2), (2, 2)], ids=["pair_g2", "pair_g2_hkv2", "single_g1"])
@pytest.mark.parametrize("D", [128, 256])
def test_bf16_forward_scores_that_outgrow_the_first_block(gpu, heads, D):
    """Late keys score far above anything in a row's first kv block (hundreds of nats): the online
    softmax must move its reference (rescale, or redo the tile in two passes) and stay exact."""
    Hq, Hkv = heads
    B, S = 1, 640
    q, k, v, _ = _qkv(B, S, Hq, Hkv, D, torch.bfloat16, 11)
    k = k.clone()
    k[:, 300:] *= 60.0          # logits of late keys have std 60 instead of 1
    k[:, 500:] *= 4.0           # and grow once more
    ids = _ids(B, S, 3, "docs")
    ids[:] = 0                  # one document: every row sees all earlier keys
    scale = D ** -0.5
    want, wl = A.dense_attention(q, k, v, ids, scale, True, None, return_lse=True)
    gids = ids.to(gpu)
    tm = build_tile_map(gids, B, S, True, None, device=gpu)
    out, lse = attention_forward(q.to(gpu), k.to(gpu), v.to(gpu), tm, gids, scale, True, None)
    _check(out, want, torch.bfloat16, ("outgrown", heads, D), flat=True)
    assert torch.isfinite(lse).all()
    assert max_abs(lse.cpu(), wl) <= 2e-2 * max(1.0, float(wl.abs().max()) / 100)


def test_launches_that_share_a_tile_map_are_ordered_across_streams(gpu):
    """The work queues live in the tile map: a launch on another stream than the previous one is made to wait for it
    (two overlapping launches would drain each other's queues and leave rows unwritten)."""
    wl = workloads.make("c2", B=2, S=4096).to(gpu)
    sp = wl.spec
    tm = build_tile_map(wl.document_ids, sp.B, sp.S, True, None)
    want, _ = attention_forward(wl.xq, wl.xk, wl.xv, tm, wl.document_ids, wl.scale, True, None)
    streams = [torch.cuda.Stream() for _ in range(3)]
    torch.cuda.synchronize()
    outs = []
    for rep in range(6):
        with torch.cuda.stream(streams[rep % 3]):
            outs.append(attention_forward(wl.xq, wl.xk, wl.xv, tm, wl.document_ids, wl.scale, True, None)[0])
    torch.cuda.synchronize()
    assert all(torch.equal(o, want) for o in outs)
    assert int(tm.work_counters.abs().sum()) == 0
