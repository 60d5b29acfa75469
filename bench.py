#!/usr/bin/env python3
"""Benchmark of the packed-SFT document-masked attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-cpu-baseline]

A step is one pass of the attention hot path over one batch of synthetic input already resident in
HBM: ``ma_attn_fwd`` followed by ``ma_attn_bwd`` (delta, dK/dV, dQ kernels) through the C ABI.
The headline value is useful TFLOP/s = 12*D*Hq*N_pairs / step time, N_pairs = unmasked (q, kv)
pairs (the MFU convention of maester/models/gemma/model.py:71-75: 2 forward + 4 backward GEMMs,
recompute not counted), for the Gemma-3-4B global-layer shape.  The same run also times, each in
its own bracket: every kernel alone (HIP events on the launch stream), the fused QK-RMSNorm+RoPE
prologue (HBM roofline), the tile-map build, the whole autograd Function, and a bounded CPU sample
of the oracle on the host cores.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_DENSE_TFLOPS = 2500.0   # MI355X bf16 dense MFMA: 256 CU x 4096 FLOP/clk/CU x 2.4 GHz
PEAK_HBM_GBPS = 8000.0            # MI355X HBM3E


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def time_region(fn, steps, warmup):
    """Average milliseconds per call, HIP events on the current (launch) stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = _events(2)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def cpu_baseline(wl, budget_seconds=12.0):
    """The reference's own CPU path on the host cores: torch's ``create_block_mask`` + eager ``flex_attention``
    (the only CPU FlexAttention with a backward; what maester/models/gemma/model.py:384-396 calls and what
    tests/test_packed_sft.py:148-155 run), driven by the oracle's restated mask mod, forward + backward, one
    (batch row, kv head) slice of the workload after the other until ``budget_seconds`` of CPU work are spent
    (a bounded sample: the whole workload is B*Hkv such slices)."""
    from torch.nn.attention.flex_attention import create_block_mask, flex_attention

    from maester_amd import workloads as W
    from oracle import masks
    sp = wl.spec
    G = sp.Hq // sp.Hkv
    slices = [(b, hk) for b in range(sp.B) for hk in range(sp.Hkv)]
    t_mask = t_fwd = t_bwd = 0.0
    flops = 0
    done = 0
    for b, hk in slices:
        q = wl.xq[b:b + 1, :, hk * G:(hk + 1) * G].float().transpose(1, 2).requires_grad_()
        k = wl.xk[b:b + 1, :, hk:hk + 1].float().transpose(1, 2).requires_grad_()
        v = wl.xv[b:b + 1, :, hk:hk + 1].float().transpose(1, 2).requires_grad_()
        do = wl.dout[b:b + 1, :, hk * G:(hk + 1) * G].float().transpose(1, 2)
        mod = masks.make_mask_mod(wl.document_ids[b:b + 1], True, sp.window)
        t0 = time.perf_counter()
        bm = create_block_mask(mod, 1, None, sp.S, sp.S, device="cpu")
        t1 = time.perf_counter()
        o = flex_attention(q, k, v, block_mask=bm, scale=wl.scale, enable_gqa=G > 1)
        t2 = time.perf_counter()
        torch.autograd.grad(o, (q, k, v), do)
        t3 = time.perf_counter()
        t_mask, t_fwd, t_bwd = t_mask + t1 - t0, t_fwd + t2 - t1, t_bwd + t3 - t2
        flops += 12 * sp.D * G * W.count_pairs([wl.doc_lengths[b]], sp.window)
        done += 1
        if t_mask + t_fwd + t_bwd >= budget_seconds:
            break
    dt = t_fwd + t_bwd
    return {
        "value": flops / dt / 1e12, "unit": "useful TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"torch {torch.__version__} eager flex_attention fwd+bwd (fp32, CPU) with the restated mask mod on {done} of "
                  f"{len(slices)} (batch row, kv head) slices of {sp.name} (S={sp.S}, G={G}, D={sp.D}): fwd {t_fwd:.2f} s + "
                  f"bwd {t_bwd:.2f} s; create_block_mask for those rows {t_mask:.2f} s (not in value)",
        "seconds": dt, "fwd_seconds": t_fwd, "bwd_seconds": t_bwd, "create_block_mask_seconds": t_mask,
        "slices_sampled": done, "slices_in_workload": len(slices),
        "whole_workload_seconds_extrapolated": dt * len(slices) / done,
        "note": "value = useful FLOPs of the sampled slices / their time; the whole workload is slices_in_workload such "
                "slices run one after the other (the factor to the whole workload is slices_in_workload / slices_sampled "
                "in time, 1 in rate)",
    }


def mfma_probe(dev, cus):
    """What the matrix cores sustain on this GPU under a pure MFMA load (see ma_probe_mfma): per operand pattern
    and number of busy compute units, the shader clock held and the resulting dense bf16 rate."""
    from maester_amd import _lib
    L = _lib.lib()
    out = torch.zeros(3, dtype=torch.int64, device=dev)
    iters, res = 20000, {}
    for label, rnd, wgs in (("ones_1cu", 0, 1), ("ones_all", 0, cus), ("random_1cu", 1, 1), ("random_all", 1, cus)):
        for _ in range(2):      # the second run is the one kept (clocks settled)
            _lib.check(L.ma_probe_mfma(iters, rnd, wgs, _lib.ptr(out), _lib.current_stream(dev)))
            torch.cuda.synchronize()
        clocks, ticks = int(out[0]), int(out[1])
        mhz = clocks / (ticks / 100.0)
        res[label] = {"cycles_per_mfma": clocks / (16.0 * iters), "shader_clock_mhz": mhz,
                      "dense_bf16_tflops_all_cus": 4 * cus * 32768 / (clocks / (16.0 * iters)) * mhz * 1e6 / 1e12}
    return res


def gpu_clock_mhz():
    """The shader clock the driver reports right now (the active line of pp_dpm_sclk), or None."""
    import glob
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            with open(path) as f:
                for line in f:
                    if line.rstrip().endswith("*"):
                        return float(line.split(":")[1].strip().rstrip("*").strip().lower().replace("mhz", ""))
        except (OSError, ValueError, IndexError):
            continue
    return None


def flex_gpu_baseline(wl, q, k, steps=30, warmup=10):
    """What maester runs today, on this GPU: torch's create_block_mask + torch.compile(flex_attention)
    (Inductor Triton templates; maester/models/gemma/model.py:384-396, 694-730) on the same inputs,
    driven by a restated mask mod.  Informational only: never part of the timed step, and skipped
    (with the reason) when the template does not compile on the box."""
    try:
        from torch.nn.attention.flex_attention import create_block_mask, flex_attention
        sp, doc, W = wl.spec, wl.document_ids, wl.spec.window

        def mod(b, h, qi, ki):
            ok = (doc[b, qi] == doc[b, ki]) & (qi >= ki)
            return ok & (qi - ki <= W) if W is not None else ok

        t_mask = time_region(lambda: create_block_mask(mod, sp.B, None, sp.S, sp.S, device=doc.device), 3, 1)
        bm = create_block_mask(mod, sp.B, None, sp.S, sp.S, device=doc.device)
        Q, K_, V = (t.transpose(1, 2).detach().requires_grad_(True) for t in (q, k, wl.xv))
        fa = torch.compile(flex_attention)
        gqa = sp.Hq != sp.Hkv
        with torch.no_grad():
            t_fwd = time_region(lambda: fa(Q, K_, V, block_mask=bm, scale=wl.scale, enable_gqa=gqa), steps, warmup)
        out = {"create_block_mask_ms": t_mask, "fwd_ms": t_fwd, "torch": torch.__version__}
        if wl.dout is not None:
            dO = wl.dout.transpose(1, 2)

            def fb():
                Q.grad = K_.grad = V.grad = None
                fa(Q, K_, V, block_mask=bm, scale=wl.scale, enable_gqa=gqa).backward(dO)
            out["fwd_bwd_ms"] = time_region(fb, steps, warmup)
        return out
    except Exception as e:  # noqa: BLE001 - a baseline that cannot run must not fail the bench
        return {"skipped": f"{type(e).__name__}: {str(e)[:200]}"}


def loss_block(dev, rows, dim, vocab, dtype, with_torch):
    """The model's last step on the same token count: fused linear + cross-entropy, loss and both gradients."""
    import math

    from maester_amd.linear_ce import ce_rows, default_chunk_rows, linear_ce_forward
    e = torch.randn(rows, dim, device=dev).to(dtype)
    c = (torch.randn(vocab, dim, device=dev) * (3.0 / math.sqrt(dim))).to(dtype)
    t = torch.randint(0, vocab, (rows,), device=dev)
    t_all = time_region(lambda: linear_ce_forward(e, c, t), 5, 2)
    step = default_chunk_rows(vocab, e.element_size(), rows)
    blk = torch.mm(e[:step], c.t())
    from maester_amd.linear_ce import transpose
    de, dc_t = torch.empty_like(e[:step]), torch.empty(dim, vocab, dtype=dtype, device=dev)
    c_t, e_t = transpose(c), transpose(e[:step].contiguous())

    def gemms():       # the three products of a block in the operand orders the loss uses
        torch.mm(e[:step], c.t(), out=blk)
        torch.mm(blk, c_t.t(), out=de)
        torch.mm(e_t, blk, out=dc_t)
    t_gemm = time_region(gemms, 5, 2)
    torch.mm(e[:step], c.t(), out=blk)
    t_rows = time_region(lambda: ce_rows(blk, t[:step]), 10, 3)
    flops = 6.0 * rows * vocab * dim
    row_bytes = 2 * e.element_size() * step * vocab
    out = {"rows": rows, "dim": dim, "vocab": vocab, "rows_per_block": step, "fwd_bwd_ms": t_all,
           "useful_flops": flops, "tflops": flops / (t_all * 1e-3) / 1e12,
           "library_gemms_ms_per_block": t_gemm, "library_gemm_tflops": 6.0 * step * vocab * dim / (t_gemm * 1e-3) / 1e12,
           "ce_rows_kernel": {"ms_per_block": t_rows, "algorithmic_bytes": row_bytes, "gbps": row_bytes / (t_rows * 1e-3) / 1e9,
                              "frac_hbm_peak": row_bytes / (t_rows * 1e-3) / 1e9 / PEAK_HBM_GBPS}}
    del blk, de, dc_t, c_t, e_t
    if with_torch:
        # the reference's materialising path (train.py:258-259) with torch's own kernels on the same inputs
        try:
            eg, cg = e.clone().requires_grad_(), c.clone().requires_grad_()

            def mat():
                eg.grad = cg.grad = None
                torch.nn.functional.cross_entropy((eg @ cg.t()).float(), t).backward()
            t_mat = time_region(mat, 2, 1)
            out["torch_materialised_fwd_bwd_ms"] = t_mat
            out["speedup_vs_torch_materialised"] = t_mat / t_all
        except RuntimeError as ex:       # out of memory on a smaller card
            out["torch_materialised_error"] = str(ex)[:200]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults long enough for the clocks to settle: the first ~50 steps of a cold GPU run 5-8 % slower
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-flex-baseline", action="store_true",
                    help="skip timing torch's compiled FlexAttention (the path maester runs today) on the same inputs")
    ap.add_argument("--no-hand-over", action="store_true",
                    help="backward without the dS workspace: the dQ kernel recomputes S and dP")
    ap.add_argument("--no-loss", action="store_true", help="skip the fused linear + cross-entropy block")
    ap.add_argument("--settle-seconds", type=float, default=2.0,
                    help="run untimed steps for this long before anything is timed, so that the clocks are at their steady state "
                         "whatever --warmup is (a GPU coming out of idle runs its first ~50 steps 5-8 %% slower)")
    ap.add_argument("--probe", action="store_true", help="also run the MFMA probe (sustained matrix-core rate and clock under load)")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay of the step)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU; --gpus N with N > 1 is not run "
              "(the path shards over batch rows / kv heads with no exchange between GPUs).", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback.", file=sys.stderr)
        sys.exit(3)

    from maester_amd import _lib, build_tile_map, packed_doc_attention, workloads
    from maester_amd.attention import (attention_backward, attention_forward, backward_workspace_bytes, prologue_backward,
                                       prologue_forward)

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    wl_cpu = workloads.make(args.workload)
    wl = wl_cpu.to(dev)
    sp = wl.spec
    K, W = args.steps, args.warmup

    # A plain 256 MiB device-to-device copy: the rate this GPU moves bytes at when nothing else is asked of it (the
    # bandwidth roof the kernels' traffic is priced against, beside the published 8 TB/s), and -- under rocprofv3
    # --pmc -- the reference point that FETCH_SIZE / WRITE_SIZE are scaled by.
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    t_copy = time_region(lambda: dst.copy_(src), 3 if args.calibrate_copy else 20, 3)
    copy_gbps = 2 * src.numel() / (t_copy * 1e-3) / 1e9
    del src, dst

    # ---- tile map (once per training step in the model; timed on its own) -------------------
    tmap = build_tile_map(wl.document_ids, sp.B, sp.S, True, sp.window)
    t_map = time_region(lambda: build_tile_map(wl.document_ids, sp.B, sp.S, True, sp.window), K, W)

    # ---- prologue --------------------------------------------------------------------------
    q, k, q_rstd, k_rstd = prologue_forward(wl.xq, wl.xk, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids)
    t_pro_f = time_region(lambda: prologue_forward(wl.xq, wl.xk, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids), K, W)
    elt = wl.xq.element_size()
    pro_bytes = 2 * elt * sp.B * sp.S * (sp.Hq + sp.Hkv) * sp.D + 8 * sp.B * sp.S + 8 * sp.B * sp.S * (sp.D // 2)

    # ---- attention: the timed step ------------------------------------------------------------
    out, lse = attention_forward(q, k, wl.xv, tmap, wl.document_ids, wl.scale, True, sp.window)
    has_bwd = wl.dout is not None
    bufs = None
    if has_bwd:
        dq, dk, dv = attention_backward(q, k, wl.xv, out, wl.dout, lse, tmap, wl.document_ids, wl.scale, True, sp.window)
        ws_bytes = backward_workspace_bytes(sp.B, sp.S, sp.Hq, sp.Hkv, sp.D, q.dtype, False if args.no_hand_over else None, tmap)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        bufs = (dq, dk, dv, ws)
        # the path the timed calls take is read off a call, not assumed
        attention_backward(q, k, wl.xv, out, wl.dout, lse, tmap, wl.document_ids, wl.scale, True, sp.window, buffers=bufs)
        hand_over = tmap.last_backward_path == "hand_over"

    def fwd():
        return attention_forward(q, k, wl.xv, tmap, wl.document_ids, wl.scale, True, sp.window)

    def bwd(stages=_lib.MA_BWD_ALL):
        return attention_backward(q, k, wl.xv, out, wl.dout, lse, tmap, wl.document_ids, wl.scale, True, sp.window,
                                  stages=stages, buffers=bufs)

    def step():
        fwd()
        if has_bwd:
            bwd()

    # steady state first: untimed steps for --settle-seconds
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()

    # per-kernel durations next (HIP events on the launch stream); the headline region below then
    # starts on a device that is already at its working clocks
    t_fwd = time_region(fwd, K, W)
    t_delta = t_dkv = t_dq = t_bwd = None
    if has_bwd:
        t_bwd = time_region(bwd, K, W)
        t_delta = time_region(lambda: bwd(_lib.MA_BWD_DELTA), K, W)
        t_dkv = time_region(lambda: bwd(_lib.MA_BWD_DKV), K, W)
        # as in the step: with the dS hand-over delta is a kernel of its own, otherwise it is fused into dQ
        t_dq = time_region(lambda: bwd(_lib.MA_BWD_DQ if hand_over else _lib.MA_BWD_DQ | _lib.MA_BWD_DELTA), K, W)
        t_pro_b = time_region(
            lambda: prologue_backward(wl.xq, wl.xk, dq, dk, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids, q_rstd,
                                      k_rstd), K, W)
    # The same kernels inside the step: the step is issued as its four launches with an event between them, so
    # that each kernel finds the caches as the kernel before it left them (a kernel repeated alone finds its own
    # inputs in the memory-side cache: the delta pass takes 1.6 times as long in the step as alone).
    in_step = None
    if has_bwd:
        stages = [("fwd", fwd), ("delta", lambda: bwd(_lib.MA_BWD_DELTA)), ("dkv", lambda: bwd(_lib.MA_BWD_DKV)),
                  ("dq", lambda: bwd(_lib.MA_BWD_DQ))] if hand_over else \
                 [("fwd", fwd), ("dq", lambda: bwd(_lib.MA_BWD_DQ | _lib.MA_BWD_DELTA)), ("dkv", lambda: bwd(_lib.MA_BWD_DKV))]
        for _ in range(W):
            step()
        n_ev = min(K, 50)
        evs = [_events(len(stages) + 1) for _ in range(n_ev)]
        for row in evs:
            row[0].record()
            for (_, f), e in zip(stages, row[1:]):
                f()
                e.record()
        torch.cuda.synchronize()
        in_step = {name: sum(row[i].elapsed_time(row[i + 1]) for row in evs) / n_ev for i, (name, _) in enumerate(stages)}
        in_step["sum_ms"] = sum(in_step.values())
    # the whole autograd Function (prologue + attention, forward + backward), for reference
    t_full = None
    if has_bwd:
        xs = [wl.xq.clone().requires_grad_(), wl.xk.clone().requires_grad_(), wl.xv.clone().requires_grad_()]
        ws_ = [None if w is None else w.clone().requires_grad_() for w in (wl.q_w, wl.k_w)]

        def full():
            o = packed_doc_attention(xs[0], xs[1], xs[2], ws_[0], ws_[1], wl.cos, wl.sin, wl.position_ids,
                                     wl.document_ids, wl.scale, True, sp.window, 1e-6, tmap)
            torch.autograd.grad(o, xs + [w for w in ws_ if w is not None], wl.dout)
        t_full = time_region(full, max(K // 2, 2), 2)

    # ---- sandwich RMSNorm + residual of the same model, on [B*S, model dim] (HBM roofline) -----------
    from maester_amd.rmsnorm import rmsnorm_backward, rmsnorm_forward
    model_dim = {"c1": 640, "c2": 2560, "c3": 2560, "c4": 3840, "c5": 4096}.get(args.workload, 2560)
    nx = torch.randn(sp.B * sp.S, model_dim, device=dev).to(wl.xq.dtype)
    nres, ndy = torch.randn_like(nx), torch.randn_like(nx)
    nw = 0.1 * torch.randn(model_dim, device=dev)
    _, nrstd = rmsnorm_forward(nx, nw, nres)
    kn = max(K // 4, 2)
    t_norm_f = time_region(lambda: rmsnorm_forward(nx, nw, nres), kn, max(W // 4, 1))
    t_norm_b = time_region(lambda: rmsnorm_backward(nx, nw, nrstd, ndy), kn, max(W // 4, 1))
    norm_bytes = 3 * nx.element_size() * nx.numel()        # x + residual in, sum out / x + dout in, dx out
    del nx, nres, ndy

    # ---- the headline region: W untimed steps, then exactly K timed steps ----------------------------
    # (the passes above left the GPU in another power state: back to the steady state of the step first)
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_seconds / 2:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    for _ in range(W):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    torch.cuda.synchronize()
    eager_ms_per_step = ms_per_step = (time.perf_counter() - t0) * 1e3 / K
    clock_after = gpu_clock_mhz()

    # Informational: the same K steps replayed from a HIP graph of one step (the library's launches are
    # graph-safe: no allocation, no host synchronisation, no memset; the work queues reset themselves on
    # the device).  Every replay must reproduce the eager step bit for bit.  The headline stays the eager
    # figure: at ~1 ms per step the four launches are queued far ahead of the GPU either way.
    launch = "eager launches through the C ABI"
    graph_error = None
    graph_ms_per_step = None
    if has_bwd and not args.no_graph:
        try:
            step()
            torch.cuda.synchronize()
            want = [t.clone() for t in (dq, dk, dv)]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            for rep in range(3):                      # replays with eager work and synchronisations in between
                for t in (dq, dk, dv):
                    t.zero_()
                graph.replay()
                torch.cuda.synchronize()
                if not all(torch.equal(a, b) for a, b in zip((dq, dk, dv), want)):
                    raise RuntimeError(f"graph replay {rep} differs from the eager step")
                step()
                torch.cuda.synchronize()
            for _ in range(W):
                graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(K):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms_per_step = (time.perf_counter() - t0) * 1e3 / K
        except Exception as e:  # noqa: BLE001 - the eager measurement stands
            graph_error = f"{type(e).__name__}: {str(e)[:200]}"

    vocab = 262144 if args.workload == "c1" else 262208
    loss = None if args.no_loss else loss_block(dev, sp.B * sp.S, model_dim, vocab, wl.xq.dtype, not args.no_flex_baseline)

    fl = wl.useful_flops()
    total_flops = fl["fwd_bwd"] if has_bwd else fl["fwd"]
    value = total_flops / (ms_per_step * 1e-3) / 1e12

    def tf(flops, ms):
        return None if ms is None else flops / (ms * 1e-3) / 1e12

    base = sp.D * sp.Hq * wl.n_pairs
    pair = (sp.Hq // sp.Hkv) % 2 == 0
    fwd_name = "attn_fwd_pair_bf16_kernel" if pair and sp.D >= 256 and sp.dtype == torch.bfloat16 else "attn_fwd_bf16_kernel"
    dq_name = (("attn_bwd_dq_ds_pair_bf16_kernel" if pair else "attn_bwd_dq_ds_bf16_kernel") if has_bwd and hand_over
               else "attn_bwd_dq_bf16_kernel")
    # Algorithmic bytes per launch: every operand and result once (what a kernel with unbounded on-chip memory moves)
    qb = elt * sp.B * sp.S * sp.Hq * sp.D             # one [B,S,Hq,D] tensor
    kb = elt * sp.B * sp.S * sp.Hkv * sp.D            # one [B,S,Hkv,D] tensor
    rowb = 4 * sp.B * sp.Hq * sp.S                    # one fp32 [B,Hq,S] array (lse, delta)
    dsb = (ws_bytes - rowb if has_bwd and hand_over else 0)   # the dS slots of the visited tiles
    kern = {
        fwd_name: {"ms": t_fwd, "algorithmic_flops": 4 * base, "algorithmic_bytes": 2 * qb + 2 * kb + rowb},    # Q, K, V in; O, lse out
        "attn_bwd_dkv_bf16_kernel": {"ms": t_dkv, "algorithmic_flops": 6 * base,                                  # dP, dV, dK
                                     "algorithmic_bytes": 2 * qb + 4 * kb + 2 * rowb + dsb},                      # Q, dO, K, V, lse, delta in; dK, dV, dS out
        dq_name: {"ms": t_dq, "algorithmic_flops": 2 * base,                                                      # dQ
                  "algorithmic_bytes": (dsb + kb + qb) if has_bwd and hand_over else (3 * qb + 2 * kb + 2 * rowb)},
    }
    if has_bwd and hand_over:
        kern["attn_delta_bf16_kernel"] = {"ms": t_delta, "algorithmic_flops": 0, "algorithmic_bytes": 2 * qb + rowb}
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    counters_file = os.path.join(ROOT, "profiles", "mfma_counters.json")
    tr, ctr = {}, {}
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            tr = json.load(f).get(sp.name, {})
    if os.path.exists(counters_file):
        with open(counters_file) as f:
            ctr = json.load(f).get(sp.name, {})
    step_name = {fwd_name: "fwd", "attn_bwd_dkv_bf16_kernel": "dkv", dq_name: "dq", "attn_delta_bf16_kernel": "delta"}
    for n, v in kern.items():
        if v["ms"] is None:
            continue
        v["tflops"] = tf(v["algorithmic_flops"], v["ms"])
        v["frac_mfma_peak"] = v["tflops"] / PEAK_BF16_DENSE_TFLOPS
        v["algorithmic_gbps"] = v["algorithmic_bytes"] / (v["ms"] * 1e-3) / 1e9
        v["frac_hbm_peak"] = v["algorithmic_gbps"] / PEAK_HBM_GBPS
        v["in_step_ms"] = None if in_step is None else in_step.get(step_name[n])
        # measured HBM traffic of a launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated, from profiles/) against
        # this run's time and this run's copy rate
        v["traffic_bytes"] = tr.get(n)
        if v["traffic_bytes"]:
            v["traffic_gbps"] = v["traffic_bytes"] / (v["ms"] * 1e-3) / 1e9
            v["traffic_frac_of_copy_rate"] = v["traffic_gbps"] / copy_gbps
            v["traffic_over_algorithmic"] = v["traffic_bytes"] / v["algorithmic_bytes"]
        if n in ctr:       # rocprofv3 --pmc counters of the same kernel and workload (profiles/*_mfma_counters.md)
            v["rocprof"] = ctr[n]
    timed = [n for n in kern if kern[n]["ms"] is not None and kern[n]["algorithmic_flops"]]
    dom_name = max(timed, key=lambda n: kern[n]["ms"])
    dom = kern[dom_name]
    # the dominant kernel against both roofs, labelled by the one it is nearer to
    roofs = {"mfma": {"achieved": dom["tflops"], "peak": PEAK_BF16_DENSE_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac_mfma_peak"]},
             "hbm": {"achieved": dom["algorithmic_gbps"], "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": dom["frac_hbm_peak"]}}
    bound = max(roofs, key=lambda r: roofs[r]["frac"])
    roofline = {
        "kernel": dom_name, "bound": bound, **roofs[bound], "traffic": dom.get("traffic_bytes"),
        "avg_launch_ms": dom["ms"], "algorithmic_flops_per_launch": dom["algorithmic_flops"],
        "algorithmic_bytes_per_launch": dom["algorithmic_bytes"], "roofs": roofs,
        "copy_gbps_this_run": copy_gbps, "traffic_gbps": dom.get("traffic_gbps"),
        "traffic_frac_of_copy_rate": dom.get("traffic_frac_of_copy_rate"),
        "mfma_utilisation_rocprof": (dom.get("rocprof") or {}).get("mfma_busy"),
    }

    T = (sp.S + 127) // 128
    n_partial, n_full = int(tmap.kv_num_blocks.sum()), int(tmap.full_kv_num_blocks.sum())
    result = {
        "metric": "useful TFLOP/s fwd+bwd doc-masked attn, Gemma3-4B S=8192 bf16; % MFMA peak",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if sp.dtype == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": sp.name, "description": sp.description, "B": sp.B, "S": sp.S, "Hq": sp.Hq,
                   "Hkv": sp.Hkv, "D": sp.D, "window": sp.window, "n_pairs": wl.n_pairs,
                   "timed_region": ("ma_attn_fwd + ma_attn_bwd (delta, dK/dV with dS hand-over, dQ) per step" if has_bwd and hand_over else
                                    "ma_attn_fwd + ma_attn_bwd (dQ with delta, dK/dV, both recomputing S and dP) per step" if has_bwd else
                                    "ma_attn_fwd per step") + ", inputs resident in HBM",
                   "launch": launch},
        "hip_graph_replay": {"ms_per_step": graph_ms_per_step, "error": graph_error,
                             "value": None if graph_ms_per_step is None else total_flops / (graph_ms_per_step * 1e-3) / 1e12},
        "pct_of_bf16_dense_peak": 100.0 * value / PEAK_BF16_DENSE_TFLOPS,
        "peak_bf16_dense_tflops": PEAK_BF16_DENSE_TFLOPS, "peak_hbm_gbps": PEAK_HBM_GBPS,
        "device_copy_gbps": copy_gbps,
        "settle_seconds": args.settle_seconds,
        "device": props.name, "gcn_arch": getattr(props, "gcnArchName", ""), "cus": props.multi_processor_count,
        "clock_mhz": clock_after, "clock_source": "pp_dpm_sclk right after the timed region (None: not readable on this box)",
        "useful_flops": fl,
        "fwd": {"ms": t_fwd, "tflops": tf(fl["fwd"], t_fwd), "pct_peak": 100 * tf(fl["fwd"], t_fwd) / PEAK_BF16_DENSE_TFLOPS},
        "bwd": None if not has_bwd else {"ms": t_bwd, "tflops": tf(fl["bwd"], t_bwd),
                                         "pct_peak": 100 * tf(fl["bwd"], t_bwd) / PEAK_BF16_DENSE_TFLOPS,
                                         "delta_ms": t_delta, "dkv_ms": t_dkv, "dq_ms": t_dq,
                                         "ds_hand_over": bool(hand_over), "path_taken": tmap.last_backward_path,
                                         "workspace_bytes": int(ws_bytes), "in_step_ms": in_step},
        "fwd_bwd_flashattn_convention_tflops": tf(fl["fwd_bwd_flashattn_convention"], ms_per_step) if has_bwd else None,
        "kernels": kern,
        "prologue": {"fwd_ms": t_pro_f, "fwd_gbps": pro_bytes / (t_pro_f * 1e-3) / 1e9,
                     "fwd_frac_hbm_peak": pro_bytes / (t_pro_f * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                     "algorithmic_bytes": pro_bytes,
                     "bwd_ms": t_pro_b if has_bwd else None},
        "sandwich_norm": {"rows": sp.B * sp.S, "dim": model_dim, "algorithmic_bytes": norm_bytes,
                          "fwd_residual_ms": t_norm_f, "fwd_gbps": norm_bytes / (t_norm_f * 1e-3) / 1e9,
                          "bwd_ms": t_norm_b, "bwd_gbps": norm_bytes / (t_norm_b * 1e-3) / 1e9},
        "tile_map": {"build_ms": t_map, "partial_tiles": n_partial, "full_tiles": n_full, "tiles": sp.B * T * T,
                     "skipped_tile_ratio": 1.0 - (n_partial + n_full) / float(sp.B * T * T),
                     "skipped_vs_causal": 1.0 - (n_partial + n_full) / float(sp.B * T * (T + 1) // 2)},
        "full_autograd_function_ms": t_full,
        "linear_cross_entropy": loss,
        "roofline": roofline,
    }
    if args.probe:
        result["mfma_probe"] = mfma_probe(dev, props.multi_processor_count)
    if not args.no_flex_baseline and sp.dtype == torch.bfloat16:
        fx = flex_gpu_baseline(wl, q, k)
        if "fwd_bwd_ms" in fx:
            fx["speedup_fwd"] = fx["fwd_ms"] / t_fwd
            fx["speedup_fwd_bwd"] = fx["fwd_bwd_ms"] / ms_per_step
            fx["speedup_tile_map"] = fx["create_block_mask_ms"] / t_map
        result["flex_gpu_baseline"] = fx
    if not args.no_cpu_baseline and has_bwd:
        result["cpu_baseline"] = cpu_baseline(wl_cpu)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
