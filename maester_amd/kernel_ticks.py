"""Where the cycles of a step go: cycle counts between marked points inside the attention kernels.

The dK/dV kernel and the pair forward kernel carry marks (``MA_TICK(n)`` in ``csrc/attn_bwd_bf16.hip``
and ``csrc/attn_fwd_pair_bf16.hip``) that compile to nothing in the library.  Built with
``-DMA_TICKS -DMA_T_BEGIN=a -DMA_T_END=b`` a kernel reads the shader-clock counter (``s_memtime``) at
marks ``a`` and ``b`` and sums the differences per wave; one interval per build keeps the cost of
measuring at one counter read per mark.  The marks:

    7 item begins            0 step begins                 2 a 32-row block begins
    8 item ends              20 own tile loads have landed 3 behind its first chain (S, dP / S^T)
                             1 behind the step's barrier   4 before its second chain (dV, dK / O^T)
                             6 step ends                   5 behind its second chain
  forward only:  9 the item's place in the schedule is known   10 its first tiles are requested (walk resolved,
                 Q rows requested)   11 the pass begins   12 the passes are over   13 epilogue begins (behind its
                 barrier)   14 / 15 first / second head is written out

``python -m maester_amd.kernel_ticks build`` (no GPU needed) builds one variant library per interval
into ``maester_amd/ticks_build/``; ``python -m maester_amd.kernel_ticks measure --workload c2`` runs
them on the GPU, each in a process of its own, and prints one line per interval: mean cycles, how
often per workgroup, share of the wave's cycles, and the clock the kernel ran at (cycles / time).
``--wave N`` (both commands) measures wave N of every workgroup instead of wave 0: the waves of a
workgroup skip different 32-row blocks of a partial tile, so what one wave spends at the step's
barrier (20 -> 1) is mostly the work another wave still has.
"""
from __future__ import annotations

import argparse
import ctypes
import os
import subprocess
import sys

from . import build as _build

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "ticks_build")
KERNELS = {"dkv": ("attn_bwd_bf16.hip", "ma_dbg_read_ticks"), "fwd": ("attn_fwd_pair_bf16.hip", "ma_dbg_read_ticks_fwd")}
INTERVALS = [(0, 1, "step begins -> behind the barrier (rows to LDS, next record, wait for the tiles)"),
             (0, 20, "step begins -> the wave's own tile loads have landed"),
             (20, 1, "-> behind the barrier (the other waves' loads and work)"),
             (1, 2, "behind the barrier -> first block (control)"),
             (2, 3, "block begins -> behind the first chain"),
             (3, 4, "elementwise between the chains"),
             (4, 5, "second chain"),
             (0, 6, "whole step"),
             (7, 0, "item begins -> first step (prologue)"),
             (6, 8, "last step ends -> item ends (epilogue)"),
             (7, 8, "whole item")]
EXTRA = {"fwd": [(7, 9, "item begins -> its place in the schedule is known (ticket, order entry)"),
                 (9, 10, "-> walk resolved, Q rows and first tiles requested"),
                 (10, 11, "-> the pass begins"),
                 (6, 12, "last step ends -> the passes are over (last wait for the tiles, barrier, redo flag)"),
                 (13, 14, "epilogue: first head scaled, turned through LDS and written out"),
                 (14, 15, "epilogue: second head")],
         "dkv": []}


def _intervals(kernel: str):
    return INTERVALS + EXTRA[kernel]


WAVE = 0     # the wave of every workgroup that is measured (set from --wave)


def _variant(kernel: str, a: int, b: int) -> str:
    return os.path.join(OUT, f"libticks_{kernel}_{a}_{b}" + (f"_w{WAVE}" if WAVE else "") + ".so")


def _build_one(job) -> str:
    kernel, src, a, b = job
    others = [os.path.join(_build.OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in _build.SOURCES if s != src]
    obj = os.path.join(OUT, f"{kernel}_{a}_{b}_w{WAVE}.o")
    flags = [f for f in _build.HIPCC_FLAGS if not f.startswith("-W")]
    cmd = [_build._hipcc(), *flags, "-DMA_TICKS", f"-DMA_T_BEGIN={a}", f"-DMA_T_END={b}", f"-DMA_T_WAVE={WAVE}", "-c",
           os.path.join(_build.CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(res.stderr)
    res = subprocess.run([_build._hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", _variant(kernel, a, b), *others, obj],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(res.stderr)
    os.remove(obj)
    return _variant(kernel, a, b)


def build_variants(jobs: int = 6) -> None:
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OUT, exist_ok=True)
    _build.build()  # the other objects come from the library's own build
    todo = [(kernel, src, a, b) for kernel, (src, _) in KERNELS.items() for a, b, _ in _intervals(kernel)]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for path in ex.map(_build_one, todo):
            print("built", path, flush=True)


def _one(kernel: str, a: int, b: int, workload: str, launches: int, settle: float) -> None:
    """Runs in a process of its own: the variant library is the only one this process loads."""
    import torch
    from . import _lib
    _lib.LIB_PATH = _variant(kernel, a, b)
    from . import build_tile_map, workloads
    from .attention import attention_backward, attention_forward, backward_workspace_bytes, prologue_forward
    wl = workloads.make(workload).to("cuda")
    sp = wl.spec
    tm = build_tile_map(wl.document_ids, sp.B, sp.S, True, sp.window, device="cuda")
    q, k = wl.xq, wl.xk
    if wl.q_w is not None:
        q, k, _, _ = prologue_forward(wl.xq, wl.xk, wl.q_w, wl.k_w, wl.cos, wl.sin, wl.position_ids)
    out, lse = attention_forward(q, k, wl.xv, tm, wl.document_ids, wl.scale, True, sp.window)
    if kernel == "dkv":
        dq, dk, dv = attention_backward(q, k, wl.xv, out, wl.dout, lse, tm, wl.document_ids, wl.scale, True, sp.window)
        ws = torch.empty(backward_workspace_bytes(sp.B, sp.S, sp.Hq, sp.Hkv, sp.D, q.dtype, None, tm), dtype=torch.uint8, device="cuda")
        bufs = (dq, dk, dv, ws)
        run = lambda: attention_backward(q, k, wl.xv, out, wl.dout, lse, tm, wl.document_ids, wl.scale, True, sp.window, stages=2, buffers=bufs)
    else:
        run = lambda: attention_forward(q, k, wl.xv, tm, wl.document_ids, wl.scale, True, sp.window)
    read = getattr(ctypes.CDLL(_lib.LIB_PATH), KERNELS[kernel][1])
    vals = (ctypes.c_ulonglong * 4)()
    import time
    t_end = time.time() + settle  # the clocks climb for a while after the GPU was idle: measure what they settle at
    while True:
        for _ in range(10):
            run()
        torch.cuda.synchronize()
        if time.time() >= t_end:
            break
    read(vals, 1)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / launches
    read(vals, 1)
    acc, cnt, tot, wgs = (int(v) for v in vals)
    print(f"{kernel} {a}->{b}: {acc / max(cnt, 1):9.1f} cycles x {cnt / max(wgs, 1):7.1f} per workgroup = {100.0 * acc / max(tot, 1):5.1f} % of "
          f"the wave's {tot / max(wgs, 1) / 1e3:8.1f} kcycles; {ms:.4f} ms per launch -> {tot / max(wgs, 1) / ms / 1e3:.0f} MHz", flush=True)


def measure(workload: str, kernels: list, launches: int, settle: float) -> None:
    for kernel in kernels:
        for a, b, what in _intervals(kernel):
            if not os.path.exists(_variant(kernel, a, b)):
                raise RuntimeError(f"{_variant(kernel, a, b)} is missing: run `python -m maester_amd.kernel_ticks build` first")
            res = subprocess.run([sys.executable, "-m", "maester_amd.kernel_ticks", "one", "--kernel", kernel, "--begin", str(a), "--end", str(b),
                                  "--wave", str(WAVE), "--workload", workload, "--launches", str(launches), "--settle-seconds", str(settle)], capture_output=True, text=True, timeout=300)
            if res.returncode != 0:
                raise RuntimeError(res.stderr[-2000:])
            print(res.stdout.strip() + f"   # {what}", flush=True)


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=["build", "measure", "one"])
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--kernel", default=None, choices=[None, "dkv", "fwd"])
    ap.add_argument("--begin", type=int, default=0)
    ap.add_argument("--end", type=int, default=6)
    ap.add_argument("--launches", type=int, default=20)
    ap.add_argument("--wave", type=int, default=0, choices=[0, 1, 2, 3], help="which wave of every workgroup is measured")
    ap.add_argument("--settle-seconds", type=float, default=1.5, help="launches repeated this long before the measured ones")
    args = ap.parse_args()
    WAVE = args.wave
    if args.what == "build":
        build_variants()
    elif args.what == "measure":
        measure(args.workload, [args.kernel] if args.kernel else ["fwd", "dkv"], args.launches, args.settle_seconds)
    else:
        _one(args.kernel, args.begin, args.end, args.workload, args.launches, args.settle_seconds)
