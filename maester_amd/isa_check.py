"""Static checks of the compiler's output for the kernels that issue instructions through ``asm``.

The compiler knows nothing about what an ``asm`` statement does, so two kinds of hazard that it
normally handles are the source's responsibility there; this module re-checks them on the generated
gfx950 assembly (``python -m maester_amd.isa_check`` or ``check_all()``):

1. **MFMA results.**  No hazard padding is inserted around ``asm`` MFMAs: between an MFMA and the
   next fence (``s_nop`` of 16 wait states), branch, label or barrier, no compiler-scheduled vector
   or memory instruction may read or write a register that one of the last two MFMAs wrote (an
   8-pass MFMA's result needs 11 wait states before the vector ALU may touch it; a register that
   two later MFMAs, 16 passes, have left alone is safe -- the kernels use that to work on a finished
   accumulator from the hooks of the chain that follows).
2. **MFMA operands.**  A fragment that the register allocator keeps in the "wrong" register file
   is copied into place right in front of the ``asm`` MFMA that names it (``v_accvgpr_write``,
   ``v_mov``), and the MFMA then reads a register the vector ALU wrote less than two wait states
   earlier.  Compiler-issued MFMAs get the padding; ``asm`` ones do not and silently compute with
   stale operands.  No ``asm`` MFMA may read, as A or B, a register that a vector-ALU instruction
   wrote within the two preceding wait states.
3. **Scalar loads in flight.**  An ``asm`` ``s_load`` returns its data some hundred cycles later,
   into the physical registers it named.  Until the next ``s_waitcnt lgkmcnt(0)`` nothing may read
   or write those registers: a spill of the (not yet loaded) tuple, followed by a reuse of the
   registers for something else, ends with the load overwriting that something else.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
SOURCES = ["attn_fwd_bf16.hip", "attn_fwd_pair_bf16.hip", "attn_bwd_bf16.hip"]
FLAGS = ("--offload-arch=gfx950 -O3 -std=c++17 -ffast-math -fno-finite-math-only -Xclang -target-feature "
         "-Xclang -packed-fp32-ops -S --cuda-device-only").split()


def _regs(text: str, classes: str) -> set:
    """(class, index) of every register of the given classes named in an operand string."""
    out = set()
    for cls, lo, hi in re.findall(r"\b([%s])\[(\d+):(\d+)\]" % classes, text):
        out |= {(cls, i) for i in range(int(lo), int(hi) + 1)}
    for cls, i in re.findall(r"\b([%s])(\d+)\b" % classes, text):
        out.add((cls, int(i)))
    return out


def check_assembly(asm: str) -> tuple[list[str], dict]:
    """Returns (violations, {kernel: (asm MFMAs, asm scalar loads)})."""
    bad, stats = [], {}
    for m in re.finditer(r"^(_ZN2ma\w+):[^\n]*\n(.*?)s_endpgm", asm, re.S | re.M):
        name, body = m.group(1), m.group(2).split("\n")
        in_asm = False
        chain = {}         # vector register written by an MFMA of the current chain -> MFMAs issued since
        pending = set()    # scalar registers of asm loads that have not been waited for
        recent = []        # (vector registers written by a VALU instruction, wait states since)
        n_mfma = n_sload = 0
        for i, ln in enumerate(body):
            t = ln.strip()
            if t.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if t.startswith(";;#ASMEND"):
                in_asm = False
                continue
            if not t or t.startswith(";"):
                continue
            if t.startswith((".LBB", "s_cbranch", "s_branch", "s_barrier")):
                chain = {}
                recent = []
                if pending and t.startswith(("s_cbranch", "s_branch")):
                    # a branch between an asm load and its wait: the linear scan no longer follows the program
                    pass
                continue
            mm = re.match(r"s_nop (\d+)", t)
            if mm:
                if int(mm.group(1)) >= 15:
                    chain = {}
                recent = [(r, d + int(mm.group(1)) + 1) for r, d in recent if d + int(mm.group(1)) + 1 < 2]
                continue
            ops = t.split(None, 1)[1] if " " in t else ""
            if t.startswith("s_waitcnt"):
                if "lgkmcnt(0)" in t:
                    pending = set()
                continue
            if pending:
                hit = _regs(ops, "s") & pending
                if hit and not (in_asm and t.startswith("s_load")):
                    bad.append(f"{name} line {i}: '{t}' touches scalar registers of a load in flight {sorted(hit)[:4]}")
            if in_asm and t.startswith("v_mfma"):
                srcs = _regs(",".join(ops.split(",")[1:3]), "va")
                for regs_written, d in recent:
                    hit = srcs & regs_written
                    if hit:
                        bad.append(f"{name} line {i}: '{t}' reads {sorted(hit)[:4]} written by the vector ALU {d} wait state(s) earlier")
            recent = [(r, d + 1) for r, d in recent if d + 1 < 2]
            if not in_asm and t.startswith("v_") and not t.startswith(("v_cmp", "v_readlane", "v_readfirstlane")):
                recent.append((_regs(ops.split(",")[0], "va"), 0))
            if in_asm:
                if t.startswith("v_mfma"):
                    n_mfma += 1
                    chain = {r: age + 1 for r, age in chain.items() if age + 1 < 2}
                    chain.update({r: 0 for r in _regs(ops.split(",")[0], "va")})
                elif t.startswith("s_load"):
                    n_sload += 1
                    pending |= _regs(ops.split(",")[0], "s")
                continue
            if chain and re.match(r"(v_|ds_|global_|buffer_|flat_|scratch_)", t):
                hit = _regs(ops, "va") & set(chain)
                if hit:
                    bad.append(f"{name} line {i}: '{t}' touches in-flight MFMA result {sorted(hit)[:4]}")
        stats[name] = (n_mfma, n_sload)
    return bad, stats


def kernel_resources(asm: str) -> dict:
    """{kernel: {"vgpr", "agpr", "sgpr", "vgpr_spill", "sgpr_spill", "lds"}} from the metadata the compiler
    appends to its assembly.  The MFMA kernels are written around the register file (accumulators that fill
    all 256 AGPRs, operand fragments that fill half of the VGPRs): a vector register that spills lands in
    scratch memory inside an MFMA chain and costs whole factors, which the numerics tests would not notice."""
    out = {}
    for m in re.finditer(r"- \.agpr_count:\s+\d+.*?\.wavefront_size", asm, re.S):
        body = m.group(0)

        def field(key, body=body):
            mm = re.search(r"\." + key + r":\s+(\S+)", body)
            return mm.group(1) if mm else None
        name = field("name")
        if name and name.startswith("_ZN2ma"):
            out[name] = {"vgpr": int(field("vgpr_count")), "agpr": int(field("agpr_count")), "sgpr": int(field("sgpr_count")),
                         "vgpr_spill": int(field("vgpr_spill_count")), "sgpr_spill": int(field("sgpr_spill_count")),
                         "lds": int(field("group_segment_fixed_size"))}
    return out


def compile_to_assembly(source: str) -> str:
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        r = subprocess.run(["hipcc", *FLAGS, os.path.join(CSRC, source), "-o", out], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc -S {source} failed:\n{r.stderr[-2000:]}")
        with open(out) as f:
            return f.read()


def check_all(sources=SOURCES, resources: dict | None = None) -> tuple[list[str], dict]:
    """Hazard check of every source; ``resources`` (a dict) is filled with ``kernel_resources`` of the same assembly."""
    bad, stats = [], {}
    with ThreadPoolExecutor(max_workers=len(sources)) as pool:
        for asm in pool.map(compile_to_assembly, sources):
            b, s = check_assembly(asm)
            bad += b
            stats.update(s)
            if resources is not None:
                resources.update(kernel_resources(asm))
    return bad, stats


if __name__ == "__main__":
    res = {}
    bad, stats = check_all(sys.argv[1:] or SOURCES, res)
    for name, (nm, ns) in stats.items():
        r = res.get(name, {})
        print(f"{name}: {nm} asm MFMAs, {ns} asm scalar loads; {r.get('vgpr')} vector registers ({r.get('agpr')} of them accumulation), "
              f"{r.get('vgpr_spill')} spilled; {r.get('sgpr_spill')} scalar registers spilled to vector lanes")
    for b in bad[:40]:
        print(b)
    print("BAD" if bad else "OK")
    sys.exit(1 if bad else 0)
