"""Seeded synthetic workloads: the five packed-SFT attention configurations the path is measured on.

Each generator reproduces one configuration exactly (document-length distribution, packing with
the last document truncated, per-document ``position_ids``, N(0,1) activations, QK-norm weights,
RoPE theta).  Ids follow the input contract of maester's packed dataset
(maester/sft/packed_dataset.py:138-185): ``document_ids`` = index of the document per token,
``position_ids`` = offset inside the document, both int64 ``[B,S]``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch

from .rope import precompute_rope_tables


@dataclass
class WorkloadSpec:
    name: str
    B: int
    S: int
    Hq: int
    Hkv: int
    D: int
    dtype: torch.dtype
    theta: float
    window: int | None = None
    qk_norm: str = "unit"       # "unit" (w = 0), "normal" (g ~ N(1, 0.02), stored w = g - 1), "none"
    backward: bool = True
    lengths: str = "uniform"    # document-length law, see _draw_length
    seed: int = 0
    description: str = ""


SPECS = {
    "c1_plumbing_fp32": WorkloadSpec(
        "c1_plumbing_fp32", 1, 2048, 4, 1, 64, torch.float32, 1e4, None, "unit", False, "uniform_64_512", 0,
        "B=1 S=2048 Hq=4 Hkv=1 D=64 fp32, forward only, docs uniform[64,512]"),
    "c2_gemma3_4b_global": WorkloadSpec(
        "c2_gemma3_4b_global", 4, 8192, 8, 4, 256, torch.bfloat16, 1e6, None, "normal", True, "lognormal_600", 0,
        "Gemma-3-4B global layer: B=4 S=8192 Hq=8 Hkv=4 D=256 bf16, docs lognormal(ln 600, 1) in [32,8192]"),
    "c3_gemma3_4b_local": WorkloadSpec(
        "c3_gemma3_4b_local", 4, 8192, 8, 4, 256, torch.bfloat16, 1e4, 1024, "normal", True, "lognormal_600", 0,
        "Gemma-3-4B local layer: config 2 plus sliding window 1024, theta 1e4"),
    "c4_gemma3_12b": WorkloadSpec(
        "c4_gemma3_12b", 2, 16384, 16, 8, 256, torch.bfloat16, 1e6, None, "normal", True, "bimodal_pareto", 0,
        "Gemma-3-12B layer: B=2 S=16384 Hq=16 Hkv=8 D=256 bf16, row 0 one full document, row 1 Pareto(1.2) docs"),
    "c4s_gemma3_12b_sampled": WorkloadSpec(
        "c4s_gemma3_12b_sampled", 2, 16384, 16, 8, 256, torch.bfloat16, 1e6, None, "normal", True, "bimodal_pareto_sampled", 0,
        "Gemma-3-12B layer, seeded default: every row is one full document with probability 0.25 (rng.random() < 0.25), "
        "Pareto(1.2) docs otherwise"),
    "c5_llama3_8b_shape": WorkloadSpec(
        "c5_llama3_8b_shape", 4, 8192, 32, 8, 128, torch.bfloat16, 5e5, None, "none", True, "uniform_128_4096", 0,
        "Llama-3-8B-shaped layer: B=4 S=8192 Hq=32 Hkv=8 D=128 bf16, no QK-norm, docs uniform[128,4096]"),
}
ALIASES = {"c1": "c1_plumbing_fp32", "c2": "c2_gemma3_4b_global", "c3": "c3_gemma3_4b_local",
           "c4": "c4_gemma3_12b", "c4s": "c4s_gemma3_12b_sampled", "c5": "c5_llama3_8b_shape"}


def spec(name: str) -> WorkloadSpec:
    return SPECS[ALIASES.get(name, name)]


def _draw_length(rng: np.random.Generator, law: str, S: int) -> int:
    if law == "uniform_64_512":
        return int(rng.integers(64, 513))
    if law == "uniform_128_4096":
        return int(rng.integers(128, 4097))
    if law == "lognormal_600":
        return int(np.clip(rng.lognormal(math.log(600.0), 1.0), 32, 8192))
    if law == "pareto":
        return int(np.clip(16.0 * (1.0 + rng.pareto(1.2)), 16, S))
    raise ValueError(law)


def pack_row(rng: np.random.Generator, law: str, S: int) -> list:
    """Draw documents until the row is full; the last one is truncated.  Returns the lengths."""
    lens, filled = [], 0
    while filled < S:
        n = min(_draw_length(rng, law, S), S - filled)
        lens.append(n)
        filled += n
    return lens


def document_lengths(sp: WorkloadSpec) -> list:
    """Per batch row, the list of document lengths."""
    rng = np.random.default_rng(sp.seed)
    rows = []
    for b in range(sp.B):
        if sp.lengths == "bimodal_pareto":
            # 25 % of rows hold one document that fills the row; with B=2 the fraction cannot be
            # met by sampling, so row 0 is the full-document row and the others are Pareto rows.
            rows.append([sp.S] if b == 0 else pack_row(rng, "pareto", sp.S))
        elif sp.lengths == "bimodal_pareto_sampled":
            # the seeded default of the same configuration: the 25 % is drawn per row
            rows.append([sp.S] if rng.random() < 0.25 else pack_row(rng, "pareto", sp.S))
        else:
            rows.append(pack_row(rng, sp.lengths, sp.S))
    return rows


def ids_from_lengths(rows: list, S: int, pad_tail: int = 0):
    """(position_ids, document_ids) int64 [B,S]; the last ``pad_tail`` tokens of every row become
    padding (document id -1, position 0) as the packed dataset marks it."""
    B = len(rows)
    pos = torch.zeros(B, S, dtype=torch.long)
    doc = torch.full((B, S), -1, dtype=torch.long)
    for b, lens in enumerate(rows):
        start = 0
        for d, n in enumerate(lens):
            pos[b, start:start + n] = torch.arange(n)
            doc[b, start:start + n] = d
            start += n
    if pad_tail:
        pos[:, S - pad_tail:] = 0
        doc[:, S - pad_tail:] = -1
    return pos, doc


def count_pairs(rows: list, window: int | None = None) -> int:
    """Number of unmasked (q, kv) pairs over the batch (per q head) for doc+causal[+window]."""
    total = 0
    for lens in rows:
        for n in lens:
            if window is None or n <= window + 1:
                total += n * (n + 1) // 2
            else:
                w1 = window + 1
                total += w1 * (w1 + 1) // 2 + (n - w1) * w1
    return total


@dataclass
class Workload:
    spec: WorkloadSpec
    xq: torch.Tensor
    xk: torch.Tensor
    xv: torch.Tensor
    dout: torch.Tensor | None
    q_w: torch.Tensor | None
    k_w: torch.Tensor | None
    cos: torch.Tensor
    sin: torch.Tensor
    position_ids: torch.Tensor
    document_ids: torch.Tensor
    scale: float
    doc_lengths: list = field(default_factory=list)
    n_pairs: int = 0

    def to(self, device):
        def mv(t):
            return None if t is None else t.to(device)
        return Workload(self.spec, mv(self.xq), mv(self.xk), mv(self.xv), mv(self.dout), mv(self.q_w), mv(self.k_w),
                        mv(self.cos), mv(self.sin), mv(self.position_ids), mv(self.document_ids), self.scale,
                        self.doc_lengths, self.n_pairs)

    def useful_flops(self):
        """fwd = 4*D*Hq*N_pairs, bwd = 8*D*Hq*N_pairs (4 GEMMs; recompute not counted -- the MFU
        convention of maester/models/gemma/model.py:71-75)."""
        base = self.spec.D * self.spec.Hq * self.n_pairs
        return {"fwd": 4 * base, "bwd": 8 * base, "fwd_bwd": 12 * base, "fwd_bwd_flashattn_convention": 14 * base}


def make(name: str, B: int | None = None, S: int | None = None, pad_tail: int = 0, rows: int | None = None) -> Workload:
    """Build a workload on the CPU.  ``B``/``S`` shrink the configuration for parity tests (same
    distributions, same seed); ``rows`` keeps only the first rows of the batch."""
    sp = spec(name)
    if B is not None or S is not None:
        sp = WorkloadSpec(**{**sp.__dict__, "B": B or sp.B, "S": S or sp.S})
    lens = document_lengths(sp)
    if rows is not None:
        lens = lens[:rows]
        sp = WorkloadSpec(**{**sp.__dict__, "B": rows})
    pos, doc = ids_from_lengths(lens, sp.S, pad_tail)
    g = torch.Generator().manual_seed(sp.seed)

    def randn(*shape):
        return torch.randn(*shape, generator=g, dtype=torch.float32).to(sp.dtype)

    xq = randn(sp.B, sp.S, sp.Hq, sp.D)
    xk = randn(sp.B, sp.S, sp.Hkv, sp.D)
    xv = randn(sp.B, sp.S, sp.Hkv, sp.D)
    dout = randn(sp.B, sp.S, sp.Hq, sp.D) if sp.backward else None
    if sp.qk_norm == "none":
        q_w = k_w = None
    elif sp.qk_norm == "unit":
        q_w, k_w = torch.zeros(sp.D), torch.zeros(sp.D)
    else:
        q_w = (1.0 + 0.02 * torch.randn(sp.D, generator=g)) - 1.0
        k_w = (1.0 + 0.02 * torch.randn(sp.D, generator=g)) - 1.0
    cos, sin = precompute_rope_tables(sp.D, max(sp.S, int(pos.max()) + 1), sp.theta)
    n_pairs = count_pairs(lens, sp.window) if pad_tail == 0 else -1
    return Workload(sp, xq, xk, xv, dout, q_w, k_w, cos, sin, pos, doc, sp.D ** -0.5, lens, n_pairs)
