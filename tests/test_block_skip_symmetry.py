"""The invariant behind the dS hand-over of the backward, checked on the CPU.

The dK/dV kernel leaves dS^T in the workspace only for the 32 x 32 blocks its waves work on; the dQ
kernel multiplies only the blocks its waves work on.  That is sound when every block the dQ side uses is
one the dK/dV side wrote.  Both kernels decide per block with ``visibility_limits`` / ``block_inside``
(``maester_amd/csrc/common.h``) and the id-range test on ``ma_tile_map.block_doc_range``
(``DkvSteps::refill`` in ``csrc/attn_bwd_bf16.hip``, ``StepTable::fill`` in ``csrc/common.h``); here the
same formulas are restated in Python, evaluated on both sides for every block of every visited tile, and
compared -- together with the other two facts the hand-over needs: a block that holds a visible pair is
used on both sides (nothing is lost), and a block the dQ side uses lies in a 64-row q step that the
dK/dV workgroup walks (so the write has happened)."""
import numpy as np
import pytest
import torch

from oracle import masks as M
from oracle import tile_map as otm

TILE, STEP, BLK = 128, 64, 32
NO_LO, NO_HI = -0x40000000, 0x7FFFFFFF


def visibility_limits(kv_side, own_lo, own_hi, rows, bounded, wlim, windowed):
    # csrc/common.h visibility_limits
    if not kv_side:
        hi = own_hi if bounded else NO_HI
        lo = own_lo - wlim - (rows - 1) if windowed else NO_LO
    else:
        lo = own_lo - (rows - 1) if bounded else NO_LO
        hi = own_hi + wlim if windowed else NO_HI
    return lo, hi


def block_inside(r0, S, partial, lo, hi):
    return r0 < S and (not partial or (lo <= r0 <= hi))


def block_ranges(doc_row, S):
    """(min, max) id of every 32-row block; blocks past the end repeat the last row (ma_tile_map.block_doc_range)."""
    n = 2 * ((S + 63) // 64)
    out = []
    for i in range(n):
        rows = doc_row[min(i * BLK, S - 1): min(i * BLK + BLK, S)] if i * BLK < S else doc_row[S - 1:S]
        out.append((int(rows.min()), int(rows.max())))
    return out


def meets(a, b):
    return a[0] <= b[1] and a[1] >= b[0]


def _ids(S, kind, seed):
    g = np.random.default_rng(seed)
    if kind == "none":
        return None
    doc = np.zeros(S, dtype=np.int64)
    at, d = 0, 0
    while at < S:
        n = int(g.integers(5, 300))
        doc[at:at + n] = d if kind != "recurring" else int(g.integers(0, 4))
        at, d = at + n, d + 1
    if kind == "padded":
        doc[S - int(g.integers(1, 100)):] = -1
    return doc


@pytest.mark.parametrize("S,window,kind,seed", [(512, None, "docs", 0), (1000, None, "docs", 1), (777, 100, "docs", 2),
                                                (640, 0, "padded", 3), (900, 300, "recurring", 4), (384, 64, "none", 5),
                                                (1500, None, "recurring", 6), (129, None, "docs", 7)])
def test_dq_side_uses_only_blocks_the_dkv_side_wrote(S, window, kind, seed):
    doc = _ids(S, kind, seed)
    ids = None if doc is None else torch.from_numpy(doc)[None]
    tl = otm.tile_lists(ids, 1, S, True, window)
    T = (S + TILE - 1) // TILE
    dense = M.dense_mask_np(None if doc is None else doc[None], 1, S, True, window)[0]
    rng = None if doc is None else block_ranges(doc, S)
    bounded, windowed = True, window is not None
    wlim = window if windowed else NO_HI
    kind_of = {}                                    # (q tile, kv tile) -> partial?
    for i in range(T):
        for n, idx, partial in ((tl["kv_num_blocks"], tl["kv_indices"], True), (tl["full_kv_num_blocks"], tl["full_kv_indices"], False)):
            for j in idx[0, 0, i, : int(n[0, 0, i])].tolist():
                kind_of[(i, j)] = partial
    used_dq = used_dkv = 0
    for (i, j), partial in kind_of.items():
        # the 64-row q steps of tile i that the dK/dV workgroup of kv tile j walks
        vis_lo, vis_hi = visibility_limits(True, j * TILE, j * TILE + TILE - 1, STEP, bounded, wlim, windowed)
        walked = {h for h in range(TILE // STEP) if block_inside(i * TILE + h * STEP, S, partial, vis_lo, vis_hi)}
        # ... and the 64-row kv steps of tile j that the dQ workgroup of q tile i walks
        qvis_lo, qvis_hi = visibility_limits(False, i * TILE, i * TILE + TILE - 1, STEP, bounded, wlim, windowed)
        qwalked = {h for h in range(TILE // STEP) if block_inside(j * TILE + h * STEP, S, partial, qvis_lo, qvis_hi)}
        for qb in range(TILE // BLK):               # 32-row q block = a wave of the dQ side
            for kb in range(TILE // BLK):           # 32-row kv block = a wave of the dK/dV side
                q0, k0 = i * TILE + qb * BLK, j * TILE + kb * BLK
                # dQ side: wave of q rows q0.., block of kv rows k0..
                lo, hi = visibility_limits(False, q0, q0 + BLK - 1, BLK, bounded, wlim, windowed)
                act_q = (k0 // STEP * STEP - j * TILE) // STEP in qwalked and block_inside(k0, S, partial, lo, hi)
                if act_q and rng is not None and partial:
                    act_q = meets(rng[k0 // BLK], rng[min(q0, S - 1) // BLK])
                # dK/dV side: wave of kv rows k0.., block of q rows q0..
                lo, hi = visibility_limits(True, k0, k0 + BLK - 1, BLK, bounded, wlim, windowed)
                act_k = (q0 // STEP * STEP - i * TILE) // STEP in walked and block_inside(q0, S, partial, lo, hi)
                if act_k and rng is not None and partial:
                    act_k = meets(rng[q0 // BLK], rng[min(k0, S - 1) // BLK])
                has_pair = bool(dense[q0:q0 + BLK, k0:k0 + BLK].any())
                own_rows_exist = q0 < S             # a dQ wave whose rows lie past the end computes columns it never stores
                if act_q and own_rows_exist:
                    assert act_k, (S, window, kind, (i, j), (qb, kb), "dQ would use a block nobody wrote")
                if has_pair:
                    assert act_q and act_k, (S, window, kind, (i, j), (qb, kb), "a visible pair would be lost")
                used_dq += act_q
                used_dkv += act_k
    assert used_dq > 0 and used_dkv > 0
