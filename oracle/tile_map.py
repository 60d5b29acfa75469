"""Block-sparse tile lists (torch ``BlockMask`` format), restated.  Test infrastructure only.

Call sites in the reference: maester/models/gemma/model.py:699-706 (global) and 723-730
(local), ``create_block_mask(fn, B, None, S, S)``.  The algorithm lives in torch
(third-party): torch/nn/attention/flex_attention.py
  _convert_mask_to_block_mask (979-1022): zero-pad to a multiple of 128, count each
      128x128 tile; full = count == 16384, partial = 0 < count < 16384 (disjoint);
  _dense_to_ordered (429-436): num = row sum, indices = stable descending argsort of the
      0/1 row  ==  set columns ascending, then unset columns ascending;
  _transpose_ordered (439-441): the q-side lists are the same on the transposed matrix.
Head dim is 1 (H=None broadcasts).  All outputs int32.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

from . import masks

BLOCK = 128
NAMES = ("kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices",
         "q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices")


def tile_classes_np(document_ids, B, S, causal=True, window=None) -> np.ndarray:
    """[B, T, T] uint8: 0 empty, 1 partial, 2 full -- brute force over the dense mask."""
    T = (S + BLOCK - 1) // BLOCK
    cls = np.zeros((B, T, T), dtype=np.uint8)
    for b in range(B):
        ids_b = None if document_ids is None else np.asarray(document_ids)[b:b + 1]
        m = masks.dense_mask_np(ids_b, 1, S, causal, window)[0]
        pad = T * BLOCK - S
        if pad:
            m = np.pad(m, ((0, pad), (0, pad)))
        cnt = m.reshape(T, BLOCK, T, BLOCK).sum(axis=(1, 3))
        cls[b][cnt > 0] = 1
        cls[b][cnt == BLOCK * BLOCK] = 2
    return cls


def _ordered(dense01: np.ndarray):
    """Row sums + stable descending argsort of a 0/1 matrix batch [..., R, C]."""
    num = dense01.sum(axis=-1).astype(np.int32)
    idx = np.argsort(-dense01.astype(np.int32), axis=-1, kind="stable").astype(np.int32)
    return num, idx


def lists_from_classes(cls: np.ndarray) -> dict:
    partial = (cls == 1)
    full = (cls == 2)
    out = {}
    out["kv_num_blocks"], out["kv_indices"] = _ordered(partial)
    out["full_kv_num_blocks"], out["full_kv_indices"] = _ordered(full)
    out["q_num_blocks"], out["q_indices"] = _ordered(np.swapaxes(partial, -1, -2))
    out["full_q_num_blocks"], out["full_q_indices"] = _ordered(np.swapaxes(full, -1, -2))
    # head dim of 1, as BlockMask carries it
    return {k: torch.from_numpy(np.ascontiguousarray(v[:, None])) for k, v in out.items()}


def tile_lists(document_ids, B, S, causal=True, window=None) -> dict:
    """The eight BlockMask tensors ([B,1,T] / [B,1,T,T] int32) from the restated predicate."""
    ids = None if document_ids is None else np.asarray(document_ids)
    return lists_from_classes(tile_classes_np(ids, B, S, causal, window))


def torch_block_mask(document_ids, B, S, causal=True, window=None):
    """torch's own ``create_block_mask`` driven by the restated predicate (CPU)."""
    from torch.nn.attention.flex_attention import create_block_mask
    mod = masks.make_mask_mod(document_ids, causal, window)
    return create_block_mask(mod, B, None, S, S, device="cpu")


def block_mask_to_dict(bm) -> dict:
    return {k: getattr(bm, k) for k in NAMES}


# ----------------------------------------------------------------------------------------------
# C restatement (oracle/tile_map_ref.c), for sizes where numpy's dense [S,S] pass is slow.
# ----------------------------------------------------------------------------------------------
_HERE = os.path.dirname(os.path.abspath(__file__))
_C_SRC = os.path.join(_HERE, "tile_map_ref.c")
_C_LIB = os.path.join(_HERE, "_build", "libtile_map_ref.so")


def build_c(force: bool = False) -> str:
    os.makedirs(os.path.dirname(_C_LIB), exist_ok=True)
    if force or not os.path.exists(_C_LIB) or os.path.getmtime(_C_LIB) < os.path.getmtime(_C_SRC):
        subprocess.check_call(["gcc", "-O2", "-shared", "-fPIC", "-o", _C_LIB, _C_SRC])
    return _C_LIB


def tile_lists_c(document_ids, B, S, causal=True, window=None) -> dict:
    lib = ctypes.CDLL(build_c())
    T = (S + BLOCK - 1) // BLOCK
    ids = None
    if document_ids is not None:
        ids = np.ascontiguousarray(np.asarray(document_ids), dtype=np.int64)
        assert ids.shape == (B, S)
    outs = {}
    ptrs = []
    for n in NAMES:
        shape = (B, 1, T) if n.endswith("num_blocks") else (B, 1, T, T)
        outs[n] = np.zeros(shape, dtype=np.int32)
        ptrs.append(outs[n].ctypes.data_as(ctypes.c_void_p))
    lib.oracle_tile_map.restype = ctypes.c_int
    rc = lib.oracle_tile_map(
        None if ids is None else ids.ctypes.data_as(ctypes.c_void_p),
        ctypes.c_int(B), ctypes.c_int(S), ctypes.c_int(1 if causal else 0),
        ctypes.c_longlong(-1 if window is None else window), *ptrs)
    assert rc == 0
    return {k: torch.from_numpy(v) for k, v in outs.items()}


def count_pairs(document_ids, B, S, causal=True, window=None) -> int:
    """N_pairs = number of allowed (q, kv) pairs over the batch (useful-FLOP accounting)."""
    total = 0
    for b in range(B):
        ids_b = None if document_ids is None else np.asarray(document_ids)[b:b + 1]
        total += int(masks.dense_mask_np(ids_b, 1, S, causal, window).sum())
    return total
