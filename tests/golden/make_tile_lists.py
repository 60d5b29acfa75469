"""Writes tests/golden/tile_lists.json: BlockMask tile lists from torch's own
``create_block_mask`` (CPU) for small id layouts, driven by the restated mask predicate.
Run from the repo root:  python tests/golden/make_tile_lists.py
"""
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import tile_map as otm  # noqa: E402


def layouts():
    rng = np.random.default_rng(7)
    out = []
    ids = torch.zeros((1, 128), dtype=torch.long)
    ids[:, 32:64] = 1; ids[:, 64:96] = 2; ids[:, 96:] = 3
    out.append(("four_docs_one_block", ids, True, None))
    ids = torch.zeros((1, 256), dtype=torch.long); ids[:, 176:] = 1
    out.append(("boundary_176", ids, True, None))
    ids = torch.zeros((2, 640), dtype=torch.long)
    ids[0, 100:333] = 1; ids[0, 333:] = 2; ids[1, 384:] = 1
    out.append(("two_rows_640", ids, True, None))
    out.append(("two_rows_640_window_200", ids, True, 200))
    ids = torch.zeros((1, 1000), dtype=torch.long)
    ids[:, 512:900] = 1; ids[:, 900:] = -1
    out.append(("ragged_1000_padding", ids, True, None))
    out.append(("ragged_1000_padding_window_128", ids, True, 128))
    out.append(("no_ids_causal_500", None, True, None))
    out.append(("no_ids_window_256_s1024", None, True, 256))
    out.append(("random_ids_300", torch.from_numpy(rng.integers(0, 3, size=(1, 300))), True, None))
    return out


def main():
    cases = []
    for name, ids, causal, window in layouts():
        B, S = (1, int(name.split("_s")[-1]) if "_s1024" in name else 500) if ids is None else ids.shape
        bm = otm.torch_block_mask(ids, B, S, causal, window)
        cases.append({
            "name": name, "B": B, "S": S, "causal": causal, "window": window,
            "document_ids": None if ids is None else ids.tolist(),
            "expect": {k: getattr(bm, k).tolist() for k in otm.NAMES},
        })
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tile_lists.json")
    with open(path, "w") as f:
        json.dump({"source": f"torch {torch.__version__} create_block_mask, BLOCK_SIZE=128", "cases": cases}, f)
    print(path, os.path.getsize(path))


if __name__ == "__main__":
    main()
