"""Pins the tile-list oracle (numpy and C) against torch's own create_block_mask, the known
layouts of the reference tests, and structural invariants."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import tile_map as otm

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "tile_lists.json")


def _layouts():
    rng = np.random.default_rng(1)
    out = {}
    ids = torch.zeros((1, 128), dtype=torch.long)
    ids[:, 32:64] = 1; ids[:, 64:96] = 2; ids[:, 96:] = 3
    out["four_docs_one_block"] = ids                                   # tests/test_packed_sft.py:112-115
    ids = torch.zeros((1, 256), dtype=torch.long); ids[:, 176:] = 1
    out["boundary_176"] = ids                                          # tests/test_packed_sft.py:170-176
    ids = torch.zeros((2, 512), dtype=torch.long)
    ids[0, 130:300] = 1; ids[0, 300:] = 2; ids[1, 256:] = 1
    out["two_rows_512"] = ids
    out["ragged_200"] = torch.from_numpy(np.sort(rng.integers(0, 3, size=(1, 200)), axis=1))
    ids = torch.zeros((1, 384), dtype=torch.long); ids[:, 128:256] = 1; ids[:, 256:300] = 2; ids[:, 300:] = -1
    out["aligned_docs_padding"] = ids
    out["non_contiguous_ids"] = torch.from_numpy(rng.integers(0, 2, size=(1, 300)))
    return out


CASES = [(True, None), (True, 50), (True, 128), (True, 0)]


@pytest.mark.parametrize("name", list(_layouts().keys()))
def test_numpy_and_c_match_torch_block_mask(name):
    ids = _layouts()[name]
    B, S = ids.shape
    for causal, window in CASES:
        want = otm.block_mask_to_dict(otm.torch_block_mask(ids, B, S, causal, window))
        got = otm.tile_lists(ids, B, S, causal, window)
        gotc = otm.tile_lists_c(ids, B, S, causal, window)
        for k in otm.NAMES:
            assert want[k].dtype == torch.int32
            assert torch.equal(got[k], want[k]), (name, causal, window, k)
            assert torch.equal(gotc[k], want[k]), (name, causal, window, k)


def test_no_document_ids_and_noncausal():
    for S in (128, 200, 384):
        for causal, window in [(True, None), (True, 100), (False, None)]:
            want = otm.block_mask_to_dict(otm.torch_block_mask(None, 1, S, causal, window))
            got = otm.tile_lists(None, 1, S, causal, window)
            gotc = otm.tile_lists_c(None, 1, S, causal, window)
            for k in otm.NAMES:
                assert torch.equal(got[k], want[k]) and torch.equal(gotc[k], want[k])
    ids = torch.zeros((1, 256), dtype=torch.long); ids[:, 100:] = 7
    want = otm.block_mask_to_dict(otm.torch_block_mask(ids, 1, 256, False, None))
    got = otm.tile_lists_c(ids, 1, 256, False, None)
    for k in otm.NAMES:
        assert torch.equal(got[k], want[k])


def test_known_layouts_closed_form():
    # one block, 4 docs of 32: a single partial tile, no full tile
    d = otm.tile_lists(_layouts()["four_docs_one_block"], 1, 128)
    assert d["kv_num_blocks"].tolist() == [[[1]]] and d["full_kv_num_blocks"].tolist() == [[[0]]]
    # boundary at 176 inside block 1: tile (1,0) partial (rows 128..175 see doc 0), diagonal partial
    d = otm.tile_lists(_layouts()["boundary_176"], 1, 256)
    assert d["kv_num_blocks"].tolist() == [[[1, 2]]]
    assert d["kv_indices"].tolist() == [[[[0, 1], [0, 1]]]]
    assert d["full_kv_num_blocks"].tolist() == [[[0, 0]]]
    # documents aligned to tiles: off-diagonal tiles inside one doc are full, never partial
    ids = torch.zeros((1, 512), dtype=torch.long); ids[:, 256:] = 1
    d = otm.tile_lists(ids, 1, 512)
    assert d["kv_num_blocks"].tolist() == [[[1, 1, 1, 1]]]
    assert d["full_kv_num_blocks"].tolist() == [[[0, 1, 0, 1]]]
    assert d["full_kv_indices"][0, 0, 1].tolist() == [0, 1, 2, 3]      # set ascending then unset ascending
    assert d["full_kv_indices"][0, 0, 3].tolist() == [2, 0, 1, 3]
    assert d["full_q_num_blocks"].tolist() == [[[1, 0, 1, 0]]]


def test_invariants_on_random_packings():
    rng = np.random.default_rng(5)
    for trial in range(4):
        S = int(rng.integers(300, 900))
        cuts = np.sort(rng.integers(1, S, size=5))
        ids = np.zeros((1, S), dtype=np.int64)
        for c in cuts:
            ids[0, c:] += 1
        window = [None, 64, 300, 129][trial]
        cls = otm.tile_classes_np(ids, 1, S, True, window)[0]
        T = cls.shape[0]
        assert np.all(np.triu(cls, 1) == 0)                 # nothing above the diagonal under causal
        assert np.all(np.diag(cls) == 1)                    # the diagonal tile is always partial
        d = otm.tile_lists(ids, 1, S, True, window)
        for i in range(T):
            n, f = int(d["kv_num_blocks"][0, 0, i]), int(d["full_kv_num_blocks"][0, 0, i])
            assert n + f <= i + 1
            p = set(d["kv_indices"][0, 0, i, :n].tolist()); fl = set(d["full_kv_indices"][0, 0, i, :f].tolist())
            assert not (p & fl)                              # lists are disjoint
            assert sorted(d["kv_indices"][0, 0, i].tolist()) == list(range(T))   # a permutation
        # q-side lists are the kv-side lists of the transposed tile matrix
        dq = otm.lists_from_classes(np.swapaxes(cls[None], -1, -2).copy())
        assert torch.equal(dq["kv_indices"], d["q_indices"]) and torch.equal(dq["kv_num_blocks"], d["q_num_blocks"])
        assert torch.equal(dq["full_kv_indices"], d["full_q_indices"])
        # the pair count of the dense mask equals the closed form used for the FLOP accounting
        assert otm.count_pairs(ids, 1, S, True, None) == sum(
            n * (n + 1) // 2 for n in np.diff(np.concatenate([[0], np.unique(cuts), [S]])))


def test_golden_fixture():
    """tests/golden/tile_lists.json was written by tests/golden/make_tile_lists.py from torch's
    create_block_mask; both restatements must reproduce it."""
    with open(GOLDEN) as f:
        gold = json.load(f)
    assert len(gold["cases"]) >= 6
    for case in gold["cases"]:
        ids = None if case["document_ids"] is None else torch.tensor(case["document_ids"], dtype=torch.long)
        B, S = case["B"], case["S"]
        for fn in (otm.tile_lists, otm.tile_lists_c):
            got = fn(ids, B, S, case["causal"], case["window"])
            for k in otm.NAMES:
                assert got[k].tolist() == case["expect"][k], (case["name"], k)
