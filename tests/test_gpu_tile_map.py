"""HIP tile map vs the oracle: bit-exact on all eight BlockMask tensors, tails included."""
import json
import os

import numpy as np
import pytest
import torch

from maester_amd import build_tile_map, workloads
from oracle import tile_map as otm

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "tile_lists.json")


def _assert_equal(tm, want, tag):
    got = tm.as_dict()
    for k in otm.NAMES:
        assert got[k].dtype == torch.int32 and got[k].is_contiguous()
        assert got[k].shape == want[k].shape, (tag, k, got[k].shape, want[k].shape)
        assert torch.equal(got[k].cpu(), want[k]), (tag, k)


def test_golden_fixture_through_c_abi(gpu):
    with open(GOLDEN) as f:
        gold = json.load(f)
    for case in gold["cases"]:
        ids = None if case["document_ids"] is None else torch.tensor(case["document_ids"], dtype=torch.long, device=gpu)
        tm = build_tile_map(ids, case["B"], case["S"], case["causal"], case["window"], device=gpu)
        want = {k: torch.tensor(v, dtype=torch.int32) for k, v in case["expect"].items()}
        _assert_equal(tm, want, case["name"])


def test_against_torch_create_block_mask_small(gpu):
    rng = np.random.default_rng(11)
    for S in (128, 200, 256, 384, 512, 1000):
        ids = torch.from_numpy(np.sort(rng.integers(0, 4, size=(2, S)), axis=1))
        for causal, window in [(True, None), (True, 100), (True, 0), (False, None)]:
            want = otm.block_mask_to_dict(otm.torch_block_mask(ids, 2, S, causal, window))
            tm = build_tile_map(ids.to(gpu), 2, S, causal, window)
            _assert_equal(tm, want, (S, causal, window))
    # arbitrary (non-contiguous) ids and the no-ids masks
    ids = torch.from_numpy(rng.integers(0, 3, size=(1, 700)))
    _assert_equal(build_tile_map(ids.to(gpu), 1, 700), otm.tile_lists(ids, 1, 700), "random ids")
    for window in (None, 300):
        _assert_equal(build_tile_map(None, 3, 900, True, window, device=gpu), otm.tile_lists(None, 3, 900, True, window),
                      ("no ids", window))


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c4s", "c5"])
def test_full_size_configs(gpu, name):
    sp = workloads.spec(name)
    rows = workloads.document_lengths(sp)
    _, doc = workloads.ids_from_lengths(rows, sp.S)
    want = otm.tile_lists_c(doc, sp.B, sp.S, True, sp.window)
    tm = build_tile_map(doc.to(gpu), sp.B, sp.S, True, sp.window)
    _assert_equal(tm, want, name)
    # the survey's tile census for these seeded layouts
    census = {"c1": (35, 4), "c2": (684, 1014), "c3": (632, 752), "c4": (420, 8296), "c4s": (593, 2639),
              "c5": (602, 2437)}      # c4: row 0 one document (forced); c4s: the seeded per-row draw of the same configuration
    assert (int(tm.kv_num_blocks.sum()), int(tm.full_kv_num_blocks.sum())) == census[name]
    assert int(tm.q_num_blocks.sum()) == census[name][0] and int(tm.full_q_num_blocks.sum()) == census[name][1]


def test_padding_tail_and_large_T(gpu):
    sp = workloads.spec("c2")
    rows = workloads.document_lengths(sp)
    _, doc = workloads.ids_from_lengths(rows, sp.S, pad_tail=777)
    assert (doc[:, -777:] == -1).all()
    _assert_equal(build_tile_map(doc.to(gpu), sp.B, sp.S, True, 1024), otm.tile_lists_c(doc, sp.B, sp.S, True, 1024), "pad")
    # more than 64 tiles per row exercises the multi-pass ordered-list kernel
    S = 128 * 150 + 17
    ids = torch.zeros((1, S), dtype=torch.long)
    ids[:, 5000:12000] = 1; ids[:, 12000:] = 2
    _assert_equal(build_tile_map(ids.to(gpu), 1, S, True, 4096), otm.tile_lists_c(ids, 1, S, True, 4096), "T=151")


def _expected_order(num_a, num_b):
    """The launch-schedule rule restated: rows by descending work (tiles in the row's lists, partial
    + full), ties by ascending index."""
    work = (num_a + num_b).reshape(-1)
    return np.array(sorted(range(work.size), key=lambda e: (-work[e], e)), dtype=np.int32)


@pytest.mark.parametrize("name,S", [("c2", 8192), ("c3", 8192), ("c1", 2048), ("c2", 1000)])
def test_launch_schedule_orders(gpu, name, S):
    wl = workloads.make(name, S=S)
    sp = wl.spec
    tm = build_tile_map(wl.document_ids.to(gpu), sp.B, sp.S, True, sp.window)
    T = (sp.S + 127) // 128
    d = {k: v.cpu().numpy() for k, v in tm.as_dict().items()}
    q_order, kv_order = tm.q_tile_order.cpu().numpy(), tm.kv_tile_order.cpu().numpy()
    assert sorted(q_order.tolist()) == list(range(sp.B * T)) and sorted(kv_order.tolist()) == list(range(sp.B * T))
    assert np.array_equal(q_order, _expected_order(d["kv_num_blocks"], d["full_kv_num_blocks"]))
    assert np.array_equal(kv_order, _expected_order(d["q_num_blocks"], d["full_q_num_blocks"]))


@pytest.mark.parametrize("name,S", [("c2", 8192), ("c1", 2048), ("c2", 1000), ("c2", 970)])
def test_block_document_ranges(gpu, name, S):
    """(min, max) document id per 32-row block, two blocks per 64-row step, tail rows repeat the last id."""
    wl = workloads.make(name, S=S, pad_tail=17)
    sp = wl.spec
    tm = build_tile_map(wl.document_ids.to(gpu), sp.B, sp.S, True, sp.window)
    got = tm.block_doc_range.cpu().numpy()
    nblk = 2 * ((S + 63) // 64)
    assert got.shape == (sp.B, nblk, 2)
    ids = wl.document_ids.numpy()
    padded = np.concatenate([ids, np.repeat(ids[:, -1:], nblk * 32 - S, axis=1)], axis=1).reshape(sp.B, nblk, 32)
    assert np.array_equal(got[..., 0], padded.min(-1)) and np.array_equal(got[..., 1], padded.max(-1))
    assert build_tile_map(None, sp.B, sp.S, True, None, device=gpu).block_doc_range is None


@pytest.mark.parametrize("name,S,window", [("c2", 8192, None), ("c3", 8192, 1024), ("c4s", 16384, None), ("c2", 1000, 64)])
def test_compact_numbering_of_visited_tiles(gpu, name, S, window):
    """tile_slot numbers the visited (partial or full) tiles in (b, i, j) order, -1 elsewhere; tile_count is their
    number -- restated here from the oracle's tile classes."""
    wl = workloads.make(name, S=S)
    sp = wl.spec
    tm = build_tile_map(wl.document_ids.to(gpu), sp.B, sp.S, True, window)
    visited = (otm.tile_classes_np(wl.document_ids, sp.B, sp.S, True, window) != 0).reshape(-1)
    want = np.where(visited, np.cumsum(visited) - 1, -1).astype(np.int32)
    assert np.array_equal(tm.tile_slot.cpu().numpy().reshape(-1), want)
    assert tm.visited_tiles() == int(visited.sum()) == int(tm.kv_num_blocks.sum()) + int(tm.full_kv_num_blocks.sum())
