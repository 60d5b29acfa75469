"""Device-side position_ids / document_ids from document boundaries, bit-exact against the oracle's
restatement of PackedSFTDataset._generate_position_ids / _generate_document_ids
(maester/sft/packed_dataset.py:138-185)."""
import numpy as np
import pytest
import torch

from maester_amd import boundaries_to_tensors, build_tile_map, device_packed_ids, packed_collate_ids
from oracle import packed_ids as OP

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


def _oracle(rows, S):
    return (torch.stack([OP.position_ids(r, S) for r in rows]), torch.stack([OP.document_ids(r, S) for r in rows]))


def _check(rows, S, gpu):
    pos, doc = device_packed_ids(*boundaries_to_tensors(rows, gpu), S)
    wpos, wdoc = _oracle(rows, S)
    assert pos.dtype == doc.dtype == torch.int64
    assert torch.equal(pos.cpu(), wpos) and torch.equal(doc.cpu(), wdoc)
    return pos, doc


def test_reference_expectations(gpu):
    # the cases of the reference's own tests (tests/test_packed_sft.py:22-66): three conversations and a padded tail
    rows = [[(0, 0, 10), (1, 10, 15), (2, 25, 5)]]
    pos, doc = _check(rows, 40, gpu)
    assert pos[0, :10].tolist() == list(range(10)) and pos[0, 10:25].tolist() == list(range(15))
    assert doc[0, 30:].tolist() == [-1] * 10 and pos[0, 30:].tolist() == [0] * 10


def test_edge_cases(gpu):
    S = 300
    rows = [
        [],                                              # nothing but padding
        [(0, 0, 300)],                                   # one document, whole row
        [(0, 0, 500)],                                   # truncated at the end of the row
        [(0, 250, 100), (1, 0, 10)],                     # out of order, truncated
        [(0, 0, 100), (1, 50, 100), (2, 75, 10)],        # overlapping: the later boundary wins
        [(0, 10, 0), (1, 20, 5), (2, 400, 5)],           # empty, and one that starts past the end
        [(i, 3 * i, 3) for i in range(100)],             # many short documents
    ]
    _check(rows, S, gpu)


def test_more_boundaries_than_one_chunk(gpu):
    S = 4096
    rows = [[(i, 2 * i, 2) for i in range(2000)], [(i, 4 * i, 3) for i in range(1024)], [(0, 5, 4000)]]
    _check(rows, S, gpu)


def test_random_rows_and_the_tile_map_built_from_them(gpu):
    rng = np.random.default_rng(3)
    S = 2048
    rows = []
    for _ in range(4):
        row, t = [], 0
        while t < S - 64:
            n = int(rng.integers(1, 400))
            row.append((len(row), t, n))
            t += n
        rows.append(row)
    pos, doc = _check(rows, S, gpu)
    hpos, hdoc = packed_collate_ids(rows, S)             # the host-side generator agrees too
    assert torch.equal(pos.cpu(), hpos) and torch.equal(doc.cpu(), hdoc)
    a = build_tile_map(doc, 4, S)
    b = build_tile_map(hdoc.to(gpu), 4, S)
    assert all(torch.equal(x, y) for x, y in zip(a.as_dict().values(), b.as_dict().values()))
