"""Pins id generation (oracle and the package's host code) to the exact expectations of
maester tests/test_packed_sft.py:22-66 and the collate expectations of :315-408."""
import torch

from oracle import packed_ids as O
from maester_amd import packed_ids as H

BOUNDS = [(100, 0, 10), (101, 10, 15), (102, 25, 8)]


def _check(mod_pos, mod_doc):
    pos = mod_pos(BOUNDS, 40)
    assert pos[0] == 0 and pos[10] == 0 and pos[25] == 0
    assert torch.equal(pos[0:10], torch.arange(10)) and torch.equal(pos[10:25], torch.arange(15))
    assert torch.equal(pos[25:33], torch.arange(8))
    assert torch.equal(pos[33:40], torch.zeros(7, dtype=torch.long))
    doc = mod_doc(BOUNDS, 40)
    assert torch.equal(doc[0:10], torch.zeros(10, dtype=torch.long))
    assert torch.equal(doc[10:25], torch.ones(15, dtype=torch.long))
    assert torch.equal(doc[25:33], torch.full((8,), 2, dtype=torch.long))
    assert torch.equal(doc[33:40], torch.full((7,), -1, dtype=torch.long))
    assert pos.dtype == torch.long and doc.dtype == torch.long


def test_oracle_ids():
    _check(O.position_ids, O.document_ids)


def test_host_ids_and_truncation():
    _check(H.generate_position_ids, H.generate_document_ids)
    # a boundary running past the row is clipped (packed_dataset.py:157,181)
    pos = H.generate_position_ids([(1, 0, 30), (2, 30, 50)], 40)
    doc = H.generate_document_ids([(1, 0, 30), (2, 30, 50)], 40)
    assert torch.equal(pos, O.position_ids([(1, 0, 30), (2, 30, 50)], 40))
    assert torch.equal(doc, O.document_ids([(1, 0, 30), (2, 30, 50)], 40))
    assert pos[39] == 9 and doc[39] == 1


def test_collate_expectations():
    # tests/test_packed_sft.py:315-408: two packed rows of 100 tokens
    rows = [[(1, 0, 30), (2, 30, 30), (3, 60, 25)], [(4, 0, 35), (5, 35, 25)]]
    pos, doc = H.packed_collate_ids(rows, 100)
    assert pos.shape == (2, 100) and doc.shape == (2, 100)
    assert pos[0, 0] == 0 and pos[0, 30] == 0 and pos[0, 60] == 0 and pos[1, 35] == 0
    assert (doc[0, :30] == 0).all() and (doc[0, 30:60] == 1).all() and (doc[0, 60:85] == 2).all()
    assert (doc[0, 85:] == -1).all()
    assert (doc[1, :35] == 0).all() and (doc[1, 35:60] == 1).all() and (doc[1, 60:] == -1).all()
