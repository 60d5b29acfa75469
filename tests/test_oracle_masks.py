"""Pins oracle.masks against the truth tables the reference's own tests hold."""
import numpy as np
import torch

from oracle import masks


def test_document_mask_prevents_cross_attention():
    # maester tests/test_packed_sft.py:72-92
    ids = torch.tensor([[0, 0, 0, 1, 1, 2, 2, 2]])
    ok = lambda q, kv: masks.allowed(ids, 0, q, kv)
    assert ok(2, 1) and ok(4, 3) and ok(7, 6)
    assert not ok(3, 2) and not ok(5, 4) and not ok(5, 2)
    assert not ok(1, 2) and not ok(6, 7)


def test_mask_without_documents():
    # tests/test_packed_sft.py:94-102: None ids -> pure causal
    ok = lambda q, kv: masks.allowed(None, 0, q, kv)
    assert ok(5, 3) and not ok(3, 5) and ok(4, 4)


def test_attention_masking_with_documents():
    # tests/test_packed_sft.py:410-430
    ids = torch.tensor([[0, 0, 0, 1, 1, 1]])
    ok = lambda q, kv: masks.allowed(ids, 0, q, kv)
    assert ok(1, 0) and ok(2, 1) and ok(4, 3)
    assert not ok(3, 2) and not ok(4, 1)
    assert not ok(0, 1) and not ok(3, 4)


def test_sliding_window_with_document_boundaries():
    # tests/test_packed_attention.py:279-336 (W=50 inclusive, docs 0-99 / 100-199)
    ids = torch.zeros((1, 200), dtype=torch.long)
    ids[0, 100:] = 1
    ok = lambda q, kv: masks.allowed(ids, 0, q, kv, True, 50)
    assert ok(50, 40) and ok(150, 140)
    assert not ok(90, 20)
    assert not ok(100, 99) and not ok(105, 98) and not ok(120, 95)
    assert ok(99, 99) and ok(100, 100)
    assert not ok(40, 50)
    # the window is inclusive: distance exactly W is visible, W+1 is not (model.py:207)
    assert ok(60, 10) and not ok(61, 10)


def test_padding_id_is_an_ordinary_document():
    ids = torch.tensor([[0, 0, -1, -1, -1]])
    assert masks.allowed(ids, 0, 3, 2) and masks.allowed(ids, 0, 4, 2)
    assert not masks.allowed(ids, 0, 2, 1)


def test_dense_forms_agree_with_scalar_predicate():
    rng = np.random.default_rng(0)
    ids = torch.from_numpy(np.sort(rng.integers(0, 4, size=(2, 37)), axis=1))
    for causal, window in [(True, None), (True, 5), (False, None), (True, 0)]:
        dn = masks.dense_mask_np(ids.numpy(), 2, 37, causal, window)
        dt = masks.dense_mask(ids, 2, 37, causal, window)[:, 0].numpy()
        mod = masks.make_mask_mod(ids, causal, window)
        for b in range(2):
            for q in range(37):
                for kv in range(37):
                    want = masks.allowed(ids, b, q, kv, causal, window)
                    assert dn[b, q, kv] == want and dt[b, q, kv] == want
                    assert bool(mod(torch.tensor(b), torch.tensor(0), torch.tensor(q), torch.tensor(kv))) == want


def test_dense_mask_matches_reference_known_layout():
    # tests/test_packed_sft.py:110-131: 4 documents of 32 tokens, causal & same_doc
    S = 128
    ids = torch.zeros((1, S), dtype=torch.long)
    ids[:, 32:64] = 1
    ids[:, 64:96] = 2
    ids[:, 96:] = 3
    same = ids.unsqueeze(2) == ids.unsqueeze(1)
    pos = torch.arange(S)
    causal = pos.view(1, S, 1) >= pos.view(1, 1, S)
    assert torch.equal(masks.dense_mask(ids, 1, S)[:, 0], causal & same)
