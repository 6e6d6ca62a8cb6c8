"""Oracle masks against the reference's golden vectors and brute force."""

import pytest
import torch

from oracle import masks as M


def _doc_ids(lengths, total=None):
    lengths = torch.tensor(lengths)
    ids = torch.repeat_interleave(torch.arange(len(lengths)), lengths)
    if total is not None and total > ids.numel():
        ids = torch.cat([ids, torch.full((total - ids.numel(),), -1)])
    return ids


def test_ttt_mask_literal_6x6():
    # expected matrix of tests/unit/models/test_eagle3_attention.py:24-31
    expected = torch.tensor([
        [1, 0, 0, 0, 0, 0],
        [0, 1, 0, 0, 0, 0],
        [0, 1, 1, 0, 0, 0],
        [0, 0, 0, 1, 0, 0],
        [0, 0, 0, 1, 1, 0],
        [0, 0, 0, 1, 1, 1],
    ], dtype=torch.bool)
    got = M.ttt_mask_dense(_doc_ids([1, 2, 3]), 6, 0)
    assert torch.equal(got, expected)


@pytest.mark.parametrize("lengths", [[1, 2, 3], [2, 2, 2], [5]])
def test_ttt_mask_diagonal_rule(lengths):
    # tests/unit/models/test_eagle3_attention.py:41-65: for kv in [N, 3N) only kv % N == q
    n = sum(lengths)
    got = M.ttt_mask_dense(_doc_ids(lengths), n, 2)
    for q in range(n):
        for kv in range(n, 3 * n):
            assert bool(got[q, kv]) == (kv % n == q)


def test_ttt_mask_extension_keeps_original_and_adds_identity():
    # tests/unit/models/test_eagle3_attention.py:122-152
    t = 8
    doc = torch.zeros(t, dtype=torch.long)
    base = M.ttt_mask_dense(doc, t, 0)
    assert torch.equal(base, torch.tril(torch.ones(t, t, dtype=torch.bool)))
    for step in range(1, 4):
        m = M.ttt_mask_dense(doc, t, step)
        assert m.shape == (t, t * (step + 1))
        assert torch.equal(m[:, :t], base)
        for j in range(1, step + 1):
            assert torch.equal(m[:, j * t:(j + 1) * t], torch.eye(t, dtype=torch.bool))


@pytest.mark.parametrize("window", [None, 1, 3, 5, 100])
@pytest.mark.parametrize("lengths,total", [([1, 2, 3], 6), ([4, 1, 5], 13), ([7], 7), ([3, 3], 9)])
def test_ttt_row_lo_is_the_interval_form_of_the_mask(lengths, total, window):
    doc = _doc_ids(lengths, total)
    mask = M.ttt_mask_dense(doc, total, 0, window)
    lo = M.ttt_row_lo(doc, window)
    for i in range(total):
        expect = torch.zeros(total, dtype=torch.bool)
        expect[int(lo[i]): i + 1] = True
        assert torch.equal(mask[i], expect), (i, lo[i])
    # no row is ever fully masked
    assert mask.any(dim=1).all()


def test_ttt_mask_padding_rows_see_only_their_diagonal():
    doc = _doc_ids([3, 2], 8)
    m = M.ttt_mask_dense(doc, 8, 2)
    for q in range(5, 8):
        assert m[q].nonzero().reshape(-1).tolist() == [q, 8 + q, 16 + q]


def _dflash_bruteforce(total, anchors, bs, doc, window=None, non_causal_flag=False):
    # pure-Python restatement of the loops in
    # tests/integration/models/test_dflash_vllm_parity.py:29-61, plus the window rule
    non_causal = window is None or non_causal_flag
    q_len = len(anchors) * bs
    out = torch.zeros(q_len, total + q_len, dtype=torch.bool)
    for q in range(q_len):
        a = int(anchors[q // bs])
        qd = int(doc[a])
        for kv in range(total + q_len):
            if kv < total:
                ok = qd == int(doc[kv]) and qd != -1 and kv < a
                if window is not None:
                    ok = ok and kv >= a - window
                out[q, kv] = ok
            else:
                same = (q // bs) == ((kv - total) // bs)
                out[q, kv] = same and (non_causal or kv <= q + total)
    return out


@pytest.mark.parametrize("window,ncf", [(None, False), (4, False), (4, True), (2, False)])
def test_dflash_mask_matches_bruteforce(window, ncf):
    total, bs = 16, 4
    doc = _doc_ids([10, 6])
    anchors = torch.tensor([3, 8, 12])
    got = M.dflash_mask_dense(doc, total, anchors, bs, window, ncf)
    assert torch.equal(got, _dflash_bruteforce(total, anchors, bs, doc, window, ncf))
    # every query sees its own block (tests/unit/models/test_dflash_attention.py:103-126)
    for q in range(got.shape[0]):
        assert got[q, total + q]


@pytest.mark.parametrize("window", [None, 3, 6])
def test_dflash_row_range_is_the_interval_form(window):
    total, bs = 24, 4
    doc = _doc_ids([10, 6, 4], total)
    anchors = torch.tensor([0, 3, 8, 12, 17, 21])  # 21 is padding
    mask = M.dflash_mask_dense(doc, total, anchors, bs, window)
    lo, hi = M.dflash_row_range(doc, anchors, bs, window)
    for r in range(mask.shape[0]):
        expect = torch.zeros(total, dtype=torch.bool)
        expect[int(lo[r]): int(hi[r])] = True
        assert torch.equal(mask[r, :total], expect), r
