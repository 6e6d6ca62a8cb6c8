"""Oracle DFlash helpers against the reference's known answers."""

import torch

from oracle import dflash as D
from oracle.eagle3 import DraftShape


def test_base_indices_known_answers():
    # tests/unit/models/test_dflash_utils.py:12-48
    f = D.base_indices_for_anchored_blocks
    assert f(torch.tensor([[3]]), 4).tolist() == [3, 4, 5, 6]
    assert f(torch.tensor([[0, 5, 10]]), 3).tolist() == [0, 1, 2, 5, 6, 7, 10, 11, 12]
    assert f(torch.tensor([[2, 7, 9]]), 1).tolist() == [2, 7, 9]
    assert f(torch.tensor([1, 4]), 2).tolist() == [1, 2, 4, 5]
    assert f(torch.tensor([[2.0, 5.0]]), 2).dtype == torch.long


def test_select_anchors_sorted_valid_and_bounded():
    # tests/unit/models/test_dflash_utils.py:51-59 and the rules of dflash/utils.py:21-67
    g = torch.Generator().manual_seed(0)
    mask = torch.ones(1, 64)
    a, v = D.select_anchors(mask, 8, 4, g)
    sel = a[v]
    assert torch.equal(sel, sel.sort().values) and sel.numel() == 8 and sel.max() < 60
    mask = torch.zeros(1, 64); mask[0, [3, 9, 62]] = 1
    a, v = D.select_anchors(mask, 8, 4, g)
    assert v.tolist() == [True, True] + [False] * 6 and a[:2].tolist() == [3, 9] and a[2:].sum() == 0


def test_targets_are_rolled_full_logits():
    # tests/unit/models/test_dflash_targets.py:37-63: targets == roll(full, 1)[:, idx]
    shape = DraftShape(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                       intermediate_size=64, vocab_size=50, draft_vocab_size=20, num_aux=2)
    w = D.random_weights(shape, 0)
    g = torch.Generator().manual_seed(1)
    vl = torch.randn(1, 24, 32, generator=g)
    idx = D.base_indices_for_anchored_blocks(torch.tensor([0, 5, 17]), 4)
    full = D.dflash_targets(w, shape, vl, torch.arange(24), sample_from_anchor=True)
    got = D.dflash_targets(w, shape, vl, idx)
    assert torch.allclose(got, torch.roll(full, 1, dims=1)[:, idx], atol=1e-6)


def test_forward_runs():
    shape = DraftShape(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                       intermediate_size=64, vocab_size=50, draft_vocab_size=20, num_aux=2,
                       num_hidden_layers=2, sliding_window=6, sliding_layers=(1,), qk_norm=True)
    w = D.random_weights(shape, 0)
    g = torch.Generator().manual_seed(2)
    t = 40
    hs = torch.randn(1, t, 64, generator=g)
    ids = torch.randint(0, 50, (1, t), generator=g)
    vl = torch.randn(1, t, 32, generator=g)
    mask = (torch.rand(1, t, generator=g) < 0.8).float()
    doc = torch.tensor([[0] * 22 + [1] * 14 + [-1] * 4])
    mask[0, 36:] = 0
    _, loss, m = D.dflash_forward(w, shape, hs, ids, mask, vl, doc, block_size=4, mask_token_id=7,
                                  max_anchors=6, generator=g)
    assert torch.isfinite(loss) and "eal_sum" in m and "position_3_acc_total" in m
