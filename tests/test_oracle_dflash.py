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


# ---------------------------------------------------------------- layer wiring pinned on HF blocks
#
# The layer of the oracle against the HF Qwen3 library blocks (Qwen3RMSNorm, Qwen3MLP,
# Qwen3RotaryEmbedding, nn.Linear, the library's eager attention) wired the way
# Qwen3DFlashAttention / Qwen3DFlashDecoderLayer wire them
# (models/dflash/model_definitions.py:97-155,170-207): q-norm then transpose, k and v of the
# context and of the mask tokens concatenated along the sequence, k-norm over the concatenation,
# rotary over all T + Q positions for k and over the LAST Q positions for q.


def _pin_shape(**kw):
    base = dict(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                intermediate_size=64, vocab_size=50, draft_vocab_size=20, num_aux=2,
                num_hidden_layers=2, sliding_window=6, sliding_layers=(1,), qk_norm=True,
                rms_norm_eps=1e-6, rope_theta=10000.0)
    base.update(kw)
    return DraftShape(**base)


def _nontrivial_gains(w, seed=3):
    g = torch.Generator().manual_seed(seed)
    for name in list(w):
        if name.endswith("norm.weight") or "layernorm" in name:
            w[name] = 1 + 0.2 * torch.randn(w[name].shape, generator=g)
    return w


from hf_blocks import HFDFlashLayer as _HFDFlashLayer  # noqa: E402
from hf_blocks import qwen3_cfg as _qwen3_cfg  # noqa: E402


def _packed_case(shape, t=40, seed=2):
    g = torch.Generator().manual_seed(seed)
    hs = torch.randn(1, t, shape.num_aux * shape.hidden_size, generator=g)
    ids = torch.randint(0, shape.vocab_size, (1, t), generator=g)
    vl = torch.randn(1, t, shape.hidden_size, generator=g)
    mask = (torch.rand(1, t, generator=g) < 0.8).float()
    doc = torch.tensor([[0] * 22 + [1] * 14 + [-1] * 4])
    pos = torch.cat([torch.arange(22), torch.arange(14), torch.zeros(4, dtype=torch.long)])[None]
    mask[0, 36:] = 0
    return hs, ids, vl, mask, doc, pos


def test_layer_equals_hf_qwen3_blocks_wired_like_the_reference():
    from transformers.models.qwen3.modeling_qwen3 import Qwen3RotaryEmbedding

    from oracle import masks as M
    from oracle.eagle3 import rope_tables

    shape = _pin_shape()
    w = _nontrivial_gains(D.random_weights(shape, 0, std=0.2))
    cfg = _qwen3_cfg(shape)
    rot = Qwen3RotaryEmbedding(cfg)
    hs, ids, vl, mask, doc, pos = _packed_case(shape)
    t, bs = 40, 4
    # two documents, anchors in both, one padded (invalid) anchor at position 0
    anchors = torch.tensor([3, 9, 17, 25, 30, 0])
    g = torch.Generator().manual_seed(11)
    noise = torch.randn(1, anchors.numel() * bs, shape.hidden_size, generator=g)
    ctx = torch.randn(1, t, shape.hidden_size, generator=g)
    block_pos = D.base_indices_for_anchored_blocks(pos[0, anchors], bs)
    all_pos = torch.cat([pos, block_pos[None]], 1)
    cos_hf, sin_hf = rot(ctx, all_pos)
    cos, sin = rope_tables(all_pos, shape.head_dim, shape.rope_theta, torch.float32, None)
    assert torch.allclose(cos, cos_hf, atol=1e-6) and torch.allclose(sin, sin_hf, atol=1e-6)
    with torch.no_grad():
        x_or, x_hf = noise, noise
        for li in range(2):
            win = shape.sliding_window if li in shape.sliding_layers else None
            for non_causal in ((False, True) if win else (False,)):
                m = M.dflash_mask_dense(doc.reshape(-1), t, anchors, bs, win, non_causal)
                got = D._dflash_layer(x_or, ctx, w, li, shape, cos, sin, m)
                ref = _HFDFlashLayer(cfg, w, li)(x_hf, ctx, cos_hf, sin_hf, m)
                assert torch.allclose(got, ref, atol=2e-5), (li, non_causal, (got - ref).abs().max())
            x_or, x_hf = got, ref
        # sensitivity: the comparison notices rotary tables shifted along the sequence (a q
        # rotated by other than the last Q positions)
        bad = D._dflash_layer(noise, ctx, w, 0, shape, torch.roll(cos, 7, 1), torch.roll(sin, 7, 1), m)
        assert (bad - _HFDFlashLayer(cfg, w, 0)(noise, ctx, cos_hf, sin_hf, m)).abs().max() > 1e-3


def test_layer_without_context_is_the_hf_qwen3_decoder_layer():
    """When no context key is visible (every anchor is the first position of its document) the
    DFlash layer is an ordinary Qwen3 decoder layer over the mask tokens alone under a
    block-diagonal mask: a library class nobody here wired."""
    from transformers.models.qwen3.modeling_qwen3 import Qwen3DecoderLayer, Qwen3RotaryEmbedding

    from oracle import masks as M
    from oracle.eagle3 import rope_tables

    shape = _pin_shape(num_hidden_layers=1, sliding_layers=())
    w = _nontrivial_gains(D.random_weights(shape, 5, std=0.2))
    cfg = _qwen3_cfg(shape)
    layer = Qwen3DecoderLayer(cfg, 0)
    sd = {k[len("layers.0."):]: v for k, v in w.items() if k.startswith("layers.0.")}
    layer.load_state_dict(sd, strict=True)
    t, bs = 24, 4
    doc = torch.tensor([0] * 6 + [1] * 6 + [2] * 6 + [3] * 6)
    pos = torch.arange(6).repeat(4)[None] + 2  # positions need not start at 0
    anchors = torch.tensor([0, 6, 12, 18])
    g = torch.Generator().manual_seed(4)
    noise = torch.randn(1, 16, shape.hidden_size, generator=g)
    ctx = torch.randn(1, t, shape.hidden_size, generator=g)
    block_pos = D.base_indices_for_anchored_blocks(pos[0, anchors], bs)[None]
    cos, sin = rope_tables(torch.cat([pos, block_pos], 1), shape.head_dim, shape.rope_theta,
                           torch.float32, None)
    m = M.dflash_mask_dense(doc, t, anchors, bs)
    assert not m[:, :t].any()
    blockdiag = torch.zeros(1, 1, 16, 16).masked_fill(~m[None, None, :, t:], float("-inf"))
    with torch.no_grad():
        got = D._dflash_layer(noise, ctx, w, 0, shape, cos, sin, m)
        ref = layer(noise, attention_mask=blockdiag,
                    position_embeddings=Qwen3RotaryEmbedding(cfg)(noise, block_pos))
    ref = ref[0] if isinstance(ref, tuple) else ref
    assert torch.allclose(got, ref, atol=2e-5), (got - ref).abs().max()


def test_forward_equals_hf_blocks_end_to_end_and_aligned_mask_literal():
    """dflash_forward == embedding, fc + hidden_norm, HF-block layers, norm, lm_head composed
    as in _backbone_forward (models/dflash/core.py:330-439), fed to the (separately pinned)
    metrics; the aligned loss mask against a literal worked from core.py:425-437."""
    import torch.nn.functional as F
    from transformers.models.qwen3.modeling_qwen3 import Qwen3RMSNorm, Qwen3RotaryEmbedding

    from oracle import masks as M
    from oracle import metrics as MT

    shape = _pin_shape()
    w = _nontrivial_gains(D.random_weights(shape, 7, std=0.2))
    cfg = _qwen3_cfg(shape)
    hs, ids, vl, mask, doc, pos = _packed_case(shape, seed=9)
    t, bs, mask_id = 40, 4, 7
    anchors = (torch.tensor([2, 10, 24, 31, 0, 0]), torch.tensor([1, 1, 1, 1, 0, 0]).bool())
    _, loss, metrics, logits = D.dflash_forward(
        w, shape, hs, ids, mask, vl, doc, pos, block_size=bs, mask_token_id=mask_id,
        anchors=anchors, return_logits=True)

    def norm(name, dim):
        n = Qwen3RMSNorm(dim, eps=shape.rms_norm_eps)
        n.weight.data.copy_(w[name])
        return n

    with torch.no_grad():
        a = anchors[0]
        tok = torch.full((1, a.numel() * bs), mask_id)
        tok[:, ::bs] = ids[:, a]
        x = F.embedding(tok, w["embed_tokens.weight"])
        ctx = norm("hidden_norm.weight", shape.hidden_size)(F.linear(hs, w["fc.weight"]))
        bpos = (pos[0, a][:, None] + torch.arange(bs)[None]).reshape(1, -1)
        cos, sin = Qwen3RotaryEmbedding(cfg)(hs, torch.cat([pos, bpos], 1))
        for li in range(2):
            win = shape.sliding_window if li in shape.sliding_layers else None
            m = M.dflash_mask_dense(doc.reshape(-1), t, a, bs, win, False)
            x = _HFDFlashLayer(cfg, w, li)(x, ctx, cos, sin, m)
        ref_logits = F.linear(norm("norm.weight", shape.hidden_size)(x), w["lm_head.weight"])
        assert torch.allclose(logits, ref_logits, atol=5e-5), (logits - ref_logits).abs().max()
        idx = (a[:, None] + torch.arange(bs)[None]).reshape(-1)
        tgt = F.linear(norm("verifier_norm.weight", shape.hidden_size)(vl[:, (idx - 1) % t]),
                       w["verifier_lm_head.weight"])
        aligned = torch.stack([mask[0, i] for i in idx.tolist()])[None].clone()
        aligned[0, 16:] = 0      # two padded anchors
        aligned[0, ::bs] = 0     # the anchor slot itself is not trained
        ref_loss, ref_m = MT.dflash_compute_metrics(ref_logits, tgt, aligned, bs)
    assert torch.allclose(loss, ref_loss, rtol=1e-5)
    for k_ in ref_m:
        assert torch.allclose(metrics[k_], ref_m[k_], rtol=1e-5), k_


def test_aligned_loss_mask_literal_two_anchors():
    # core.py:425-437 by hand: T = 10, block 3, anchors (2 valid, 6 valid, 0 padded);
    # loss_mask = 1 1 0 1 1 1 1 0 1 1 -> rows [2,3,4 | 6,7,8 | 0,1,2] -> 0 1 1 | 1 0 1 | 1 1 0,
    # padded block zeroed, slot 0 of every block zeroed -> 0 1 1 | 0 0 1 | 0 0 0.
    # Read back through the per-slot totals of the metrics (slots 1 and 2).
    shape = _pin_shape(num_hidden_layers=1, sliding_layers=())
    w = D.random_weights(shape, 1)
    g = torch.Generator().manual_seed(0)
    t = 10
    hs = torch.randn(1, t, 64, generator=g)
    ids = torch.randint(0, 50, (1, t), generator=g)
    vl = torch.randn(1, t, 32, generator=g)
    mask = torch.tensor([[1, 1, 0, 1, 1, 1, 1, 0, 1, 1.0]])
    doc = torch.zeros(1, t, dtype=torch.long)
    anchors = (torch.tensor([2, 6, 0]), torch.tensor([True, True, False]))
    _, _, m = D.dflash_forward(w, shape, hs, ids, mask, vl, doc, block_size=3, anchors=anchors)
    assert m["position_1_acc_total"].item() == 1 and m["position_2_acc_total"].item() == 2
    assert m["full_acc_total"].item() == 3
    # with sample_from_anchor the anchor slot is trained too: 0 1 1 | 1 0 1 | 0 0 0
    _, _, m = D.dflash_forward(w, shape, hs, ids, mask, vl, doc, block_size=3, anchors=anchors,
                               sample_from_anchor=True)
    assert [m[f"position_{s}_acc_total"].item() for s in range(3)] == [1, 1, 2]
