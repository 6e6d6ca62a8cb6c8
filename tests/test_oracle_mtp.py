"""Oracle MTP path against the reference's known answers and library routines."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import mtp as OM
from oracle.eagle3 import DraftShape


def _shape(**kw):
    base = dict(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                intermediate_size=64, vocab_size=61, draft_vocab_size=61, rms_norm_eps=1e-6,
                rope_theta=10000.0, qk_norm=True)
    base.update(kw)
    return DraftShape(**base)


def test_step_weights_closed_form():
    # models/mtp/core.py:29-38: beta^k / sum_j beta^j
    w = OM.compute_step_weights(0.6, 3)
    assert w == pytest.approx([1 / 1.96, 0.6 / 1.96, 0.36 / 1.96])
    assert sum(OM.compute_step_weights(0.3, 5)) == pytest.approx(1.0)
    assert OM.compute_step_weights(1.0, 4) == pytest.approx([0.25] * 4)


def test_packed_mask_is_document_local_literal():
    # tests/unit/models/test_mtp_attention.py:17-55, documents of 1, 3 and 2 tokens
    pos = torch.tensor([[0, 0, 1, 2, 0, 1]])
    want = torch.tensor([
        [1, 0, 0, 0, 0, 0],
        [0, 1, 0, 0, 0, 0],
        [0, 1, 1, 0, 0, 0],
        [0, 1, 1, 1, 0, 0],
        [0, 0, 0, 0, 1, 0],
        [0, 0, 0, 0, 1, 1]], dtype=torch.bool)
    assert torch.equal(OM.packed_causal_mask(pos)[0], want)
    assert OM.packed_sequence_ids(pos).tolist() == [[1, 2, 2, 2, 3, 3]] or \
        OM.packed_sequence_ids(pos).tolist() == [[0, 1, 1, 1, 2, 2]]


def test_packed_ids_match_transformers_routine():
    from transformers.masking_utils import find_packed_sequence_indices

    g = torch.Generator().manual_seed(0)
    for _ in range(5):
        lens = torch.randint(1, 9, (6,), generator=g).tolist()
        row = torch.cat([torch.arange(n) for n in lens])
        pos = torch.stack([row, row.flip(0)])
        got = OM.packed_sequence_ids(pos)
        want = find_packed_sequence_indices(pos)
        assert torch.equal(got, want)


def test_mask_matches_transformers_create_causal_mask():
    from transformers import Qwen3Config
    from transformers.masking_utils import create_causal_mask

    cfg = Qwen3Config(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                      intermediate_size=64, vocab_size=61, num_hidden_layers=1)
    cfg._attn_implementation = "sdpa"
    pos = torch.tensor([[0, 1, 2, 0, 1, 0, 1, 2, 3, 0]])
    m = create_causal_mask(config=cfg, inputs_embeds=torch.zeros(1, 10, 32), attention_mask=None,
                           past_key_values=None, position_ids=pos)
    allow = m[0, 0] if m.dtype == torch.bool else m[0, 0] == 0
    assert torch.equal(allow, OM.packed_causal_mask(pos)[0])


def test_padding_mask_matches_transformers_create_causal_mask():
    """With a 2-D padding mask the library drops the packed-sequence detection (position restarts
    no longer split the row) and masks the padded KEYS; fully masked query rows aside (the library
    un-masks them for the sdpa kernel), the restated mask is the library's."""
    from transformers import Qwen3Config
    from transformers.masking_utils import create_causal_mask

    cfg = Qwen3Config(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                      intermediate_size=64, vocab_size=61, num_hidden_layers=1)
    cfg._attn_implementation = "eager"
    pos = torch.tensor([[0, 1, 2, 0, 1, 0, 1, 2, 3, 0], [0, 1, 2, 3, 4, 5, 6, 7, 8, 9]])
    am = torch.tensor([[1, 1, 1, 1, 1, 1, 1, 0, 0, 0], [0, 0, 0, 1, 1, 1, 1, 1, 1, 1]])
    m = create_causal_mask(config=cfg, inputs_embeds=torch.zeros(2, 10, 32), attention_mask=am,
                           past_key_values=None, position_ids=pos)
    allow = m[:, 0] if m.dtype == torch.bool else m[:, 0] == 0
    want = OM.padded_causal_mask(am)
    has_key = want.any(-1)
    assert torch.equal(allow[has_key], want[has_key])
    # row 0: the position restarts at 3 and 5 do not split the row any more
    assert want[0, 6, 0] and not OM.packed_causal_mask(pos)[0, 6, 0]


def test_layer_matches_transformers_qwen3_modules():
    """The restated layer against the library's Qwen3DecoderLayer wired like
    models/mtp/model_definitions.py:95-116."""
    from transformers import Qwen3Config
    from transformers.models.qwen3.modeling_qwen3 import (Qwen3DecoderLayer, Qwen3RMSNorm,
                                                          Qwen3RotaryEmbedding)

    shape = _shape()
    w = OM.random_weights(shape, 3, std=0.1)
    cfg = Qwen3Config(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
                      intermediate_size=64, vocab_size=61, num_hidden_layers=1, rms_norm_eps=1e-6,
                      rope_theta=10000.0, attention_bias=False)
    cfg._attn_implementation = "eager"
    layer = Qwen3DecoderLayer(cfg, 0)
    p = "mtp_layers.0."
    sd = {k[len(p):]: v for k, v in w.items()
          if k.startswith(p) and k[len(p):] in dict(layer.named_parameters())}
    layer.load_state_dict(sd, strict=True)
    norms = {}
    for name in ("hidden_layernorm", "token_layernorm", "final_layernorm"):
        norms[name] = Qwen3RMSNorm(32, eps=1e-6)
        norms[name].weight.data.copy_(w[p + name + ".weight"])
    rot = Qwen3RotaryEmbedding(cfg)
    g = torch.Generator().manual_seed(4)
    n = 9
    hidden = torch.randn(1, n, 32, generator=g)
    embeds = torch.randn(1, n, 32, generator=g)
    pos = torch.tensor([[0, 1, 2, 3, 0, 1, 2, 0, 1]])
    mask = OM.packed_causal_mask(pos)
    add = torch.zeros(1, 1, n, n).masked_fill(~mask[:, None], float("-inf"))
    with torch.no_grad():
        proj = F.linear(torch.cat([norms["token_layernorm"](embeds), norms["hidden_layernorm"](hidden)], -1),
                        w[p + "input_proj.weight"])
        out = layer(hidden_states=proj, attention_mask=add, position_ids=pos,
                    position_embeddings=rot(proj, pos))
        out = out[0] if isinstance(out, tuple) else out
        want = norms["final_layernorm"](out)
        cos, sin = OM.rope_tables(pos[0], 8, 10000.0, torch.float32)
        got = OM.mtp_layer(hidden, embeds, w, shape, cos, sin, mask[0])
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-4), (got - want).abs().max()


def _inputs(shape, b, n, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randint(0, shape.vocab_size, (b, n), generator=g),
            torch.randn(b, n, shape.hidden_size, generator=g))


def test_forward_output_structure_and_short_sequences():
    # tests/unit/models/test_mtp_model.py:14-44,105-116
    shape = _shape()
    w = OM.random_weights(shape, 0)
    ids, hs = _inputs(shape, 1, 10, 1)
    logits, loss, m = OM.mtp_forward(w, shape, ids, hs)
    assert len(logits) == 3 and all(l.shape == (1, 6, 61) for l in logits)
    assert loss.dim() == 0 and torch.isfinite(loss) and loss >= 0
    assert set(m) == {"loss_step_0", "loss_step_1", "loss_step_2", "loss_sum", "loss_total"}
    assert all(math.isfinite(float(v)) for v in m.values())
    ids, hs = _inputs(shape, 1, 3, 2)
    logits, _, _ = OM.mtp_forward(w, shape, ids, hs)
    assert len(logits) == 1
    with pytest.raises(ValueError, match="expected exactly 3 weights"):
        OM.mtp_forward(w, shape, *_inputs(shape, 1, 10, 1), step_weights=[1.0])


def test_loss_masking_and_step_weights():
    # tests/unit/models/test_mtp_model.py:47-102
    shape = _shape()
    w = OM.random_weights(shape, 0)
    ids, hs = _inputs(shape, 1, 10, 3)
    _, l0, _ = OM.mtp_forward(w, shape, ids, hs, loss_mask=torch.zeros(1, 10))
    assert l0 == 0.0
    _, lfull, _ = OM.mtp_forward(w, shape, ids, hs)
    mask = torch.ones(1, 10)
    mask[:, -3:] = 0
    _, lpart, _ = OM.mtp_forward(w, shape, ids, hs, loss_mask=mask)
    assert lfull != lpart
    _, _, m = OM.mtp_forward(w, shape, ids, hs, step_weights=[1.0, 0.0, 0.0])
    assert m["loss_step_0"] > 0 and m["loss_step_1"] == 0.0 and m["loss_step_2"] == 0.0


def test_step_loss_is_mean_cross_entropy_of_shifted_targets():
    """Step k predicts input_ids[t + k + 2] from position t (models/mtp/core.py:198-218)."""
    shape = _shape()
    w = OM.random_weights(shape, 5)
    ids, hs = _inputs(shape, 2, 12, 6)
    logits, loss, m = OM.mtp_forward(w, shape, ids, hs, step_weights=[0.5, 0.3, 0.2])
    total = 0.0
    for k, wk in enumerate([0.5, 0.3, 0.2]):
        lp = torch.log_softmax(logits[k].double(), -1)
        tgt = ids[:, k + 2:k + 2 + 8]
        nll = -lp.gather(-1, tgt.unsqueeze(-1)).squeeze(-1)
        assert float(m[f"loss_step_{k}"]) == pytest.approx(wk * nll.mean().item(), rel=1e-5)
        total += wk * nll.mean().item()
    assert loss.item() == pytest.approx(total, rel=1e-5)


def test_dense_and_sdpa_attention_agree_and_rows_are_independent():
    shape = _shape()
    w = OM.random_weights(shape, 7)
    ids, hs = _inputs(shape, 2, 14, 8)
    pos = torch.tensor([[0, 1, 2, 3, 0, 1, 2, 3, 4, 5, 0, 1, 2, 3],
                        list(range(14))])
    a = OM.mtp_forward(w, shape, ids, hs, position_ids=pos, attn="dense")
    b = OM.mtp_forward(w, shape, ids, hs, position_ids=pos, attn="sdpa")
    assert torch.allclose(a[1], b[1], rtol=1e-5)
    for x, y in zip(a[0], b[0]):
        assert torch.allclose(x, y, atol=1e-5)
    # a batch row alone gives the same logits as inside the batch
    solo = OM.mtp_forward(w, shape, ids[1:], hs[1:], position_ids=pos[1:])
    assert torch.allclose(solo[0][2], a[0][2][1:], atol=1e-5)
