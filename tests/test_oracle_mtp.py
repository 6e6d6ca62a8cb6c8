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



def _hybrid_shape(**kw):
    base = dict(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                intermediate_size=48, vocab_size=61, draft_vocab_size=61, rms_norm_eps=1e-6,
                rope_theta=10000.0)
    base.update(kw)
    return OM.HybridShape(**base)


def _library_hybrid(model_type, shape, w):
    """(decoder layer, norm class, rotary module) of the library for one hybrid flavour, the
    layer at the last full-attention index as models/mtp/model_definitions.py:52-68 picks it,
    loaded with the oracle's weights."""
    common = dict(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                  intermediate_size=48, vocab_size=61, num_hidden_layers=4, rms_norm_eps=1e-6,
                  attention_bias=False, layer_types=["linear_attention", "full_attention"] * 2,
                  rope_parameters={"rope_type": "default", "rope_theta": 10000.0,
                                   "partial_rotary_factor": shape.partial_rotary_factor})
    moe = dict(num_experts=shape.num_experts, num_experts_per_tok=shape.num_experts_per_tok,
               moe_intermediate_size=shape.moe_intermediate_size,
               shared_expert_intermediate_size=shape.shared_expert_intermediate_size)
    if model_type == "qwen3_next":
        from transformers import Qwen3NextConfig
        from transformers.models.qwen3_next import modeling_qwen3_next as M
        cfg = Qwen3NextConfig(**common, **moe, norm_topk_prob=shape.norm_topk_prob,
                              decoder_sparse_step=1, mlp_only_layers=[])
        classes = (M.Qwen3NextDecoderLayer, M.Qwen3NextRMSNorm, M.Qwen3NextRotaryEmbedding)
    elif model_type == "qwen3_5_text":
        from transformers.models.qwen3_5 import modeling_qwen3_5 as M
        from transformers.models.qwen3_5.configuration_qwen3_5 import Qwen3_5TextConfig
        cfg = Qwen3_5TextConfig(**common)
        classes = (M.Qwen3_5DecoderLayer, M.Qwen3_5RMSNorm, M.Qwen3_5TextRotaryEmbedding)
    else:
        from transformers.models.qwen3_5_moe import modeling_qwen3_5_moe as M
        from transformers.models.qwen3_5_moe.configuration_qwen3_5_moe import Qwen3_5MoeTextConfig
        cfg = Qwen3_5MoeTextConfig(**common, **moe)
        classes = (M.Qwen3_5MoeDecoderLayer, M.Qwen3_5MoeRMSNorm, M.Qwen3_5MoeTextRotaryEmbedding)
    cfg._attn_implementation = "eager"
    layer = classes[0](cfg, 3)
    p = "mtp_layers.0."
    own = dict(layer.named_parameters())
    sd = {k[len(p):]: v for k, v in w.items() if k.startswith(p) and k[len(p):] in own}
    assert set(sd) == set(own), set(own) ^ set(sd)
    layer.load_state_dict(sd, strict=True)
    return layer, classes[1], classes[2](cfg)


@pytest.mark.parametrize("model_type,kw", [
    ("qwen3_next", dict(num_experts=6, num_experts_per_tok=2, moe_intermediate_size=24,
                        shared_expert_intermediate_size=40, norm_topk_prob=True)),
    ("qwen3_next", dict(num_experts=5, num_experts_per_tok=3, moe_intermediate_size=16,
                        shared_expert_intermediate_size=16, norm_topk_prob=False,
                        partial_rotary_factor=0.5)),
    ("qwen3_5_text", dict()),
    ("qwen3_5_moe_text", dict(num_experts=6, num_experts_per_tok=2, moe_intermediate_size=24,
                              shared_expert_intermediate_size=40)),
])
def test_hybrid_layer_matches_transformers_modules(model_type, kw):
    """The restated hybrid layer (gain 1 + w norms, gated attention, partial rotary embedding,
    sparse MoE with a shared expert) against the library's decoder layer of each flavour wired
    like models/mtp/model_definitions.py:95-116, output and gradients."""
    shape = _hybrid_shape(model_type=model_type, **kw)
    w = {k: v.requires_grad_(True) for k, v in OM.random_weights(shape, 5, std=0.1).items()}
    layer, norm_class, rot = _library_hybrid(model_type, shape, w)
    p = "mtp_layers.0."
    norms = {}
    for name in ("hidden_layernorm", "token_layernorm", "final_layernorm"):
        norms[name] = norm_class(32, eps=1e-6)
        norms[name].weight.data.copy_(w[p + name + ".weight"])
    g = torch.Generator().manual_seed(6)
    n = 11
    hidden = torch.randn(1, n, 32, generator=g)
    embeds = torch.randn(1, n, 32, generator=g)
    pos = torch.tensor([[0, 1, 2, 3, 0, 1, 2, 0, 1, 2, 3]])
    mask = OM.packed_causal_mask(pos)
    add = torch.zeros(1, 1, n, n).masked_fill(~mask[:, None], float("-inf"))
    proj = F.linear(torch.cat([norms["token_layernorm"](embeds), norms["hidden_layernorm"](hidden)], -1),
                    w[p + "input_proj.weight"].detach())
    out = layer(hidden_states=proj, attention_mask=add, position_ids=pos,
                position_embeddings=rot(proj, pos))
    out = out[0] if isinstance(out, tuple) else out
    want = norms["final_layernorm"](out)
    cos, sin = OM.rope_tables(pos[0], OM.rotary_dim(shape), 10000.0, torch.float32)
    assert cos.shape[-1] == int(16 * shape.partial_rotary_factor)
    got = OM.mtp_layer(hidden, embeds, w, shape, cos, sin, mask[0])
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-4), (got - want).abs().max()
    probe = torch.randn(want.shape, generator=g)
    (want * probe).sum().backward()
    (got * probe).sum().backward()
    own = dict(layer.named_parameters())
    for name, param in own.items():
        assert torch.allclose(w[p + name].grad, param.grad, atol=2e-5, rtol=1e-3), name
    assert torch.allclose(w[p + "final_layernorm.weight"].grad, norms["final_layernorm"].weight.grad,
                          atol=2e-5, rtol=1e-3)


def test_hybrid_routing_and_norm_against_closed_forms():
    """What the mathematics fixes: zero weights make the norm a plain normalisation; routing scores
    are the k largest soft-max probabilities, in descending order, summing to 1 when renormalised;
    one expert with top-1 routing and a zero shared gate weight reduces the block to that expert's
    SwiGLU MLP plus half the shared expert's."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 7, 32, generator=g)
    y = OM.zero_centered_rms_norm(x, torch.zeros(32), 1e-6)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(1, 7), atol=1e-4)
    wr = torch.randn(6, 32, generator=g)
    scores, idx = OM.moe_routing(x[0], wr, 3, True)
    probs = F.softmax(x[0] @ wr.t(), dim=-1)
    assert torch.equal(idx, probs.argsort(dim=-1, descending=True)[:, :3])
    assert torch.allclose(scores.sum(-1), torch.ones(7), atol=1e-6)
    raw, _ = OM.moe_routing(x[0], wr, 3, False)
    assert torch.allclose(raw, probs.gather(1, idx), atol=1e-7)
    shape = _hybrid_shape(num_experts=1, num_experts_per_tok=1, moe_intermediate_size=24,
                          shared_expert_intermediate_size=40)
    w = OM.random_weights(shape, 2, std=0.1)
    p = "mtp_layers.0.mlp."
    w[p + "shared_expert_gate.weight"].zero_()
    got = OM.sparse_moe(x, w, p, shape)
    gu, dn = w[p + "experts.gate_up_proj"][0], w[p + "experts.down_proj"][0]
    a, b = F.linear(x, gu).chunk(2, dim=-1)
    want = F.linear(F.silu(a) * b, dn) + 0.5 * OM.swiglu_mlp(x, w, p + "shared_expert.")
    assert torch.allclose(got, want, atol=1e-5)


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
