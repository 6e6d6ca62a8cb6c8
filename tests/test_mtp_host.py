"""Host logic of the MTP path that needs no GPU: the configuration derived from the library's
configs, the router arithmetic and the expert sort."""

import pytest


def test_config_from_the_library_configs():
    """``MTPConfig.from_transformer_config`` picks what the reference's layer classes would build
    (models/mtp/model_definitions.py:52-68,159-205): the last full-attention index, sparse or
    dense by the library's rule."""
    from transformers import Qwen3Config, Qwen3NextConfig
    from transformers.models.qwen3_5.configuration_qwen3_5 import Qwen3_5TextConfig
    from transformers.models.qwen3_5_moe.configuration_qwen3_5_moe import Qwen3_5MoeTextConfig

    from speculators_amd.mtp import MTPConfig

    common = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64, vocab_size=1000,
                  num_hidden_layers=4, intermediate_size=512)
    moe = dict(num_experts=8, num_experts_per_tok=2, moe_intermediate_size=64, shared_expert_intermediate_size=128)
    c = MTPConfig.from_transformer_config(Qwen3NextConfig(**common, **moe))
    assert (c.model_type, c.num_experts, c.partial_rotary_factor, c.rotary_dim) == ("qwen3_next", 8, 0.25, 16)
    c = MTPConfig.from_transformer_config(Qwen3NextConfig(**common, **moe, mlp_only_layers=[3]))
    assert c.num_experts == 0 and c.intermediate_size == 512
    c = MTPConfig.from_transformer_config(Qwen3NextConfig(**common, **moe, decoder_sparse_step=3))
    assert c.num_experts == 0  # last full-attention layer is index 3: (3 + 1) % 3 != 0
    c = MTPConfig.from_transformer_config(Qwen3_5TextConfig(**common))
    assert (c.model_type, c.num_experts, c.rotary_dim) == ("qwen3_5_text", 0, 16)
    c = MTPConfig.from_transformer_config(Qwen3_5MoeTextConfig(**common, **moe))
    assert (c.model_type, c.num_experts, c.norm_topk_prob) == ("qwen3_5_moe_text", 8, True)
    c = MTPConfig.from_transformer_config(Qwen3Config(**common))
    assert (c.model_type, c.rotary_dim, c.num_experts) == ("qwen3", 64, 0)
    with pytest.raises(ValueError, match="Unsupported MTP model type"):
        MTPConfig.from_transformer_config(type("C", (), {"model_type": "llama"})())


def test_route_equals_the_oracle_router_and_sort_pairs_is_a_stable_expert_sort():
    import torch

    from oracle import mtp as OM
    from speculators_amd import moe

    g = torch.Generator().manual_seed(0)
    x = torch.randn(50, 32, generator=g)
    wr = torch.randn(12, 32, generator=g)
    for renorm in (True, False):
        scores, idx = moe.route(x @ wr.t(), 4, renorm)
        want_s, want_i = OM.moe_routing(x, wr, 4, renorm)
        assert torch.equal(idx, want_i) and torch.equal(scores, want_s)
    order, src_row, pos, off = moe.sort_pairs(idx, 12)
    flat = idx.reshape(-1)
    # sorted by expert, token order kept inside an expert (what makes the weight gradients reproducible)
    assert torch.equal(flat[order], flat.sort(stable=True).values)
    keys = flat[order] * 1000 + order
    assert (keys.diff() > 0).all()
    assert torch.equal(src_row.long(), order // 4)
    assert off[0] == 0 and off[-1] == 200 and torch.equal(off[1:].long(), torch.bincount(flat, minlength=12).cumsum(0))
    assert torch.equal(order[pos.reshape(-1).long()], torch.arange(200))
    # an expert nobody chose is an empty group
    idx2 = idx.clone()
    idx2[idx2 == 3] = 5
    _, _, _, off2 = moe.sort_pairs(idx2, 12)
    assert off2[4] == off2[3]
