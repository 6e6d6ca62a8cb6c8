"""Host logic of the MTP model configuration (no GPU)."""

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
