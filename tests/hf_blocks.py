"""HF transformers library blocks composed the way the reference composes them: shared by the
oracle-pinning tests (CPU) and the attention plug-in tests (GPU).  Test infrastructure."""

import torch


def qwen3_cfg(shape):
    from transformers import Qwen3Config

    cfg = Qwen3Config(hidden_size=shape.hidden_size, num_attention_heads=shape.num_attention_heads,
                      num_key_value_heads=shape.num_key_value_heads, head_dim=shape.head_dim,
                      intermediate_size=shape.intermediate_size, vocab_size=shape.vocab_size,
                      rms_norm_eps=shape.rms_norm_eps, num_hidden_layers=shape.num_hidden_layers,
                      rope_parameters={"rope_type": "default", "rope_theta": shape.rope_theta},
                      attention_bias=False, attention_dropout=0.0)
    cfg._attn_implementation = "eager"
    return cfg


class HFDFlashLayer(torch.nn.Module):
    """HF library blocks holding the oracle's weights of layer ``li``, wired the way
    Qwen3DFlashAttention / Qwen3DFlashDecoderLayer wire them
    (models/dflash/model_definitions.py:97-155,170-207).  ``attn_impl``: "eager" = the library's
    eager attention under a dense additive mask; any other name is looked up in HF's global
    attention registry, as the reference does (model_definitions.py:134-152), and receives the
    mask object as it is."""

    def __init__(self, cfg, w, li, attn_impl: str = "eager"):
        super().__init__()
        self.attn_impl = attn_impl
        from transformers.models.qwen3.modeling_qwen3 import Qwen3MLP, Qwen3RMSNorm

        h, d = cfg.hidden_size, cfg.head_dim
        p = f"layers.{li}."
        self.num_key_value_groups = cfg.num_attention_heads // cfg.num_key_value_heads
        self.d = d
        self.proj = torch.nn.ModuleDict({
            "q": torch.nn.Linear(h, cfg.num_attention_heads * d, bias=False),
            "k": torch.nn.Linear(h, cfg.num_key_value_heads * d, bias=False),
            "v": torch.nn.Linear(h, cfg.num_key_value_heads * d, bias=False),
            "o": torch.nn.Linear(cfg.num_attention_heads * d, h, bias=False)})
        for n, lin in self.proj.items():
            lin.weight.data.copy_(w[p + f"self_attn.{n}_proj.weight"])
        self.q_norm, self.k_norm = Qwen3RMSNorm(d, eps=cfg.rms_norm_eps), Qwen3RMSNorm(d, eps=cfg.rms_norm_eps)
        self.q_norm.weight.data.copy_(w[p + "self_attn.q_norm.weight"])
        self.k_norm.weight.data.copy_(w[p + "self_attn.k_norm.weight"])
        self.mlp = Qwen3MLP(cfg)
        for n in ("gate", "up", "down"):
            getattr(self.mlp, n + "_proj").weight.data.copy_(w[p + f"mlp.{n}_proj.weight"])
        self.ln1, self.ln2 = Qwen3RMSNorm(h, eps=cfg.rms_norm_eps), Qwen3RMSNorm(h, eps=cfg.rms_norm_eps)
        self.ln1.weight.data.copy_(w[p + "input_layernorm.weight"])
        self.ln2.weight.data.copy_(w[p + "post_attention_layernorm.weight"])

    def forward(self, noise, ctx, cos, sin, bool_mask):
        from transformers.models.qwen3.modeling_qwen3 import eager_attention_forward, rotate_half

        n_q, n_ctx = noise.shape[1], ctx.shape[1]
        x = self.ln1(noise)
        q = self.q_norm(self.proj["q"](x).view(1, n_q, -1, self.d)).transpose(1, 2)
        k = torch.cat([self.proj["k"](ctx), self.proj["k"](x)], 1).view(1, n_ctx + n_q, -1, self.d)
        v = torch.cat([self.proj["v"](ctx), self.proj["v"](x)], 1).view(1, n_ctx + n_q, -1, self.d)
        k, v = self.k_norm(k).transpose(1, 2), v.transpose(1, 2)
        c, s = cos.unsqueeze(1), sin.unsqueeze(1)
        q = q * c[..., -n_q:, :] + rotate_half(q) * s[..., -n_q:, :]
        k = k * c + rotate_half(k) * s
        if self.attn_impl == "eager":
            fmask = torch.zeros(1, 1, n_q, n_ctx + n_q, device=q.device, dtype=q.dtype).masked_fill(
                ~bool_mask[None, None], float("-inf"))
            a, _ = eager_attention_forward(self, q, k, v, fmask, scaling=self.d ** -0.5, dropout=0.0)
        else:
            from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

            a, _ = ALL_ATTENTION_FUNCTIONS[self.attn_impl](self, q, k, v, bool_mask, dropout=0.0,
                                                           scaling=self.d ** -0.5, sliding_window=None)
        y = noise + self.proj["o"](a.reshape(1, n_q, -1))
        return y + self.mlp(self.ln2(y))
