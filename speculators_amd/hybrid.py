"""The full-attention decoder layer of the hybrid MTP flavours on the HIP path.

``qwen3_next``, ``qwen3_5_text`` and ``qwen3_5_moe_text`` MTP layers are the library's
``Qwen3NextDecoderLayer`` / ``Qwen3_5DecoderLayer`` / ``Qwen3_5MoeDecoderLayer`` built at the last
``full_attention`` index and mixed with ``MTPLayerMixin`` (models/mtp/model_definitions.py:52-68,
118-205).  What they change against the dense Qwen3 layer:

  * every RMSNorm has the gain ``1 + weight`` (``Qwen3NextRMSNorm``, weights start at zero);
  * ``q_proj`` is twice as wide: per head the query and a gate, and the attention output is
    multiplied by ``sigmoid(gate)`` before ``o_proj`` (``Qwen3NextAttention``);
  * the rotary embedding covers the first ``partial_rotary_factor`` of each head;
  * the MLP is dense (``qwen3_5_text``, or a ``qwen3_next`` layer outside the sparse pattern) or
    the sparse MoE block with a shared expert (``Qwen3NextSparseMoeBlock``).

Parameter names are the library's, so a reference checkpoint's ``mtp_layers.0.*`` loads as is.
"""

from __future__ import annotations

from types import SimpleNamespace

import torch
from torch import nn

from . import attention as A
from . import fused_ops as FO
from . import gemm, moe
from .eagle3 import MLP, RMSNorm
from .weights import WeightStager


class ZeroCenteredRMSNorm(RMSNorm):
    """``Qwen3NextRMSNorm``: ``norm(x) * (1 + weight)``."""

    def __init__(self, dim: int, eps: float, stager: WeightStager | None = None):
        super().__init__(dim, eps, stager)
        self.weight = nn.Parameter(torch.zeros(dim))

    @property
    def gain(self) -> torch.Tensor:
        if self._stager is None:
            return (1.0 + self.weight.float()).to(torch.bfloat16)
        return self._stager.gain(self.weight, plus_one=True)


class GatedAttention(nn.Module):
    """``Qwen3NextAttention`` (``modeling_qwen3_next.py``)."""

    def __init__(self, cfg, stager: WeightStager):
        super().__init__()
        h, hq, hkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        self.hq, self.hkv, self.d = hq, hkv, d
        self.q_proj = nn.Linear(h, hq * d * 2, bias=False)
        self.k_proj = nn.Linear(h, hkv * d, bias=False)
        self.v_proj = nn.Linear(h, hkv * d, bias=False)
        self.o_proj = nn.Linear(hq * d, h, bias=False)
        self.q_norm = ZeroCenteredRMSNorm(d, cfg.rms_norm_eps, stager)
        self.k_norm = ZeroCenteredRMSNorm(d, cfg.rms_norm_eps, stager)
        self.scaling = d ** -0.5
        self.attn_fn = A.ALL_ATTENTION_FUNCTIONS[cfg.attn_implementation]
        self._stager = stager

    def forward(self, x, position_ids, inv_freq, mask):
        t = x.shape[1]
        hq, hkv, d = self.hq, self.hkv, self.d
        W = self._stager.get
        q, gate = FO.split_query_gate(gemm.linear_staged(x, W(self.q_proj.weight)), hq)
        k = gemm.linear_staged(x, W(self.k_proj.weight))
        v = gemm.linear_staged(x, W(self.v_proj.weight))
        q = self.q_norm(q).reshape(1, t, hq * d)
        k = self.k_norm(k.view(1, t, hkv, d)).view(1, t, hkv * d)
        # rotary embedding of the first 2 * len(inv_freq) elements of every head, fused with the
        # [T, heads * D] -> [heads, T, D] relayout
        q = FO.rope_relayout(q, position_ids, inv_freq, hq, True, 0)
        k = FO.rope_relayout(k, position_ids, inv_freq, hkv, True, 0)
        v = FO.rope_relayout(v, position_ids, inv_freq, hkv, False, 0)
        out, _ = self.attn_fn(self, q, k, v, mask, scaling=self.scaling)
        out = FO.sigmoid_gate(out.reshape(1, t, hq * d), gate)
        return gemm.linear_staged(out, W(self.o_proj.weight))


class _Router(nn.Module):
    def __init__(self, num_experts: int, hidden: int):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(num_experts, hidden))


class _Experts(nn.Module):
    """The expert weights as two stacks (``Qwen3NextExperts``): gate and up merged row-wise."""

    def __init__(self, num_experts: int, hidden: int, inter: int):
        super().__init__()
        self.gate_up_proj = nn.Parameter(torch.empty(num_experts, 2 * inter, hidden))
        self.down_proj = nn.Parameter(torch.empty(num_experts, hidden, inter))
        for p in (self.gate_up_proj, self.down_proj):
            nn.init.normal_(p, std=0.02)


class SparseMoeBlock(nn.Module):
    """``Qwen3NextSparseMoeBlock``: routed experts plus a shared expert behind a sigmoid gate."""

    def __init__(self, cfg, stager: WeightStager):
        super().__init__()
        h = cfg.hidden_size
        self.top_k = cfg.num_experts_per_tok
        self.renormalise = cfg.norm_topk_prob
        self.gate = _Router(cfg.num_experts, h)
        self.experts = _Experts(cfg.num_experts, h, cfg.moe_intermediate_size)
        self.shared_expert = MLP(SimpleNamespace(hidden_size=h,
                                                 intermediate_size=cfg.shared_expert_intermediate_size), stager)
        self.shared_expert_gate = nn.Linear(h, 1, bias=False)
        self._stager = stager
        self.routing_log: list | None = None  # set to a list to collect every call's expert ids

    def forward(self, x):
        W = self._stager.get
        x2 = x.reshape(-1, x.shape[-1])
        scores, idx = moe.route(gemm.linear_staged(x2, W(self.gate.weight)), self.top_k, self.renormalise)
        if self.routing_log is not None:
            self.routing_log.append(idx)
        routed = moe.experts_mlp(x2, scores, idx, W(self.experts.gate_up_proj), W(self.experts.down_proj))
        shared = self.shared_expert(x).reshape(x2.shape)
        shared = torch.sigmoid(gemm.linear_staged(x2, W(self.shared_expert_gate.weight))) * shared
        return (routed + shared).view(x.shape)


class HybridMTPLayer(nn.Module):
    """``Qwen3NextMTPLayer`` / ``Qwen35MTPLayer`` / ``Qwen35MoeMTPLayer``
    (models/mtp/model_definitions.py:95-116 around the library's decoder layer)."""

    def __init__(self, cfg, stager: WeightStager):
        super().__init__()
        h, eps = cfg.hidden_size, cfg.rms_norm_eps
        self._stager = stager
        self.hidden_layernorm = ZeroCenteredRMSNorm(h, eps, stager)
        self.token_layernorm = ZeroCenteredRMSNorm(h, eps, stager)
        self.input_proj = nn.Linear(2 * h, h, bias=False)
        self.final_layernorm = ZeroCenteredRMSNorm(h, eps, stager)
        self.input_layernorm = ZeroCenteredRMSNorm(h, eps, stager)
        self.post_attention_layernorm = ZeroCenteredRMSNorm(h, eps, stager)
        self.self_attn = GatedAttention(cfg, stager)
        self.mlp = SparseMoeBlock(cfg, stager) if cfg.num_experts > 0 else MLP(cfg, stager)

    def forward(self, hidden, embeds, position_ids, inv_freq, mask):
        rows = hidden.shape[-2]
        w_in = self._stager.get(self.input_proj.weight)
        x = gemm.linear_staged(
            FO.pair_norm_cat(embeds, hidden, self.token_layernorm.gain, self.hidden_layernorm.gain,
                             self.token_layernorm.eps, out=w_in.x_slot(rows)), w_in)
        a = self.self_attn(self.input_layernorm(x), position_ids, inv_freq, mask)
        post, final = self.post_attention_layernorm, self.final_layernorm
        y, z = FO.add_rms_norm(x, a, post.gain, post.eps)
        _, out = FO.add_rms_norm(y, self.mlp(z), final.gain, final.eps)
        return out
