"""MTP (multi-token prediction) draft model: host side of the HIP training path.

Keeps the call contract of ``MTPDraftModel.forward`` (models/mtp/core.py:114-231):

    forward(input_ids, hidden_states, attention_mask=None, position_ids=None,
            loss_mask=None, step_weights=None) -> (logits_list, loss, metrics)

with the reference's metric keys (``loss_step_{k}``, ``loss_sum``, ``loss_total``) and
state-dict names (``mtp_layers.0.*``, ``embed_tokens``, ``lm_head``).  The layer is
``MTPLayerMixin`` (models/mtp/model_definitions.py:78-151) around a decoder layer:
two RMSNorms, ``input_proj (2H -> H)``, the layer, a final RMSNorm.  The layer is the
Qwen3 one with per-head q/k RMSNorm (``qwen3``) or the full-attention layer of the hybrid
flavours (``qwen3_next``, ``qwen3_5_text``, ``qwen3_5_moe_text``, models/mtp/model_definitions.py:
159-205; ``hybrid.py``): gain ``1 + w`` norms, gated attention, partial rotary embedding,
dense or sparse-MoE MLP.  Attention runs on the HIP interval-masked kernel (causal
inside each packed sequence, sequences found from the position restarts as
``create_causal_mask`` does at models/mtp/core.py:180-186), ``lm_head`` on the MFMA
GEMM, the loss on the label cross-entropy kernel.

A batch ``[B, L]`` is laid out as one packed row ``[1, B*L]`` whose sequences never
cross a batch row: every op other than attention is row-wise, and attention sees
the same keys.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn

from . import attention as A
from . import fused_ops as FO
from . import gemm
from . import losses as L
from .eagle3 import MLP, Attention, RMSNorm
from .hybrid import HybridMTPLayer
from .weights import WeightStager, compute_input

IGNORE_INDEX = -100


def compute_step_weights(beta: float = 0.6, num_steps: int = 3) -> list[float]:
    """Normalised exponential-decay step weights (models/mtp/core.py:29-38)."""
    raw = [beta**k for k in range(num_steps)]
    total = sum(raw)
    return [w / total for w in raw]


@dataclass
class MTPConfig:
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    num_speculative_steps: int = 3
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1000000.0
    rope_scaling: dict | None = None  # HF rope parameters (any rope_type of the library; see fused_ops.rope_inv_freq)
    model_type: str = "qwen3"
    attn_implementation: str = A.ATTN_IMPL_TTT
    qk_norm: bool = True  # Qwen3 attention
    # hybrid flavours (qwen3_next, qwen3_5_text, qwen3_5_moe_text)
    partial_rotary_factor: float = 1.0
    num_experts: int = 0  # 0: dense MLP of intermediate_size
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    shared_expert_intermediate_size: int = 0
    norm_topk_prob: bool = True

    @property
    def rotary_dim(self) -> int:
        return int(self.head_dim * self.partial_rotary_factor)

    @classmethod
    def from_transformer_config(cls, tc, num_speculative_steps: int = 3, **overrides) -> "MTPConfig":
        """From the verifier's (text) layer config, as ``MTPDraftModel.__init__`` reads
        ``config.transformer_layer_config`` (models/mtp/core.py:82-90).  The hybrid flavours take
        the layer at the last ``full_attention`` index (models/mtp/model_definitions.py:52-68); a
        ``qwen3_next`` layer there is sparse when the library's ``Qwen3NextDecoderLayer`` makes it
        so (``mlp_only_layers`` / ``decoder_sparse_step``), a ``qwen3_5_moe_text`` layer always."""
        model_type = resolve_model_type(tc.model_type)
        rope = dict(getattr(tc, "rope_parameters", None) or getattr(tc, "rope_scaling", None) or {})
        theta = rope.pop("rope_theta", None) or getattr(tc, "rope_theta", 10000.0)
        factor = rope.pop("partial_rotary_factor", None) or getattr(tc, "partial_rotary_factor", 1.0)
        rope.pop("mrope_section", None)
        rope.pop("mrope_interleaved", None)
        kind = rope.get("rope_type", rope.get("type", "default"))
        if kind in ("dynamic", "longrope"):  # the trained context travels with the rope parameters here
            rope.setdefault("max_position_embeddings", tc.max_position_embeddings)
        head_dim = getattr(tc, "head_dim", None) or tc.hidden_size // tc.num_attention_heads
        kw = dict(hidden_size=tc.hidden_size, num_attention_heads=tc.num_attention_heads,
                  num_key_value_heads=tc.num_key_value_heads, head_dim=head_dim,
                  intermediate_size=tc.intermediate_size, vocab_size=tc.vocab_size,
                  num_speculative_steps=num_speculative_steps, rms_norm_eps=tc.rms_norm_eps,
                  rope_theta=float(theta), rope_scaling=None if kind == "default" else rope,
                  model_type=model_type)
        if model_type != "qwen3":
            kw["partial_rotary_factor"] = float(factor)
            sparse = model_type == "qwen3_5_moe_text"
            if model_type == "qwen3_next":
                types = list(getattr(tc, "layer_types", None) or [])
                idx = max((i for i, t in enumerate(types) if t == "full_attention"), default=0)
                if types and "full_attention" not in types:
                    raise ValueError("Hybrid MTP layer requires at least one 'full_attention' entry in "
                                     f"config.layer_types, got: {types}")
                sparse = (idx not in (getattr(tc, "mlp_only_layers", None) or [])
                          and tc.num_experts > 0 and (idx + 1) % tc.decoder_sparse_step == 0)
            if sparse:
                kw.update(num_experts=tc.num_experts, num_experts_per_tok=tc.num_experts_per_tok,
                          moe_intermediate_size=tc.moe_intermediate_size,
                          shared_expert_intermediate_size=tc.shared_expert_intermediate_size,
                          norm_topk_prob=getattr(tc, "norm_topk_prob", True))
        kw.update(overrides)
        return cls(**kw)


MODEL_TYPES = ("qwen3", "qwen3_next", "qwen3_5_text", "qwen3_5_moe_text")


def resolve_model_type(model_type: str) -> str:
    """models/mtp/model_definitions.py:31-35."""
    if model_type in MODEL_TYPES:
        return model_type
    raise ValueError(f"Unsupported MTP model type '{model_type}'. Supported types: {sorted(MODEL_TYPES)}")


class MTPLayer(nn.Module):
    """``Qwen3MTPLayer`` (models/mtp/model_definitions.py:78-151)."""

    def __init__(self, cfg: MTPConfig, stager: WeightStager):
        super().__init__()
        h, eps = cfg.hidden_size, cfg.rms_norm_eps
        self._stager = stager
        self.hidden_layernorm = RMSNorm(h, eps, stager)
        self.token_layernorm = RMSNorm(h, eps, stager)
        self.input_proj = nn.Linear(2 * h, h, bias=False)
        self.final_layernorm = RMSNorm(h, eps, stager)
        self.input_layernorm = RMSNorm(h, eps, stager)
        self.post_attention_layernorm = RMSNorm(h, eps, stager)
        self.self_attn = Attention(cfg, h, stager)
        self.mlp = MLP(cfg, stager)

    def forward(self, hidden, embeds, position_ids, inv_freq, mask):
        # both norms write into the halves of the 2H-wide projection input; each residual add is
        # fused into the norm that follows it
        rows = hidden.shape[-2]
        w_in = self._stager.get(self.input_proj.weight)
        x = gemm.linear_staged(
            FO.pair_norm_cat(embeds, hidden, self.token_layernorm.gain, self.hidden_layernorm.gain,
                             self.token_layernorm.eps, out=w_in.x_slot(rows)), w_in)
        a = self.self_attn(self.input_layernorm(x), position_ids, 0, inv_freq, {}, mask)
        post, final = self.post_attention_layernorm, self.final_layernorm
        w_gu = self._stager.get(self.mlp.gate_proj.weight, self.mlp.up_proj.weight)
        y, z = FO.add_rms_norm(x, a, post.gain, post.eps, out=w_gu.x_slot(rows))
        _, out = FO.add_rms_norm(y, self.mlp(z), final.gain, final.eps)
        return out


class MTPDraftModel(nn.Module):
    def __init__(self, config: MTPConfig):
        super().__init__()
        resolve_model_type(config.model_type)
        self.config = config
        self._stager = WeightStager()
        self._rotary = FO.RotaryFrequencies(config.rotary_dim, config.rope_theta, config.rope_scaling)
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        layer_class = MTPLayer if config.model_type == "qwen3" else HybridMTPLayer
        self.mtp_layers = nn.ModuleList([layer_class(config, self._stager)])
        # the verifier's embedding and head are frozen (model.py:70-71)
        self.embed_tokens.weight.requires_grad_(False)
        self.lm_head.weight.requires_grad_(False)
        # lm_head and the loss as one autograd node while the head is frozen (False: two nodes, logits
        # returned with their own gradient path as in the reference)
        self.fuse_head_loss = True

    @property
    def layers(self) -> nn.ModuleList:
        return self.mtp_layers

    def invalidate_weight_caches(self):
        """Drop the kept bf16 / transposed copies of the frozen weights.  They are keyed on the
        parameter's address and version counter, which a write through ``param.data`` does not
        change: call this after such a write.  ``train()`` / ``eval()`` and ``load_state_dict``
        call it."""
        self._stager.invalidate()

    def train(self, mode: bool = True):
        self._stager.invalidate()
        return super().train(mode)

    def load_state_dict(self, *args, **kwargs):
        self._stager.invalidate()
        return super().load_state_dict(*args, **kwargs)

    def forward(self, input_ids, hidden_states, attention_mask=None, position_ids=None,
                loss_mask=None, step_weights=None, return_dict: bool = True, **_kwargs):
        cfg = self.config
        self._stager.begin(uses=cfg.num_speculative_steps)
        hidden_states = compute_input(hidden_states)
        input_ids = input_ids.long()
        device = input_ids.device
        b, n = input_ids.shape
        num_steps = cfg.num_speculative_steps
        if step_weights is not None and len(step_weights) != num_steps:
            raise ValueError(
                f"step_weights has {len(step_weights)} entries but num_speculative_steps={num_steps}; "
                f"expected exactly {num_steps} weights.")
        if position_ids is None:
            position_ids = torch.arange(n, device=device).unsqueeze(0).expand(b, -1)

        all_logits: list[torch.Tensor] = []
        total_loss = torch.tensor(0.0, device=device)
        metrics: dict = {}
        steps = min(num_steps, max(0, n - 2))
        valid = n - steps - 1
        if valid <= 0 or steps == 0:
            metrics["loss_sum"] = total_loss.detach().clone()
            metrics["loss_total"] = torch.tensor(1.0, device=device)
            return all_logits, total_loss, metrics

        pos = position_ids[:, :valid].to(torch.int64)
        if attention_mask is None:
            # sequence index inside each row (a new sequence wherever the position does not grow
            # by one), made unique across rows: the packed row [1, B * valid] never mixes rows
            diff = torch.diff(pos, prepend=pos[:, :1] - 1, dim=-1)
            seq = (diff != 1).cumsum(-1) + torch.arange(b, device=device).unsqueeze(1) * (valid + 1)
            mask = A.create_ttt_mask(seq.reshape(-1), b * valid, None)
        else:
            # a padding mask switches the packed-sequence detection off (create_causal_mask only
            # looks at position restarts when no mask is given): key j <= i with attention_mask[j]
            if attention_mask.shape != (b, n):
                raise ValueError(f"attention_mask must be {(b, n)}, got {tuple(attention_mask.shape)}")
            mask = A.create_padding_span_mask(attention_mask[:, :valid].to(device))
        flat_pos = pos.reshape(-1).contiguous()
        rope_top = self._rotary.top(flat_pos)
        layer = self.mtp_layers[0]

        current = hidden_states
        for step in range(steps):
            hid = current[:, :valid].reshape(1, b * valid, cfg.hidden_size)
            with torch.no_grad():
                emb = F.embedding(input_ids[:, step + 1:step + 1 + valid], self.embed_tokens.weight)
                emb = emb.to(hidden_states.dtype).reshape(1, b * valid, cfg.hidden_size)
            # (asked once per step, like the rotary module: models/mtp/core.py:196)
            inv_freq = self._rotary.select(device, rope_top)
            out = layer(hid, emb, flat_pos, inv_freq, mask)
            targets = input_ids[:, step + 2:step + 2 + valid]
            if loss_mask is not None:
                targets = targets.clone()
                targets[loss_mask[:, step + 2:step + 2 + valid] == 0] = IGNORE_INDEX
            weight = step_weights[step] if step_weights is not None else 1.0
            head = self._stager.get(self.lm_head.weight)
            if self.fuse_head_loss and out.requires_grad and not head.trainable:
                # head + loss as one autograd node: the backward skips the ignored positions in the
                # input-gradient product of the head (the returned logits carry no gradient)
                unreduced, logits = L.head_label_cross_entropy(
                    out.view(b, valid, cfg.hidden_size), head.w, head.wt, targets, IGNORE_INDEX)
            else:
                logits = gemm.linear_staged(out, head, hip=True).view(b, valid, cfg.vocab_size)
                unreduced = L.label_cross_entropy(logits, targets, IGNORE_INDEX)
            all_logits.append(logits)
            valid_count = (targets != IGNORE_INDEX).sum()
            step_loss = weight * unreduced.sum() / valid_count.clamp(min=1)
            total_loss = total_loss + step_loss
            metrics[f"loss_step_{step}"] = step_loss.detach().clone()
            current = out.view(b, valid, cfg.hidden_size)

        metrics["loss_sum"] = total_loss.detach().clone()
        metrics["loss_total"] = torch.tensor(1.0, device=device)
        return all_logits, total_loss, metrics

    @staticmethod
    def get_trainer_kwargs(**kwargs):
        """(train_call_kwargs, val_call_kwargs): ``step_weights`` as given, else computed from
        ``step_weight_beta`` and ``num_speculative_steps`` (models/mtp/core.py:280-304)."""
        step_weights = kwargs.get("step_weights")
        if step_weights is None:
            if "num_speculative_steps" not in kwargs:
                raise ValueError("num_speculative_steps must be set from the model config "
                                 "before calling get_trainer_kwargs")
            step_weights = compute_step_weights(beta=kwargs.get("step_weight_beta", 0.6),
                                                num_steps=kwargs["num_speculative_steps"])
        train_kwargs = {"step_weights": step_weights}
        return train_kwargs, train_kwargs.copy()
