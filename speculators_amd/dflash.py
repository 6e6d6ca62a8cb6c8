"""DFlash draft model: host side of the HIP anchored-block training path.

Keeps the call contract of ``DFlashDraftModel.forward``
(models/dflash/core.py:441-478):

    forward(hidden_states, input_ids, loss_mask, verifier_last_hidden_states,
            document_ids, position_ids, loss_config, gamma, max_anchors,
            per_position_loss_weight, dpace_alpha) -> (None, loss, metrics)

and the reference's state-dict names (models/dflash/core.py:36-120).  The
anchored-block attention of every layer runs on the HIP interval-masked
kernel, fc / lm_head / verifier head on the MFMA GEMM, loss and per-slot
acceptance counts on the fused vocabulary loss kernel.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch
import torch.nn.functional as F
from torch import nn

from . import attention as A
from . import fused_ops as FO
from . import gemm
from . import losses as L
from . import metrics as MT
from .eagle3 import MLP, RMSNorm
from .weights import WeightStager, compute_input


@dataclass
class DFlashConfig:
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    draft_vocab_size: int
    num_aux: int = 5
    num_hidden_layers: int = 5
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1000000.0
    rope_scaling: dict | None = None  # HF rope parameters (any rope_type of the library; see fused_ops.rope_inv_freq)
    block_size: int = 8
    mask_token_id: int | None = None
    sliding_window: int | None = None
    sliding_layers: tuple = field(default_factory=tuple)
    sliding_window_non_causal: bool = False
    sample_from_anchor: bool = False
    attn_implementation: str = A.ATTN_IMPL_DFLASH


def get_base_indices_for_anchored_blocks(anchor_positions: torch.Tensor, block_size: int):
    """[a, a+1, ..., a+bs-1] per anchor, flattened (models/dflash/utils.py:6-18)."""
    a = anchor_positions.to(dtype=torch.long).view(-1)
    off = torch.arange(block_size, device=a.device, dtype=torch.long)
    return (a[:, None] + off[None, :]).reshape(-1)


def select_anchors(loss_mask: torch.Tensor, num_anchors: int, block_size: int):
    """Random anchors among the positions with loss_mask set, excluding the last
    ``block_size`` positions; sorted; padded with position 0 / invalid
    (models/dflash/utils.py:21-67)."""
    if loss_mask.ndim != 2:
        raise ValueError(f"Expected [B, T], got {loss_mask.shape}")
    if block_size <= 0:
        raise ValueError(f"Expected block size > 0, got {block_size}")
    valid = loss_mask.bool().clone()
    valid[:, -block_size:] = False
    idx = torch.nonzero(valid.squeeze(0), as_tuple=False).squeeze(-1)
    dev = loss_mask.device
    anchors = torch.zeros(num_anchors, dtype=torch.long, device=dev)
    ok = torch.zeros(num_anchors, dtype=torch.bool, device=dev)
    k = min(num_anchors, idx.numel())
    perm = torch.randperm(idx.numel(), device=dev)
    anchors[:k] = torch.sort(idx[perm[:k]]).values
    ok[:k] = True
    return anchors, ok


class DFlashAttention(nn.Module):
    """q from the mask tokens; k/v from ``cat([context, mask tokens])``; per-head q/k
    RMSNorm; RoPE with the last q_len positions for q
    (models/dflash/model_definitions.py:47-155)."""

    def __init__(self, cfg: DFlashConfig, stager: WeightStager):
        super().__init__()
        hq, hkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        self.hq, self.hkv, self.d = hq, hkv, d
        self._stager = stager
        self.q_proj = nn.Linear(cfg.hidden_size, hq * d, bias=False)
        self.k_proj = nn.Linear(cfg.hidden_size, hkv * d, bias=False)
        self.v_proj = nn.Linear(cfg.hidden_size, hkv * d, bias=False)
        self.o_proj = nn.Linear(hq * d, cfg.hidden_size, bias=False)
        self.q_norm = RMSNorm(d, cfg.rms_norm_eps, stager)
        self.k_norm = RMSNorm(d, cfg.rms_norm_eps, stager)
        self.scaling = d ** -0.5
        self.attn_fn = A.ALL_ATTENTION_FUNCTIONS[cfg.attn_implementation]

    def forward(self, x, ctx, q_pos, kv_pos, inv_freq, mask):
        ql, tl = x.shape[1], ctx.shape[1]
        lin, W = gemm.linear_staged, self._stager.get
        q = self.q_norm(lin(x, W(self.q_proj.weight)).view(1, ql, self.hq, self.d)).view(1, ql, self.hq * self.d)
        # one projection of cat([context, mask tokens]) instead of two per weight
        both = torch.cat([ctx, x], dim=1)
        k = lin(both, W(self.k_proj.weight))
        v = lin(both, W(self.v_proj.weight))
        k = self.k_norm(k.view(1, tl + ql, self.hkv, self.d)).view(1, tl + ql, self.hkv * self.d)
        q = FO.rope_relayout(q, q_pos, inv_freq, self.hq, True, 0)
        k = FO.rope_relayout(k, kv_pos, inv_freq, self.hkv, True, 0)
        v = FO.rope_relayout(v, kv_pos, inv_freq, self.hkv, False, 0)
        out, _ = self.attn_fn(self, q, k, v, mask, scaling=self.scaling)
        return lin(out.reshape(1, ql, self.hq * self.d), W(self.o_proj.weight))


class DFlashDecoderLayer(nn.Module):
    def __init__(self, cfg: DFlashConfig, stager: WeightStager):
        super().__init__()
        self.self_attn = DFlashAttention(cfg, stager)
        self.mlp = MLP(cfg, stager)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, stager)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, stager)

    def forward(self, x, ctx, q_pos, kv_pos, inv_freq, mask, x_normed=None, next_norm=None):
        """``x_normed``: ``input_layernorm(x)`` when the previous layer already produced it;
        ``next_norm``: the RMSNorm that reads this layer's output -- the result is then
        ``(out, next_norm(out))`` with the last residual add fused into that norm."""
        if x_normed is None:
            x_normed = self.input_layernorm(x)
        a = self.self_attn(x_normed, ctx, q_pos, kv_pos, inv_freq, mask)
        post = self.post_attention_layernorm
        y, z = FO.add_rms_norm(x, a, post.gain, post.eps)  # residual add fused into the norm
        m = self.mlp(z)
        if next_norm is None:
            return y + m
        return FO.add_rms_norm(y, m, next_norm.gain, next_norm.eps)


class DFlashDraftModel(nn.Module):
    def __init__(self, config: DFlashConfig):
        super().__init__()
        self.config = config
        h = config.hidden_size
        self.block_size = config.block_size
        self._stager = st = WeightStager()
        self._rotary = FO.RotaryFrequencies(config.head_dim, config.rope_theta, config.rope_scaling)
        self.draft_vocab_size = config.draft_vocab_size
        self.verifier_vocab_size = config.vocab_size
        self.use_draft_vocab = config.draft_vocab_size != config.vocab_size
        if self.use_draft_vocab:
            self.register_buffer("t2d", torch.zeros(config.vocab_size, dtype=torch.bool))
            self.register_buffer("d2t", torch.zeros(config.draft_vocab_size, dtype=torch.long))
        else:
            self.t2d = self.d2t = None
        self.embed_tokens = nn.Embedding(config.vocab_size, h)
        self.lm_head = nn.Linear(h, config.draft_vocab_size, bias=False)
        self.verifier_lm_head = nn.Linear(h, config.draft_vocab_size, bias=False)
        self.fc = nn.Linear(config.num_aux * h, h, bias=False)
        self.hidden_norm = RMSNorm(h, config.rms_norm_eps, st)
        self.layers = nn.ModuleList(DFlashDecoderLayer(config, st) for _ in range(config.num_hidden_layers))
        self.norm = RMSNorm(h, config.rms_norm_eps, st)
        self.verifier_norm = RMSNorm(h, config.rms_norm_eps, st)
        for p in (self.embed_tokens.weight, self.lm_head.weight, self.verifier_lm_head.weight,
                  self.verifier_norm.weight):
            p.requires_grad_(False)
        self.uses_sliding_window_attn = bool(config.sliding_layers)
        self.uses_full_attn = config.num_hidden_layers > len(config.sliding_layers)
        # lm_head and the loss as one autograd node while the head is frozen and the loss is a single
        # fused reduction (False: always two nodes)
        self.fuse_head_loss = True

    @property
    def mask_token_id(self) -> int:
        if self.config.mask_token_id is None:
            raise ValueError(
                "mask_token_id is not set on the config. Pass --mask-token-id during training or "
                "ensure the config was saved with mask_token_id set.")
        return self.config.mask_token_id

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

    def _linear(self, x, weight):
        """``x @ weight.T`` on the MFMA kernel of this library (fc, lm_head, verifier head)."""
        return gemm.linear_staged(x, self._stager.get(weight), hip=True)

    def forward(self, hidden_states, input_ids, loss_mask, verifier_last_hidden_states,
                document_ids, position_ids=None, loss_config: L.LossConfig | None = None,
                gamma: float = 4.0, max_anchors: int = 512,
                per_position_loss_weight: str = "fixed-exp-decay", dpace_alpha: float = 0.5,
                anchors=None, **_kwargs):
        """``anchors=(positions, valid)`` overrides the random anchor selection."""
        cfg = self.config
        device = hidden_states.device
        t = hidden_states.shape[1]
        bs = self.block_size
        self._stager.begin()
        hidden_states = compute_input(hidden_states)
        verifier_last_hidden_states = compute_input(verifier_last_hidden_states)
        if position_ids is None:
            position_ids = torch.arange(t, dtype=torch.long, device=device).unsqueeze(0)
        if anchors is None:
            anchors = select_anchors(loss_mask, max_anchors, bs)
        anchor_pos, anchor_valid = anchors
        doc = document_ids.reshape(-1).to(device)
        full_mask = (A.create_dflash_mask(doc, t, anchor_pos, bs, None)
                     if self.uses_full_attn else None)
        sw_mask = (A.create_dflash_mask(doc, t, anchor_pos, bs, cfg.sliding_window,
                                        cfg.sliding_window_non_causal)
                   if self.uses_sliding_window_attn else None)
        n_q = anchor_pos.numel() * bs
        ids = torch.full((1, n_q), self.mask_token_id, dtype=torch.long, device=device)
        ids[:, ::bs] = input_ids[:, anchor_pos]
        with torch.no_grad():
            noise = F.embedding(ids, self.embed_tokens.weight).to(hidden_states.dtype)
        ctx = self.hidden_norm(self._linear(hidden_states, self.fc.weight))
        block_pos = get_base_indices_for_anchored_blocks(position_ids[0, anchor_pos], bs)
        kv_pos = torch.cat([position_ids.reshape(-1), block_pos]).to(torch.int64).contiguous()
        q_pos = block_pos.to(torch.int64).contiguous()
        inv_freq = self._rotary.select(device, self._rotary.top(kv_pos))
        block_idx = get_base_indices_for_anchored_blocks(anchor_pos, bs)
        with torch.no_grad():
            idx = block_idx if cfg.sample_from_anchor else (block_idx - 1) % t
            targets = self._linear(self.verifier_norm(verifier_last_hidden_states[:, idx]),
                                   self.verifier_lm_head.weight)
        normed = None
        last = len(self.layers) - 1
        for li, layer in enumerate(self.layers):
            # the norm that reads this layer's output: the next layer's input norm or the final one
            nxt = self.norm if li == last else self.layers[li + 1].input_layernorm
            noise, normed = layer(noise, ctx, q_pos, kv_pos, inv_freq,
                                  sw_mask if li in cfg.sliding_layers else full_mask,
                                  x_normed=normed, next_norm=nxt)
        head = self._stager.get(self.lm_head.weight)
        if self.fuse_head_loss and normed.requires_grad and not head.trainable:
            # head + loss as one autograd node while the head is frozen (see metrics.Head)
            logits = MT.Head(normed, head.w, head.wt)
        else:
            logits = gemm.linear_staged(normed, head, hip=True)
        aligned = loss_mask.clone()[:, block_idx]
        aligned = aligned * anchor_valid.repeat_interleave(bs).unsqueeze(0).to(aligned.dtype)
        if not cfg.sample_from_anchor:
            aligned[:, ::bs] = 0
        loss, metrics = MT.dflash_compute_metrics(
            logits, targets, aligned, bs, gamma=gamma, loss_config=loss_config,
            per_position_loss_weight=per_position_loss_weight, dpace_alpha=dpace_alpha,
            sample_from_anchor=cfg.sample_from_anchor)
        return None, loss, metrics

    @staticmethod
    def get_trainer_kwargs(**kwargs):
        """(train_call_kwargs, val_call_kwargs) like models/dflash/core.py:234-262."""
        shared = {
            "loss_config": L.resolve_loss_config(kwargs["loss_fn"], kwargs.get("loss_implementation", "hip")),
            "gamma": kwargs.get("dflash_decay_gamma", 4.0),
            "max_anchors": kwargs.get("max_anchors", 512),
            "per_position_loss_weight": kwargs.get("per_position_loss_weight", "fixed-exp-decay"),
            "dpace_alpha": kwargs.get("dpace_alpha", 0.5),
        }
        return dict(shared), dict(shared)
