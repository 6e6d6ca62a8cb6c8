"""EAGLE3 draft model: host side of the HIP training hot path.

Keeps the reference model's call contract
(``Eagle3DraftModel.forward``, models/eagle3/core.py:192-365):

    forward(hidden_states, input_ids, document_ids, loss_mask, position_ids,
            verifier_last_hidden_states, ttt_steps, ttt_step_loss_decay,
            loss_config) -> (draft_tokens, loss, metrics)

and its state-dict names (models/eagle3/core.py:31-42), so a checkpoint of the
reference loads with ``load_state_dict``.  The attention of every TTT step
runs on the HIP TTT kernel, fc / lm_head / verifier head on the MFMA GEMM, the
per-step loss, arg-maxes and acceptance counts on the fused vocabulary loss.
The decoder-internal projections use PyTorch's (hipBLASLt) matmul.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import NamedTuple

import torch
import torch.nn.functional as F
from torch import nn

from . import attention as A
from . import fused_ops as FO
from . import gemm
from . import losses as L
from . import metrics as MT
from .weights import WeightStager, compute_input


@dataclass
class Eagle3Config:
    """Shape and switches of the draft (the subset of Eagle3SpeculatorConfig +
    transformer_layer_config the forward reads; models/eagle3/config.py)."""

    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int  # verifier vocabulary
    draft_vocab_size: int
    num_aux: int = 3
    num_hidden_layers: int = 1
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = None  # HF rope parameters (any rope_type of the library; see fused_ops.rope_inv_freq)
    norm_before_residual: bool = False
    norm_before_fc: bool = False
    fc_norm: bool = False
    norm_output: bool = False
    qk_norm: bool = False
    sliding_window: int | None = None
    sliding_layers: tuple = field(default_factory=tuple)
    attn_implementation: str = A.ATTN_IMPL_TTT
    embed_requires_grad: bool = False  # requires_grad of embed_tokens.weight (models/eagle3/core.py:68)


class RMSNorm(nn.Module):
    """``stager``: the model's ``WeightStager`` (the gain is then read through it: bf16 compute copy
    of an fp32 master gain); None for a stand-alone norm on bf16 tensors."""

    def __init__(self, dim: int, eps: float, stager: WeightStager | None = None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps
        self._stager = stager

    @property
    def gain(self) -> torch.Tensor:
        return self.weight if self._stager is None else self._stager.gain(self.weight)

    def forward(self, x):
        return FO.rms_norm(x, self.gain, self.eps)


class Attention(nn.Module):
    def __init__(self, cfg: Eagle3Config, in_features: int, stager: WeightStager):
        super().__init__()
        hq, hkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        self.hq, self.hkv, self.d = hq, hkv, d
        self.q_proj = nn.Linear(in_features, hq * d, bias=False)
        self.k_proj = nn.Linear(in_features, hkv * d, bias=False)
        self.v_proj = nn.Linear(in_features, hkv * d, bias=False)
        self.o_proj = nn.Linear(hq * d, cfg.hidden_size, bias=False)
        if cfg.qk_norm:
            self.q_norm = RMSNorm(d, cfg.rms_norm_eps, stager)
            self.k_norm = RMSNorm(d, cfg.rms_norm_eps, stager)
        self.qk_norm = cfg.qk_norm
        self.scaling = d ** -0.5
        self.attn_fn = A.ALL_ATTENTION_FUNCTIONS[cfg.attn_implementation]
        self._stager = stager

    def forward(self, x, position_ids, pos_offset, inv_freq, cache: dict, mask):
        t = x.shape[1]
        W = self._stager.get
        if not self.qk_norm:
            # one GEMM for q, k and v; rotary embedding + [T, heads*D] -> [heads, T, D] fused behind it
            pos = position_ids.reshape(-1)
            if pos.dtype != torch.int64:
                pos = pos.to(torch.int64)
            kvc = cache.get("kv")
            # (a head size the kernels are not built for goes the general way below: the attention
            # function widens it with zero columns)
            if (kvc is None and cache.get("steps") and self.attn_fn is A.ttt_hip_attention_forward
                    and self.d in A.KERNEL_HEAD_DIMS):
                # all TTT steps' keys / values of this layer in one buffer, written in place
                kvc = cache["kv"] = A.TTTKVCache(self.hkv, t, self.d, cache["steps"], x.device)
            q, k, v = gemm.qkv_rope(x, W(self.q_proj.weight, self.k_proj.weight, self.v_proj.weight),
                                    pos.contiguous(), inv_freq, self.hq, self.hkv, self.d, pos_offset,
                                    kv_out=None if kvc is None else kvc.window(pos_offset))
            if kvc is not None:
                wo = W(self.o_proj.weight)
                out = A.ttt_attention_cached(q, k, v, kvc, mask, self.scaling, out=wo.x_slot(t))
                return gemm.linear_staged(out.reshape(1, t, self.hq * self.d), wo)
        else:
            q = gemm.linear_staged(x, W(self.q_proj.weight))
            k = gemm.linear_staged(x, W(self.k_proj.weight))
            v = gemm.linear_staged(x, W(self.v_proj.weight))
            q = self.q_norm(q.view(1, t, self.hq, self.d)).view(1, t, self.hq * self.d)
            k = self.k_norm(k.view(1, t, self.hkv, self.d)).view(1, t, self.hkv * self.d)
            # rotary embedding + [T, heads*D] -> [heads, T, D] in one pass each
            q = FO.rope_relayout(q, position_ids, inv_freq, self.hq, True, pos_offset)
            k = FO.rope_relayout(k, position_ids, inv_freq, self.hkv, True, pos_offset)
            v = FO.rope_relayout(v, position_ids, inv_freq, self.hkv, False, 0)
        # the K/V cache grows by T keys per TTT step (DynamicCache.update in the reference)
        cache["k"] = k if "k" not in cache else torch.cat([cache["k"], k], dim=2)
        cache["v"] = v if "v" not in cache else torch.cat([cache["v"], v], dim=2)
        out, _ = self.attn_fn(self, q, cache["k"], cache["v"], mask, scaling=self.scaling)
        return gemm.linear_staged(out.reshape(1, t, self.hq * self.d), W(self.o_proj.weight))


class MLP(nn.Module):
    def __init__(self, cfg, stager: WeightStager):
        super().__init__()
        self.gate_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.up_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False)
        self._stager = stager

    def forward(self, x):
        W = self._stager.get
        # gate and up as one GEMM, SwiGLU on the two halves of its output
        wd = W(self.down_proj.weight)
        act = gemm.gate_up_swiglu(x, W(self.gate_proj.weight, self.up_proj.weight),
                                  out=wd.x_slot(x.numel() // x.shape[-1]))
        return gemm.linear_staged(act, wd)


class _Prenormed(NamedTuple):
    """A hidden state together with the next layer's input norm of it."""

    value: torch.Tensor
    normed: torch.Tensor


class DecoderLayer(nn.Module):
    """Layer 0 carries the EAGLE3 first-layer changes
    (models/eagle3/model_definitions.py:14-110): q/k/v read ``cat([embeds, hidden])``
    (2H wide), embeds and hidden are normalised separately, the residual is the
    (optionally normalised) hidden half."""

    def __init__(self, cfg: Eagle3Config, layer_idx: int, stager: WeightStager):
        super().__init__()
        self.first = layer_idx == 0
        self.cfg = cfg
        self._stager = stager
        self.self_attn = Attention(cfg, (2 if self.first else 1) * cfg.hidden_size, stager)
        self.mlp = MLP(cfg, stager)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, stager)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, stager)
        if self.first:
            self.hidden_norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, stager)

    def forward(self, x, position_ids, pos_offset, inv_freq, cache, mask, next_norm=None):
        """``x``: the hidden state, or for the first layer the pair ``(embeds, hidden)`` (their
        concatenation is what the reference passes).  With ``next_norm`` (the RMSNorm that
        consumes this layer's output) the result is ``(out, next_norm(out))``: the last
        residual add is fused into that norm."""
        if self.first:
            embeds, hidden = x
            eps = self.cfg.rms_norm_eps
            if self.cfg.norm_before_residual:
                embeds = self.input_layernorm(embeds)
                hidden = self.hidden_norm(hidden)
                residual = hidden
                xin = torch.cat([embeds, hidden], dim=-1)
            else:
                # both norms write straight into the halves of the 2H-wide projection input; the
                # residual goes through the same node (its gradient is folded into the norm's)
                att = self.self_attn
                wqkv = self._stager.get(att.q_proj.weight, att.k_proj.weight, att.v_proj.weight)
                xin, residual = FO.pair_norm_cat(
                    embeds, hidden, self.input_layernorm.gain, self.hidden_norm.gain, eps,
                    out=None if att.qk_norm else wqkv.x_slot(hidden.shape[-2]), residual=True)
            a = self.self_attn(xin, position_ids, pos_offset, inv_freq, cache, mask)
        else:
            if isinstance(x, _Prenormed):  # the previous layer already applied this layer's input norm
                residual, xn = x
            else:
                residual, xn = x, self.input_layernorm(x)
            a = self.self_attn(xn, position_ids, pos_offset, inv_freq, cache, mask)
        post = self.post_attention_layernorm
        wgu = self._stager.get(self.mlp.gate_proj.weight, self.mlp.up_proj.weight)
        y, z = FO.add_rms_norm(residual, a, post.gain, post.eps, out=wgu.x_slot(a.shape[-2]))
        m = self.mlp(z)
        if next_norm is None:
            return y + m
        return FO.add_rms_norm(y, m, next_norm.gain, next_norm.eps)


class Eagle3DraftModel(nn.Module):
    def __init__(self, config: Eagle3Config):
        super().__init__()
        self.config = config
        h = config.hidden_size
        self.hidden_size = h
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
        self.layers = nn.ModuleList(DecoderLayer(config, i, st) for i in range(config.num_hidden_layers))
        self.norm = RMSNorm(h, config.rms_norm_eps, st)
        self.verifier_norm = RMSNorm(h, config.rms_norm_eps, st)
        self.input_norm = (RMSNorm(config.num_aux * h, config.rms_norm_eps, st)
                           if config.norm_before_fc else None)
        self.fc_norm = (nn.ModuleList(RMSNorm(h, config.rms_norm_eps, st) for _ in range(config.num_aux))
                        if config.fc_norm else None)
        # frozen, as in model.py:63-71 and models/eagle3/core.py:68,120
        for p in (self.embed_tokens.weight, self.lm_head.weight, self.verifier_lm_head.weight,
                  self.verifier_norm.weight):
            p.requires_grad_(False)
        self.embed_tokens.weight.requires_grad_(config.embed_requires_grad)
        self.uses_sliding_window_attn = bool(config.sliding_layers)
        self.uses_full_attn = config.num_hidden_layers > len(config.sliding_layers)
        # lm_head and the loss as one autograd node while the head is frozen and the loss is a single
        # fused reduction (False: always two nodes)
        self.fuse_head_loss = True
        # True: every forward leaves its per-step draft logits ([1, T, Vd], detached) in
        # ``last_logits`` (for parity checks; the reference returns no logits either)
        self.keep_logits = False
        self.last_logits: list = []

    # ------------------------------------------------------------------ helpers
    def load_vocab_mappings(self, t2d, d2t):
        """Validation rules of model.py:81-121."""
        if t2d is None and d2t is None:
            return
        if t2d is None or d2t is None:
            raise ValueError("Both t2d and d2t must be provided together, or both must be None.")
        if not self.use_draft_vocab:
            return
        if t2d.shape[0] != self.verifier_vocab_size:
            raise ValueError(f"t2d.shape[0] ({t2d.shape[0]}) must match verifier_vocab_size "
                             f"({self.verifier_vocab_size}).")
        if int(t2d.sum(dtype=torch.long).item()) != self.draft_vocab_size:
            raise ValueError(f"t2d has {int(t2d.sum(dtype=torch.long).item())} non-zero values, "
                             f"expected {self.draft_vocab_size}.")
        if d2t.shape[0] != self.draft_vocab_size:
            raise ValueError(f"d2t.shape[0] ({d2t.shape[0]}) must match draft_vocab_size "
                             f"({self.draft_vocab_size}).")
        self.t2d.copy_(t2d.to(self.t2d.device))
        self.d2t.copy_(d2t.to(self.d2t.device))

    def invalidate_weight_caches(self):
        """Drop the kept bf16 / transposed copies of the frozen weights (``lm_head``,
        ``verifier_lm_head``, ``verifier_norm``).  They are keyed on the parameter's address and
        version counter, which a write through ``param.data`` does not change: call this after
        such a write.  ``train()`` / ``eval()`` and ``load_state_dict`` call it."""
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

    # ------------------------------------------------------------------ forward
    def forward(self, hidden_states, input_ids, document_ids, loss_mask=None, position_ids=None,
                verifier_last_hidden_states=None, ttt_steps: int = 3,
                ttt_step_loss_decay: float = 1.0, loss_config: L.LossConfig | None = None,
                verifier_logits=None, **_kwargs):
        """See the module docstring.  ``verifier_logits`` (``[1, T, Vt]`` over the target
        vocabulary) is an alternative to ``verifier_last_hidden_states``: the targets are
        then the d2t gather of those logits instead of the row-sliced verifier head."""
        cfg = self.config
        device = hidden_states.device
        t = hidden_states.shape[1]
        self._stager.begin(uses=ttt_steps)
        hidden_states = compute_input(hidden_states)
        if verifier_last_hidden_states is not None:
            verifier_last_hidden_states = compute_input(verifier_last_hidden_states)
        if position_ids is None:
            position_ids = 1 + torch.arange(t, dtype=torch.long, device=device).unsqueeze(0)
        doc = document_ids.reshape(-1).to(device)
        full_mask = A.create_ttt_mask(doc, t, None) if self.uses_full_attn else None
        sw_mask = (A.create_ttt_mask(doc, t, cfg.sliding_window)
                   if self.uses_sliding_window_attn else None)

        x = hidden_states
        if self.input_norm is not None:
            x = self.input_norm(x)
        if self.fc_norm is not None:
            chunks = x.chunk(len(self.fc_norm), dim=-1)
            x = torch.cat([n(c) for n, c in zip(self.fc_norm, chunks, strict=True)], dim=-1)
        hidden = self._linear(x, self.fc.weight)

        original_ids = input_ids.detach().clone()
        return_loss = verifier_last_hidden_states is not None or verifier_logits is not None
        if return_loss:
            with torch.no_grad():
                if verifier_logits is not None:
                    # gathered through d2t inside the first step's loss pass (metrics.TargetGather)
                    targets = (MT.TargetGather(compute_input(verifier_logits), self.d2t)
                               if self.use_draft_vocab else compute_input(verifier_logits))
                else:
                    # applied lazily: a cross-entropy loss takes the target rows' statistics from the
                    # head product's epilogue and never sees the rows (metrics.VerifierHead)
                    targets = MT.VerifierHead(self.verifier_norm(verifier_last_hidden_states),
                                              self._stager.get(self.verifier_lm_head.weight).w)
            loss = torch.zeros((), device=device)
            prev_correct = (loss_mask.clone() if loss_mask is not None
                            else torch.ones(1, t, device=device, dtype=torch.bool))
            metrics: dict = {}

        caches = [{"steps": ttt_steps} for _ in self.layers]
        stats_cache: dict = {}
        position_ids = position_ids.reshape(-1).to(torch.int64).contiguous()
        rope_top = self._rotary.top(position_ids)
        draft_tokens = []
        self.last_logits = []
        for step in range(ttt_steps):
            # looked up without a graph whatever embed_requires_grad says, as the reference does
            # (models/eagle3/core.py:270-271): the flag only marks the parameter as trainable
            with torch.no_grad():
                # (the looked-up rows are cast to bf16 before the norm either way)
                table = self.embed_tokens.weight
                if not table.requires_grad:
                    table = self._stager.get(table).w  # frozen: its bf16 copy is made once and kept
                embeds = F.embedding(input_ids, table)
            y = (embeds.to(hidden.dtype), hidden)
            normed = None
            last = len(self.layers) - 1
            # (the positions of step j are position_ids + j; a length-dependent rope type looks at them)
            inv_freq = self._rotary.select(device, rope_top, step)
            for li, layer in enumerate(self.layers):
                mask = sw_mask if li in cfg.sliding_layers else full_mask
                # the norm that reads this layer's output: the next layer's input norm, or the
                # final norm -- the layer fuses its last residual add into it
                nxt = self.norm if li == last else self.layers[li + 1].input_layernorm
                y, normed = layer(y, position_ids, step, inv_freq, caches[li], mask, next_norm=nxt)
                if li != last:
                    y = _Prenormed(y, normed)
            hidden = normed if cfg.norm_output else y
            head = self._stager.get(self.lm_head.weight)
            fuse = (return_loss and self.fuse_head_loss and normed.requires_grad
                    and not head.trainable)
            if not fuse:
                logits = gemm.linear_staged(normed, head, hip=True)

            if return_loss:
                # head + loss as one autograd node while the head is frozen (see metrics.Head)
                lg = MT.Head(normed, head.w, head.wt) if fuse else logits
                s_loss, s_metrics, pred = MT.compute_metrics(
                    lg, targets, loss_mask, prev_correct, step, ttt_step_loss_decay,
                    loss_config=loss_config, target_stats_cache=stats_cache, return_pred=True)
                if fuse:
                    logits = lg.logits
                loss = loss + s_loss
                metrics.update(s_metrics)
                # draft tokens: the loss kernel's arg-max for the aligned rows, plus the
                # last `step` rows (which have no target) on their own
                pred = pred.to(torch.int64)
                if step:
                    pred = torch.cat([pred, MT.argmax_rows(logits.detach()[0, t - step:])])
                draft_tokens.append(pred.view(1, t))
            else:
                draft_tokens.append(MT.argmax_rows(logits.detach()))

            if self.keep_logits:
                self.last_logits.append(logits.detach())
            input_ids = torch.cat(
                [original_ids[:, 1 + step:], original_ids.new_zeros(1, 1 + step)], dim=-1)
            if full_mask is not None:
                full_mask = full_mask.extended()
            if sw_mask is not None:
                sw_mask = sw_mask.extended()

        if not return_loss:
            return draft_tokens
        metrics["loss_sum"] = loss.detach().clone()
        metrics["loss_total"] = torch.ones((), device=device)
        return draft_tokens, loss, metrics

    @staticmethod
    def get_trainer_kwargs(**kwargs):
        """(train_call_kwargs, val_call_kwargs) like models/eagle3/core.py:428-451."""
        loss_config = L.resolve_loss_config(kwargs["loss_fn"], kwargs.get("loss_implementation", "hip"))
        shared = {"ttt_steps": kwargs["ttt_steps"],
                  "ttt_step_loss_decay": kwargs["ttt_step_loss_decay"],
                  "loss_config": loss_config}
        return dict(shared), dict(shared)
