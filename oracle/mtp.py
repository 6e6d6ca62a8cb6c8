"""CPU restatement of the MTP (multi-token prediction) training forward.

TEST INFRASTRUCTURE ONLY: nothing under ``speculators_amd`` may import this.

Follows, in plain PyTorch on the CPU:
  * ``compute_step_weights``            models/mtp/core.py:29-38
  * ``MTPDraftModel.forward``           models/mtp/core.py:114-231
  * ``MTPLayerMixin.forward``           models/mtp/model_definitions.py:95-116
  * the Qwen3 decoder layer it wraps    transformers ``modeling_qwen3.py``
    (pre-norm attention with per-head q/k RMSNorm, SwiGLU MLP)
  * the hybrid flavours' full-attention decoder layer (models/mtp/model_definitions.py:159-205
    wrap ``Qwen3NextDecoderLayer`` / ``Qwen3_5DecoderLayer`` / ``Qwen3_5MoeDecoderLayer`` at the
    last ``full_attention`` index): transformers ``modeling_qwen3_next.py`` -- RMSNorm with gain
    ``1 + w`` and one rounding, q_proj twice as wide with a sigmoid output gate, rotary embedding
    on the first ``partial_rotary_factor`` of each head, and the sparse MoE block (soft-max
    router, top-k, optional renormalisation, experts with a merged gate/up weight, a shared
    expert behind a sigmoid gate)
  * the packed-sequence causal mask     transformers ``masking_utils.py``
    ``find_packed_sequence_indices`` (called through ``create_causal_mask`` with
    ``attention_mask=None`` at models/mtp/core.py:180-186)

Pinned by: the library's own ``Qwen3DecoderLayer``, ``Qwen3NextDecoderLayer``,
``Qwen3_5DecoderLayer`` and ``Qwen3_5MoeDecoderLayer`` (with their rotary modules) wired like
the mixin, ``create_causal_mask`` of the library itself for the padding-mask form, the
block-diagonal causal matrix of
tests/unit/models/test_mtp_attention.py:17-55 (documents [1, 3, 2]), the loss
properties of tests/unit/models/test_mtp_model.py (all-zero mask -> exactly 0,
zero step weight -> that step's loss 0, short sequences give fewer steps), the
closed form of the step weights, ``F.cross_entropy`` (a library routine) for the
loss, and agreement of the dense attention with ``F.scaled_dot_product_attention``.
Whole-model values on random weights have no golden vector in the reference.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from .attention import dense_attention
from .eagle3 import DraftShape, RotaryState, apply_rope, rms_norm, rope_tables, swiglu_mlp

IGNORE_INDEX = -100


def compute_step_weights(beta: float = 0.6, num_steps: int = 3) -> list[float]:
    """alpha_k = beta^k / sum_j beta^j, k = 0..K-1 (models/mtp/core.py:29-38)."""
    raw = [beta**k for k in range(num_steps)]
    total = sum(raw)
    return [r / total for r in raw]


def packed_sequence_ids(position_ids: torch.Tensor) -> torch.Tensor:
    """``[B, L]`` positions -> ``[B, L]`` sequence index inside each row: a new sequence
    starts wherever the position does not grow by exactly one."""
    first = position_ids[:, :1] - 1
    diff = torch.diff(position_ids, prepend=first, dim=-1)
    return (diff != 1).cumsum(-1)


def packed_causal_mask(position_ids: torch.Tensor) -> torch.Tensor:
    """Dense bool ``[B, L, L]``: query i sees key j iff j <= i and both lie in the same
    packed sequence of the row."""
    seq = packed_sequence_ids(position_ids)
    n = position_ids.shape[1]
    idx = torch.arange(n)
    causal = idx[:, None] >= idx[None, :]
    return causal[None] & (seq[:, :, None] == seq[:, None, :])


def padded_causal_mask(attention_mask: torch.Tensor) -> torch.Tensor:
    """Dense bool ``[B, L, L]`` for a 2-D padding mask ``[B, L]``: query i sees key j iff j <= i
    and ``attention_mask[b, j]`` is non-zero.  With a mask given, ``create_causal_mask`` does not
    look for packed sequences in the positions (transformers ``masking_utils.py``: the detection
    runs only for ``attention_mask is None``), so there is no same-sequence term."""
    n = attention_mask.shape[1]
    idx = torch.arange(n)
    causal = idx[:, None] >= idx[None, :]
    return causal[None] & (attention_mask != 0)[:, None, :]


@dataclass
class HybridShape(DraftShape):
    """Shape of a hybrid-flavour MTP layer (``qwen3_next``, ``qwen3_5_text``,
    ``qwen3_5_moe_text``).  ``num_experts == 0``: dense SwiGLU MLP of ``intermediate_size``."""

    model_type: str = "qwen3_next"
    partial_rotary_factor: float = 0.25
    num_experts: int = 0
    num_experts_per_tok: int = 2
    moe_intermediate_size: int = 0
    shared_expert_intermediate_size: int = 0
    norm_topk_prob: bool = True


def zero_centered_rms_norm(x, weight, eps):
    """``Qwen3NextRMSNorm``: fp32 inside, gain ``1 + w``, one cast at the end."""
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * (1.0 + weight.float())).type_as(x)


def apply_partial_rope(x, cos, sin):
    """x ``[1, heads, T, D]``, tables ``[1, T, R]`` with R <= D: the first R elements of every head
    are rotated (pairs i, i + R/2), the rest passes (``apply_rotary_pos_emb`` of
    ``modeling_qwen3_next.py``)."""
    r = cos.shape[-1]
    rot, rest = x[..., :r], x[..., r:]
    h = r // 2
    rotated = torch.cat([-rot[..., h:], rot[..., :h]], dim=-1)
    return torch.cat([rot * cos.unsqueeze(1) + rotated * sin.unsqueeze(1), rest], dim=-1)


def moe_routing(x2, router_weight, top_k: int, renormalise: bool):
    """``Qwen3NextTopKRouter``: soft-max over all experts in fp32, the ``top_k`` largest
    probabilities, optionally renormalised to sum 1, cast to the dtype of the router logits.
    -> (scores ``[rows, top_k]``, expert ids ``[rows, top_k]``)."""
    logits = F.linear(x2, router_weight)
    probs = F.softmax(logits, dtype=torch.float, dim=-1)
    top, idx = torch.topk(probs, top_k, dim=-1)
    if renormalise:
        top = top / top.sum(dim=-1, keepdim=True)
    return top.to(logits.dtype), idx


def sparse_moe(x, w, prefix, shape: HybridShape, routing: dict | None = None):
    """``Qwen3NextSparseMoeBlock`` on ``[1, L, H]``: every token's ``top_k`` experts (SwiGLU with
    the merged ``gate_up_proj [E, 2I, H]``, ``down_proj [E, H, I]``) weighted by the router scores,
    plus the shared expert scaled by ``sigmoid(shared_expert_gate(x))``.

    ``routing`` (tests of a bf16 implementation, whose top-k may differ from the fp32 one where two
    probabilities nearly tie): ``routing["forced"]``, expert ids ``[L, k]`` to use instead of this
    function's own top-k (the scores are still this function's probabilities at those experts);
    the function's own choice, all probabilities and the router logits are left in
    ``routing["own"]`` / ``routing["probs"]`` / ``routing["logits"]``."""
    x2 = x.reshape(-1, x.shape[-1])
    scores, idx = moe_routing(x2, w[prefix + "gate.weight"], shape.num_experts_per_tok,
                              shape.norm_topk_prob)
    if routing is not None:
        logits = F.linear(x2, w[prefix + "gate.weight"])
        probs = F.softmax(logits, dtype=torch.float, dim=-1)
        routing["own"], routing["probs"], routing["logits"] = idx, probs.detach(), logits.detach()
        if routing.get("forced") is not None:
            idx = routing["forced"]
            scores = probs.gather(1, idx)
            if shape.norm_topk_prob:
                scores = scores / scores.sum(dim=-1, keepdim=True)
            scores = scores.to(logits.dtype)
    out = torch.zeros_like(x2)
    # (one unbind per stack: its backward stacks the experts' gradients once, where indexing the
    # stack per expert would materialise a stack-sized gradient for every expert)
    gate_up = w[prefix + "experts.gate_up_proj"].unbind(0)
    down = w[prefix + "experts.down_proj"].unbind(0)
    for e in range(shape.num_experts):
        rows, slot = torch.where(idx == e)
        if rows.numel() == 0:
            continue
        g, u = F.linear(x2[rows], gate_up[e]).chunk(2, dim=-1)
        y = F.linear(F.silu(g) * u, down[e]) * scores[rows, slot, None]
        out.index_add_(0, rows, y.to(out.dtype))
    shared = swiglu_mlp(x2, w, prefix + "shared_expert.")
    shared = torch.sigmoid(F.linear(x2, w[prefix + "shared_expert_gate.weight"])) * shared
    return (out + shared).reshape(x.shape)


def _hybrid_layer(x, w, p, shape: HybridShape, cos, sin, mask, attn, routing=None):
    """One row ``[1, L, H]`` through the full-attention decoder layer of the hybrid flavours."""
    n = x.shape[1]
    hq, hkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    eps = shape.rms_norm_eps
    a = p + "self_attn."
    y = zero_centered_rms_norm(x, w[p + "input_layernorm.weight"], eps)
    q, gate = torch.chunk(F.linear(y, w[a + "q_proj.weight"]).view(1, n, hq, 2 * d), 2, dim=-1)
    gate = gate.reshape(1, n, hq * d)
    q = zero_centered_rms_norm(q, w[a + "q_norm.weight"], eps).transpose(1, 2)
    k = zero_centered_rms_norm(F.linear(y, w[a + "k_proj.weight"]).view(1, n, hkv, d),
                               w[a + "k_norm.weight"], eps).transpose(1, 2)
    v = F.linear(y, w[a + "v_proj.weight"]).view(1, n, hkv, d).transpose(1, 2)
    q, k = apply_partial_rope(q, cos, sin), apply_partial_rope(k, cos, sin)
    if attn == "sdpa":
        g = hq // hkv
        o = F.scaled_dot_product_attention(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1),
                                           attn_mask=mask[None, None], scale=d**-0.5)
        o = o.transpose(1, 2).contiguous()
    else:
        o = dense_attention(q, k, v, mask, d**-0.5)
    o = o.reshape(1, n, hq * d) * torch.sigmoid(gate)
    x = x + F.linear(o, w[a + "o_proj.weight"])
    z = zero_centered_rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    if shape.num_experts > 0:
        return x + sparse_moe(z, w, p + "mlp.", shape, routing)
    return x + swiglu_mlp(z, w, p + "mlp.")


def rotary_dim(shape: DraftShape) -> int:
    """Rotated elements per head: ``int(head_dim * partial_rotary_factor)``
    (``compute_default_rope_parameters`` of the hybrid flavours' rotary modules)."""
    return int(shape.head_dim * getattr(shape, "partial_rotary_factor", 1.0))


def _qwen3_layer(x, w, p, shape: DraftShape, cos, sin, mask, attn):
    """One row ``[1, L, H]`` through the Qwen3 decoder layer."""
    n = x.shape[1]
    hq, hkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    a = p + "self_attn."
    y = rms_norm(x, w[p + "input_layernorm.weight"], shape.rms_norm_eps)
    q = rms_norm(F.linear(y, w[a + "q_proj.weight"]).view(1, n, hq, d), w[a + "q_norm.weight"],
                 shape.rms_norm_eps).transpose(1, 2)
    k = rms_norm(F.linear(y, w[a + "k_proj.weight"]).view(1, n, hkv, d), w[a + "k_norm.weight"],
                 shape.rms_norm_eps).transpose(1, 2)
    v = F.linear(y, w[a + "v_proj.weight"]).view(1, n, hkv, d).transpose(1, 2)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    if attn == "sdpa":
        g = hq // hkv
        o = F.scaled_dot_product_attention(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1),
                                           attn_mask=mask[None, None], scale=d**-0.5)
        o = o.transpose(1, 2).contiguous()
    else:
        o = dense_attention(q, k, v, mask, d**-0.5)
    x = x + F.linear(o.reshape(1, n, hq * d), w[a + "o_proj.weight"])
    z = rms_norm(x, w[p + "post_attention_layernorm.weight"], shape.rms_norm_eps)
    return x + swiglu_mlp(z, w, p + "mlp.")


def mtp_layer(hidden, embeds, w, shape: DraftShape, cos, sin, mask, attn="dense", routing=None):
    """models/mtp/model_definitions.py:95-116 on one row."""
    p = "mtp_layers.0."
    hybrid = isinstance(shape, HybridShape)
    norm = zero_centered_rms_norm if hybrid else rms_norm
    hn = norm(hidden, w[p + "hidden_layernorm.weight"], shape.rms_norm_eps)
    en = norm(embeds, w[p + "token_layernorm.weight"], shape.rms_norm_eps)
    proj = F.linear(torch.cat([en, hn], dim=-1), w[p + "input_proj.weight"])
    if hybrid:
        out = _hybrid_layer(proj, w, p, shape, cos, sin, mask, attn, routing)
    else:
        out = _qwen3_layer(proj, w, p, shape, cos, sin, mask, attn)
    return norm(out, w[p + "final_layernorm.weight"], shape.rms_norm_eps)


def mtp_forward(w, shape: DraftShape, input_ids, hidden_states, position_ids=None, loss_mask=None,
                step_weights=None, num_steps: int = 3, attn: str = "dense", attention_mask=None,
                routing=None):
    """``(logits_list, loss, metrics)`` of models/mtp/core.py:114-231.  ``attention_mask``
    (``[B, L]`` padding mask) replaces the packed-sequence mask as in core.py:180-186.
    ``routing``: a list with one dict per (step, batch row), in that order, handed to
    ``sparse_moe`` (see there)."""
    input_ids = input_ids.long()
    b, n = input_ids.shape
    if step_weights is not None and len(step_weights) != num_steps:
        raise ValueError(f"step_weights has {len(step_weights)} entries but num_speculative_steps="
                         f"{num_steps}; expected exactly {num_steps} weights.")
    if position_ids is None:
        position_ids = torch.arange(n).unsqueeze(0).expand(b, -1)
    logits_list = []
    total = torch.tensor(0.0)
    metrics = {}
    steps = min(num_steps, max(0, n - 2))
    valid = n - steps - 1
    if valid <= 0 or steps == 0:
        metrics["loss_sum"] = total.clone()
        metrics["loss_total"] = torch.tensor(1.0)
        return logits_list, total, metrics
    pos = position_ids[:, :valid]
    masks = packed_causal_mask(pos) if attention_mask is None else \
        padded_causal_mask(attention_mask[:, :valid])
    current = hidden_states
    rotary = RotaryState(rotary_dim(shape), shape.rope_theta, shape.rope_scaling)
    for step in range(steps):
        hid = current[:, :valid]
        emb = F.embedding(input_ids[:, step + 1:step + 1 + valid], w["embed_tokens.weight"])
        rows = []
        # the rotary module is called once per step with the positions of the whole batch
        # (models/mtp/core.py:196): a length-dependent rope type sees their maximum
        inv = rotary.inv_freq(pos)
        for r in range(b):
            cos, sin = rope_tables(pos[r], rotary_dim(shape), shape.rope_theta, hid.dtype,
                                   shape.rope_scaling, inv_freq=inv)
            rows.append(mtp_layer(hid[r:r + 1], emb[r:r + 1].to(hid.dtype), w, shape, cos, sin,
                                  masks[r], attn, None if routing is None else routing[step * b + r]))
        out = torch.cat(rows, dim=0)
        logits = F.linear(out, w["lm_head.weight"])
        logits_list.append(logits)
        tgt = input_ids[:, step + 2:step + 2 + valid]
        if loss_mask is not None:
            tgt = tgt.clone()
            tgt[loss_mask[:, step + 2:step + 2 + valid] == 0] = IGNORE_INDEX
        weight = step_weights[step] if step_weights is not None else 1.0
        unreduced = F.cross_entropy(logits.permute(0, 2, 1).float(), tgt, ignore_index=IGNORE_INDEX,
                                    reduction="none")
        count = (tgt != IGNORE_INDEX).sum()
        step_loss = weight * unreduced.sum() / count.clamp(min=1)
        total = total + step_loss
        metrics[f"loss_step_{step}"] = step_loss.detach().clone()
        current = out
    metrics["loss_sum"] = total.detach().clone()
    metrics["loss_total"] = torch.tensor(1.0)
    return logits_list, total, metrics


def random_weights(shape: DraftShape, seed: int = 0, dtype=torch.float32, std: float = 0.02):
    """Seeded weights keyed by the MTP state-dict names (models/mtp/core.py:41-96,
    models/mtp/model_definitions.py:85-93).  Norm weights are 1 + noise so that a missing
    or swapped norm shows."""
    g = torch.Generator().manual_seed(seed)
    h, hq, hkv, d = (shape.hidden_size, shape.num_attention_heads,
                     shape.num_key_value_heads, shape.head_dim)
    f = shape.intermediate_size

    def rnd(*s):
        return (torch.randn(*s, generator=g) * std).to(dtype)

    def nrm(k):
        return (1.0 + 0.1 * torch.randn(k, generator=g)).to(dtype)

    p = "mtp_layers.0."
    if isinstance(shape, HybridShape):
        def zc(k):  # gains are 1 + w: w itself is noise around zero
            return (0.1 * torch.randn(k, generator=g)).to(dtype)

        out = {
            "embed_tokens.weight": (torch.randn(shape.vocab_size, h, generator=g)).to(dtype),
            "lm_head.weight": rnd(shape.vocab_size, h),
            p + "hidden_layernorm.weight": zc(h),
            p + "token_layernorm.weight": zc(h),
            p + "input_proj.weight": rnd(h, 2 * h),
            p + "final_layernorm.weight": zc(h),
            p + "input_layernorm.weight": zc(h),
            p + "post_attention_layernorm.weight": zc(h),
            p + "self_attn.q_proj.weight": rnd(hq * d * 2, h),
            p + "self_attn.k_proj.weight": rnd(hkv * d, h),
            p + "self_attn.v_proj.weight": rnd(hkv * d, h),
            p + "self_attn.o_proj.weight": rnd(h, hq * d),
            p + "self_attn.q_norm.weight": zc(d),
            p + "self_attn.k_norm.weight": zc(d),
        }
        if shape.num_experts > 0:
            e, fi, fs = shape.num_experts, shape.moe_intermediate_size, shape.shared_expert_intermediate_size
            out.update({
                p + "mlp.gate.weight": (torch.randn(e, h, generator=g) * 10 * std).to(dtype),
                p + "mlp.experts.gate_up_proj": rnd(e, 2 * fi, h),
                p + "mlp.experts.down_proj": rnd(e, h, fi),
                p + "mlp.shared_expert.gate_proj.weight": rnd(fs, h),
                p + "mlp.shared_expert.up_proj.weight": rnd(fs, h),
                p + "mlp.shared_expert.down_proj.weight": rnd(h, fs),
                p + "mlp.shared_expert_gate.weight": rnd(1, h),
            })
        else:
            out.update({
                p + "mlp.gate_proj.weight": rnd(f, h),
                p + "mlp.up_proj.weight": rnd(f, h),
                p + "mlp.down_proj.weight": rnd(h, f),
            })
        return out
    return {
        "embed_tokens.weight": (torch.randn(shape.vocab_size, h, generator=g)).to(dtype),
        "lm_head.weight": rnd(shape.vocab_size, h),
        p + "hidden_layernorm.weight": nrm(h),
        p + "token_layernorm.weight": nrm(h),
        p + "input_proj.weight": rnd(h, 2 * h),
        p + "final_layernorm.weight": nrm(h),
        p + "input_layernorm.weight": nrm(h),
        p + "post_attention_layernorm.weight": nrm(h),
        p + "self_attn.q_proj.weight": rnd(hq * d, h),
        p + "self_attn.k_proj.weight": rnd(hkv * d, h),
        p + "self_attn.v_proj.weight": rnd(hkv * d, h),
        p + "self_attn.o_proj.weight": rnd(h, hq * d),
        p + "self_attn.q_norm.weight": nrm(d),
        p + "self_attn.k_norm.weight": nrm(d),
        p + "mlp.gate_proj.weight": rnd(f, h),
        p + "mlp.up_proj.weight": rnd(f, h),
        p + "mlp.down_proj.weight": rnd(h, f),
    }
