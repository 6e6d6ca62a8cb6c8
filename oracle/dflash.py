"""DFlash anchored-block draft forward (oracle, CPU).

Functional restatement of ``DFlashDraftModel._backbone_forward`` / ``forward``
(models/dflash/core.py:330-478) with ``Qwen3DFlashAttention`` /
``Qwen3DFlashDecoderLayer`` (models/dflash/model_definitions.py:97-207) and
the anchor helpers of models/dflash/utils.py:6-67.

Pinned by: index-helper known answers and the sortedness of sampled anchors
(tests/unit/models/test_dflash_utils.py:12-59), the targets alignment rule
``targets == roll(full_logits, 1)[:, idx]``
(tests/unit/models/test_dflash_targets.py:37-63), the mask brute force,
dense attention == SDPA; the layer against the HF Qwen3 library blocks wired like
``Qwen3DFlashAttention`` / ``Qwen3DFlashDecoderLayer`` (two layers, one windowed, causal and
non-causal blocks, packed documents, a padded anchor, non-trivial norm gains), against HF
``Qwen3DecoderLayer`` itself where no context key is visible, the whole forward against
the same blocks composed as ``_backbone_forward``, and the aligned loss mask by a
hand-worked literal.  ``select_anchors`` consumes torch's RNG stream the way
the reference does (one ``randperm`` over the valid positions), so the same
seed selects the same anchors.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from . import masks as M
from . import metrics as MT
from .attention import dense_attention
from .eagle3 import DraftShape, apply_rope, rms_norm, rope_tables, swiglu_mlp


def base_indices_for_anchored_blocks(anchor_positions, block_size: int):
    """[a, a+1, .., a+bs-1] for every anchor, flattened; dflash/utils.py:6-18."""
    a = anchor_positions.to(torch.long).reshape(-1)
    return (a[:, None] + torch.arange(block_size, dtype=torch.long)[None, :]).reshape(-1)


def select_anchors(loss_mask, num_anchors: int, block_size: int, generator=None):
    """Up to ``num_anchors`` random positions with loss_mask set, excluding the
    last ``block_size`` positions, ascending; the rest padded with position 0
    and flagged invalid; dflash/utils.py:21-67."""
    if loss_mask.ndim != 2:
        raise ValueError(f"Expected [B, T], got {tuple(loss_mask.shape)}")
    if block_size <= 0:
        raise ValueError(f"Expected block size > 0, got {block_size}")
    ok = loss_mask.bool().clone()
    ok[:, -block_size:] = False
    candidates = torch.nonzero(ok[0]).reshape(-1)
    anchors = torch.zeros(num_anchors, dtype=torch.long)
    valid = torch.zeros(num_anchors, dtype=torch.bool)
    k = min(num_anchors, candidates.numel())
    perm = torch.randperm(candidates.numel(), generator=generator)
    anchors[:k] = candidates[perm[:k]].sort().values
    valid[:k] = True
    return anchors, valid


def dflash_targets(w, shape, verifier_last_hidden_states, block_indices,
                   sample_from_anchor: bool = False):
    """Verifier logits for every mask-token slot: the slot at base position i is
    trained on the verifier's output at i-1 (wrapping); core.py:389-406."""
    t = verifier_last_hidden_states.shape[1]
    idx = block_indices if sample_from_anchor else (block_indices - 1) % t
    x = rms_norm(verifier_last_hidden_states[:, idx], w["verifier_norm.weight"],
                 shape.rms_norm_eps)
    return F.linear(x, w["verifier_lm_head.weight"])


def _dflash_layer(noise, ctx, w, idx, shape, cos, sin, mask):
    p = f"layers.{idx}."
    hq, hkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    ql, tl = noise.shape[1], ctx.shape[1]
    x = rms_norm(noise, w[p + "input_layernorm.weight"], shape.rms_norm_eps)
    a = p + "self_attn."
    q = F.linear(x, w[a + "q_proj.weight"]).view(1, ql, hq, d)
    q = rms_norm(q, w[a + "q_norm.weight"], shape.rms_norm_eps).transpose(1, 2)
    k = torch.cat([F.linear(ctx, w[a + "k_proj.weight"]),
                   F.linear(x, w[a + "k_proj.weight"])], dim=1).view(1, tl + ql, hkv, d)
    v = torch.cat([F.linear(ctx, w[a + "v_proj.weight"]),
                   F.linear(x, w[a + "v_proj.weight"])], dim=1).view(1, tl + ql, hkv, d)
    k = rms_norm(k, w[a + "k_norm.weight"], shape.rms_norm_eps).transpose(1, 2)
    v = v.transpose(1, 2)
    q = apply_rope(q, cos[:, -ql:], sin[:, -ql:])
    k = apply_rope(k, cos, sin)
    o = dense_attention(q, k, v, mask, d**-0.5).reshape(1, ql, hq * d)
    y = noise + F.linear(o, w[a + "o_proj.weight"])
    z = rms_norm(y, w[p + "post_attention_layernorm.weight"], shape.rms_norm_eps)
    return y + swiglu_mlp(z, w, p + "mlp.")


def dflash_forward(w, shape: DraftShape, hidden_states, input_ids, loss_mask,
                   verifier_last_hidden_states, document_ids, position_ids=None,
                   block_size: int = 8, mask_token_id: int = 0, loss_config=None,
                   gamma: float = 4.0, max_anchors: int = 512,
                   per_position_loss_weight: str = "fixed-exp-decay",
                   dpace_alpha: float = 0.5, sliding_window_non_causal: bool = False,
                   sample_from_anchor: bool = False, anchors=None, generator=None,
                   return_logits: bool = False):
    """-> (None, loss, metrics); core.py:330-478.  ``anchors=(positions, valid)``
    overrides the random selection (for tests that share anchors with the HIP
    path)."""
    t = hidden_states.shape[1]
    dtype = hidden_states.dtype
    if position_ids is None:
        position_ids = torch.arange(t, dtype=torch.long).unsqueeze(0)
    if anchors is None:
        anchors = select_anchors(loss_mask, max_anchors, block_size, generator)
    anchor_pos, anchor_valid = anchors
    n_q = anchor_pos.numel() * block_size
    doc = document_ids.reshape(-1)

    ids = torch.full((1, n_q), mask_token_id, dtype=torch.long)
    ids[:, ::block_size] = input_ids[:, anchor_pos]
    noise = F.embedding(ids, w["embed_tokens.weight"])
    ctx = rms_norm(F.linear(hidden_states, w["fc.weight"]), w["hidden_norm.weight"],
                   shape.rms_norm_eps)
    block_pos = base_indices_for_anchored_blocks(position_ids[0, anchor_pos], block_size)
    all_pos = torch.cat([position_ids, block_pos.unsqueeze(0)], dim=1)
    cos, sin = rope_tables(all_pos, shape.head_dim, shape.rope_theta, dtype, shape.rope_scaling)
    block_idx = base_indices_for_anchored_blocks(anchor_pos, block_size)
    with torch.no_grad():
        targets = dflash_targets(w, shape, verifier_last_hidden_states, block_idx,
                                 sample_from_anchor)
    for li in range(shape.num_hidden_layers):
        win = shape.sliding_window if li in shape.sliding_layers else None
        mask = M.dflash_mask_dense(doc, t, anchor_pos, block_size, win,
                                   sliding_window_non_causal)
        noise = _dflash_layer(noise, ctx, w, li, shape, cos, sin, mask)
    logits = F.linear(rms_norm(noise, w["norm.weight"], shape.rms_norm_eps),
                      w["lm_head.weight"])
    aligned = loss_mask.clone()[:, block_idx]
    aligned = aligned * anchor_valid.repeat_interleave(block_size).unsqueeze(0).to(aligned.dtype)
    if not sample_from_anchor:
        aligned[:, ::block_size] = 0
    loss, metrics = MT.dflash_compute_metrics(
        logits, targets, aligned, block_size, gamma, loss_config,
        per_position_loss_weight, dpace_alpha, sample_from_anchor,
    )
    if return_logits:
        return None, loss, metrics, logits
    return None, loss, metrics


def random_weights(shape: DraftShape, seed: int = 0, dtype=torch.float32, std: float = 0.02):
    """Seeded weights keyed by the DFlash state-dict names (core.py:36-120)."""
    g = torch.Generator().manual_seed(seed)
    h, hq, hkv, d = (shape.hidden_size, shape.num_attention_heads,
                     shape.num_key_value_heads, shape.head_dim)
    f = shape.intermediate_size

    def rnd(*s):
        return (torch.randn(*s, generator=g) * std).to(dtype)

    w = {
        "embed_tokens.weight": rnd(shape.vocab_size, h),
        "fc.weight": rnd(h, shape.num_aux * h),
        "lm_head.weight": rnd(shape.draft_vocab_size, h),
        "verifier_lm_head.weight": rnd(shape.draft_vocab_size, h),
        "norm.weight": torch.ones(h, dtype=dtype),
        "hidden_norm.weight": torch.ones(h, dtype=dtype),
        "verifier_norm.weight": torch.ones(h, dtype=dtype),
    }
    for li in range(shape.num_hidden_layers):
        p = f"layers.{li}."
        w[p + "self_attn.q_proj.weight"] = rnd(hq * d, h)
        w[p + "self_attn.k_proj.weight"] = rnd(hkv * d, h)
        w[p + "self_attn.v_proj.weight"] = rnd(hkv * d, h)
        w[p + "self_attn.o_proj.weight"] = rnd(h, hq * d)
        w[p + "self_attn.q_norm.weight"] = torch.ones(d, dtype=dtype)
        w[p + "self_attn.k_norm.weight"] = torch.ones(d, dtype=dtype)
        w[p + "mlp.gate_proj.weight"] = rnd(f, h)
        w[p + "mlp.up_proj.weight"] = rnd(f, h)
        w[p + "mlp.down_proj.weight"] = rnd(h, f)
        w[p + "input_layernorm.weight"] = torch.ones(h, dtype=dtype)
        w[p + "post_attention_layernorm.weight"] = torch.ones(h, dtype=dtype)
    return w
