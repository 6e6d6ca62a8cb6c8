"""EAGLE3 draft forward with the TTT loop (oracle, CPU).

A functional restatement of ``Eagle3DraftModel.forward``
(models/eagle3/core.py:192-365) over a plain ``{state_dict_name: tensor}``
mapping, with the first-layer changes of ``Eagle3FirstLayerMixin``
(models/eagle3/model_definitions.py:54-110) and the closed forms of the HF
Llama blocks it is built from (RMSNorm fp32-inside, half-split RoPE computed in
fp32 and cast, SwiGLU MLP, K/V cache that grows by T keys per step).

Pinned by (tests/test_oracle_eagle3.py): ``first_layer`` == the HF ``LlamaAttention`` /
``LlamaMLP`` / ``LlamaRMSNorm`` / ``LlamaRotaryEmbedding`` modules patched the way the
reference patches them, and with ``qk_norm`` == ``Qwen3Attention`` (q/k RMSNorm before the
rotation) wired the same way; ``later_layer`` == the library's whole ``LlamaDecoderLayer`` /
``Qwen3DecoderLayer`` over three TTT steps on one ``DynamicCache`` (output and every
gradient); agreement of the dense-mask attention with
``F.scaled_dot_product_attention``, the reference's mask / loss / metric golden
vectors through the modules it calls, and shift / alignment invariants
(step-k rows only see targets k positions later).  The whole-model loss on
random weights has no golden vector anywhere in the reference (its tests
assert finiteness and cross-backend agreement only).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import math

import torch
import torch.nn.functional as F

from . import masks as M
from . import metrics as MT
from .attention import dense_attention


@dataclass
class DraftShape:
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
    norm_before_residual: bool = False
    norm_before_fc: bool = False
    fc_norm: bool = False
    norm_output: bool = False
    qk_norm: bool = False  # Qwen3-style per-head RMSNorm of q and k
    sliding_window: int | None = None
    sliding_layers: tuple = field(default_factory=tuple)  # indices of windowed layers
    rope_scaling: dict | None = None  # HF rope parameters: {"rope_type": "llama3" | "linear", ...}


def rms_norm(x, weight, eps):
    """fp32 inside, result cast back then scaled (HF LlamaRMSNorm)."""
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return weight * xf.to(x.dtype)


def rope_kind(scaling=None) -> str:
    return (scaling or {}).get("rope_type", (scaling or {}).get("type", "default"))


def rope_inv_freq(head_dim, theta, scaling=None, seq_len=None):
    """fp32 inverse frequencies of the rotary embedding.  ``scaling`` follows the HF rope
    parameters the draft inherits from its verifier (models/eagle3/core.py:105-112 keeps them
    in the layer config; Llama-3.1 ships ``rope_type = "llama3"``):
      linear:   every frequency divided by ``factor``;
      yarn:     see ``_yarn_inv_freq``; its table factor is ``rope_table_scale``;
      llama3:   wavelengths above ``L / low_freq_factor`` (L = original_max_position_embeddings)
                are divided by ``factor``, those below ``L / high_freq_factor`` kept, and the band
                between is blended linearly in ``L / wavelength``;
      dynamic:  the base grows with the running length ``seq_len`` once that passes
                ``max_position_embeddings`` (a key of ``scaling`` here; the library keeps it on the
                model config): ``theta * (factor * n / L - (factor - 1)) ** (d / (d - 2))``;
      longrope: per-frequency divisors, ``long_factor`` when ``seq_len`` is beyond
                ``original_max_position_embeddings``, ``short_factor`` otherwise; table factor
                ``sqrt(1 + ln(factor) / ln(L_original))``.
    ``seq_len`` only matters to the last two; which length a rotary module runs with from call to call
    is ``RotaryState``.  Pinned against ``transformers.modeling_rope_utils.ROPE_INIT_FUNCTIONS``."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    kind = rope_kind(scaling)
    if kind == "default":
        return inv
    if kind == "longrope":
        long = seq_len is not None and int(seq_len) > int(scaling["original_max_position_embeddings"])
        ext = torch.tensor(scaling["long_factor" if long else "short_factor"], dtype=torch.float32)
        shape = torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim
        return 1.0 / (ext * theta ** shape)
    factor = float(scaling["factor"])
    if kind == "linear":
        return inv / factor
    if kind == "yarn":
        return _yarn_inv_freq(inv, head_dim, theta, scaling)
    if kind == "dynamic":
        ctx = int(scaling["max_position_embeddings"])
        if seq_len is None:
            base = theta * ((factor * ctx / ctx) - (factor - 1)) ** (head_dim / (head_dim - 2))
        else:
            # (the library's update hands the length over as an int64 tensor: the base is an fp32 value)
            n = torch.maximum(torch.as_tensor(int(seq_len), dtype=torch.int64), torch.tensor(ctx, dtype=torch.int64))
            base = theta * ((factor * n / ctx) - (factor - 1)) ** (head_dim / (head_dim - 2))
        return 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    if kind != "llama3":
        raise NotImplementedError(f"rope_type '{kind}'")
    lo, hi = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
    ctx = float(scaling["original_max_position_embeddings"])
    wavelen = 2 * math.pi / inv
    out = torch.where(wavelen > ctx / lo, inv / factor, inv)
    blend = (ctx / wavelen - lo) / (hi - lo)
    mid = (1 - blend) * out / factor + blend * out
    band = ~(wavelen < ctx / hi) & ~(wavelen > ctx / lo)
    return torch.where(band, mid, out)


def _yarn_inv_freq(inv, dim, theta, scaling):
    """YaRN frequencies (transformers ``_compute_yarn_parameters``): a linear ramp over the
    frequency index between the index whose wavelength fits the original context ``beta_fast``
    times and the one that fits it ``beta_slow`` times; below the ramp the frequency is kept,
    above it divided by ``factor``."""
    factor = float(scaling["factor"])
    ctx = float(scaling["original_max_position_embeddings"])
    fast, slow = scaling.get("beta_fast") or 32, scaling.get("beta_slow") or 1

    def index_of(rotations):
        return dim * math.log(ctx / (rotations * 2 * math.pi)) / (2 * math.log(theta))

    lo, hi = index_of(fast), index_of(slow)
    if scaling.get("truncate", True):
        lo, hi = math.floor(lo), math.ceil(hi)
    lo, hi = max(lo, 0), min(hi, dim - 1)
    if lo == hi:
        hi += 0.001
    ramp = torch.clamp((torch.arange(dim // 2, dtype=torch.float32) - lo) / (hi - lo), 0, 1)
    keep = 1 - ramp
    freqs = theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim)
    return (1.0 / (factor * freqs)) * (1 - keep) + (1.0 / freqs) * keep


def rope_table_scale(scaling=None) -> float:
    """The factor on both tables (``attention_scaling`` of the HF rotary modules): 1 except for
    yarn, where it is ``attention_factor`` if given, else ``0.1 ln(factor) + 1`` (with ``mscale`` /
    ``mscale_all_dim``: the ratio of the two such terms), and longrope, where it is
    ``attention_factor`` if given, else ``sqrt(1 + ln(factor) / ln(L_original))`` for a factor above 1
    (``factor`` defaults to ``max_position_embeddings / L_original``)."""
    kind = rope_kind(scaling)
    if kind == "longrope":
        if scaling.get("attention_factor") is not None:
            return float(scaling["attention_factor"])
        ctx0 = scaling["original_max_position_embeddings"]
        factor = scaling.get("factor")
        if factor is None:
            factor = scaling["max_position_embeddings"] / ctx0
        return 1.0 if factor <= 1.0 else math.sqrt(1 + math.log(factor) / math.log(ctx0))
    if kind != "yarn":
        return 1.0
    if scaling.get("attention_factor") is not None:
        return float(scaling["attention_factor"])
    factor = float(scaling["factor"])

    def term(m=1.0):
        return 1.0 if factor <= 1 else 0.1 * m * math.log(factor) + 1.0

    if scaling.get("mscale") and scaling.get("mscale_all_dim"):
        return term(scaling["mscale"]) / term(scaling["mscale_all_dim"])
    return term()


class RotaryState:
    """The frequencies one rotary module runs with from call to call (``dynamic_rope_update`` of
    transformers' ``modeling_rope_utils.py``, which wraps the forward of every HF rotary module).
    With ``n = max(position_ids) + 1`` of the call:
      longrope: the long divisors if ``n > original_max_position_embeddings``, else the short ones;
      dynamic:  recomputed for ``n`` whenever ``n`` exceeds every length seen so far (starting from
                ``max_position_embeddings``), kept otherwise -- until a call with
                ``n < max_position_embeddings`` puts the original frequencies back;
      every other type: fixed."""

    def __init__(self, head_dim, theta, scaling=None):
        self.head_dim, self.theta, self.scaling = head_dim, theta, scaling
        self.kind = rope_kind(scaling)
        self.original = rope_inv_freq(head_dim, theta, scaling)
        self.current = self.original
        if self.kind == "dynamic":
            self.ctx = int(scaling["max_position_embeddings"])
            self.seen = self.ctx

    def inv_freq(self, position_ids):
        if self.kind == "longrope":
            n = int(position_ids.max()) + 1
            if n > int(self.scaling["original_max_position_embeddings"]):
                return rope_inv_freq(self.head_dim, self.theta, self.scaling,
                                     int(self.scaling["original_max_position_embeddings"]) + 1)
            return self.original
        if self.kind == "dynamic":
            n = int(position_ids.max()) + 1
            if n > self.seen:
                self.current = rope_inv_freq(self.head_dim, self.theta, self.scaling, n)
                self.seen = n
            if n < self.ctx and self.seen > self.ctx:
                self.current, self.seen = self.original, self.ctx
            return self.current
        return self.original


def rope_tables(position_ids, head_dim, theta, dtype, scaling=None, state=None, inv_freq=None):
    """cos/sin ``[1, T, D]``: fp32 outer product, duplicated halves, table scale, cast.  ``state``: the
    ``RotaryState`` of the module when several calls follow each other (a fresh one otherwise);
    ``inv_freq``: the frequencies themselves, where the caller has asked the state already."""
    if inv_freq is None:
        if state is None:
            state = RotaryState(head_dim, theta, scaling)
        inv_freq = state.inv_freq(position_ids)
    inv = inv_freq
    ang = position_ids.reshape(1, -1, 1).float() * inv.reshape(1, 1, -1)
    ang = torch.cat([ang, ang], dim=-1)
    scale = rope_table_scale(scaling)
    return (ang.cos() * scale).to(dtype), (ang.sin() * scale).to(dtype)


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat([-x[..., h:], x[..., :h]], dim=-1)


def apply_rope(x, cos, sin):
    """x ``[1, heads, T, D]``, tables ``[1, T, D]``."""
    return x * cos.unsqueeze(1) + rotate_half(x) * sin.unsqueeze(1)


def swiglu_mlp(x, w, prefix):
    g = F.linear(x, w[prefix + "gate_proj.weight"])
    u = F.linear(x, w[prefix + "up_proj.weight"])
    return F.linear(F.silu(g) * u, w[prefix + "down_proj.weight"])


def _attention_block(x, w, prefix, shape, cos, sin, cache, mask, attn):
    t = x.shape[1]
    hq, hkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    q = F.linear(x, w[prefix + "q_proj.weight"]).view(1, t, hq, d)
    k = F.linear(x, w[prefix + "k_proj.weight"]).view(1, t, hkv, d)
    v = F.linear(x, w[prefix + "v_proj.weight"]).view(1, t, hkv, d)
    if shape.qk_norm:
        q = rms_norm(q, w[prefix + "q_norm.weight"], shape.rms_norm_eps)
        k = rms_norm(k, w[prefix + "k_norm.weight"], shape.rms_norm_eps)
    q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    cache["k"] = k if cache.get("k") is None else torch.cat([cache["k"], k], dim=2)
    cache["v"] = v if cache.get("v") is None else torch.cat([cache["v"], v], dim=2)
    if attn == "sdpa":
        group = hq // hkv
        o = F.scaled_dot_product_attention(
            q, cache["k"].repeat_interleave(group, 1), cache["v"].repeat_interleave(group, 1),
            attn_mask=mask[None, None], scale=d**-0.5,
        ).transpose(1, 2).contiguous()
    else:
        o = dense_attention(q, cache["k"], cache["v"], mask, d**-0.5)
    return F.linear(o.reshape(1, t, hq * d), w[prefix + "o_proj.weight"])


def first_layer(x2h, w, shape, cos, sin, cache, mask, attn="dense"):
    """models/eagle3/model_definitions.py:54-110 on ``[1, T, 2H]`` input."""
    p = "layers.0."
    h = shape.hidden_size
    embeds, hidden = x2h[..., :h], x2h[..., h:]
    residual = hidden
    embeds = rms_norm(embeds, w[p + "input_layernorm.weight"], shape.rms_norm_eps)
    hidden = rms_norm(hidden, w[p + "hidden_norm.weight"], shape.rms_norm_eps)
    if shape.norm_before_residual:
        residual = hidden
    a = _attention_block(torch.cat([embeds, hidden], -1), w, p + "self_attn.", shape,
                         cos, sin, cache, mask, attn)
    y = residual + a
    z = rms_norm(y, w[p + "post_attention_layernorm.weight"], shape.rms_norm_eps)
    return y + swiglu_mlp(z, w, p + "mlp.")


def later_layer(x, w, idx, shape, cos, sin, cache, mask, attn="dense"):
    """A standard pre-norm decoder layer (HF LlamaDecoderLayer.forward)."""
    p = f"layers.{idx}."
    a = _attention_block(rms_norm(x, w[p + "input_layernorm.weight"], shape.rms_norm_eps),
                         w, p + "self_attn.", shape, cos, sin, cache, mask, attn)
    y = x + a
    z = rms_norm(y, w[p + "post_attention_layernorm.weight"], shape.rms_norm_eps)
    return y + swiglu_mlp(z, w, p + "mlp.")


def eagle3_forward(w, shape: DraftShape, hidden_states, input_ids, document_ids,
                   loss_mask=None, position_ids=None, verifier_last_hidden_states=None,
                   ttt_steps: int = 3, ttt_step_loss_decay: float = 1.0,
                   loss_config=None, attn: str = "dense", return_logits: bool = False,
                   verifier_logits=None, d2t=None, rotary_state=None):
    """-> (draft_tokens, loss, metrics[, logits per step]).
    models/eagle3/core.py:192-365.  ``verifier_logits`` (``[1, T, Vt]``, with the ``d2t`` offset
    table) stands in for ``verifier_last_hidden_states``: the targets are then those logits at
    the draft ids ``i + d2t[i]`` -- what the row-sliced verifier head computes, by the identity
    ``(W h)[t2d] == W[t2d] h`` (model.py:161-169; pinned in tests/test_oracle_metrics.py)."""
    t = hidden_states.shape[1]
    dtype = hidden_states.dtype
    if position_ids is None:
        position_ids = 1 + torch.arange(t, dtype=torch.long).unsqueeze(0)
    doc = document_ids.reshape(-1)

    def mask_for(layer_idx, step):
        win = shape.sliding_window if layer_idx in shape.sliding_layers else None
        return M.ttt_mask_dense(doc, t, step, win)

    x = hidden_states
    if shape.norm_before_fc:
        x = rms_norm(x, w["input_norm.weight"], shape.rms_norm_eps)
    if shape.fc_norm:
        chunks = x.chunk(shape.num_aux, dim=-1)
        x = torch.cat([rms_norm(c, w[f"fc_norm.{i}.weight"], shape.rms_norm_eps)
                       for i, c in enumerate(chunks)], dim=-1)
    hidden = F.linear(x, w["fc.weight"])

    original_ids = input_ids.detach().clone()
    with_loss = verifier_last_hidden_states is not None or verifier_logits is not None
    if verifier_logits is not None:
        from .vocab import gather_targets

        targets = (gather_targets(verifier_logits, d2t) if d2t is not None else verifier_logits).detach()
    elif with_loss:
        with torch.no_grad():
            targets = F.linear(
                rms_norm(verifier_last_hidden_states, w["verifier_norm.weight"],
                         shape.rms_norm_eps),
                w["verifier_lm_head.weight"],
            )
    if with_loss:
        loss = torch.zeros(())
        prev_correct = (loss_mask.clone() if loss_mask is not None
                        else torch.ones(1, t, dtype=torch.bool))
        metrics: dict = {}

    caches = [dict() for _ in range(shape.num_hidden_layers)]
    draft_tokens, all_logits = [], []
    # one rotary module serves every step (and every later forward pass: hand the state in again)
    if rotary_state is None:
        rotary_state = RotaryState(shape.head_dim, shape.rope_theta, shape.rope_scaling)
    for step in range(ttt_steps):
        with torch.no_grad():
            embeds = F.embedding(input_ids, w["embed_tokens.weight"])
        cos, sin = rope_tables(position_ids, shape.head_dim, shape.rope_theta, dtype, shape.rope_scaling,
                               rotary_state)
        y = first_layer(torch.cat([embeds, hidden], -1), w, shape, cos, sin,
                        caches[0], mask_for(0, step), attn)
        for li in range(1, shape.num_hidden_layers):
            y = later_layer(y, w, li, shape, cos, sin, caches[li], mask_for(li, step), attn)
        if shape.norm_output:
            hidden = rms_norm(y, w["norm.weight"], shape.rms_norm_eps)
            logits = F.linear(hidden, w["lm_head.weight"])
        else:
            hidden = y
            logits = F.linear(rms_norm(y, w["norm.weight"], shape.rms_norm_eps),
                              w["lm_head.weight"])
        if return_logits:
            all_logits.append(logits)
        if with_loss:
            s_loss, s_metrics = MT.eagle3_compute_metrics(
                logits, targets, loss_mask, prev_correct, step, ttt_step_loss_decay,
                loss_config,
            )
            loss = loss + s_loss
            metrics.update(s_metrics)
        draft_tokens.append(logits.argmax(-1).detach().clone())
        # teacher forcing: ground-truth ids shifted left by 1 + step, zero padded
        input_ids = torch.cat(
            [original_ids[:, 1 + step:], original_ids.new_zeros(1, 1 + step)], dim=-1
        )
        position_ids = position_ids + 1

    if not with_loss:
        return draft_tokens
    metrics["loss_sum"] = loss.detach().clone()
    metrics["loss_total"] = torch.tensor(1.0)
    if return_logits:
        return draft_tokens, loss, metrics, all_logits
    return draft_tokens, loss, metrics


def random_weights(shape: DraftShape, seed: int = 0, dtype=torch.float32, std: float = 0.02):
    """Seeded N(0, std) weights with unit RMSNorm gains, keyed by the
    reference's state-dict names (models/eagle3/core.py:31-42; the fill rule of
    tests/integration/conftest.py:85-93)."""
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
        "verifier_norm.weight": torch.ones(h, dtype=dtype),
    }
    if shape.norm_before_fc:
        w["input_norm.weight"] = torch.ones(shape.num_aux * h, dtype=dtype)
    if shape.fc_norm:
        for i in range(shape.num_aux):
            w[f"fc_norm.{i}.weight"] = torch.ones(h, dtype=dtype)
    for li in range(shape.num_hidden_layers):
        p = f"layers.{li}."
        in_dim = 2 * h if li == 0 else h
        w[p + "self_attn.q_proj.weight"] = rnd(hq * d, in_dim)
        w[p + "self_attn.k_proj.weight"] = rnd(hkv * d, in_dim)
        w[p + "self_attn.v_proj.weight"] = rnd(hkv * d, in_dim)
        w[p + "self_attn.o_proj.weight"] = rnd(h, hq * d)
        if shape.qk_norm:
            w[p + "self_attn.q_norm.weight"] = torch.ones(d, dtype=dtype)
            w[p + "self_attn.k_norm.weight"] = torch.ones(d, dtype=dtype)
        w[p + "mlp.gate_proj.weight"] = rnd(f, h)
        w[p + "mlp.up_proj.weight"] = rnd(f, h)
        w[p + "mlp.down_proj.weight"] = rnd(h, f)
        w[p + "input_layernorm.weight"] = torch.ones(h, dtype=dtype)
        w[p + "post_attention_layernorm.weight"] = torch.ones(h, dtype=dtype)
        if li == 0:
            w[p + "hidden_norm.weight"] = torch.ones(h, dtype=dtype)
    return w
