"""The oracle's EAGLE3 forward against the HF library blocks it restates, and
its alignment invariants."""

import pytest
import torch

from oracle import eagle3 as E
from oracle import masks as M
from oracle.attention import dense_attention


def _tiny_shape(**kw):
    base = dict(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                intermediate_size=128, vocab_size=128, draft_vocab_size=48, rms_norm_eps=1e-6,
                rope_theta=10000.0)
    base.update(kw)
    return E.DraftShape(**base)


def _batch(shape, t, seed=0, docs=None):
    g = torch.Generator().manual_seed(seed)
    hs = torch.randn(1, t, shape.num_aux * shape.hidden_size, generator=g)
    ids = torch.randint(0, shape.vocab_size, (1, t), generator=g)
    vl = torch.randn(1, t, shape.hidden_size, generator=g)
    mask = (torch.rand(1, t, generator=g) < 0.7).float()
    if docs is None:
        doc = torch.zeros(1, t, dtype=torch.long)
        pos = 1 + torch.arange(t).unsqueeze(0)
    else:
        doc = torch.full((1, t), -1, dtype=torch.long)
        pos = torch.zeros(1, t, dtype=torch.long)
        o = 0
        for i, n in enumerate(docs):
            doc[0, o:o + n] = i
            pos[0, o:o + n] = 1 + torch.arange(n)
            o += n
        mask[0, o:] = 0
    return hs, ids, doc, mask, pos, vl


def test_dense_attention_equals_sdpa_library_routine():
    g = torch.Generator().manual_seed(0)
    t = 24
    q = torch.randn(1, 4, t, 16, generator=g)
    k = torch.randn(1, 2, 3 * t, 16, generator=g)
    v = torch.randn(1, 2, 3 * t, 16, generator=g)
    doc = torch.tensor([0] * 10 + [1] * 9 + [-1] * 5)
    mask = M.ttt_mask_dense(doc, t, 2, sliding_window=6)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), attn_mask=mask[None, None],
        scale=0.25).transpose(1, 2)
    assert torch.allclose(dense_attention(q, k, v, mask, 0.25), ref, atol=1e-5)


def test_first_layer_equals_hf_llama_blocks():
    from transformers import DynamicCache, LlamaConfig
    from transformers.models.llama.modeling_llama import (
        LlamaAttention, LlamaMLP, LlamaRMSNorm, LlamaRotaryEmbedding)

    shape = _tiny_shape(norm_before_residual=True)
    w = E.random_weights(shape, seed=1)
    for k_ in list(w):
        if k_.endswith("norm.weight") or "layernorm" in k_:
            w[k_] = 1 + 0.1 * torch.randn_like(w[k_])
    cfg = LlamaConfig(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                      intermediate_size=128, vocab_size=128, rms_norm_eps=1e-6,
                      rope_parameters={"rope_type": "default", "rope_theta": 10000.0},
                      num_hidden_layers=1, attention_bias=False)
    cfg._attn_implementation = "eager"
    attn = LlamaAttention(cfg, 0)
    attn.q_proj = torch.nn.Linear(128, 64, bias=False)
    attn.k_proj = torch.nn.Linear(128, 32, bias=False)
    attn.v_proj = torch.nn.Linear(128, 32, bias=False)
    p = "layers.0."
    for n in "qkvo":
        getattr(attn, n + "_proj").weight.data.copy_(w[p + f"self_attn.{n}_proj.weight"])
    mlp = LlamaMLP(cfg)
    for n in ("gate", "up", "down"):
        getattr(mlp, n + "_proj").weight.data.copy_(w[p + f"mlp.{n}_proj.weight"])
    norms = {}
    for n in ("input_layernorm", "hidden_norm", "post_attention_layernorm"):
        norms[n] = LlamaRMSNorm(64, eps=1e-6)
        norms[n].weight.data.copy_(w[p + n + ".weight"])
    rot_cfg = LlamaConfig(**{**cfg.to_dict(), "hidden_size": 128})
    rot = LlamaRotaryEmbedding(rot_cfg)

    t = 20
    g = torch.Generator().manual_seed(5)
    doc = torch.tensor([0] * 8 + [1] * 9 + [-1] * 3)
    pos = torch.cat([1 + torch.arange(8), 1 + torch.arange(9), torch.zeros(3, dtype=torch.long)]).unsqueeze(0)
    cache_hf, cache_or = DynamicCache(), {}
    with torch.no_grad():
        for step in range(3):
            x = torch.randn(1, t, 128, generator=g)
            mask = M.ttt_mask_dense(doc, t, step)
            fmask = torch.zeros(1, 1, t, (step + 1) * t).masked_fill(~mask[None, None], float("-inf"))
            cos, sin = rot(x, pos + step)
            e, h = x.split(64, -1)
            e, h = norms["input_layernorm"](e), norms["hidden_norm"](h)
            a, _ = attn(hidden_states=torch.cat([e, h], -1), attention_mask=fmask,
                        position_embeddings=(cos, sin), past_key_values=cache_hf,
                        cache_position=torch.arange(step * t, (step + 1) * t))
            y = h + a
            ref = y + mlp(norms["post_attention_layernorm"](y))
            c2, s2 = E.rope_tables(pos + step, 16, 10000.0, torch.float32)
            assert torch.allclose(c2, cos, atol=1e-6) and torch.allclose(s2, sin, atol=1e-6)
            got = E.first_layer(x, w, shape, c2, s2, cache_or, mask)
            assert torch.allclose(got, ref, atol=2e-5), (step, (got - ref).abs().max())


@pytest.mark.parametrize("attn", ["dense", "sdpa"])
def test_forward_runs_and_backends_agree(attn):
    shape = _tiny_shape(norm_output=True, norm_before_fc=True, norm_before_residual=True,
                        sliding_window=8, sliding_layers=(0,), num_hidden_layers=2)
    w = E.random_weights(shape, seed=0)
    hs, ids, doc, mask, pos, vl = _batch(shape, 32, docs=[12, 15])
    toks, loss, m = E.eagle3_forward(w, shape, hs, ids, doc, mask, pos, vl, ttt_steps=3,
                                     ttt_step_loss_decay=0.9, attn=attn)
    toks2, loss2, m2 = E.eagle3_forward(w, shape, hs, ids, doc, mask, pos, vl, ttt_steps=3,
                                        ttt_step_loss_decay=0.9, attn="dense")
    assert torch.isfinite(loss) and len(toks) == 3 and toks[0].shape == (1, 32)
    # whole-model loss agreement across attention backends, the reference's own
    # tolerance (tests/integration/models/test_model_forward.py:360-366)
    assert torch.allclose(loss, loss2, atol=1e-3, rtol=1e-3)
    for k in ("loss_0_sum", "full_acc_2_total", "cond_acc_1_total", "loss_sum", "loss_total"):
        assert k in m
    assert m["loss_sum"].item() == pytest.approx(sum(m[f"loss_{k}_sum"].item() for k in range(3)), rel=1e-6)


def test_documents_are_independent_and_padding_is_inert():
    """Packing invariant: the loss of a packed row equals what each document
    contributes alone (the mask is block diagonal by document)."""
    shape = _tiny_shape()
    w = E.random_weights(shape, seed=2)
    hs, ids, doc, mask, pos, vl = _batch(shape, 24, docs=[10, 9])
    _, _, _, logits = E.eagle3_forward(w, shape, hs, ids, doc, mask, pos, vl, ttt_steps=2,
                                       return_logits=True)
    # document 1 alone (rows 10..18)
    sl = slice(10, 19)
    _, _, _, lg1 = E.eagle3_forward(w, shape, hs[:, sl], ids[:, sl], torch.zeros(1, 9, dtype=torch.long),
                                    mask[:, sl], pos[:, sl], vl[:, sl], ttt_steps=2, return_logits=True)
    # step 0 is identical row by row; step 1 is too except the last row of the
    # document, whose teacher-forced input id comes from the neighbour in the packed row
    assert torch.allclose(logits[0][:, sl], lg1[0], atol=1e-5)
    assert torch.allclose(logits[1][:, 10:18], lg1[1][:, :8], atol=1e-5)


def test_teacher_forcing_shift():
    """Step k consumes input_ids shifted left by k (zero padded) and positions + k."""
    shape = _tiny_shape()
    w = E.random_weights(shape, seed=3)
    hs, ids, doc, mask, pos, vl = _batch(shape, 16)
    toks, loss, m = E.eagle3_forward(w, shape, hs, ids, doc, mask, pos, vl, ttt_steps=2)
    ids2 = ids.clone(); ids2[0, 0] = (ids2[0, 0] + 1) % shape.vocab_size
    toks2, loss2, _ = E.eagle3_forward(w, shape, hs, ids2, doc, mask, pos, vl, ttt_steps=2)
    # token 0 is only ever used as the step-0 input of row 0
    assert not torch.equal(toks[0], toks2[0]) or loss.item() != loss2.item()


# ---------------------------------------------------------------- rope frequency scaling
_LLAMA31 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
            "original_max_position_embeddings": 8192}


_YARN = {"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 32768}


@pytest.mark.parametrize("scaling", [None, {"rope_type": "linear", "factor": 4.0}, _LLAMA31,
                                     dict(_LLAMA31, factor=32.0, original_max_position_embeddings=64),
                                     _YARN, dict(_YARN, factor=40.0, beta_fast=16, beta_slow=2,
                                                 original_max_position_embeddings=4096, mscale=1.0,
                                                 mscale_all_dim=0.7),
                                     dict(_YARN, attention_factor=1.25, truncate=False)])
@pytest.mark.parametrize("head_dim,theta", [(128, 500000.0), (64, 10000.0)])
def test_rope_inv_freq_matches_transformers(scaling, head_dim, theta):
    """The oracle's inverse frequencies == the HF rotary initialisation (library routine), and
    the product's host-side evaluation == the oracle's, bit for bit."""
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    from speculators_amd.fused_ops import rope_inv_freq

    got = E.rope_inv_freq(head_dim, theta, scaling)
    params = {"rope_type": "default", "rope_theta": theta}
    params.update(scaling or {})
    cfg = LlamaConfig(hidden_size=head_dim * 4, num_attention_heads=4, head_dim=head_dim,
                      rope_parameters=params, max_position_embeddings=131072)
    kind = params["rope_type"]
    if kind == "default":
        from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding

        want = LlamaRotaryEmbedding(cfg).inv_freq
        factor = 1.0
    else:
        want, factor = ROPE_INIT_FUNCTIONS[kind](cfg, "cpu")
    assert (factor == 1.0) == (kind != "yarn")
    assert E.rope_table_scale(scaling) == pytest.approx(factor, rel=1e-12)
    assert torch.equal(got, want)
    mine = rope_inv_freq(head_dim, theta, "cpu", scaling)
    assert torch.equal(mine, got) and mine.attention_scaling == pytest.approx(factor, rel=1e-12)
    if kind == "yarn":  # the tables of the library's rotary module, attention factor included
        from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding

        pos = torch.tensor([[0, 1, 5, 1000, 40000]])
        cos, sin = LlamaRotaryEmbedding(cfg)(torch.zeros(1, 5, 8), pos)
        mc, ms = E.rope_tables(pos[0], head_dim, theta, torch.float32, scaling)
        assert torch.allclose(mc, cos, atol=1e-6) and torch.allclose(ms, sin, atol=1e-6)
    if kind == "llama3":  # the scaling does something: low frequencies shrink by `factor`
        base = E.rope_inv_freq(head_dim, theta, None)
        assert torch.equal(got[0], base[0]) and torch.isclose(got[-1], base[-1] / scaling["factor"])


def test_rope_scaling_rejects_unknown_types():
    from speculators_amd.fused_ops import rope_inv_freq

    with pytest.raises(NotImplementedError):
        rope_inv_freq(64, 10000.0, "cpu", {"rope_type": "no-such-type", "factor": 2.0})
    with pytest.raises(NotImplementedError):
        E.rope_inv_freq(64, 10000.0, {"rope_type": "no-such-type", "factor": 2.0})


def _length_dependent_cases(head_dim):
    g = torch.Generator().manual_seed(head_dim)
    long = (1 + 3 * torch.rand(head_dim // 2, generator=g)).tolist()
    short = (1 + 0.2 * torch.rand(head_dim // 2, generator=g)).tolist()
    longrope = {"rope_type": "longrope", "long_factor": long, "short_factor": short,
                "original_max_position_embeddings": 128}
    return [({"rope_type": "dynamic", "factor": 2.0}, 256),
            ({"rope_type": "dynamic", "factor": 4.0}, 64),
            (longrope, 1024),                                    # factor = 1024 / 128
            (dict(longrope, factor=8.0, attention_factor=1.3), 1024),
            (dict(longrope, factor=1.0), 1024)]                  # no table factor


@pytest.mark.parametrize("head_dim,theta", [(64, 10000.0), (128, 500000.0)])
@pytest.mark.parametrize("case", range(5))
def test_length_dependent_rope_follows_the_library_module_call_by_call(case, head_dim, theta):
    """"dynamic" and "longrope": the frequencies the HF rotary module runs with over a sequence of
    calls (growth, a shorter call that keeps the grown base, the reset below the trained context;
    either side of the longrope threshold) == the oracle's ``RotaryState`` == the product's
    ``RotaryFrequencies``, bit for bit, tables and table factor included."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding

    from speculators_amd.fused_ops import RotaryFrequencies

    scaling, ctx = _length_dependent_cases(head_dim)[case]
    params = {"rope_theta": theta}
    params.update(scaling)
    cfg = LlamaConfig(hidden_size=head_dim * 4, num_attention_heads=4, head_dim=head_dim,
                      rope_parameters=params, max_position_embeddings=ctx)
    module = LlamaRotaryEmbedding(cfg)
    mine = dict(scaling, max_position_embeddings=ctx)
    state = E.RotaryState(head_dim, theta, mine)
    product = RotaryFrequencies(head_dim, theta, mine)
    assert product.by_length and torch.equal(module.inv_freq, state.original)
    assert E.rope_table_scale(mine) == pytest.approx(module.attention_scaling, rel=1e-12)
    for top in (50, 300, 280, 1000, 400, 100, 260, 63, 64, 65, 127, 128, 129, 255, 256, 257):
        pos = torch.arange(top - 20, top).unsqueeze(0)
        cos, sin = module(torch.zeros(1, 20, 8), pos)
        assert torch.equal(state.inv_freq(pos), module.inv_freq), top
        mc, ms = E.rope_tables(pos[0], head_dim, theta, torch.float32, mine, inv_freq=module.inv_freq)
        assert torch.equal(mc, cos) and torch.equal(ms, sin)
        # the product is asked with the highest position split into base + offset (a TTT step)
        got = product.select("cpu", product.top(pos) - 3, 3)
        assert torch.equal(got, module.inv_freq), top
        assert got.attention_scaling == pytest.approx(module.attention_scaling, rel=1e-12)


def test_fixed_rope_types_never_read_the_positions():
    from speculators_amd.fused_ops import RotaryFrequencies

    for scaling in (None, _LLAMA31, _YARN, {"rope_type": "linear", "factor": 2.0}):
        r = RotaryFrequencies(64, 10000.0, scaling)
        assert not r.by_length and r.top(None) is None
        assert r.select("cpu") is r.select("cpu", None, 5)
        assert torch.equal(r.select("cpu"), E.rope_inv_freq(64, 10000.0, scaling))


# ---------------------------------------------------------------- layers after the first, q/k norm
def _randomise_gains(w, seed):
    g = torch.Generator().manual_seed(seed)
    for name in list(w):
        if name.endswith("norm.weight") or "layernorm" in name:
            w[name] = 1 + 0.2 * torch.randn(w[name].shape, generator=g)
    return w


def _ttt_batch(t, docs, pad):
    doc = torch.tensor(sum(([i] * n for i, n in enumerate(docs)), []) + [-1] * pad)
    pos = torch.cat([1 + torch.arange(n) for n in docs] + [torch.zeros(pad, dtype=torch.long)]).unsqueeze(0)
    assert doc.numel() == t
    return doc, pos


def _additive(mask):
    return torch.zeros(1, 1, *mask.shape).masked_fill(~mask[None, None], float("-inf"))


@pytest.mark.parametrize("family", ["llama", "qwen3"])
def test_later_layer_equals_hf_decoder_layer(family):
    """``later_layer`` (every EAGLE3 layer after the first: models/eagle3/core.py:286-300 runs the
    unpatched ``decoder_layer_class`` of models/base_components.py:39-52) against the library's own
    ``LlamaDecoderLayer`` / ``Qwen3DecoderLayer`` -- classes used whole, nothing wired here -- over
    three TTT steps sharing one ``DynamicCache``, packed documents plus padding, a windowed mask,
    random norm gains.  Output and the gradient of the input and of every parameter."""
    from transformers import DynamicCache, LlamaConfig, Qwen3Config
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer, LlamaRotaryEmbedding
    from transformers.models.qwen3.modeling_qwen3 import Qwen3DecoderLayer, Qwen3RotaryEmbedding

    qk = family == "qwen3"
    shape = _tiny_shape(num_hidden_layers=2, qk_norm=qk)
    w = _randomise_gains(E.random_weights(shape, seed=11, std=0.2), 12)
    common = dict(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                  intermediate_size=128, vocab_size=128, rms_norm_eps=1e-6, num_hidden_layers=2,
                  attention_bias=False,
                  rope_parameters={"rope_type": "default", "rope_theta": 10000.0})
    if qk:
        cfg = Qwen3Config(**common, layer_types=["full_attention"] * 2, sliding_window=None)
        layer, rot = Qwen3DecoderLayer(cfg, 1), Qwen3RotaryEmbedding(cfg)
    else:
        cfg = LlamaConfig(**common)
        layer, rot = LlamaDecoderLayer(cfg, 1), LlamaRotaryEmbedding(cfg)
    cfg._attn_implementation = "eager"
    layer.self_attn.config._attn_implementation = "eager"
    p = "layers.1."
    names = {n: prm for n, prm in layer.named_parameters()}
    assert set(names) == {k[len(p):] for k in w if k.startswith(p)}
    for n, prm in names.items():
        prm.data.copy_(w[p + n])
    wl = {k: v.clone().requires_grad_(True) for k, v in w.items() if k.startswith(p)}

    t = 20
    doc, pos = _ttt_batch(t, [8, 9], 3)
    g = torch.Generator().manual_seed(13)
    xs = [torch.randn(1, t, 64, generator=g) for _ in range(3)]
    xs_hf = [x.clone().requires_grad_(True) for x in xs]
    xs_or = [x.clone().requires_grad_(True) for x in xs]
    cache_hf, cache_or = DynamicCache(), {}
    probe = torch.randn(3, 1, t, 64, generator=g)
    total_hf = total_or = 0.0
    for step in range(3):
        mask = M.ttt_mask_dense(doc, t, step, sliding_window=5)
        cos, sin = rot(xs[step], pos + step)
        ref = layer(xs_hf[step], attention_mask=_additive(mask), position_ids=pos + step,
                    past_key_values=cache_hf, use_cache=True, position_embeddings=(cos, sin))
        ref = ref[0] if isinstance(ref, tuple) else ref
        c2, s2 = E.rope_tables(pos + step, 16, 10000.0, torch.float32)
        got = E.later_layer(xs_or[step], wl, 1, shape, c2, s2, cache_or, mask)
        assert torch.allclose(got, ref, atol=3e-5), (step, (got - ref).abs().max())
        total_hf = total_hf + (ref * probe[step]).sum()
        total_or = total_or + (got * probe[step]).sum()
    total_hf.backward()
    total_or.backward()
    for a, b in zip(xs_or, xs_hf):   # step 0's input also reaches steps 1, 2 through the cache
        assert torch.allclose(a.grad, b.grad, atol=1e-4, rtol=1e-4)
    for n, prm in names.items():
        assert torch.allclose(wl[p + n].grad, prm.grad, atol=2e-4, rtol=1e-4), n


def test_later_layer_pin_notices_a_post_norm_or_a_dropped_residual():
    """The comparison above has teeth: the plausible slips (normalising after the attention
    instead of before it, a residual taken from the normalised input) move the output by far
    more than its tolerance."""
    shape = _tiny_shape(num_hidden_layers=2)
    w = _randomise_gains(E.random_weights(shape, seed=11, std=0.2), 12)
    t = 12
    doc, pos = _ttt_batch(t, [7, 5], 0)
    x = torch.randn(1, t, 64, generator=torch.Generator().manual_seed(1))
    cos, sin = E.rope_tables(pos, 16, 10000.0, torch.float32)
    mask = M.ttt_mask_dense(doc, t, 0)
    good = E.later_layer(x, w, 1, shape, cos, sin, {}, mask)
    p = "layers.1."
    a = E._attention_block(x, w, p + "self_attn.", shape, cos, sin, {}, mask, "dense")
    post = x + E.rms_norm(a, w[p + "input_layernorm.weight"], shape.rms_norm_eps)
    post = post + E.swiglu_mlp(E.rms_norm(post, w[p + "post_attention_layernorm.weight"], 1e-6), w, p + "mlp.")
    xn = E.rms_norm(x, w[p + "input_layernorm.weight"], shape.rms_norm_eps)
    y = xn + E._attention_block(xn, w, p + "self_attn.", shape, cos, sin, {}, mask, "dense")
    wrong_res = y + E.swiglu_mlp(E.rms_norm(y, w[p + "post_attention_layernorm.weight"], 1e-6), w, p + "mlp.")
    assert (good - post).abs().max() > 1e-2 and (good - wrong_res).abs().max() > 1e-2


def test_first_layer_with_qk_norm_equals_hf_qwen3_blocks():
    """EAGLE3 on Qwen3 layers: ``Eagle3FirstLayerMixin`` (models/eagle3/model_definitions.py:14-110)
    mixed into ``Qwen3DecoderLayer`` (models/base_components.py:46-51) swaps q/k/v for projections
    of the 2H input and otherwise runs the library's ``Qwen3Attention.forward``: per-head RMSNorm
    of q and k BEFORE the rotary embedding.  The oracle's first layer with ``qk_norm`` against the
    library's ``Qwen3Attention`` / ``Qwen3MLP`` / ``Qwen3RMSNorm`` / ``Qwen3RotaryEmbedding``
    composed that way, three TTT steps on one ``DynamicCache``, non-trivial q/k gains; a
    norm-after-RoPE variant is noticed."""
    from transformers import DynamicCache, Qwen3Config
    from transformers.models.qwen3.modeling_qwen3 import (
        Qwen3Attention, Qwen3MLP, Qwen3RMSNorm, Qwen3RotaryEmbedding)

    shape = _tiny_shape(qk_norm=True, norm_before_residual=False)
    w = _randomise_gains(E.random_weights(shape, seed=21, std=0.2), 22)
    cfg = Qwen3Config(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                      intermediate_size=128, vocab_size=128, rms_norm_eps=1e-6, num_hidden_layers=1,
                      attention_bias=False, layer_types=["full_attention"], sliding_window=None,
                      rope_parameters={"rope_type": "default", "rope_theta": 10000.0})
    cfg._attn_implementation = "eager"
    attn = Qwen3Attention(cfg, 0)
    attn.q_proj = torch.nn.Linear(128, 64, bias=False)
    attn.k_proj = torch.nn.Linear(128, 32, bias=False)
    attn.v_proj = torch.nn.Linear(128, 32, bias=False)
    p = "layers.0."
    for n in "qkvo":
        getattr(attn, n + "_proj").weight.data.copy_(w[p + f"self_attn.{n}_proj.weight"])
    attn.q_norm.weight.data.copy_(w[p + "self_attn.q_norm.weight"])
    attn.k_norm.weight.data.copy_(w[p + "self_attn.k_norm.weight"])
    mlp = Qwen3MLP(cfg)
    for n in ("gate", "up", "down"):
        getattr(mlp, n + "_proj").weight.data.copy_(w[p + f"mlp.{n}_proj.weight"])
    norms = {}
    for n in ("input_layernorm", "hidden_norm", "post_attention_layernorm"):
        norms[n] = Qwen3RMSNorm(64, eps=1e-6)
        norms[n].weight.data.copy_(w[p + n + ".weight"])
    rot = Qwen3RotaryEmbedding(cfg)

    t = 20
    doc, pos = _ttt_batch(t, [8, 9], 3)
    g = torch.Generator().manual_seed(23)
    cache_hf, cache_or, cache_bad = DynamicCache(), {}, {}
    with torch.no_grad():
        for step in range(3):
            x = torch.randn(1, t, 128, generator=g)
            mask = M.ttt_mask_dense(doc, t, step)
            cos, sin = rot(x, pos + step)
            e, h = x.split(64, -1)
            residual = h                                # norm_before_residual = False
            e, h = norms["input_layernorm"](e), norms["hidden_norm"](h)
            a, _ = attn(hidden_states=torch.cat([e, h], -1), attention_mask=_additive(mask),
                        position_embeddings=(cos, sin), past_key_values=cache_hf)
            y = residual + a
            ref = y + mlp(norms["post_attention_layernorm"](y))
            c2, s2 = E.rope_tables(pos + step, 16, 10000.0, torch.float32)
            got = E.first_layer(x, w, shape, c2, s2, cache_or, mask)
            assert torch.allclose(got, ref, atol=3e-5), (step, (got - ref).abs().max())
            # the slip this pin is for: normalising after the rotation
            xin = torch.cat([e, h], -1)
            q = torch.nn.functional.linear(xin, w[p + "self_attn.q_proj.weight"]).view(1, t, 4, 16).transpose(1, 2)
            k = torch.nn.functional.linear(xin, w[p + "self_attn.k_proj.weight"]).view(1, t, 2, 16).transpose(1, 2)
            v = torch.nn.functional.linear(xin, w[p + "self_attn.v_proj.weight"]).view(1, t, 2, 16).transpose(1, 2)
            q = E.rms_norm(E.apply_rope(q, c2, s2), w[p + "self_attn.q_norm.weight"], 1e-6)
            k = E.rms_norm(E.apply_rope(k, c2, s2), w[p + "self_attn.k_norm.weight"], 1e-6)
            cache_bad["k"] = k if "k" not in cache_bad else torch.cat([cache_bad["k"], k], 2)
            cache_bad["v"] = v if "v" not in cache_bad else torch.cat([cache_bad["v"], v], 2)
            o = dense_attention(q, cache_bad["k"], cache_bad["v"], mask, 16 ** -0.5)
            bad = torch.nn.functional.linear(o.reshape(1, t, 64), w[p + "self_attn.o_proj.weight"])
            assert (bad - a).abs().max() > 1e-2
