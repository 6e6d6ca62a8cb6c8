"""Whole EAGLE3 draft forward + backward on the HIP path against the CPU oracle."""

import pytest
import torch

from oracle import eagle3 as OE
from oracle import losses as OL

pytestmark = pytest.mark.gpu


def _shape(**kw):
    base = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
                intermediate_size=512, vocab_size=2000, draft_vocab_size=704, rms_norm_eps=1e-5,
                rope_theta=10000.0)
    base.update(kw)
    return OE.DraftShape(**base)


_HALF = 32  # frequencies per head at the head size of `_shape`


def _batch(shape, t, seed, docs):
    g = torch.Generator().manual_seed(seed)
    hs = torch.randn(1, t, shape.num_aux * shape.hidden_size, generator=g)
    ids = torch.randint(0, shape.vocab_size, (1, t), generator=g)
    vl = torch.randn(1, t, shape.hidden_size, generator=g)
    mask = (torch.rand(1, t, generator=g) < 0.7).float()
    doc = torch.full((1, t), -1, dtype=torch.long)
    pos = torch.zeros(1, t, dtype=torch.long)
    o = 0
    for i, n in enumerate(docs):
        doc[0, o:o + n] = i
        pos[0, o:o + n] = 1 + torch.arange(n)
        o += n
    mask[0, o:] = 0
    return hs, ids, doc, mask, pos, vl


def _make(shape, w, param_dtype=torch.bfloat16, **extra):
    from speculators_amd.eagle3 import Eagle3Config, Eagle3DraftModel

    cfg = Eagle3Config(**extra, **{k: getattr(shape, k) for k in (
        "hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
        "vocab_size", "draft_vocab_size", "num_aux", "num_hidden_layers", "rms_norm_eps", "rope_theta",
        "norm_before_residual", "norm_before_fc", "fc_norm", "norm_output", "qk_norm",
        "sliding_window", "sliding_layers", "rope_scaling")})
    model = Eagle3DraftModel(cfg)
    missing, unexpected = model.load_state_dict(w, strict=False)
    assert not unexpected and set(missing) <= {"t2d", "d2t"}, (missing, unexpected)
    return model.to(param_dtype).cuda()


VARIANTS = [
    dict(),
    dict(norm_before_residual=True, norm_output=True, norm_before_fc=True),
    dict(num_hidden_layers=2, sliding_window=48, sliding_layers=(0,), qk_norm=True),
    # Llama-3.1 style frequency scaling, with a short original context so that it matters here
    dict(num_hidden_layers=2, rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                            "high_freq_factor": 4.0,
                                            "original_max_position_embeddings": 64}),
    # YaRN: blended frequencies and the attention factor on both tables (q/k/v as one product, and
    # with per-head q/k norms the stand-alone rotary kernel)
    dict(rope_scaling={"rope_type": "yarn", "factor": 16.0, "original_max_position_embeddings": 32}),
    dict(qk_norm=True, rope_scaling={"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 64,
                                     "attention_factor": 1.3}),
    dict(embed_requires_grad=True),  # marks the parameter trainable; the lookup itself has no graph
    # length-dependent types (the batch's highest position is 170, + 1 per TTT step): longrope whose
    # long divisors set in between step 0 and step 1, NTK-dynamic whose base grows at every step
    dict(rope_scaling={"rope_type": "longrope", "original_max_position_embeddings": 171,
                       "max_position_embeddings": 1368,
                       "short_factor": [1.0 + 0.01 * i for i in range(_HALF)],
                       "long_factor": [1.5 + 0.2 * i for i in range(_HALF)]}),
    dict(num_hidden_layers=2, rope_scaling={"rope_type": "dynamic", "factor": 2.0,
                                            "max_position_embeddings": 100}),
    # a head size the kernels are not built for: the attention function widens it with zero columns
    dict(num_hidden_layers=2, head_dim=96),
]


@pytest.mark.parametrize("variant", VARIANTS)
def test_forward_backward_matches_oracle(variant):
    variant = dict(variant)
    extra = {k_: variant.pop(k_) for k_ in ("embed_requires_grad",) if k_ in variant}
    shape = _shape(**variant)
    w32 = OE.random_weights(shape, seed=1, std=0.05)
    g = torch.Generator().manual_seed(11)
    for k_ in w32:  # non-trivial norm gains
        if k_.endswith("norm.weight") or "layernorm" in k_:
            w32[k_] = 1 + 0.1 * torch.randn(w32[k_].shape, generator=g)
    w = {k_: v.bfloat16() for k_, v in w32.items()}  # both sides start from the same bf16 values
    t, steps = 320, 3
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 2, [120, 170])
    hs, vl = hs.bfloat16(), vl.bfloat16()

    model = _make(shape, w, **extra)
    assert model.embed_tokens.weight.requires_grad == bool(extra.get("embed_requires_grad"))
    toks, loss, m = model(hs.cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.cuda(),
                          ttt_steps=steps, ttt_step_loss_decay=0.9)
    loss.backward()

    wf = {k_: v.float().requires_grad_(v.dtype.is_floating_point) for k_, v in w.items()}
    rt, rloss, rm, rlogits = OE.eagle3_forward(
        wf, shape, hs.float(), ids, doc, mask, pos, vl.float(), ttt_steps=steps,
        ttt_step_loss_decay=0.9, return_logits=True)
    rloss.backward()

    rel = abs(loss.item() - rloss.item()) / abs(rloss.item())
    print("loss", loss.item(), rloss.item(), rel)
    assert rel < 1e-3  # bf16 activations against an fp32 oracle
    assert set(m) == set(rm)
    for key in rm:
        if key.endswith("_total"):
            assert m[key].item() == rm[key].item(), key  # mask / row counts: exact
    # the same oracle in bf16 on the CPU gives the rounding noise floor of this model
    wb = {k_: v.clone().requires_grad_(v.dtype.is_floating_point) for k_, v in w.items()}
    _, bloss, _ = OE.eagle3_forward(wb, shape, hs, ids, doc, mask, pos, vl, ttt_steps=steps,
                                    ttt_step_loss_decay=0.9)
    bloss.backward()
    for name, p in model.named_parameters():
        if not p.requires_grad or name == "embed_tokens.weight":
            assert p.grad is None  # the embedding lookup runs without a graph (core.py:270-271)
            continue
        want = wf[name].grad
        scale = want.abs().max().item()
        err = (p.grad.float().cpu() - want).abs().max().item()
        floor = (wb[name].grad.float() - want).abs().max().item()
        # 2e-2 relative max-norm, or twice the error a bf16 PyTorch run of the oracle makes
        assert err <= max(2e-2 * scale, 2 * floor) + 1e-6, (name, err, floor, scale)
    assert len(toks) == steps and toks[0].shape == (1, t) and toks[0].dtype == torch.int64
    # draft tokens are an arg-max of bf16 logits: compare where the oracle's top-2 margin is clear
    for k in range(steps):
        top2 = rlogits[k].topk(2, dim=-1).values
        clear = (top2[..., 0] - top2[..., 1]) > 0.05 * top2[..., 0].abs().clamp_min(1.0)
        assert torch.equal(toks[k].cpu()[clear], rt[k][clear])


@pytest.mark.parametrize("variant", [VARIANTS[1], VARIANTS[2]])
def test_fp32_master_weights_under_autocast_match_oracle(variant):
    """The trainer's regime (train/trainer.py:459-465): fp32 master parameters, forward under
    ``torch.autocast(bf16)``, fp32 gradients.  Against the fp32 oracle (loss 1e-3, gradients 2e-2
    relative max-norm or twice the error of the same oracle under CPU autocast), and through
    ``torch.autograd.grad`` as well as ``backward()``."""
    shape = _shape(**variant)
    w32 = OE.random_weights(shape, seed=1, std=0.05)
    g = torch.Generator().manual_seed(11)
    for k_ in w32:
        if k_.endswith("norm.weight") or "layernorm" in k_:
            w32[k_] = 1 + 0.1 * torch.randn(w32[k_].shape, generator=g)
    t, steps = 320, 3
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 2, [120, 170])
    hs, vl = hs.bfloat16(), vl.bfloat16()  # hidden states are stored in bf16 (train/data.py)

    model = _make(shape, w32, param_dtype=torch.float32)
    assert model.fc.weight.dtype == torch.float32
    args = (hs.cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.cuda())
    with pytest.raises(RuntimeError, match="autocast"):
        model(*args, ttt_steps=1)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        toks, loss, m = model(*args, ttt_steps=steps, ttt_step_loss_decay=0.9)
    assert loss.dtype == torch.float32
    params = {n: p for n, p in model.named_parameters() if p.requires_grad}
    via_grad = torch.autograd.grad(loss, list(params.values()), retain_graph=True)
    loss.backward()
    for (n, p), gg in zip(params.items(), via_grad, strict=True):
        assert p.grad.dtype == torch.float32 and torch.equal(p.grad, gg), n

    def oracle(autocast):
        wf = {k_: v.clone().requires_grad_(v.dtype.is_floating_point) for k_, v in w32.items()}
        with torch.autocast("cpu", dtype=torch.bfloat16, enabled=autocast):
            _, rl, rm = OE.eagle3_forward(wf, shape, hs.float(), ids, doc, mask, pos, vl.float(),
                                          ttt_steps=steps, ttt_step_loss_decay=0.9)
        rl.backward()
        return rl, rm, wf

    rloss, rm, wf = oracle(False)
    _, _, wa = oracle(True)
    # the kernels keep every activation in bf16 (CPU autocast keeps norms and residuals in fp32):
    # the second noise floor is the same oracle run entirely in bf16
    wb = {k_: v.bfloat16().requires_grad_(v.dtype.is_floating_point) for k_, v in w32.items()}
    _, bl, _ = OE.eagle3_forward(wb, shape, hs, ids, doc, mask, pos, vl, ttt_steps=steps,
                                 ttt_step_loss_decay=0.9)
    bl.backward()
    rel = abs(loss.item() - rloss.item()) / abs(rloss.item())
    print("loss", loss.item(), rloss.item(), rel)
    assert rel < 1e-3
    for key in rm:
        if key.endswith("_total"):
            assert m[key].item() == rm[key].item(), key
    for name, p in params.items():
        want = wf[name].grad
        err = (p.grad.cpu() - want).abs().max().item()
        floor = max((wa[name].grad - want).abs().max().item(),
                    (wb[name].grad.float() - want).abs().max().item())
        assert err <= max(2e-2 * want.abs().max().item(), 2 * floor) + 1e-6, (name, err, floor)
    # validation: no graph, same loss
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        _, vloss, _ = model(*args, ttt_steps=steps, ttt_step_loss_decay=0.9)
    # (the training forward reads each row pair once, 512 threads to a row; the one without a graph streams
    # it, 256 to a row: the same sums in another order)
    assert abs(vloss.item() - loss.item()) <= 1e-6 * abs(loss.item())
    # an optimizer step on the fp32 masters is seen by the next forward (nothing stale is kept)
    torch.optim.SGD(params.values(), lr=0.05).step()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        _, vloss2, _ = model(*args, ttt_steps=steps, ttt_step_loss_decay=0.9)
    assert vloss2.item() < vloss.item()


@pytest.mark.parametrize("regime", ["bf16", "autocast"])
def test_configs0_in_full_matches_oracle(regime):
    """The reference's own CPU-runnable case at its real size: Llama-3.2-1B shape (hidden 2048,
    32 q / 8 kv heads, head_dim 64, FFN 8192), target vocabulary 128 256 -> draft 32 000 through
    a sorted random d2t subset, seq 512, 3 TTT steps, verifier logits ~ N(0, 2^2) over the target
    vocabulary, hidden states ~ N(0, 1), loss_mask Bernoulli(0.7), seeded.  Whole model on the
    HIP path against the fp32 oracle: loss 1e-3, per-step logits and every gradient 2e-2 relative
    max-norm, mask / row counts exact, the gathered targets bit-exact."""
    from oracle import vocab as OV
    from speculators_amd import losses as L

    shape = OE.DraftShape(hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
                          intermediate_size=8192, vocab_size=128256, draft_vocab_size=32000,
                          rms_norm_eps=1e-5, rope_theta=500000.0)
    t, steps = 512, 3
    g = torch.Generator().manual_seed(0)
    w32 = {k_: v.bfloat16().float() for k_, v in OE.random_weights(shape, seed=0).items()}
    hs = torch.randn(1, t, 3 * shape.hidden_size, generator=g).bfloat16()
    ids = torch.randint(0, shape.vocab_size, (1, t), generator=g)
    vlogits = (torch.randn(1, t, shape.vocab_size, generator=g) * 2).bfloat16()
    mask = (torch.rand(1, t, generator=g) < 0.7).float()
    doc = torch.zeros(1, t, dtype=torch.long)
    sel = torch.randperm(shape.vocab_size, generator=g)[: shape.draft_vocab_size]
    d2t, t2d = OV.build_vocab_mappings(sel.tolist(), shape.vocab_size)

    auto = regime == "autocast"
    model = _make(shape, w32, param_dtype=torch.float32 if auto else torch.bfloat16)
    model.load_vocab_mappings(t2d, d2t)
    model.keep_logits = True
    # index mapping: bit-exact against the oracle's gather
    got_targets = L.vocab_gather(vlogits.cuda(), model.d2t)
    assert torch.equal(got_targets.cpu(), OV.gather_targets(vlogits, d2t))
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=auto):
        toks, loss, m = model(hs.cuda(), ids.cuda(), doc.cuda(), mask.cuda(), None,
                              verifier_logits=vlogits.cuda(), ttt_steps=steps)
    loss.backward()

    wf = {k_: v.clone().requires_grad_(True) for k_, v in w32.items()}
    rt, rloss, rm, rlogits = OE.eagle3_forward(wf, shape, hs.float(), ids, doc, mask, None,
                                               ttt_steps=steps, verifier_logits=vlogits.float(), d2t=d2t,
                                               return_logits=True, attn="sdpa")
    rloss.backward()
    rel = abs(loss.item() - rloss.item()) / abs(rloss.item())
    print(regime, "loss", loss.item(), rloss.item(), rel)
    assert rel < 1e-3
    assert set(m) == set(rm)
    for key in rm:
        if key.endswith("_total"):
            assert m[key].item() == rm[key].item(), key
    for k_ in range(steps):
        got, want = model.last_logits[k_].float().cpu(), rlogits[k_].detach()
        assert (got - want).abs().max() <= 2e-2 * want.abs().max(), k_
    for name, p in model.named_parameters():
        if not p.requires_grad:
            continue
        want = wf[name].grad
        err = (p.grad.float().cpu() - want).abs().max().item()
        assert err <= 2e-2 * want.abs().max().item() + 1e-7, (name, err, want.abs().max().item())


def test_verifier_logits_entry_point_equals_row_sliced_head():
    """targets from a d2t gather of full-vocab verifier logits == the row-sliced verifier head."""
    from oracle import vocab as OV

    shape = _shape()
    w = {k_: v.bfloat16() for k_, v in OE.random_weights(shape, seed=3, std=0.05).items()}
    g = torch.Generator().manual_seed(5)
    sel = torch.randperm(shape.vocab_size, generator=g)[: shape.draft_vocab_size]
    d2t, t2d = OV.build_vocab_mappings(sel.tolist(), shape.vocab_size)
    full_head = (torch.randn(shape.vocab_size, shape.hidden_size, generator=g) * 0.05).bfloat16()
    w["verifier_lm_head.weight"] = full_head[t2d]
    model = _make(shape, w)
    model.load_vocab_mappings(t2d, d2t)
    t = 128
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 6, [128])
    hs, vl = hs.bfloat16().cuda(), vl.bfloat16().cuda()
    args = (hs, ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda())
    _, loss_a, m_a = model(*args, verifier_last_hidden_states=vl, ttt_steps=2)
    with torch.no_grad():
        full_logits = torch.nn.functional.linear(model.verifier_norm(vl), full_head.cuda())
    _, loss_b, m_b = model(*args, verifier_logits=full_logits, ttt_steps=2)
    assert loss_a.item() == pytest.approx(loss_b.item(), rel=2e-3)
    for key in m_a:
        if "acc" in key and key.endswith("_total"):
            assert m_a[key].item() == m_b[key].item()


def test_requires_bf16_and_hip_tensors():
    from speculators_amd._lib import SpxError

    shape = _shape()
    w = OE.random_weights(shape, seed=3)
    from speculators_amd.eagle3 import Eagle3Config, Eagle3DraftModel
    model = _make(shape, {k_: v.bfloat16() for k_, v in w.items()})
    hs, ids, doc, mask, pos, vl = _batch(shape, 128, 6, [128])
    with pytest.raises(RuntimeError):
        model(hs.cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.cuda(), ttt_steps=1)


def test_weight_gradient_over_all_steps_in_one_product():
    """The decoder projections' weight gradients come from one product over the stacked inputs and
    output gradients of all TTT steps, run when autograd reaches the staging node.  That must be
    invisible: ``torch.autograd.grad`` and ``backward()`` agree bit for bit, a retained graph can be
    walked twice, a hook on the parameter sees the gradient, and the result equals the step-by-step
    sum (the same model run with one use per weight expected, i.e. one product per step)."""
    shape = _shape()
    w = {k_: v.bfloat16() for k_, v in OE.random_weights(shape, seed=6, std=0.05).items()}
    hs, ids, doc, mask, pos, vl = _batch(shape, 160, 3, [90, 60])
    args = (hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda())
    for dtype, auto in ((torch.bfloat16, False), (torch.float32, True)):
        model = _make(shape, w, dtype)
        names = [n for n, p in model.named_parameters() if p.requires_grad]
        params = [p for _, p in model.named_parameters() if p.requires_grad]

        def fwd():
            with torch.autocast("cuda", dtype=torch.bfloat16, enabled=auto):
                return model(*args, ttt_steps=3, ttt_step_loss_decay=0.8)[1]

        seen = {}
        layer = model.layers[0]
        handle = layer.mlp.gate_proj.weight.register_hook(lambda g: seen.setdefault("gate", g.clone()))
        loss = fwd()
        loss.backward(retain_graph=True)
        handle.remove()
        g_bwd = [p.grad.clone() for p in params]
        assert torch.equal(seen["gate"], layer.mlp.gate_proj.weight.grad)
        assert all(g.dtype == dtype for g in g_bwd)
        # the same graph again: the gradients double (to one more rounding of the sum)
        loss.backward()
        for n, p, g in zip(names, params, g_bwd, strict=True):
            want = 2 * g.float()
            assert (p.grad.float() - want).abs().max() <= 2 ** -7 * want.abs().max() + 1e-12, n
        model.zero_grad(set_to_none=True)
        g_fn = torch.autograd.grad(fwd(), params)
        for n, a, b in zip(names, g_fn, g_bwd, strict=True):
            assert torch.equal(a, b), n
        # one product per step instead (no stacking): same sums up to fp32 summation order
        ref = _make(shape, w, dtype)
        begin = ref._stager.begin
        ref._stager.begin = lambda uses=1: begin(1)
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=auto):
            ref(*args, ttt_steps=3, ttt_step_loss_decay=0.8)[1].backward()
        ref_grads = {n: p.grad for n, p in ref.named_parameters() if p.requires_grad}
        for n, g in zip(names, g_bwd, strict=True):
            r = ref_grads[n].float()
            tol = (2 ** -7 if dtype == torch.bfloat16 else 1e-5) * r.abs().max() + 1e-12
            assert (g.float() - r).abs().max() <= tol, n


def test_backward_of_a_single_step_loss_reaches_only_the_steps_before_it():
    """A loss that stops after the first TTT step of a three-step forward: the later steps never
    run a backward, and the stacked weight-gradient product covers the first step's rows only.
    The gradients equal those of a one-step forward."""
    from speculators_amd import metrics as MT

    shape = _shape()
    w = {k_: v.bfloat16() for k_, v in OE.random_weights(shape, seed=8, std=0.05).items()}
    hs, ids, doc, mask, pos, vl = _batch(shape, 128, 5, [70, 50])
    args = (hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda())
    model = _make(shape, w)
    params = {n: p for n, p in model.named_parameters() if p.requires_grad}
    step_losses = []
    orig = MT.compute_metrics

    def spy(*a, **k):
        out = orig(*a, **k)
        step_losses.append(out[0])
        return out

    MT.compute_metrics = spy
    try:
        model(*args, ttt_steps=3)
    finally:
        MT.compute_metrics = orig
    assert len(step_losses) == 3
    step_losses[0].backward()
    got = {n: p.grad.clone() for n, p in params.items() if p.grad is not None}
    model.zero_grad(set_to_none=True)
    model(*args, ttt_steps=1)[1].backward()
    for n, p in params.items():
        if p.grad is None:
            assert n not in got, n
            continue
        assert torch.equal(got[n], p.grad), n


def test_gradient_accumulation_semantics_across_iterations():
    """The weight gradients are written into ``.grad`` by the GEMMs themselves (merged q/k/v
    buffer, beta = 1 accumulation over TTT steps): a second backward without ``zero_grad`` must
    add to them, ``zero_grad(set_to_none=False)`` must be honoured, and a fresh run must give the
    first run's bits again (every kernel reduces in a fixed order)."""
    shape = _shape(num_hidden_layers=2)
    w = {k_: v.bfloat16() for k_, v in OE.random_weights(shape, seed=4, std=0.05).items()}
    model = _make(shape, w)
    hs, ids, doc, mask, pos, vl = _batch(shape, 192, 9, [100, 80])
    args = (hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda())

    def run():
        _, loss, _ = model(*args, ttt_steps=3, ttt_step_loss_decay=0.9)
        loss.backward()
        return loss.item()

    params = {n: p for n, p in model.named_parameters() if p.requires_grad}
    l1 = run()
    g1 = {n: p.grad.clone() for n, p in params.items()}
    assert all(torch.isfinite(g).all() for g in g1.values())
    l2 = run()  # accumulates
    assert l2 == l1
    for n, p in params.items():
        want = 2 * g1[n].float()
        err = (p.grad.float() - want).abs().max().item()
        assert err <= 2 ** -7 * want.abs().max().item() + 1e-8, (n, err)  # one more bf16 rounding
    model.zero_grad(set_to_none=False)
    assert all(not p.grad.any() for p in params.values())
    run()
    for n, p in params.items():
        assert torch.equal(p.grad, g1[n]), n
    model.zero_grad(set_to_none=True)
    run()
    for n, p in params.items():
        assert torch.equal(p.grad, g1[n]), n
    # a plain optimizer step works on the (view) gradients and changes the next loss
    opt = torch.optim.SGD(params.values(), lr=0.05)
    opt.step()
    model.zero_grad(set_to_none=True)
    l3 = run()
    assert l3 < l1


@pytest.mark.parametrize("loss_fn", ["kl_div", "ce", "tv"])
def test_head_and_loss_as_one_node_changes_nothing(loss_fn, monkeypatch):
    """lm_head + fused loss as one autograd node (packed loss backward, row-counted head product)
    against the two-node form: loss, metrics, draft tokens and every parameter gradient bit for bit.
    (The node's streaming form, which shares its kernels with the two-node path; the form that writes
    the gradient in the forward row pass is compared with it below.)"""
    from speculators_amd import losses as L

    monkeypatch.setattr(L, "HEAD_LOSS_ONE_PASS", False)
    shape = _shape(num_hidden_layers=2)
    w = {k: v.bfloat16() for k, v in OE.random_weights(shape, seed=1, std=0.05).items()}
    t = 300
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 3, [120, 140])
    mask[0, :7] = 0  # a dead run at the start
    got = []
    for fuse in (True, False):
        model = _make(shape, w)
        model.fuse_head_loss = fuse
        toks, loss, metrics = model(
            hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda(),
            ttt_steps=3, ttt_step_loss_decay=0.8, loss_config=L.resolve_loss_config(loss_fn))
        loss.backward()
        got.append((loss.detach(), [x.clone() for x in toks], {k: v.clone() for k, v in metrics.items()},
                    {k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(got[0][0], got[1][0])
    for a, b in zip(got[0][1], got[1][1]):
        assert torch.equal(a, b)
    assert got[0][2].keys() == got[1][2].keys()
    for k in got[0][2]:
        assert torch.equal(got[0][2][k], got[1][2][k]), k
    assert got[0][3].keys() == got[1][3].keys() and len(got[0][3]) > 5
    for k in got[0][3]:
        assert torch.equal(got[0][3][k], got[1][3][k]), k


@pytest.mark.parametrize("loss_fn", ["kl_div", "ce"])
@pytest.mark.parametrize("master", [False, True])
def test_logits_gradient_written_in_the_forward_row_pass(loss_fn, master, monkeypatch):
    """The head + loss node in its one-pass form (the row pair read once: loss, statistics, acceptance
    chain AND the unit-weight logits gradient of the unmasked rows, the row weights applied after the
    input-gradient product) against its streaming form: draft tokens and every count identical, the
    loss within 1e-6, every parameter gradient within bf16 rounding of the largest entry.  With a
    loss scale on top (the upstream gradient of the loss is not one) and a second backward over the
    retained graph."""
    from speculators_amd import losses as L

    shape = _shape(num_hidden_layers=2)
    w32 = OE.random_weights(shape, seed=1, std=0.05)
    t = 300
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 3, [120, 140])
    mask[0, :7] = 0
    mask[0, 150:190] = 0
    got = []
    for one_pass in (True, False):
        monkeypatch.setattr(L, "HEAD_LOSS_ONE_PASS", one_pass)
        if master:
            model = _make(shape, w32, param_dtype=torch.float32)
        else:
            model = _make(shape, {k: v.bfloat16() for k, v in w32.items()})
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=master):
            toks, loss, metrics = model(
                hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda(),
                ttt_steps=3, ttt_step_loss_decay=0.8, loss_config=L.resolve_loss_config(loss_fn))
        (loss * 3.0).backward(retain_graph=True)
        first = {k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None}
        model.zero_grad(set_to_none=True)
        (loss * 3.0).backward()
        for k, p in model.named_parameters():
            if p.grad is not None:
                assert torch.equal(p.grad, first[k]), k
        got.append((loss.detach(), [x.clone() for x in toks], {k: v.clone() for k, v in metrics.items()}, first))
    assert abs(got[0][0].item() - got[1][0].item()) <= 1e-6 * abs(got[1][0].item())
    for a, b in zip(got[0][1], got[1][1]):
        assert torch.equal(a, b)
    for k in got[1][2]:
        if "loss" in k and k.endswith("_sum"):
            assert abs(got[0][2][k].item() - got[1][2][k].item()) <= 1e-6 * abs(got[1][2][k].item()) + 1e-9, k
        else:
            assert torch.equal(got[0][2][k], got[1][2][k]), k
    assert got[0][3].keys() == got[1][3].keys() and len(got[0][3]) > 5
    for k in got[1][3]:
        a, b = got[0][3][k].float(), got[1][3][k].float()
        assert (a - b).abs().max().item() <= 2 ** -6 * b.abs().max().item() + 1e-12, k


def test_a_backward_pass_for_some_inputs_leaves_nothing_behind():
    """``autograd.grad`` for ONE parameter over a retained graph runs the uses' backwards but never
    reaches the staging nodes of the other weights and gains: what those uses recorded (output
    gradients of the one-product weight gradient, partial sums of the gain gradients, the shared dK / dV
    buffer) belongs to that pass and must not enter the full ``backward()`` that follows."""
    shape = _shape(num_hidden_layers=2)
    w = {k: v.bfloat16() for k, v in OE.random_weights(shape, seed=1, std=0.05).items()}
    t = 200
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 3, [90, 100])
    args = (hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda())
    grads = []
    for partial_first in (False, True):
        model = _make(shape, w)
        _, loss, _ = model(*args, ttt_steps=3, ttt_step_loss_decay=0.8)
        if partial_first:
            (one,) = torch.autograd.grad(loss, [model.fc.weight], retain_graph=True)
        loss.backward()
        grads.append({k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None})
        if partial_first:
            assert torch.equal(one, grads[-1]["fc.weight"])
    assert grads[0].keys() == grads[1].keys() and len(grads[0]) > 5
    for k in grads[0]:
        assert torch.equal(grads[0][k], grads[1][k]), k


def test_head_node_falls_back_for_compound_losses():
    """A weighted sum of losses keeps the two-node form (the logits feed several reductions)."""
    from speculators_amd import losses as L

    shape = _shape()
    w = {k: v.bfloat16() for k, v in OE.random_weights(shape, seed=2, std=0.05).items()}
    hs, ids, doc, mask, pos, vl = _batch(shape, 200, 4, [200])
    got = []
    for fuse in (True, False):
        model = _make(shape, w)
        model.fuse_head_loss = fuse
        _, loss, _ = model(hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(),
                           vl.bfloat16().cuda(), ttt_steps=2,
                           loss_config=L.resolve_loss_config('{"ce": 0.3, "tv": 0.7}'))
        loss.backward()
        got.append((loss.detach(), {k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(got[0][0], got[1][0])
    for k in got[0][1]:
        assert torch.equal(got[0][1][k], got[1][1][k]), k


def test_decoder_projections_on_the_library_gemm(monkeypatch):
    """``SPX_DECODER_GEMM``: the decoder-layer projections and their input gradients on this
    library's MFMA kernel (``spx``), on the library GEMM behind ``torch.matmul`` (``hipblaslt``), or
    the forward products there and the input gradients here (``mixed``, the default).  Same loss and
    gradients up to the rounding of a bf16 product evaluated in another order."""
    from speculators_amd import gemm

    shape = _shape(num_hidden_layers=2)
    w = {k_: v.bfloat16() for k_, v in OE.random_weights(shape, seed=8, std=0.05).items()}
    hs, ids, doc, mask, pos, vl = _batch(shape, 200, 3, [120, 70])
    args = (hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda())
    results = {}
    assert gemm.DECODER_GEMM in ("hipblaslt", "spx", "mixed")
    for kind in ("hipblaslt", "spx", "mixed"):
        monkeypatch.setattr(gemm, "DECODER_GEMM", kind)
        model = _make(shape, w, torch.bfloat16)
        _, loss, metrics = model(*args, ttt_steps=3, ttt_step_loss_decay=0.8)
        loss.backward()
        results[kind] = (loss.item(), {n: p.grad.float() for n, p in model.named_parameters() if p.grad is not None},
                         metrics)
    la, ga, ma = results["hipblaslt"]
    for other in ("spx", "mixed"):
        lb, gb, mb = results[other]
        assert abs(la - lb) <= 2e-3 * abs(la), other
        assert ga.keys() == gb.keys()
        for n in ga:
            assert (ga[n] - gb[n]).abs().max() <= 3e-2 * ga[n].abs().max() + 1e-6, (other, n)
        for k_ in ma:
            if k_.endswith("_total"):
                assert torch.equal(ma[k_], mb[k_]), (other, k_)


def test_cross_entropy_loss_never_materialises_the_verifier_logits(monkeypatch):
    """With ``ce`` as the only loss the verifier head is reduced to per-row statistics in the
    epilogue of its product (``metrics.VerifierHead`` -> ``spx_gemm_bf16_nt_stats`` with no output):
    no ``[T, Vd]`` target tensor is made at any step.  Loss within 1e-3 of the fp32 oracle, the
    ``_total`` counts exact, and against the same model with the target logits materialised: loss,
    every metric, the draft tokens and every gradient bit for bit."""
    from speculators_amd import losses as L
    from speculators_amd import metrics as MT

    shape = _shape(num_hidden_layers=2, norm_output=True)
    w32 = OE.random_weights(shape, seed=4, std=0.05)
    w = {k: v.bfloat16() for k, v in w32.items()}
    t = 300
    hs, ids, doc, mask, pos, vl = _batch(shape, t, 9, [150, 130])
    args = (hs.bfloat16().cuda(), ids.cuda(), doc.cuda(), mask.cuda(), pos.cuda(), vl.bfloat16().cuda())
    cfg = L.resolve_loss_config("ce")

    def run(model):
        toks, loss, metrics = model(*args, ttt_steps=3, ttt_step_loss_decay=0.8, loss_config=cfg)
        loss.backward()
        return (loss.detach(), toks, metrics,
                {k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None})

    calls = {"materialize": 0, "stats": 0}
    real_mat, real_stats = MT.VerifierHead.materialize, MT.VerifierHead.stats

    def mat(self):
        calls["materialize"] += 1
        return real_mat(self)

    def stats(self):
        calls["stats"] += 1
        return real_stats(self)

    monkeypatch.setattr(MT.VerifierHead, "materialize", mat)
    monkeypatch.setattr(MT.VerifierHead, "stats", stats)
    got = run(_make(shape, w))
    assert calls == {"materialize": 0, "stats": 1}

    # the same with the target logits in memory (the statistics then come from the loss kernel's pass)
    monkeypatch.setattr(MT.VerifierHead, "stats", lambda self: (_ for _ in ()).throw(AssertionError("unused")))
    real_cm = MT.compute_metrics

    def cm(logits, targets, *a, **kw):
        if isinstance(targets, MT.VerifierHead):
            targets = targets.materialize()
        return real_cm(logits, targets, *a, **kw)

    import speculators_amd.eagle3 as E3
    monkeypatch.setattr(E3.MT, "compute_metrics", cm)
    want = run(_make(shape, w))
    assert calls["materialize"] == 3
    assert torch.equal(got[0], want[0])
    for a, b in zip(got[1], want[1]):
        assert torch.equal(a, b)
    assert got[2].keys() == want[2].keys()
    for k in got[2]:
        assert torch.equal(got[2][k], want[2][k]), k
    assert got[3].keys() == want[3].keys() and len(got[3]) > 5
    for k in got[3]:
        assert torch.equal(got[3][k], want[3][k]), k

    wf = {k: v.float() for k, v in w.items()}
    _, rloss, rm = OE.eagle3_forward(wf, shape, hs.bfloat16().float(), ids, doc, mask, pos, vl.bfloat16().float(),
                                     ttt_steps=3, ttt_step_loss_decay=0.8, loss_config=OL.resolve_loss_config("ce"))
    assert abs(got[0].item() - rloss.item()) <= 1e-3 * abs(rloss.item())
    for k in range(3):
        assert got[2][f"full_acc_{k}_total"].item() == rm[f"full_acc_{k}_total"].item()
        assert got[2][f"cond_acc_{k}_total"].item() == rm[f"cond_acc_{k}_total"].item()
