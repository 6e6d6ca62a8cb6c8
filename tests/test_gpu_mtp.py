"""HIP MTP path (label cross-entropy kernel, head_dim-256 attention, whole model) against
the CPU oracle, through the C ABI."""

import pytest
import torch
import torch.nn.functional as F

from oracle import masks as OMK
from oracle import mtp as OM
from oracle.attention import dense_attention
from oracle.eagle3 import DraftShape

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,vocab,dtype", [(37, 1000, torch.float32), (64, 50257, torch.bfloat16),
                                              (16, 151936, torch.bfloat16), (5, 7, torch.float32)])
def test_label_ce_matches_torch_cross_entropy(rows, vocab, dtype):
    from speculators_amd.losses import label_cross_entropy

    g = torch.Generator().manual_seed(rows + vocab)
    x = (torch.randn(rows, vocab, generator=g) * 3).to(dtype)
    lab = torch.randint(0, vocab, (rows,), generator=g)
    lab[::5] = -100
    go = torch.randn(rows, generator=g)
    go[1::7] = 0
    xg = x.cuda().requires_grad_(True)
    loss = label_cross_entropy(xg, lab.cuda())
    loss.backward(go.cuda())
    xr = x.float().requires_grad_(True)
    ref = F.cross_entropy(xr, lab, ignore_index=-100, reduction="none")
    ref.backward(go)
    assert loss.dtype == torch.float32 and loss.shape == (rows,)
    torch.testing.assert_close(loss.cpu(), ref, rtol=1e-5, atol=2e-5)
    assert (loss.cpu()[lab == -100] == 0).all()
    tol = 1e-6 if dtype == torch.float32 else 4e-3  # bf16 gradient rounding: 2^-8 relative
    err = (xg.grad.float().cpu() - xr.grad).abs().max().item()
    assert err <= tol * xr.grad.abs().max().item() + 1e-9, err
    # ignored rows and rows without upstream gradient are exact zeros
    dead = (lab == -100) | (go == 0)
    assert (xg.grad.cpu()[dead] == 0).all()


def test_label_ce_strided_rows_and_argmax_first_index():
    from speculators_amd import _lib

    g = torch.Generator().manual_seed(1)
    full = torch.randn(9, 300, generator=g).bfloat16()
    full[2, 17] = full[2, 250] = 9.0   # tie: the first index wins
    full[4, :] = 1.0                   # all equal
    x = full.cuda()[:, 3:203]          # unaligned, strided rows
    lab = torch.randint(0, 200, (9,), generator=g).cuda()
    out = torch.empty(2, 9, device="cuda")
    am = torch.empty(9, dtype=torch.int32, device="cuda")
    _lib.call("spx_label_ce_fwd", _lib.ptr(x), x.stride(0), _lib.ptr(lab), 9, 200, 0, -100,
              _lib.ptr(out[0]), _lib.ptr(out[1]), _lib.ptr(am), _lib.stream_ptr(x.device))
    xs = full[:, 3:203].float()
    assert torch.equal(am.cpu().long(), xs.argmax(-1))
    assert am[2].item() == 14 and am[4].item() == 0
    torch.testing.assert_close(out[1].cpu(), torch.logsumexp(xs, -1), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(out[0].cpu(), F.cross_entropy(xs, lab.cpu(), reduction="none"),
                               rtol=1e-5, atol=2e-5)


def test_label_ce_bad_label_is_nan_and_errors():
    from speculators_amd import _lib
    from speculators_amd.losses import label_cross_entropy

    x = torch.randn(3, 40).cuda()
    lab = torch.tensor([1, 40, -5]).cuda()
    out = label_cross_entropy(x, lab)
    assert torch.isfinite(out[0]) and torch.isnan(out[1]) and torch.isnan(out[2])
    with pytest.raises(ValueError):
        label_cross_entropy(x, lab[:2])
    with pytest.raises(_lib.SpxError):
        label_cross_entropy(x.half(), lab)


def test_gemm_operand_above_2_gib_in_one_launch():
    """A logits-gradient-sized first operand (2.2 GB) goes through ONE launch: the kernel's 32-bit
    offsets are relative to the tile.  Rows on both sides of the 2 GiB line against an fp32
    product of the same rows."""
    from speculators_amd import gemm

    g = torch.Generator(device="cuda").manual_seed(0)
    m, k, n = 8200, 131080, 264
    a = torch.randn(m, k, device="cuda", generator=g).bfloat16()
    b = (torch.randn(n, k, device="cuda", generator=g) * 0.05).bfloat16()
    assert a.numel() * 2 > 2 ** 31
    got = gemm.gemm_nt(a, b)
    rows = torch.tensor([0, 255, 256, 8190, 8191, 8192, 8193, m - 1], device="cuda")
    want = a[rows].float() @ b.float().t()
    assert (got[rows].float() - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-3
    count = torch.tensor([8195], dtype=torch.int32, device="cuda")
    out = torch.full((m, n), 3.0, dtype=torch.bfloat16, device="cuda")
    gemm.gemm_nt(a, b, out, m_live=count)
    assert (out[8195:] == 3).all()
    assert (out[rows[:-1]].float() - want[:-1]).abs().max() <= 2 ** -8 * want.abs().max() + 1e-3
    # the same rows under a count that keeps all of them: bit for bit (the call without a count
    # may cut its last tiles along the contraction, which sums in another order)
    every = gemm.gemm_nt(a, b, m_live=torch.tensor([m], dtype=torch.int32, device="cuda"))
    assert torch.equal(out[:8195], every[:8195])
    assert (every.float() - got.float()).abs().max() <= 2 ** -7 * want.abs().max()


@pytest.mark.parametrize("t,hq,hkv,docs", [(192, 2, 1, [192]), (300, 4, 2, [100, 130, 70])])
def test_attention_head_dim_256(t, hq, hkv, docs):
    from speculators_amd.attention import create_ttt_mask, ttt_attention

    d = 256
    g = torch.Generator().manual_seed(t)
    doc = torch.cat([torch.full((n,), i) for i, n in enumerate(docs)])
    mask = create_ttt_mask(doc.cuda(), t, None)
    q = torch.randn(1, hq, t, d, generator=g).bfloat16()
    k = torch.randn(1, hkv, t, d, generator=g).bfloat16()
    v = torch.randn(1, hkv, t, d, generator=g).bfloat16()
    go = torch.randn(1, t, hq, d, generator=g).bfloat16()
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = ttt_attention(qg, kg, vg, mask, d ** -0.5)
    out.backward(go.cuda())
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = dense_attention(qr, kr, vr, OMK.ttt_mask_dense(doc, t, 0, None), d ** -0.5)
    ref.backward(go.float())
    err = (out.float().cpu() - ref).abs().max().item()
    assert err <= 2e-2 * ref.abs().max().item(), err
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        err = (got.float().cpu() - want).abs().max().item()
        assert err <= 2e-2 * want.abs().max().item(), (name, err, want.abs().max().item())


@pytest.mark.parametrize("d,hq,hkv", [(64, 4, 2), (128, 2, 1), (256, 2, 1)])
def test_span_attention_under_a_padding_mask(d, hq, hkv):
    """Attention with one key interval per query (right- and left-padded rows, an all-padding row):
    forward and backward against the dense oracle under the padding-mask form of the causal mask."""
    from speculators_amd.attention import create_padding_span_mask, span_attention

    b, n = 4, 96
    am = torch.ones(b, n, dtype=torch.long)
    am[0, 70:] = 0   # right padding
    am[1, :25] = 0   # left padding
    am[3, :] = 0     # nothing but padding
    t = b * n
    g = torch.Generator().manual_seed(d)
    q = torch.randn(1, hq, t, d, generator=g).bfloat16()
    k = torch.randn(1, hkv, t, d, generator=g).bfloat16()
    v = torch.randn(1, hkv, t, d, generator=g).bfloat16()
    go = torch.randn(1, t, hq, d, generator=g).bfloat16()
    mask = create_padding_span_mask(am.cuda())
    # the packed row never mixes batch rows: block diagonal of the per-row masks
    dense = torch.zeros(t, t, dtype=torch.bool)
    per_row = OM.padded_causal_mask(am)
    for r in range(b):
        dense[r * n:(r + 1) * n, r * n:(r + 1) * n] = per_row[r]
    lo, hi = mask.row_lo.cpu(), mask.row_hi.cpu()
    idx = torch.arange(t)
    assert torch.equal(dense, (idx[None, :] >= lo[:, None]) & (idx[None, :] < hi[:, None]))
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = span_attention(qg, kg, vg, mask, d ** -0.5)
    out.backward(go.cuda())
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = dense_attention(qr, kr, vr, dense, d ** -0.5)
    ref.backward(go.float())
    assert (out.float().cpu() - ref).abs().max() <= 2e-2 * ref.abs().max()
    assert not out[0, 3 * n:].any()  # queries that see nothing give zeros
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        err = (got.float().cpu() - want).abs().max().item()
        assert err <= 2e-2 * want.abs().max().item(), (name, err, want.abs().max().item())
    with pytest.raises(ValueError, match="contiguous run"):
        create_padding_span_mask(torch.tensor([[1, 0, 1, 1]]).cuda())


def test_model_with_a_padding_mask_matches_oracle():
    """``attention_mask`` (models/mtp/core.py:119,180-186): right- and left-padded rows.  The padded
    positions are kept out of the loss; logits are compared where the mask marks a token."""
    shape = _shape()
    steps = 2
    w = {k: v.bfloat16() for k, v in OM.random_weights(shape, seed=4, std=0.05).items()}
    g = torch.Generator().manual_seed(9)
    b, n = 2, 150
    ids = torch.randint(0, shape.vocab_size, (b, n), generator=g)
    hs = torch.randn(b, n, shape.hidden_size, generator=g).bfloat16()
    am = torch.ones(b, n, dtype=torch.long)
    am[0, 110:] = 0
    am[1, :30] = 0
    lm = ((torch.rand(b, n, generator=g) < 0.7) & (am != 0)).float()
    model = _make(shape, w, steps)
    logits, loss, m = model(ids.cuda(), hs.cuda(), attention_mask=am.cuda(), loss_mask=lm.cuda())
    loss.backward()
    wf = {k: v.float().requires_grad_(True) for k, v in w.items()}
    rl, rloss, rm = OM.mtp_forward(wf, shape, ids, hs.float(), loss_mask=lm, num_steps=steps,
                                   attention_mask=am)
    rloss.backward()
    assert abs(loss.item() - rloss.item()) <= 1e-3 * abs(rloss.item())
    valid = n - steps - 1
    tok = am[:, :valid] != 0
    for k in range(steps):
        got, want = logits[k].float().cpu()[tok], rl[k][tok]
        assert (got - want).abs().max() <= 2e-2 * want.abs().max(), k
    for name, p in model.named_parameters():
        if p.requires_grad:
            want = wf[name].grad
            assert (p.grad.float().cpu() - want).abs().max() <= 3e-2 * want.abs().max() + 1e-6, name
    # without the mask the same call splits the rows at position restarts instead: a different result
    with pytest.raises(ValueError, match="attention_mask must be"):
        model(ids.cuda(), hs.cuda(), attention_mask=am[:, :10].cuda())


def _shape(**kw):
    base = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
                intermediate_size=512, vocab_size=1000, draft_vocab_size=1000, rms_norm_eps=1e-6,
                rope_theta=10000.0, qk_norm=True)
    base.update(kw)
    return DraftShape(**base)


def _make(shape, w, steps):
    from speculators_amd.mtp import MTPConfig, MTPDraftModel

    cfg = MTPConfig(hidden_size=shape.hidden_size, num_attention_heads=shape.num_attention_heads,
                    num_key_value_heads=shape.num_key_value_heads, head_dim=shape.head_dim,
                    intermediate_size=shape.intermediate_size, vocab_size=shape.vocab_size,
                    num_speculative_steps=steps, rms_norm_eps=shape.rms_norm_eps,
                    rope_theta=shape.rope_theta)
    model = MTPDraftModel(cfg)
    missing, unexpected = model.load_state_dict(w, strict=True)
    return model.to(torch.bfloat16).cuda()


@pytest.mark.parametrize("variant", [dict(), dict(head_dim=128, num_attention_heads=2, num_key_value_heads=1),
                                     dict(head_dim=256, num_attention_heads=2, num_key_value_heads=1),
                                     dict(head_dim=96, num_attention_heads=2, num_key_value_heads=1)])
def test_model_forward_backward_matches_oracle(variant):
    shape = _shape(**variant)
    steps = 3
    w32 = OM.random_weights(shape, seed=2, std=0.05)
    w = {k: v.bfloat16() for k, v in w32.items()}
    g = torch.Generator().manual_seed(5)
    b, n = 2, 200
    ids = torch.randint(0, shape.vocab_size, (b, n), generator=g)
    hs = torch.randn(b, n, shape.hidden_size, generator=g).bfloat16()
    pos = torch.stack([torch.cat([torch.arange(70), torch.arange(90), torch.arange(40)]),
                       torch.arange(n)])
    lm = (torch.rand(b, n, generator=g) < 0.7).float()
    sw = OM.compute_step_weights(0.6, steps)

    model = _make(shape, w, steps)
    logits, loss, m = model(ids.cuda(), hs.cuda(), position_ids=pos.cuda(), loss_mask=lm.cuda(),
                            step_weights=sw)
    loss.backward()

    wf = {k: v.float().requires_grad_(True) for k, v in w.items()}
    rl, rloss, rm = OM.mtp_forward(wf, shape, ids, hs.float(), position_ids=pos, loss_mask=lm,
                                   step_weights=sw, num_steps=steps)
    rloss.backward()
    rel = abs(loss.item() - rloss.item()) / abs(rloss.item())
    print("loss", loss.item(), rloss.item(), rel)
    assert rel < 1e-3
    assert set(m) == set(rm)
    for k in range(steps):
        assert logits[k].shape == rl[k].shape == (b, n - steps - 1, shape.vocab_size)
        err = (logits[k].float().cpu() - rl[k]).abs().max().item()
        assert err <= 2e-2 * rl[k].abs().max().item(), (k, err)
        assert abs(m[f"loss_step_{k}"].item() - rm[f"loss_step_{k}"].item()) <= 1e-3 * rm[f"loss_step_{k}"].item()
    # the same oracle in bf16 on the CPU gives the rounding noise floor of this model
    wb = {k: v.clone().requires_grad_(True) for k, v in w.items()}
    _, bloss, _ = OM.mtp_forward(wb, shape, ids, hs, position_ids=pos, loss_mask=lm, step_weights=sw,
                                 num_steps=steps)
    bloss.backward()
    for name, p in model.named_parameters():
        if not p.requires_grad:
            assert p.grad is None
            continue
        want = wf[name].grad
        scale = want.abs().max().item()
        err = (p.grad.float().cpu() - want).abs().max().item()
        floor = (wb[name].grad.float() - want).abs().max().item()
        assert err <= max(2e-2 * scale, 2 * floor) + 1e-6, (name, err, floor, scale)


def test_model_properties_of_the_reference_tests():
    # tests/unit/models/test_mtp_model.py on the HIP path
    shape = _shape()
    w = {k: v.bfloat16() for k, v in OM.random_weights(shape, seed=3, std=0.05).items()}
    model = _make(shape, w, 3)
    g = torch.Generator().manual_seed(9)
    ids = torch.randint(0, shape.vocab_size, (1, 40), generator=g).cuda()
    hs = torch.randn(1, 40, shape.hidden_size, generator=g).bfloat16().cuda()
    with torch.no_grad():
        logits, loss, m = model(ids, hs)
        assert len(logits) == 3 and logits[0].shape == (1, 36, shape.vocab_size)
        assert set(m) == {"loss_step_0", "loss_step_1", "loss_step_2", "loss_sum", "loss_total"}
        _, l0, _ = model(ids, hs, loss_mask=torch.zeros(1, 40, device="cuda"))
        assert l0.item() == 0.0
        _, _, mz = model(ids, hs, step_weights=[1.0, 0.0, 0.0])
        assert mz["loss_step_0"] > 0 and mz["loss_step_1"] == 0.0 and mz["loss_step_2"] == 0.0
        short, _, _ = model(ids[:, :3], hs[:, :3])
        assert len(short) == 1
        with pytest.raises(ValueError, match="expected exactly 3 weights"):
            model(ids, hs, step_weights=[1.0])
        # an all-ones padding mask and a single packed sequence are the same mask
        with_mask, _, _ = model(ids, hs, attention_mask=torch.ones_like(ids))
        plain, _, _ = model(ids, hs)
        assert all(torch.equal(a, b_) for a, b_ in zip(with_mask, plain, strict=True))
        with pytest.raises(RuntimeError, match="bf16"):
            model(ids, hs.float())


def test_head_and_loss_as_one_node_equals_the_two_node_path():
    """Frozen head + label cross-entropy as one autograd node (packed loss backward, row-counted
    input-gradient product) against linear + label_cross_entropy: same losses, same logits, and
    the same input gradient bit for bit -- zero rows included.  (With the row statistics taken from
    the head product's epilogue the log-sum-exp is summed in another order: that form is compared in
    test_head_cross_entropy_with_epilogue_statistics_equals_the_streaming_form.)"""
    from speculators_amd import gemm
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(3)
    rows, h, v = 700, 128, 1000
    x = torch.randn(2, rows // 2, h, generator=g).bfloat16().cuda()
    w = (torch.randn(v, h, generator=g) * 0.05).bfloat16().cuda()
    wt = w.t().contiguous()
    labels = torch.randint(0, v, (2, rows // 2), generator=g)
    labels[torch.rand(2, rows // 2, generator=g) < 0.35] = -100
    labels[0, :5] = -100           # a dead run at the very start
    labels = labels.cuda()
    gw = torch.rand(2, rows // 2, generator=g).cuda()
    gw[1, 7] = 0.0                  # a live label with a zero incoming gradient

    x1 = x.clone().requires_grad_(True)
    loss1, logits1 = L.head_label_cross_entropy(x1, w, wt, labels, epilogue_stats=False)
    (loss1 * gw).sum().backward()
    x2 = x.clone().requires_grad_(True)
    logits2 = gemm.linear(x2, w, wt)
    loss2 = L.label_cross_entropy(logits2, labels)
    (loss2 * gw).sum().backward()
    assert torch.equal(loss1, loss2) and torch.equal(logits1, logits2.detach())
    assert not logits1.requires_grad
    assert torch.equal(x1.grad, x2.grad)
    dead = (labels == -100) | (gw == 0)
    assert (x1.grad[dead] == 0).all() and (x1.grad[~dead] != 0).any()


@pytest.mark.parametrize("frac", [0.0, 1.0])
def test_head_and_loss_node_with_no_or_all_rows_live(frac):
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, 300, 64, generator=g).bfloat16().cuda().requires_grad_(True)
    w = (torch.randn(520, 64, generator=g) * 0.05).bfloat16().cuda()
    labels = torch.randint(0, 520, (1, 300), generator=g).cuda()
    if frac == 0.0:
        labels[:] = -100
    loss, _ = L.head_label_cross_entropy(x, w, w.t().contiguous(), labels)
    loss.sum().backward()
    ref = x.detach().clone().requires_grad_(True)
    L.label_cross_entropy((ref.float() @ w.float().t()).bfloat16(), labels)  # shape / dtype check only
    if frac == 0.0:
        assert (x.grad == 0).all() and (loss == 0).all()
    else:
        assert torch.isfinite(x.grad.float()).all() and (x.grad != 0).any()


def test_model_with_and_without_the_fused_head_node_agree(monkeypatch):
    """The MTP model's loss, logits and parameter gradients do not depend on whether the head and
    the loss are one autograd node or two (bit for bit: the packed product computes the same
    dot products in the same order; the row statistics streamed in both, not taken from the head
    product's epilogue, whose sum runs in another order)."""
    from speculators_amd import losses as L

    monkeypatch.setattr(L, "HEAD_CE_EPILOGUE_STATS", False)
    shape = _shape()
    steps = 2
    w = {k: v.bfloat16() for k, v in OM.random_weights(shape, seed=4, std=0.05).items()}
    g = torch.Generator().manual_seed(9)
    b, n = 2, 150
    ids = torch.randint(0, shape.vocab_size, (b, n), generator=g).cuda()
    hs = torch.randn(b, n, shape.hidden_size, generator=g).bfloat16().cuda()
    lm = (torch.rand(b, n, generator=g) < 0.6).float().cuda()
    got = []
    for fuse in (True, False):
        model = _make(shape, w, steps)
        model.fuse_head_loss = fuse
        logits, loss, _ = model(ids, hs, loss_mask=lm)
        loss.backward()
        got.append((loss.detach(), [x.detach() for x in logits],
                    {k: p.grad.clone() for k, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(got[0][0], got[1][0])
    for x, y in zip(got[0][1], got[1][1]):
        assert torch.equal(x, y)
    assert got[0][2].keys() == got[1][2].keys() and len(got[0][2]) > 0
    for k in got[0][2]:
        assert torch.equal(got[0][2][k], got[1][2][k]), k


@pytest.mark.parametrize("rows,hidden,vocab", [(300, 128, 5000), (520, 256, 151936)])
def test_head_cross_entropy_with_epilogue_statistics_equals_the_streaming_form(rows, hidden, vocab):
    """The frozen head + label cross-entropy node with the row log-sum-exp taken from the head
    product's epilogue (``spx_gemm_bf16_nt_stats`` + ``spx_label_ce_from_lse``) against the form
    that streams the logits again (``spx_label_ce_fwd``): same logits bit for bit, losses within
    1e-6 relative (exact zeros at ignored labels, NaN at a bad label in both), input gradients within
    the rounding of one bf16 step, and the loss against ``F.cross_entropy`` on the same logits."""
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, hidden, generator=g).bfloat16().cuda()
    w = (torch.randn(vocab, hidden, generator=g) * 0.05).bfloat16().cuda()
    wt = w.t().contiguous()
    labels = torch.randint(0, vocab, (rows,), generator=g)
    labels[::7] = -100
    labels = labels.cuda()
    gr = torch.randn(rows, generator=g).cuda()
    res = []
    for epi in (True, False):
        xi = x.clone().requires_grad_(True)
        loss, logits = L.head_label_cross_entropy(xi, w, wt, labels, -100, epilogue_stats=epi)
        (loss * gr).sum().backward()
        res.append((loss.detach(), logits, xi.grad))
    (la, ga, da), (lb, gb, db) = res
    assert torch.equal(ga.view(torch.int16), gb.view(torch.int16))
    assert (la[::7] == 0).all() and (lb[::7] == 0).all()
    assert ((la - lb).abs() <= 1e-6 * lb.abs() + 1e-6).all()
    ref = torch.nn.functional.cross_entropy(ga.float(), labels, ignore_index=-100, reduction="none")
    assert ((la - ref).abs() <= 2e-6 * ref.abs() + 2e-6).all()
    assert (da.float() - db.float()).abs().max() <= 1e-2 * db.float().abs().max()
    bad = labels.clone()
    bad[1] = vocab + 3
    lo, _ = L.head_label_cross_entropy(x, w, wt, bad, -100, epilogue_stats=True)
    assert torch.isnan(lo[1]) and torch.isfinite(lo[2])
