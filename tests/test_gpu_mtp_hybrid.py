"""HIP path of the hybrid MTP flavours (gated attention, partial rotary embedding, gain 1 + w
norms, sparse MoE with grouped expert products) against the CPU oracle, through the C ABI."""

import pytest
import torch
import torch.nn.functional as F

from oracle import mtp as OM

pytestmark = pytest.mark.gpu


def _groups(sizes):
    off = torch.zeros(len(sizes) + 1, dtype=torch.int32)
    off[1:] = torch.tensor(sizes).cumsum(0)
    return off


@pytest.mark.parametrize("sizes,n,k", [([5, 0, 300, 256, 1, 0, 77], 264, 136), ([512], 512, 64),
                                       ([0, 0, 3], 8, 8), ([257, 255, 256, 700], 1000, 520)])
def test_grouped_nt_product(sizes, n, k):
    """Rows sorted by group, every group against its own weight: empty groups, groups below,
    at and above the 256-row tile, ragged N and K."""
    from speculators_amd.moe import gemm_nt_grouped

    g = torch.Generator().manual_seed(sum(sizes) + n)
    rows = sum(sizes)
    a = torch.randn(rows, k, generator=g).bfloat16()
    b = torch.randn(len(sizes), n, k, generator=g).bfloat16()
    off = _groups(sizes)
    out = torch.full((rows + 3, n), 7.0, dtype=torch.bfloat16, device="cuda")
    got = gemm_nt_grouped(a.cuda(), b.cuda(), off.cuda(), out=out[:rows])
    assert (out[rows:] == 7).all()
    r0 = 0
    for e, sz in enumerate(sizes):
        want = a[r0:r0 + sz].float() @ b[e].float().t()
        if sz:
            err = (got[r0:r0 + sz].float().cpu() - want).abs().max().item()
            assert err <= 2 ** -8 * want.abs().max().item() + 1e-3, (e, err)
        r0 += sz


@pytest.mark.parametrize("sizes,m,n", [([5, 0, 300, 64, 1, 0, 77], 264, 136), ([0, 0, 3], 8, 8),
                                       ([130, 255, 70], 512, 520)])
@pytest.mark.parametrize("fp32", [False, True])
def test_grouped_tn_product(sizes, m, n, fp32):
    """Per-group weight gradients dY_e^T X_e: an empty group gets zeros, or is left alone when the
    product is added."""
    from speculators_amd.moe import gemm_tn_grouped

    g = torch.Generator().manual_seed(sum(sizes) + m)
    rows = sum(sizes)
    a = torch.randn(rows, m, generator=g).bfloat16()
    b = torch.randn(rows, n, generator=g).bfloat16()
    off = _groups(sizes).cuda()
    dt = torch.float32 if fp32 else torch.bfloat16
    out = torch.full((len(sizes), m, n), 3.0, dtype=dt, device="cuda")
    gemm_tn_grouped(a.cuda(), b.cuda(), off, out)
    tol = 2e-6 * max(sizes) ** 0.5 if fp32 else 2 ** -8
    want = torch.zeros(len(sizes), m, n)
    r0 = 0
    for e, sz in enumerate(sizes):
        want[e] = a[r0:r0 + sz].float().t() @ b[r0:r0 + sz].float()
        r0 += sz
    for e in range(len(sizes)):
        err = (out[e].float().cpu() - want[e]).abs().max().item()
        assert err <= tol * want[e].abs().max().item() + 1e-3, (e, err)
    first = out.clone()
    gemm_tn_grouped(a.cuda(), b.cuda(), off, out, accumulate=True)
    for e in range(len(sizes)):
        err = (out[e].float().cpu() - 2 * first[e].float().cpu()).abs().max().item()
        assert err <= 2 ** -7 * want[e].abs().max().item() + 1e-3, (e, err)


@pytest.mark.parametrize("fp32", [False, True])
def test_grouped_tn_product_over_several_segments(fp32):
    """One product over the sorted rows of several uses: segments with different group sizes, a
    group that is empty in some segments or in all, a segment that contributes nothing (offsets
    all zero), group sizes around the 64-row slab."""
    from speculators_amd.moe import gemm_tn_grouped_multi

    seg_sizes = [[5, 0, 130, 64, 1, 0, 56], [0, 0, 7, 200, 49, 0, 0], [0] * 7, [63, 0, 65, 0, 128, 0, 0]]
    rows, m, n = 256, 264, 136
    g = torch.Generator().manual_seed(11)
    a = torch.randn(len(seg_sizes) * rows, m, generator=g).bfloat16()
    b = torch.randn(len(seg_sizes) * rows, n, generator=g).bfloat16()
    off = torch.stack([_groups(sz) for sz in seg_sizes])
    off[2] = 0
    want = torch.zeros(7, m, n, dtype=torch.float64)
    for s_, sz in enumerate(seg_sizes):
        if s_ == 2:
            continue
        r0 = s_ * rows
        for e, c in enumerate(sz):
            want[e] += a[r0:r0 + c].double().t() @ b[r0:r0 + c].double()
            r0 += c
    dt = torch.float32 if fp32 else torch.bfloat16
    out = torch.full((7, m, n), 3.0, dtype=dt, device="cuda")
    gemm_tn_grouped_multi(a.cuda(), b.cuda(), off.cuda(), out)
    tol = 1e-5 if fp32 else 2 ** -8
    for e in range(7):
        err = (out[e].double().cpu() - want[e]).abs().max().item()
        assert err <= tol * want[e].abs().max().item() + 1e-3, (e, err)
    assert (out[1] == 0).all() and (out[5] == 0).all()  # empty everywhere: zeros written
    first = out.clone()
    gemm_tn_grouped_multi(a.cuda(), b.cuda(), off.cuda(), out, accumulate=True)
    assert (out.double() - 2 * first.double()).abs().max() <= 2 ** -7 * want.abs().max() + 1e-3


def test_row_movement_kernels():
    """gather / combine / pair dot against index arithmetic; bad indices give zero rows."""
    from speculators_amd import moe

    g = torch.Generator().manual_seed(0)
    t, k, h, e = 37, 3, 72, 5
    x = torch.randn(t, h, generator=g).bfloat16().cuda()
    idx = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(t)]).cuda()
    order, src_row, pos, off = moe.sort_pairs(idx, e)
    flat = idx.reshape(-1)
    assert torch.equal(flat[order], flat[order].sort().values)
    assert torch.equal(off.cpu()[1:], torch.bincount(flat.cpu(), minlength=e).cumsum(0).int())
    assert torch.equal(order[pos.reshape(-1).long()], torch.arange(t * k, device="cuda"))
    xs = moe.gather_rows(x, src_row)
    assert torch.equal(xs, x[src_row.long()])
    scale = torch.rand(t * k, generator=g).cuda()
    xs2 = moe.gather_rows(x, src_row, scale)
    assert torch.equal(xs2, (x[src_row.long()].float() * scale[:, None]).bfloat16())
    bad = src_row.clone()
    bad[3] = -1
    bad[5] = t
    xb = moe.gather_rows(x, bad)
    assert (xb[3] == 0).all() and (xb[5] == 0).all() and torch.equal(xb[4], xs[4])
    w = torch.rand(t, k, generator=g).cuda()
    ys = torch.randn(t * k, h, generator=g).bfloat16().cuda()
    want = (ys[pos.long()].float() * w[:, :, None]).sum(1)
    got = moe.combine_rows(ys, pos, w)
    assert (got.float() - want).abs().max() <= 2 ** -8 * want.abs().max()
    got1 = moe.combine_rows(ys, pos, None)
    want1 = ys[pos.long()].float().sum(1)
    assert (got1.float() - want1).abs().max() <= 2 ** -8 * want1.abs().max()
    d = moe.pair_dot(x, ys, pos)
    wantd = (x.float()[:, None, :] * ys[pos.long()].float()).sum(-1)
    assert torch.allclose(d, wantd, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("d,rot", [(64, 16), (128, 64), (256, 64), (64, 64)])
def test_partial_rotary_relayout(d, rot):
    """Rotation of the first ``rot`` elements of every head + relayout, forward and backward,
    against the oracle's partial rotary embedding."""
    from speculators_amd import fused_ops as FO

    g = torch.Generator().manual_seed(d + rot)
    t, heads = 50, 3
    x = torch.randn(1, t, heads * d, generator=g).bfloat16()
    pos = torch.randint(0, 4000, (t,), generator=g)
    inv = FO.rope_inv_freq(rot, 10000.0, "cuda")
    xg = x.cuda().requires_grad_(True)
    out = FO.rope_relayout(xg, pos.cuda(), inv, heads, True, 0)
    go = torch.randn(out.shape, generator=g).bfloat16()
    out.backward(go.cuda())
    cos, sin = OM.rope_tables(pos, rot, 10000.0, torch.bfloat16)
    xr = x.float().requires_grad_(True)
    want = OM.apply_partial_rope(xr.view(1, t, heads, d).transpose(1, 2), cos.float(), sin.float())
    want.backward(go.float())
    assert (out.float().cpu() - want).abs().max() <= 2e-2 * want.abs().max()
    assert torch.equal(out[..., rot:].cpu(), x.view(1, t, heads, d).transpose(1, 2)[..., rot:])
    assert (xg.grad.float().cpu() - xr.grad).abs().max() <= 2e-2 * xr.grad.abs().max()


def test_query_gate_split_and_sigmoid_gate():
    from speculators_amd import fused_ops as FO

    g = torch.Generator().manual_seed(3)
    t, heads, d = 33, 3, 64
    y = torch.randn(1, t, heads * 2 * d, generator=g).bfloat16()
    o = torch.randn(1, t, heads * d, generator=g).bfloat16()
    go = torch.randn(1, t, heads * d, generator=g).bfloat16()
    yg, og = y.cuda().requires_grad_(True), o.cuda().requires_grad_(True)
    q, gate = FO.split_query_gate(yg, heads)
    out = FO.sigmoid_gate(og, gate)
    (out * go.cuda()).sum().backward(retain_graph=True)
    qsum = (q.float() * 2).sum()
    qsum.backward()
    yr, orf = y.float().requires_grad_(True), o.float().requires_grad_(True)
    qr, gr = torch.chunk(yr.view(1, t, heads, 2 * d), 2, dim=-1)
    want = orf * torch.sigmoid(gr.reshape(1, t, heads * d))
    ((want * go.float()).sum() + (qr * 2).sum()).backward()
    assert torch.equal(q.cpu(), qr.detach().bfloat16().view(t, heads, d))
    # the bf16 eager form: sigmoid rounded, product rounded
    eager = o * torch.sigmoid(gr.detach().reshape(1, t, heads * d).bfloat16())
    assert (out.cpu() == eager).float().mean() > 0.995
    assert (og.grad.float().cpu() - orf.grad).abs().max() <= 1e-2 * orf.grad.abs().max()
    assert (yg.grad.float().cpu() - yr.grad).abs().max() <= 1e-2 * yr.grad.abs().max()


def _hybrid_shape(**kw):
    base = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
                intermediate_size=512, vocab_size=1000, draft_vocab_size=1000, rms_norm_eps=1e-6,
                rope_theta=10000.0)
    base.update(kw)
    return OM.HybridShape(**base)


_MOE = dict(num_experts=8, num_experts_per_tok=2, moe_intermediate_size=64, shared_expert_intermediate_size=128)


def _make(shape, w, steps, dtype=torch.bfloat16):
    from speculators_amd.mtp import MTPConfig, MTPDraftModel

    cfg = MTPConfig(hidden_size=shape.hidden_size, num_attention_heads=shape.num_attention_heads,
                    num_key_value_heads=shape.num_key_value_heads, head_dim=shape.head_dim,
                    intermediate_size=shape.intermediate_size, vocab_size=shape.vocab_size,
                    num_speculative_steps=steps, rms_norm_eps=shape.rms_norm_eps, rope_theta=shape.rope_theta,
                    model_type=shape.model_type, partial_rotary_factor=shape.partial_rotary_factor,
                    num_experts=shape.num_experts, num_experts_per_tok=shape.num_experts_per_tok,
                    moe_intermediate_size=shape.moe_intermediate_size,
                    shared_expert_intermediate_size=shape.shared_expert_intermediate_size,
                    norm_topk_prob=shape.norm_topk_prob)
    model = MTPDraftModel(cfg)
    model.load_state_dict(w, strict=True)
    return model.to(dtype).cuda()


def _check_routing(rt):
    """The HIP top-k is a top-k of the oracle's router logits up to near ties: the sets agree for
    almost every token, and where they differ the logits of the exchanged experts lie within a few
    bf16 steps of each other (the HIP router works on bf16 logits of bf16 activations)."""
    own, hip_idx, logits = rt["own"], rt["forced"], rt["logits"]
    same = (own.sort(-1).values == hip_idx.sort(-1).values).all(-1)
    assert same.float().mean() >= 0.95, same.float().mean()
    for t in (~same).nonzero().flatten().tolist():
        mine, theirs = set(own[t].tolist()), set(hip_idx[t].tolist())
        lo = min(logits[t, e].item() for e in mine - theirs)
        hi = max(logits[t, e].item() for e in theirs - mine)
        assert abs(lo - hi) <= 2 ** -5 * max(abs(lo), abs(hi), 1.0), (t, lo, hi)


@pytest.mark.parametrize("renorm", [True, False])
def test_sparse_moe_block_matches_oracle(renorm):
    """The block alone, forward and backward, every parameter's gradient; the oracle is given the
    HIP path's expert choice where the two differ on a near tie."""
    from speculators_amd.hybrid import SparseMoeBlock
    from speculators_amd.weights import WeightStager

    shape = _hybrid_shape(num_experts=6, num_experts_per_tok=3, moe_intermediate_size=72,
                          shared_expert_intermediate_size=40, norm_topk_prob=renorm)
    p = "mtp_layers.0.mlp."
    w32 = {k[len(p):]: v for k, v in OM.random_weights(shape, 4, std=0.05).items() if k.startswith(p)}
    w = {k: v.bfloat16() for k, v in w32.items()}
    stager = WeightStager()
    block = SparseMoeBlock(shape, stager)
    block.load_state_dict(w, strict=True)
    block = block.bfloat16().cuda()
    block.routing_log = []
    g = torch.Generator().manual_seed(8)
    t = 300
    x = torch.randn(1, t, shape.hidden_size, generator=g).bfloat16()
    go = torch.randn(1, t, shape.hidden_size, generator=g).bfloat16()
    stager.begin()
    xg = x.cuda().requires_grad_(True)
    out = block(xg)
    out.backward(go.cuda())
    hip_idx = block.routing_log[0].cpu()

    wf = {p + k: v.float().requires_grad_(True) for k, v in w.items()}
    xr = x.float().requires_grad_(True)
    routing = {"forced": hip_idx}
    want = OM.sparse_moe(xr, wf, p, shape, routing)
    want.backward(go.float())
    _check_routing(routing)
    assert (out.float().cpu() - want).abs().max() <= 2e-2 * want.abs().max()
    assert (xg.grad.float().cpu() - xr.grad).abs().max() <= 2e-2 * xr.grad.abs().max()
    for name, prm in block.named_parameters():
        ref = wf[p + name].grad
        err = (prm.grad.float().cpu() - ref).abs().max().item()
        assert err <= 2e-2 * ref.abs().max().item() + 1e-6, (name, err, ref.abs().max().item())


@pytest.mark.parametrize("model_type,kw,master", [
    ("qwen3_next", dict(_MOE), False),
    ("qwen3_next", dict(_MOE, norm_topk_prob=False, head_dim=128, num_attention_heads=2, num_key_value_heads=1,
                        partial_rotary_factor=0.5), False),
    ("qwen3_next", dict(head_dim=256, num_attention_heads=2, num_key_value_heads=1), False),
    ("qwen3_5_text", dict(), False),
    ("qwen3_5_moe_text", dict(_MOE), False),
    ("qwen3_5_moe_text", dict(_MOE), True),
])
def test_hybrid_model_forward_backward_matches_oracle(model_type, kw, master):
    """Whole model of every hybrid flavour (``master``: fp32 master weights under bf16 autocast,
    the trainer's regime): loss, per-step losses, logits and every gradient against the fp32
    oracle run with the HIP path's expert choice."""
    shape = _hybrid_shape(model_type=model_type, **kw)
    steps = 3
    w32 = OM.random_weights(shape, seed=2, std=0.05)
    w = {k: v.bfloat16() for k, v in w32.items()}
    g = torch.Generator().manual_seed(5)
    b, n = 2, 200
    ids = torch.randint(0, shape.vocab_size, (b, n), generator=g)
    hs = torch.randn(b, n, shape.hidden_size, generator=g).bfloat16()
    pos = torch.stack([torch.cat([torch.arange(70), torch.arange(90), torch.arange(40)]), torch.arange(n)])
    lm = (torch.rand(b, n, generator=g) < 0.7).float()
    sw = OM.compute_step_weights(0.6, steps)
    valid = n - steps - 1

    if master:
        model = _make(shape, {k: v.float() for k, v in w.items()}, steps, torch.float32)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            moe_block = model.mtp_layers[0].mlp
            moe_block.routing_log = []
            logits, loss, m = model(ids.cuda(), hs.cuda(), position_ids=pos.cuda(), loss_mask=lm.cuda(),
                                    step_weights=sw)
    else:
        model = _make(shape, w, steps)
        moe_block = model.mtp_layers[0].mlp
        if shape.num_experts:
            moe_block.routing_log = []
        logits, loss, m = model(ids.cuda(), hs.cuda(), position_ids=pos.cuda(), loss_mask=lm.cuda(),
                                step_weights=sw)
    loss.backward()

    routing = None
    if shape.num_experts:
        routing = [{"forced": moe_block.routing_log[s].cpu().view(b, valid, -1)[r]}
                   for s in range(steps) for r in range(b)]
    wf = {k: v.float().requires_grad_(True) for k, v in w.items()}
    rl, rloss, rm = OM.mtp_forward(wf, shape, ids, hs.float(), position_ids=pos, loss_mask=lm, step_weights=sw,
                                   num_steps=steps, routing=routing)
    rloss.backward()
    if routing:
        for s in range(steps):
            for r in range(b):
                _check_routing(routing[s * b + r])
    rel = abs(loss.item() - rloss.item()) / abs(rloss.item())
    print("loss", loss.item(), rloss.item(), rel)
    assert rel < 1e-3
    assert set(m) == set(rm)
    for k in range(steps):
        err = (logits[k].float().cpu() - rl[k]).abs().max().item()
        assert err <= 2e-2 * rl[k].abs().max().item(), (k, err)
        assert abs(m[f"loss_step_{k}"].item() - rm[f"loss_step_{k}"].item()) <= 1e-3 * rm[f"loss_step_{k}"].item()
    # the same oracle in bf16 on the CPU (same expert choice) gives the rounding noise floor
    wb = {k: v.clone().requires_grad_(True) for k, v in w.items()}
    rb = None if routing is None else [{"forced": rt["forced"]} for rt in routing]
    _, bloss, _ = OM.mtp_forward(wb, shape, ids, hs, position_ids=pos, loss_mask=lm, step_weights=sw,
                                 num_steps=steps, routing=rb)
    bloss.backward()
    for name, prm in model.named_parameters():
        if not prm.requires_grad:
            assert prm.grad is None
            continue
        assert prm.grad.dtype == prm.dtype
        want = wf[name].grad
        scale = want.abs().max().item()
        err = (prm.grad.float().cpu() - want).abs().max().item()
        floor = (wb[name].grad.float() - want).abs().max().item()
        assert err <= max(2e-2 * scale, 2 * floor) + 1e-6, (name, err, floor, scale)


def test_moe_block_at_the_qwen3_next_sizes():
    """512 experts, top-10, hidden 2048, expert width 512 (the Qwen3-Next-80B-A3B MTP layer) on 6000
    tokens: sampled tokens against a per-token fp32 evaluation with the block's own expert choice,
    equivariance under a permutation of the tokens, and a sampled expert's weight gradient against
    the fp32 product over exactly the tokens routed to it."""
    from types import SimpleNamespace

    from speculators_amd.hybrid import SparseMoeBlock
    from speculators_amd.weights import WeightStager

    cfg = SimpleNamespace(hidden_size=2048, num_experts=512, num_experts_per_tok=10, moe_intermediate_size=512,
                          shared_expert_intermediate_size=512, norm_topk_prob=True)
    torch.manual_seed(0)
    stager = WeightStager()
    block = SparseMoeBlock(cfg, stager)
    with torch.no_grad():
        for name, prm in block.named_parameters():
            prm.normal_(0.0, 0.3 if name == "gate.weight" else 0.03)
        # expert 7 is a favourite (more than one 256-row tile of tokens), experts 500.. are avoided
        block.gate.weight[7, 0] = 4.0
        block.gate.weight[500:, 0] = -40.0
    block = block.bfloat16().cuda()
    block.routing_log = []
    t = 6000
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(1, t, 2048, device="cuda", generator=g)
    x[..., 0] = x[..., 0].abs() + 0.5
    x = x.bfloat16().requires_grad_(True)
    go = torch.randn(1, t, 2048, device="cuda", generator=g).bfloat16()
    stager.begin()
    out = block(x)
    out.backward(go)
    idx = block.routing_log[0]
    assert idx.shape == (t, 10) and (idx.sort(-1).values.diff(dim=-1) > 0).all()  # ten distinct experts
    counts = torch.bincount(idx.reshape(-1), minlength=512)
    assert counts.sum() == t * 10 and counts.max() > 256  # some expert spans more than one tile

    w = {k: v.detach().float() for k, v in block.named_parameters()}
    rows = torch.randint(0, t, (24,), device="cuda", generator=g)
    xs = x.detach()[0, rows].float()
    probs = F.softmax((x.detach()[0, rows] @ block.gate.weight.t()).float(), dim=-1)
    sc = probs.gather(1, idx[rows])
    sc = (sc / sc.sum(-1, keepdim=True)).bfloat16().float()
    want = torch.zeros(24, 2048, device="cuda")
    for i in range(24):
        for j in range(10):
            e = int(idx[rows[i], j])
            a, b = (w["experts.gate_up_proj"][e] @ xs[i]).chunk(2)
            want[i] += sc[i, j] * (w["experts.down_proj"][e] @ (F.silu(a) * b))
        a, b = w["shared_expert.gate_proj.weight"] @ xs[i], w["shared_expert.up_proj.weight"] @ xs[i]
        gate = torch.sigmoid(w["shared_expert_gate.weight"] @ xs[i])
        want[i] += gate * (w["shared_expert.down_proj.weight"] @ (F.silu(a) * b))
    err = (out[0, rows].float() - want).abs().max().item()
    assert err <= 2e-2 * want.abs().max().item(), err

    # a permutation of the tokens permutes the output rows (bit for bit: every row's arithmetic is its own)
    perm = torch.randperm(t, device="cuda", generator=g)
    stager.begin()
    with torch.no_grad():
        out_p = block(x.detach()[:, perm])
    assert torch.equal(out_p, out.detach()[:, perm])

    # weight gradient of the busiest expert: d(down_proj[e]) = sum over its (token, slot) pairs of
    # score * go_t (outer) act_t
    e = int(counts.argmax())
    tok, slot = (idx == e).nonzero(as_tuple=True)
    xe = x.detach()[0, tok].float()
    a, b = (xe @ w["experts.gate_up_proj"][e].t()).chunk(2, dim=-1)
    act = (F.silu(a) * b).bfloat16().float()
    pe = F.softmax((x.detach()[0, tok] @ block.gate.weight.t()).float(), dim=-1)
    se = pe.gather(1, idx[tok])
    se = (se / se.sum(-1, keepdim=True)).bfloat16().float()[torch.arange(tok.numel()), slot]
    want_dw = (go[0, tok].float() * se[:, None]).t() @ act
    got_dw = block.experts.down_proj.grad[e].float()
    assert (got_dw - want_dw).abs().max() <= 3e-2 * want_dw.abs().max()
    # an expert nobody chose has a zero gradient
    unused = (counts == 0).nonzero().flatten()
    assert unused.numel() >= 12
    assert (block.experts.down_proj.grad[unused] == 0).all()
    assert (block.experts.gate_up_proj.grad[unused] == 0).all()


def test_hybrid_model_with_a_padding_mask_matches_oracle():
    """``attention_mask`` (models/mtp/core.py:119,180-186) through the gated-attention layer:
    right- and left-padded rows, dense MLP flavour (no routing in the way)."""
    shape = _hybrid_shape(model_type="qwen3_5_text")
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
    logits, loss, _ = model(ids.cuda(), hs.cuda(), attention_mask=am.cuda(), loss_mask=lm.cuda())
    loss.backward()
    wf = {k: v.float().requires_grad_(True) for k, v in w.items()}
    rl, rloss, _ = OM.mtp_forward(wf, shape, ids, hs.float(), loss_mask=lm, num_steps=steps, attention_mask=am)
    rloss.backward()
    assert abs(loss.item() - rloss.item()) <= 1e-3 * abs(rloss.item())
    tok = am[:, :n - steps - 1] != 0
    for k in range(steps):
        got, want = logits[k].float().cpu()[tok], rl[k][tok]
        assert (got - want).abs().max() <= 2e-2 * want.abs().max(), k
    for name, prm in model.named_parameters():
        if prm.requires_grad:
            want = wf[name].grad
            assert (prm.grad.float().cpu() - want).abs().max() <= 3e-2 * want.abs().max() + 1e-6, name


def test_hybrid_projections_on_this_librarys_gemm_agree_with_the_default(monkeypatch):
    """``SPX_DECODER_GEMM=spx`` on a hybrid MoE layer: every projection the kernel can take runs on
    it, and the ones it cannot (the shared expert's gate of width 1: a contraction of one element
    in its input gradient) stay with PyTorch's matmul inside the same mode.  Loss, logits and every
    gradient against the default mode."""
    from speculators_amd import gemm

    shape = _hybrid_shape(model_type="qwen3_5_moe_text", **_MOE)
    steps = 2
    w = {k: v.bfloat16() for k, v in OM.random_weights(shape, seed=3, std=0.05).items()}
    g = torch.Generator().manual_seed(6)
    b, n = 2, 150
    ids = torch.randint(0, shape.vocab_size, (b, n), generator=g).cuda()
    hs = torch.randn(b, n, shape.hidden_size, generator=g).bfloat16().cuda()
    lm = (torch.rand(b, n, generator=g) < 0.7).float().cuda()
    sw = OM.compute_step_weights(0.6, steps)
    seen = []
    real_back = gemm._project_back

    def spy(dy2, staged):
        seen.append((gemm.DECODER_GEMM, dy2.shape[1]))
        return real_back(dy2, staged)

    monkeypatch.setattr(gemm, "_project_back", spy)
    results = {}
    for kind in ("mixed", "spx"):
        monkeypatch.setattr(gemm, "DECODER_GEMM", kind)
        model = _make(shape, w, steps)
        logits, loss, _ = model(ids, hs, loss_mask=lm, step_weights=sw)
        loss.backward()
        results[kind] = (loss.item(), [l.float() for l in logits],
                         {nm: p.grad.float() for nm, p in model.named_parameters() if p.grad is not None})
    assert ("spx", 1) in seen, seen      # the width-1 gate went through the fall-back branch under spx
    la, lga, ga = results["mixed"]
    lb, lgb, gb = results["spx"]
    assert abs(la - lb) <= 2e-3 * abs(la)
    for a, b_ in zip(lga, lgb):
        assert (a - b_).abs().max() <= 3e-2 * a.abs().max()
    assert ga.keys() == gb.keys()
    for nm in ga:
        assert (ga[nm] - gb[nm]).abs().max() <= 3e-2 * ga[nm].abs().max() + 1e-6, nm
