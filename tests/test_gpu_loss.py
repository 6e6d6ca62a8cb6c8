"""HIP fused vocabulary loss against the CPU oracle (through the C ABI)."""

import pytest
import torch

from oracle import losses as OL
from oracle import metrics as OM
from oracle import vocab as OV

pytestmark = pytest.mark.gpu

LOSS_TOL = dict(atol=1e-4, rtol=1e-3)  # tests/unit/models/test_fused_losses.py:35
GRAD_TOL = dict(atol=1e-3, rtol=1e-2)  # tests/unit/models/test_fused_losses.py:36
NAMES = ["kl_div", "rkl", "jsd", "ce", "tv", "nla", "lk_hybrid"]


def _check(name, logits, targets, loss_tol=LOSS_TOL, grad_tol=GRAD_TOL):
    from speculators_amd import losses as L

    fn = L.resolve_loss_config(name)[name][0]
    lg = logits.cuda().detach().clone().requires_grad_(True)
    out = fn(lg, targets.cuda())
    assert out.dtype == torch.float32 and out.shape == logits.shape[:-1]
    lo = logits.float().detach().clone().requires_grad_(True)
    ref = OL.LOSS_FNS[name](lo, targets.float())
    torch.testing.assert_close(out.cpu(), ref.detach(), **loss_tol)
    g = torch.Generator().manual_seed(9)
    go = torch.randn(ref.shape, generator=g)
    go[:, ::3] = 0.0  # rows that take the zero-gradient early-out
    (ref * go).sum().backward()
    (out * go.cuda()).sum().backward()
    got = lg.grad.float().cpu()
    torch.testing.assert_close(got, lo.grad, **grad_tol)
    assert (got[:, ::3] == 0).all()


@pytest.mark.parametrize("name", NAMES)
def test_fp32_with_saturated_rows(name):
    # the regime of tests/unit/models/test_fused_losses.py:71-79
    g = torch.Generator().manual_seed(0)
    a = torch.randn(1, 32, 512, generator=g) * 3
    b = torch.randn(1, 32, 512, generator=g) * 3
    a[0, -2:] = -30.0; b[0, -2:] = -30.0
    a[0, -2:, 0] = 30.0; b[0, -2, 0] = 30.0; b[0, -1, 7] = 30.0
    _check(name, a, b)


@pytest.mark.parametrize("name", NAMES)
def test_bf16(name):
    g = torch.Generator().manual_seed(1)
    a = (torch.randn(1, 64, 512, generator=g) * 3).bfloat16()
    b = (torch.randn(1, 64, 512, generator=g) * 3).bfloat16()
    # the oracle computes in fp32 from the same bf16 inputs; the gradient is rounded to bf16
    _check(name, a, b, grad_tol=dict(atol=1e-3, rtol=1e-2))


@pytest.mark.parametrize("name", NAMES)
def test_wide_vocab_151936(name):
    g = torch.Generator().manual_seed(2)
    a = torch.randn(1, 3, 151936, generator=g) * 3
    b = torch.randn(1, 3, 151936, generator=g) * 3
    _check(name, a, b)


@pytest.mark.parametrize("vocab", [1, 7, 8, 9, 250, 32000 + 3])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ragged_vocab_and_unaligned_rows(vocab, dtype):
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(vocab)
    a = (torch.randn(1, 5, vocab, generator=g) * 2).to(dtype)
    b = (torch.randn(1, 5, vocab, generator=g) * 2).to(dtype)
    rows, am_d, am_t, _ = L.fused_rows(L.OP_KL, a.cuda(), b.cuda())
    torch.testing.assert_close(rows.cpu(), OL.kl_div(a, b), **LOSS_TOL)
    assert torch.equal(am_d.cpu().long(), a.float().argmax(-1))
    assert torch.equal(am_t.cpu().long(), b.float().argmax(-1))


def test_argmax_first_index_on_ties_bit_exact():
    from speculators_amd import losses as L
    from speculators_amd.metrics import argmax_rows

    g = torch.Generator().manual_seed(3)
    # coarse bf16 values: many exact ties per row
    a = (torch.randint(-4, 5, (1, 257, 32000), generator=g).float() * 0.5).bfloat16()
    b = (torch.randint(-4, 5, (1, 257, 32000), generator=g).float() * 0.5).bfloat16()
    _, am_d, am_t, _ = L.fused_rows(L.OP_KL, a.cuda(), b.cuda())
    assert torch.equal(am_d.cpu().long(), a.float().argmax(-1))
    assert torch.equal(am_t.cpu().long(), b.float().argmax(-1))
    assert torch.equal(argmax_rows(a.cuda()).cpu(), a.float().argmax(-1))
    # a late unique maximum and an early one
    a[0, 0, :] = 0; a[0, 0, 31999] = 1
    a[0, 1, :] = 0; a[0, 1, 0] = 1
    assert argmax_rows(a.cuda())[0, :2].tolist() == [31999, 0]


def test_vocab_gather_bit_exact():
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(4)
    vt, vd = 128256, 32000
    sel = torch.randperm(vt, generator=g)[:vd]
    d2t, t2d = OV.build_vocab_mappings(sel.tolist(), vt)
    full = (torch.randn(1, 9, vt, generator=g) * 2).bfloat16()
    got = L.vocab_gather(full.cuda(), d2t.cuda()).cpu()
    assert torch.equal(got, OV.gather_targets(full, d2t))
    assert torch.equal(got, full[..., t2d])
    full32 = torch.randn(3, vt, generator=g)
    assert torch.equal(L.vocab_gather(full32.cuda(), d2t.cuda()).cpu(), full32[..., t2d])


@pytest.mark.parametrize("op_name", ["kl_div", "rkl", "jsd", "ce", "tv"])
@pytest.mark.parametrize("dtype,vt,vd", [(torch.bfloat16, 128256, 32000), (torch.float32, 1000, 333),
                                         (torch.bfloat16, 5003, 1001)])
def test_step_pass_gathers_and_counts_in_the_row_pass(op_name, dtype, vt, vd):
    """The one-pass form (targets read through d2t, acceptance chain inside the row pass) against
    the three-kernel form (gather, loss, chain reduce): gathered rows bit-exact against the
    oracle's index mapping, row losses / statistics / arg-maxes bit-identical, counts and the
    in-place ``prev_correct`` identical."""
    from speculators_amd import _lib
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(vt + vd)
    rows = 37
    sel = torch.randperm(vt, generator=g)[:vd]
    d2t, t2d = OV.build_vocab_mappings(sel.tolist(), vt)
    full = (torch.randn(rows, vt, generator=g) * 2).to(dtype).cuda()
    logits = (torch.randn(rows, vd, generator=g) * 2).to(dtype).cuda()
    compact = L.vocab_gather(full, d2t.cuda())
    assert torch.equal(compact.cpu(), OV.gather_targets(full.cpu(), d2t))
    for i in range(0, rows, 3):  # a third of the rows agree with their target
        logits[i, compact[i].float().argmax()] = 30.0
    mask = (torch.rand(rows, generator=g) < 0.7).float().cuda()
    prev0 = (torch.rand(rows, generator=g) < 0.8).cuda()
    op = L.PRIMITIVE_OP[op_name]

    ref = L.fused_loss_forward(op, logits, compact)
    out = torch.empty(6, device="cuda")
    prev_ref = prev0.clone()
    _lib.call("spx_ttt_step_reduce", _lib.ptr(ref[0]), _lib.ptr(ref[4]), _lib.ptr(ref[5]), _lib.ptr(mask),
              _lib.kind_code(mask), _lib.ptr(prev_ref), _lib.kind_code(prev_ref), rows, 0.7,
              _lib.ptr(out), None, _lib.stream_ptr(mask.device))

    prev_got = prev0.clone()
    step = L.StepPass(d2t=d2t.cuda(), mask=mask, prev=prev_got,
                      counts=torch.zeros(3, dtype=torch.int32, device="cuda"))
    got = L.fused_loss_forward(op, logits, full, step=step)
    assert torch.equal(step.gathered, compact)
    for a, b in zip(got[:6], ref[:6], strict=True):
        assert torch.equal(a, b)
    assert torch.equal(prev_got, prev_ref)
    assert step.counts.tolist() == [int(out[1]), int(out[2]), int(out[4])]
    out2 = torch.empty(6, device="cuda")
    _lib.call("spx_ttt_step_mean", _lib.ptr(got[0]), _lib.ptr(mask), _lib.kind_code(mask), rows, 0.7,
              _lib.ptr(step.counts), _lib.ptr(out2), None, _lib.stream_ptr(mask.device))
    assert torch.equal(out2, out)


@pytest.mark.parametrize("op_name", ["kl_div", "ce"])
@pytest.mark.parametrize("known", [False, True])
@pytest.mark.parametrize("vocab", [32000, 32768, 8, 1000])
def test_row_pass_that_also_writes_the_logits_gradient(op_name, known, vocab):
    """``spx_vocab_loss_step_fwd_grad`` (a workgroup keeps the row pair in registers: loss, statistics,
    acceptance chain and the unit-weight logits gradient of the unmasked rows in ONE read of the rows)
    against the streaming kernels: arg-maxes, counts and ``prev_correct`` identical, row losses and
    log-sum-exps within 1e-5 (another summation order), masked rows with known statistics report a
    zero loss; the packed gradient rows against ``softmax(x) - softmax(y)`` / ``softmax(x) - onehot``
    in fp32 (one bf16 rounding); the scaled unpack."""
    from speculators_amd import _lib
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(vocab + 7 * known)
    rows = 41
    logits = (torch.randn(rows, vocab, generator=g) * 2).bfloat16().cuda()
    targets = (torch.randn(rows, vocab, generator=g) * 2).bfloat16().cuda()
    for i in range(0, rows, 3):
        logits[i, targets[i].float().argmax()] = 30.0
    targets[5, 1] = targets[5].float().max()  # a tie inside the target row: the first index wins
    targets[5, 0] = targets[5, 1]
    mask = (torch.rand(rows, generator=g) < 0.7).float().cuda()
    mask[0], mask[1] = 0.0, 1.0
    prev0 = (torch.rand(rows, generator=g) < 0.8).cuda()
    op = L.PRIMITIVE_OP[op_name]

    base = L.fused_loss_forward(op, logits, targets)  # the statistics of step 0
    stats = (base[2].clone(), base[5].clone()) if known else None
    prev_ref = prev0.clone()
    step_ref = L.StepPass(mask=mask, prev=prev_ref, counts=torch.zeros(3, dtype=torch.int32, device="cuda"))
    ref = L.fused_loss_forward(op, logits, targets, stats, step=step_ref)

    prev_got = prev0.clone()
    step = L.StepPass(mask=mask, prev=prev_got, counts=torch.zeros(3, dtype=torch.int32, device="cuda"),
                      grad_in_pass=True)
    assert L._one_pass_ok(op, logits, targets, step)
    loss, lse_t, am_d, am_t, packed, row_map, count = L._loss_forward_with_grad(
        op, logits, None if (known and op_name == "ce") else targets, stats, step)
    live = mask.bool()
    n_live = int(live.sum())
    assert int(count) == n_live
    assert torch.equal(am_d, ref[4]) and torch.equal(am_t, ref[5])
    assert torch.equal(prev_got, prev_ref) and step.counts.tolist() == step_ref.counts.tolist()
    want_loss = ref[0] if not known else torch.where(live, ref[0], torch.zeros_like(ref[0]))
    if op_name == "ce" and not known:
        want_loss = ref[0]  # without known statistics every row is reduced in full
    assert (loss - want_loss).abs().max().item() <= 1e-5 * max(1.0, want_loss.abs().max().item())
    assert (lse_t - ref[2]).abs().max().item() <= 1e-5 * max(1.0, ref[2].abs().max().item())

    p = torch.softmax(logits.float(), -1)
    if op_name == "ce":
        q = torch.nn.functional.one_hot(ref[5].long(), vocab).float()
    else:
        q = torch.softmax(targets.float(), -1)
    want = (p - q)[live]
    got = packed[:n_live].float()
    assert (got - want).abs().max().item() <= 2 ** -8 * want.abs().max().item() + 1e-6
    assert torch.equal(row_map[live].long().cpu(), torch.arange(n_live)) and (row_map[~live] == -1).all()

    scale = torch.randn(rows, generator=g).cuda()
    cols = packed[:, :8].contiguous()
    out = L._unpack_rows_scaled(cols, row_map, scale, rows + 3)
    want_out = torch.zeros(rows + 3, 8, device="cuda")
    want_out[:rows][live] = cols[:n_live].float() * scale[live, None]
    assert torch.equal(out, want_out.bfloat16())


def test_compute_metrics_with_target_gather_equals_materialised_targets():
    """compute_metrics over three TTT steps with the targets given as full-vocabulary logits +
    d2t (first step reads through the table and leaves the draft-vocabulary rows behind) against
    the same call on gathered targets: every metric, the loss and the gradients bit for bit."""
    from speculators_amd import losses as L
    from speculators_amd.metrics import TargetGather, compute_metrics

    g = torch.Generator().manual_seed(8)
    t, vt, vd, steps = 130, 4000, 1000, 3
    sel = torch.randperm(vt, generator=g)[:vd]
    d2t, _ = OV.build_vocab_mappings(sel.tolist(), vt)
    full = (torch.randn(1, t, vt, generator=g) * 2).bfloat16().cuda()
    mask = (torch.rand(1, t, generator=g) < 0.7).float().cuda()
    logits = [(torch.randn(1, t, vd, generator=g) * 2).bfloat16().cuda() for _ in range(steps)]
    runs = []
    for form in ("gather", "materialised"):
        tg = TargetGather(full, d2t.cuda()) if form == "gather" else L.vocab_gather(full, d2t.cuda())
        prev, cache, res = mask.clone(), {}, []
        for k in range(steps):
            lg = logits[k].clone().requires_grad_(True)
            loss, m = compute_metrics(lg, tg, mask, prev, k, 0.9, L.resolve_loss_config("kl_div"),
                                      target_stats_cache=cache)
            loss.backward()
            res.append((loss.detach(), m, lg.grad, prev.clone()))
        if form == "gather":
            assert torch.equal(tg.compact, L.vocab_gather(full, d2t.cuda()))
        runs.append(res)
    for (la, ma, ga, pa), (lb, mb, gb, pb) in zip(*runs, strict=True):
        assert torch.equal(la, lb) and torch.equal(ga, gb) and torch.equal(pa, pb)
        assert ma.keys() == mb.keys()
        for key in ma:
            assert torch.equal(ma[key], mb[key]), key


@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.bool, torch.int64, torch.bfloat16])
def test_eagle3_compute_metrics_chain_matches_oracle(mask_dtype):
    from speculators_amd import losses as L
    from speculators_amd.metrics import compute_metrics

    g = torch.Generator().manual_seed(5)
    t, v, steps = 300, 1000, 4
    targets = (torch.randn(1, t, v, generator=g) * 2).bfloat16()
    mask = (torch.rand(1, t, generator=g) < 0.7).to(mask_dtype)
    prev_ref = mask.clone()
    prev_gpu = mask.clone().cuda()
    for k in range(steps):
        logits = (torch.randn(1, t, v, generator=g) * 2).bfloat16()
        for i in range(0, t - k, 2):  # make half the rows agree with the shifted target
            logits[0, i, targets[0, i + k].float().argmax()] = 20.0
        lg = logits.cuda().requires_grad_(True)
        loss, m = compute_metrics(lg, targets.cuda(), mask.cuda(), prev_gpu, k, 0.8,
                                  L.resolve_loss_config("kl_div"))
        lo = logits.float().requires_grad_(True)
        rloss, rm = OM.eagle3_compute_metrics(lo, targets.float(), mask, prev_ref, k, 0.8)
        assert loss.item() == pytest.approx(rloss.item(), rel=1e-3)
        for key in rm:
            if "acc" in key:  # integer counts: bit exact
                assert m[key].item() == rm[key].item(), key
            else:
                assert m[key].item() == pytest.approx(rm[key].item(), rel=1e-3), key
        assert set(m) == set(rm)
        assert torch.equal(prev_gpu.cpu(), prev_ref) and prev_gpu.dtype == mask_dtype
        loss.backward(); rloss.backward()
        torch.testing.assert_close(lg.grad.float().cpu(), lo.grad, atol=1e-5, rtol=2e-2)


def test_compound_loss_config_and_no_mask():
    from speculators_amd import losses as L
    from speculators_amd.metrics import compute_metrics

    g = torch.Generator().manual_seed(6)
    logits = torch.randn(1, 40, 333, generator=g)
    targets = torch.randn(1, 40, 333, generator=g)
    cfg = L.resolve_loss_config('{"ce": 0.25, "tv": 0.75}')
    loss, m = compute_metrics(logits.cuda(), targets.cuda(), None, None, 2, 0.5, cfg)
    rloss, rm = OM.eagle3_compute_metrics(logits, targets, None, None, 2, 0.5,
                                          OL.resolve_loss_config({"ce": 0.25, "tv": 0.75}))
    assert set(m) == set(rm)
    for key in rm:
        assert m[key].item() == pytest.approx(rm[key].item(), rel=1e-3, abs=1e-6), key


@pytest.mark.parametrize("weighting", ["fixed-exp-decay", "dpace"])
def test_dflash_compute_metrics_matches_oracle(weighting):
    from speculators_amd import losses as L
    from speculators_amd.metrics import dflash_compute_metrics

    g = torch.Generator().manual_seed(7)
    bs, a, v = 8, 37, 2000
    logits = (torch.randn(1, a * bs, v, generator=g) * 2).bfloat16()
    targets = (torch.randn(1, a * bs, v, generator=g) * 2).bfloat16()
    for i in range(0, a * bs, 3):
        logits[0, i, targets[0, i].float().argmax()] = 20.0
    mask = (torch.rand(1, a * bs, generator=g) < 0.8).float()
    mask[:, ::bs] = 0
    name = "ce" if weighting == "dpace" else "kl_div"
    lg = logits.cuda().requires_grad_(True)
    loss, m = dflash_compute_metrics(lg, targets.cuda(), mask.cuda(), bs, 4.0,
                                     L.resolve_loss_config(name), weighting, 0.5)
    lo = logits.float().requires_grad_(True)
    rloss, rm = OM.dflash_compute_metrics(lo, targets.float(), mask, bs, 4.0,
                                          OL.resolve_loss_config(name), weighting, 0.5)
    assert set(m) == set(rm)
    for key in rm:
        if "acc" in key:
            assert m[key].item() == rm[key].item(), key
        else:
            assert m[key].item() == pytest.approx(rm[key].item(), rel=1e-3, abs=1e-6), key
    loss.backward(); rloss.backward()
    torch.testing.assert_close(lg.grad.float().cpu(), lo.grad, atol=1e-5, rtol=2e-2)


def test_full_size_rows_properties():
    """Config[1] row shape (32000-wide bf16): properties that need no oracle at size --
    KL(x, x) == 0, loss >= 0, gradient rows sum to ~0, determinism."""
    from speculators_amd import losses as L

    g = torch.Generator(device="cuda").manual_seed(8)
    x = (torch.randn(1, 4096, 32000, device="cuda", generator=g) * 2).bfloat16().requires_grad_(True)
    y = (torch.randn(1, 4096, 32000, device="cuda", generator=g) * 2).bfloat16()
    same = L.kl_div_loss(x.detach(), x.detach())
    assert same.abs().max().item() < 1e-4
    rows, am_d, _, _ = L.fused_rows(L.OP_KL, x, y)
    rows2, am_d2, _, _ = L.fused_rows(L.OP_KL, x, y)
    assert torch.equal(rows, rows2) and torch.equal(am_d, am_d2)
    assert (rows >= 0).all()
    rows.sum().backward()
    assert x.grad.float().sum(-1).abs().max().item() < 2e-2
    # a 64-row sample against the oracle
    idx = torch.arange(0, 4096, 64)
    ref = OL.kl_div(x.detach()[:, idx].cpu(), y[:, idx].cpu())
    torch.testing.assert_close(rows[:, idx].detach().cpu(), ref, **LOSS_TOL)


def test_full_size_row_pass_with_gradient_properties():
    """The one-read row pass at the config[1] row shape (4096 x 32000 bf16, 70 % of the rows live, target
    statistics of an earlier step handed in): against the streaming kernels on the same rows -- arg-maxes,
    counts and chain identical, row losses within 1e-5 -- and through what needs no oracle at size: KL rows
    >= 0, every gradient row sums to ~0 (two soft-maxes), the gradient of a row paired with itself is zero,
    two runs agree bit for bit."""
    from speculators_amd import losses as L

    g = torch.Generator(device="cuda").manual_seed(9)
    t, v = 4096, 32000
    x = (torch.randn(t, v, device="cuda", generator=g) * 2).bfloat16()
    y = (torch.randn(t, v, device="cuda", generator=g) * 2).bfloat16()
    y[7] = x[7]  # a row paired with itself
    mask = (torch.rand(t, device="cuda", generator=g) < 0.7).float()
    mask[7] = 1.0
    base = L.fused_loss_forward(L.OP_KL, x, y)
    known = (base[2].clone(), base[5].clone())
    prev0 = torch.rand(t, device="cuda", generator=g) < 0.8

    def run(one_pass):
        prev = prev0.clone()
        step = L.StepPass(mask=mask, prev=prev, counts=torch.zeros(3, dtype=torch.int32, device="cuda"),
                          grad_in_pass=one_pass)
        if one_pass:
            out = L._loss_forward_with_grad(L.OP_KL, x, y, known, step)
            return out, prev, step.counts
        return L.fused_loss_forward(L.OP_KL, x, y, known, step=step), prev, step.counts

    (loss, _lse_t, am_d, am_t, packed, row_map, count), prev_a, counts_a = run(True)
    ref, prev_b, counts_b = run(False)
    live = mask.bool()
    n_live = int(live.sum())
    assert int(count) == n_live and counts_a.tolist() == counts_b.tolist() and torch.equal(prev_a, prev_b)
    assert torch.equal(am_d, ref[4]) and torch.equal(am_t, ref[5])
    assert (loss[live] - ref[0][live]).abs().max().item() <= 1e-5 * ref[0].abs().max().item()
    assert (loss[~live] == 0).all() and (loss >= -1e-5).all()
    grad = packed[:n_live].float()
    assert grad.sum(-1).abs().max().item() < 2e-2
    assert grad[int(row_map[7])].abs().max().item() == 0.0
    packed2 = L._loss_forward_with_grad(L.OP_KL, x, y, known, L.StepPass(
        mask=mask, prev=prev0.clone(), counts=torch.zeros(3, dtype=torch.int32, device="cuda"), grad_in_pass=True))[4]
    assert torch.equal(packed2[:n_live], packed[:n_live])
    # a 32-row sample against the closed form in fp32
    idx = torch.nonzero(live).flatten()[::97][:32]
    want = torch.softmax(x[idx].float(), -1) - torch.softmax(y[idx].float(), -1)
    got = packed[row_map[idx].long()].float()
    assert (got - want).abs().max().item() <= 2 ** -8 * want.abs().max().item() + 1e-7


@pytest.mark.parametrize("op_name", ["kl_div", "ce"])
def test_reused_target_statistics_give_the_same_rows(op_name):
    """Steps >= 1 reuse the verifier rows' lse / arg-max from step 0: same loss, arg-maxes
    and gradient as recomputing them."""
    from speculators_amd import losses as L

    op = L.PRIMITIVE_OP[op_name]
    g = torch.Generator().manual_seed(11)
    t, v, k = 200, 4000, 3
    logits = (torch.randn(1, t, v, generator=g) * 2).bfloat16().cuda()
    targets = (torch.randn(1, t, v, generator=g) * 2).bfloat16().cuda()
    _, _, am_full, lse_full = L.fused_rows(op, logits, targets)
    a = logits[:, : t - k].detach().clone().requires_grad_(True)
    b = logits[:, : t - k].detach().clone().requires_grad_(True)
    fresh, pd_f, pt_f, _ = L.fused_rows(op, a, targets[:, k:])
    known = (lse_full.reshape(-1)[k:], am_full.reshape(-1)[k:])
    reused, pd_r, pt_r, _ = L.fused_rows(op, b, targets[:, k:], known)
    assert torch.equal(pd_f, pd_r) and torch.equal(pt_f, pt_r)
    torch.testing.assert_close(reused, fresh, atol=2e-6, rtol=1e-5)
    go = torch.randn_like(fresh)
    (fresh * go).sum().backward(); (reused * go).sum().backward()
    torch.testing.assert_close(b.grad.float(), a.grad.float(), atol=1e-6, rtol=1e-3)


@pytest.mark.parametrize("live_fraction", [0.15, 0.45, 1.0])
def test_head_and_loss_node_with_the_input_gradient_in_parts(live_fraction, monkeypatch):
    """The frozen head + loss node over a sparse loss mask: its input-gradient product runs over the
    packed live rows and, when their tiles are few, with the contraction cut into parts
    (``spx_gemm_bf16_nt_rows_split``).  Against the same node with the cut switched off (one rounding of
    a bf16 value apart) and against autograd through the fp32 oracle loss; dead rows get exact zeros."""
    from speculators_amd import gemm as G
    from speculators_amd import losses as L

    t, h, vd = 1024, 512, 4096
    g = torch.Generator().manual_seed(int(live_fraction * 100))
    x = (torch.randn(1, t, h, generator=g) * 0.5).bfloat16()
    w = (torch.randn(vd, h, generator=g) * 0.05).bfloat16()
    tg = (torch.randn(1, t, vd, generator=g) * 2).bfloat16()
    mask = (torch.rand(1, t, generator=g) < live_fraction).float()
    grads = {}
    for parts in (4, 1):
        monkeypatch.setattr(G, "SPLIT_PARTS", parts)
        xg = x.cuda().requires_grad_(True)
        wc = w.cuda()
        loss = L.head_fused_rows(L.OP_KL, xg, wc, wc.t().contiguous(), tg.cuda())[0]
        (loss * mask.cuda()).sum().backward()
        grads[parts] = xg.grad.float().cpu()
    xr = x.float().requires_grad_(True)
    # (the oracle sees the logits the kernel sees: rounded to bf16, gradient straight through)
    logits = xr @ w.float().t()
    logits = logits + (logits.detach().bfloat16().float() - logits.detach())
    ref = OL.kl_div(logits, tg.float())
    (ref * mask).sum().backward()
    want = xr.grad
    scale = want.abs().max().item()
    dead = mask[0] == 0
    for parts in (4, 1):
        assert (grads[parts][0][dead] == 0).all()
        assert (grads[parts] - want).abs().max().item() <= 2e-2 * scale + 1e-6, parts
    assert (grads[4] - grads[1]).abs().max().item() <= 1e-2 * scale + 1e-6


@pytest.mark.parametrize("op_name", ["kl_div", "ce"])
@pytest.mark.parametrize("case", ["even", "skewed", "ragged", "one_tile", "clustered"])
def test_pipelined_gather_pass_on_the_edges_of_its_tiling(op_name, case):
    """The pipelined form of the one-pass kernel (bf16, 16-byte aligned rows, kl / ce: spans of the
    full row staged two tiles deep, picks with lane = id) against the three-kernel form, bit for bit:
    a table spread evenly; one that is dense at the low ids and sparse at the high ones, so that
    the spans of the late tiles do not fit a buffer and are read directly; a draft vocabulary that
    ends inside a chunk of 8 (rows kept aligned by their stride); one smaller than a tile; ids
    clustered in two far-apart runs (a span boundary inside a tile)."""
    from speculators_amd import _lib
    from speculators_amd import losses as L

    g = torch.Generator().manual_seed(len(case) * 7 + len(op_name))
    rows = 21
    if case == "even":
        vt, vd = 40000, 9000
        sel = torch.randperm(vt, generator=g)[:vd]
    elif case == "skewed":
        vt, vd = 200000, 6144
        dense = torch.arange(4000)                                  # ids 0..3999 map to themselves
        sparse = 4000 + torch.randperm(vt - 4000, generator=g)[:vd - 4000]  # 2144 ids over 196000 columns
        sel = torch.cat([dense, sparse])
    elif case == "ragged":
        vt, vd = 30000, 4099
        sel = torch.randperm(vt, generator=g)[:vd]
    elif case == "one_tile":
        vt, vd = 3000, 700
        sel = torch.randperm(vt, generator=g)[:vd]
    else:
        vt, vd = 150000, 5000
        sel = torch.cat([torch.arange(100, 2600), torch.arange(140000, 142500)])
    d2t, _ = OV.build_vocab_mappings(sel.tolist(), vt)
    vt_ld, vd_ld = -(-vt // 8) * 8, -(-vd // 8) * 8
    full = (torch.randn(rows, vt_ld, generator=g) * 2).bfloat16().cuda()[:, :vt]
    logits = (torch.randn(rows, vd_ld, generator=g) * 2).bfloat16().cuda()[:, :vd]
    compact = L.vocab_gather(full.contiguous(), d2t.cuda())
    assert torch.equal(compact.cpu(), OV.gather_targets(full.cpu(), d2t))
    for i in range(0, rows, 3):
        logits[i, compact[i].float().argmax()] = 30.0
    mask = (torch.rand(rows, generator=g) < 0.7).float().cuda()
    prev0 = (torch.rand(rows, generator=g) < 0.8).cuda()
    op = L.PRIMITIVE_OP[op_name]
    ref = L.fused_loss_forward(op, logits, compact)
    out = torch.empty(6, device="cuda")
    prev_ref = prev0.clone()
    _lib.call("spx_ttt_step_reduce", _lib.ptr(ref[0]), _lib.ptr(ref[4]), _lib.ptr(ref[5]), _lib.ptr(mask),
              _lib.kind_code(mask), _lib.ptr(prev_ref), _lib.kind_code(prev_ref), rows, 0.7,
              _lib.ptr(out), None, _lib.stream_ptr(mask.device))
    prev_got = prev0.clone()
    step = L.StepPass(d2t=d2t.cuda(), mask=mask, prev=prev_got,
                      counts=torch.zeros(3, dtype=torch.int32, device="cuda"))
    assert full.stride(0) % 8 == 0 and logits.stride(0) % 8 == 0  # the pipelined kernel's precondition
    got = L.fused_loss_forward(op, logits, full, step=step)
    assert torch.equal(step.gathered, compact)
    names = ("loss", "lse_draft", "lse_target", "extra", "argmax_draft", "argmax_target")
    for name, a, b in zip(names, got[:6], ref[:6], strict=True):
        if op_name == "ce" and name in ("lse_target", "extra"):
            continue  # not defined for ce
        assert torch.equal(a, b), name
    assert torch.equal(prev_got, prev_ref)
    assert step.counts.tolist() == [int(out[1]), int(out[2]), int(out[4])]
