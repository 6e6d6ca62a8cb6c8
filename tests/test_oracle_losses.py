"""Oracle losses: the identities the reference's tests assert
(tests/unit/models/test_metrics.py), library routines, closed-form gradients."""

import math
from functools import partial

import pytest
import torch
import torch.nn.functional as F

from oracle import losses as L


def _pair(seed=0, shape=(1, 4, 50), scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale, torch.randn(*shape, generator=g) * scale


def test_kl_matches_library_kl_div():
    a, b = _pair(1, (1, 6, 33), 3.0)
    ref = F.kl_div(F.log_softmax(a, -1), F.softmax(b, -1), reduction="none").sum(-1)
    assert torch.allclose(L.kl_div(a, b), ref, atol=1e-6)


def test_ce_matches_library_cross_entropy_first_index_ties():
    a, b = _pair(2, (1, 5, 17))
    b[0, 0, 3] = b[0, 0, 9] = 50.0  # tie -> first index
    ref = F.cross_entropy(a.reshape(-1, 17), b.argmax(-1).reshape(-1), reduction="none")
    assert torch.allclose(L.ce(a, b).reshape(-1), ref, atol=1e-6)
    assert int(b.argmax(-1)[0, 0]) == 3


@pytest.mark.parametrize("fn", [L.kl_div, L.rkl, L.jsd])
def test_identical_zero_random_nonnegative(fn):
    x = torch.randn(1, 4, 8)
    assert fn(x, x).sum().item() == pytest.approx(0.0, abs=1e-4)
    a, b = _pair(0, (1, 4, 8))
    assert (fn(a, b) >= -1e-6).all()


def test_rkl_is_kl_swapped():
    a, b = _pair(0, (1, 4, 8))
    assert torch.allclose(L.rkl(a, b), L.kl_div(b, a), atol=1e-6)


def test_jsd_symmetric_bounded_manual():
    a, b = _pair(0, (1, 4, 50))
    assert torch.allclose(L.jsd(a, b), L.jsd(b, a), atol=1e-6)
    p = torch.full((1, 1, 4), -100.0); p[0, 0, 0] = 100.0
    q = torch.full((1, 1, 4), -100.0); q[0, 0, 1] = 100.0
    assert L.jsd(p, q).max().item() == pytest.approx(math.log(2), abs=1e-3)
    pp, qq = torch.softmax(b, -1), torch.softmax(a, -1)
    m = 0.5 * (pp + qq)
    manual = 0.5 * ((pp * (pp / m).log()).sum(-1) + (qq * (qq / m).log()).sum(-1))
    assert torch.allclose(L.jsd(a, b), manual, atol=1e-5)


def test_tv_is_half_l1_in_unit_range():
    a, b = _pair(0, (1, 4, 50))
    l1 = 0.5 * (torch.softmax(a, -1) - torch.softmax(b, -1)).abs().sum(-1)
    out = L.tv(a, b)
    assert torch.allclose(out, l1, atol=1e-6)
    assert (out >= 0).all() and (out <= 1).all()
    assert torch.allclose(L.tv(a, a), torch.zeros(1, 4), atol=1e-6)


def test_nla_forms():
    a, b = _pair(0, (1, 4, 50))
    assert torch.allclose(L.nla(a, a), torch.zeros(1, 4), atol=1e-5)
    assert torch.allclose(L.nla(a, b), -torch.log((1 - L.tv(a, b)).clamp_min(1e-5)), atol=1e-6)
    t = torch.full((1, 1, 50), -30.0); t[0, 0, 7] = 30.0
    x = torch.randn(1, 1, 50)
    assert torch.allclose(L.nla(x, t), L.ce(x, t), atol=1e-3)
    d = torch.full((1, 1, 50), -30.0); d[0, 0, 0] = 30.0
    t2 = torch.full((1, 1, 50), -30.0); t2[0, 0, 1] = 30.0
    v = L.nla(d, t2)
    assert torch.isfinite(v).all() and v.item() == pytest.approx(-math.log(1e-5), rel=1e-3)


def test_lk_hybrid_limits_and_detached_weight():
    a, b = _pair(0, (1, 4, 50))
    assert torch.allclose(L.lk_hybrid(a, b, eta=0.0), L.kl_div(a, b), atol=1e-6)
    assert torch.allclose(L.lk_hybrid(a, b, eta=1e6), L.tv(a, b), atol=1e-5)
    x = torch.randn(1, 3, 40, requires_grad=True)
    t = torch.randn(1, 3, 40)
    g_impl = torch.autograd.grad(L.lk_hybrid(x, t, 3.0).sum(), x)[0]

    def manual(detach):
        dp, tp = torch.softmax(x, -1), torch.softmax(t, -1)
        ov = torch.minimum(dp, tp).sum(-1)
        lam = torch.exp(-3.0 * (ov.detach() if detach else ov))
        return (lam * L.kl_div(x, t) + (1 - lam) * (1 - ov)).sum()

    g_det = torch.autograd.grad(manual(True), x, retain_graph=True)[0]
    g_no = torch.autograd.grad(manual(False), x)[0]
    assert torch.allclose(g_impl, g_det, atol=1e-5)
    assert not torch.allclose(g_det, g_no, atol=1e-4)


@pytest.mark.parametrize("name", ["kl_div", "rkl", "jsd", "ce", "tv"])
def test_closed_form_gradient_equals_autograd(name):
    a, b = _pair(5, (1, 6, 64), 2.0)
    a = a.double().requires_grad_(True)
    out = L.LOSS_FNS[name](a, b.double())
    # the oracle computes in fp32; compare with autograd through the same fp32 graph
    g = torch.autograd.grad(out.sum(), a)[0].float()
    closed = L.row_loss_grad(name, a.detach().float(), b)
    assert torch.allclose(closed, g, atol=2e-6), (closed - g).abs().max()


def test_saturated_rows_stay_finite():
    # the +-30 point-mass regime of tests/unit/models/test_fused_losses.py:71-79
    g = torch.Generator().manual_seed(0)
    a = torch.randn(1, 8, 512, generator=g) * 3
    b = torch.randn(1, 8, 512, generator=g) * 3
    a[0, -2:] = -30.0; b[0, -2:] = -30.0
    a[0, -2:, 0] = 30.0; b[0, -2, 0] = 30.0; b[0, -1, 7] = 30.0
    for name, fn in L.LOSS_FNS.items():
        assert torch.isfinite(fn(a, b)).all(), name
    assert L.kl_div(a, b)[0, -2].item() == pytest.approx(0.0, abs=1e-5)
    assert L.kl_div(a, b)[0, -1].item() == pytest.approx(60.0, rel=1e-4)


def test_decay_scales_loss_and_masked_mean():
    g = torch.Generator().manual_seed(42)
    a = torch.randn(1, 16, 8, generator=g); b = torch.randn(1, 16, 8, generator=g)
    m = torch.ones(1, 16)
    d = partial(L.exp_loss_decay, gamma=0.5)
    l0 = L.loss_function(a, b, m, torch.zeros(1, 16, dtype=torch.long), L.kl_div, d)
    l2 = L.loss_function(a, b, m, torch.full((1, 16), 2), L.kl_div, d)
    assert torch.isclose(l2, l0 * 0.25, rtol=1e-4)
    assert L.loss_function(a, b, torch.zeros(1, 16), torch.zeros(1, 16), L.kl_div).item() == pytest.approx(0, abs=1e-4)
    mm = torch.tensor([[1, 0, 1, 1, 0, 1.0]])
    r = L.loss_function(a[:, :6], b[:, :6], mm, torch.zeros(1, 6), L.kl_div)
    assert torch.isclose(r, (L.kl_div(a[:, :6], b[:, :6]) * mm).sum() / (mm.sum() + 1e-5))


def test_decay_known_values():
    pos = torch.arange(4, dtype=torch.float)
    d = L.dflash_loss_decay(pos, gamma=4.0)
    assert d[0].item() == 0.0 and d[1].item() == pytest.approx(1.0)
    assert d[2].item() == pytest.approx(math.exp(-0.25)) and d[3].item() == pytest.approx(math.exp(-0.5))
    s = L.dflash_loss_decay(pos, gamma=4.0, sample_from_anchor=True)
    assert s[0].item() == pytest.approx(1.0) and s[2].item() == pytest.approx(math.exp(-0.5))
    assert L.exp_loss_decay(torch.tensor(2.0), gamma=0.5).item() == pytest.approx(0.25)
    assert L.exp_loss_decay(torch.tensor(0.0), gamma=0.5).item() == pytest.approx(1.0)


def test_dpace_hand_computed_two_blocks():
    # block 0: CE = [0, ln2, ln4], mask [1,1,1], alpha=.5 -> s = [1,.75,.625]
    # prefix = [1,.75,.46875]; w = [2.21875, 1.21875, .46875]
    # block 1: mask [0,1,1], CE = [9, 0, ln2] -> s = [1,1,.75]; prefix*m = [0,1,.75]; w=[0,1.75,.75]
    ce = torch.tensor([[0.0, math.log(2), math.log(4), 9.0, 0.0, math.log(2)]])
    m = torch.tensor([[1, 1, 1, 0, 1, 1.0]])
    w = L.dpace_loss_decay(None, m, 3, 0.5, ce)
    assert torch.allclose(w, torch.tensor([[2.21875, 1.21875, 0.46875, 0.0, 1.75, 0.75]]), atol=1e-6)


def test_bf16_inputs_fp32_math_gradient_within_2_percent_of_fp64():
    # the regime of tests/unit/models/test_metrics.py:388-439
    g = torch.Generator().manual_seed(0)
    t = (torch.randn(1, 8, 4096, generator=g) * 2).bfloat16()
    x = (t.float() + torch.randn(1, 8, 4096, generator=g) * 0.1).bfloat16()
    for name in ["kl_div", "rkl", "jsd", "tv"]:
        xd = x.double().requires_grad_(True)
        pd, qd = torch.softmax(t.double(), -1), torch.softmax(xd, -1)
        if name == "kl_div":
            ref = (pd * (pd.log() - qd.log())).sum()
        elif name == "rkl":
            ref = (qd * (qd.log() - pd.log())).sum()
        elif name == "jsd":
            md = 0.5 * (pd + qd)
            ref = 0.5 * ((pd * (pd / md).log()).sum() + (qd * (qd / md).log()).sum())
        else:
            ref = (1 - torch.minimum(pd, qd).sum(-1)).sum()
        exact = torch.autograd.grad(ref, xd)[0]
        got = L.row_loss_grad(name, x, t).double()
        assert ((got - exact).norm() / exact.norm()).item() < 0.02, name


def test_dpace_equals_per_block_double_loop_on_random_masks():
    """losses/utils.py:64-112 spelled out per element in float64: within a block,
    w_i = m_i * sum_{j >= i} m_j * prod_{l <= j} s_l,  s_l = (1 - a) exp(-CE_l) + a where the
    mask is set and 1 elsewhere.  Random masks (also all-zero and all-one blocks), several block
    sizes and smoothing constants."""
    g = torch.Generator().manual_seed(0)
    for bs, blocks, alpha in [(1, 5, 0.5), (4, 7, 0.5), (16, 9, 0.1), (5, 6, 0.0), (8, 4, 1.0)]:
        n = bs * blocks
        ce = torch.rand(1, n, generator=g) * 6
        m = (torch.rand(1, n, generator=g) < 0.6).float()
        m[0, :bs] = 0
        if blocks > 1:
            m[0, bs:2 * bs] = 1
        got = L.dpace_loss_decay(None, m, bs, alpha, ce)
        want = torch.zeros(n, dtype=torch.float64)
        for b in range(blocks):
            for i in range(bs):
                if m[0, b * bs + i] == 0:
                    continue
                acc = 0.0
                for j in range(i, bs):
                    if m[0, b * bs + j] == 0:
                        continue
                    prod = 1.0
                    for l in range(j + 1):
                        if m[0, b * bs + l] != 0:
                            prod *= (1 - alpha) * math.exp(-ce[0, b * bs + l].item()) + alpha
                    acc += prod
                want[b * bs + i] = acc
        assert got.shape == (1, n)
        assert torch.allclose(got[0].double(), want, rtol=1e-5, atol=1e-7), (bs, alpha)
    # no gradient reaches the row losses through the weight
    ce = torch.rand(1, 8, generator=g, requires_grad=True)
    assert not L.dpace_loss_decay(None, torch.ones(1, 8), 4, 0.5, ce).requires_grad


def test_compound_loss_is_the_weighted_sum_and_reports_terms_only_when_several():
    """losses/utils.py:233-266: total = sum_name weight * loss_function(name); the ``{name}_loss``
    entries are the UNWEIGHTED, detached per-term values and exist only for more than one term.
    Checked against the closed form built from the single-term reduction (itself pinned above),
    with a mask, a decay and weights that do not sum to one."""
    g = torch.Generator().manual_seed(7)
    a = torch.randn(1, 12, 40, generator=g, requires_grad=True)
    b = torch.randn(1, 12, 40, generator=g)
    m = (torch.rand(1, 12, generator=g) < 0.6).float()
    pos = torch.full((1, 12), 2)
    d = partial(L.exp_loss_decay, gamma=0.8)
    single = {n: L.loss_function(a, b, m, pos, L.LOSS_FNS[n], d) for n in ("ce", "tv", "kl_div")}

    cfg = L.resolve_loss_config({"ce": 0.25, "tv": 0.75})
    total, terms = L.compound_loss(a, b, m, pos, cfg, d)
    assert torch.isclose(total, 0.25 * single["ce"] + 0.75 * single["tv"], rtol=1e-6)
    assert set(terms) == {"ce_loss", "tv_loss"}
    assert torch.equal(terms["ce_loss"], single["ce"].detach()) and not terms["ce_loss"].requires_grad
    assert torch.equal(terms["tv_loss"], single["tv"].detach())
    # the weights are applied as given: no renormalisation, order of the mapping irrelevant
    cfg3 = L.resolve_loss_config({"tv": 2.0, "kl_div": 0.5, "ce": 1.5})
    total3, terms3 = L.compound_loss(a, b, m, pos, cfg3, d)
    assert torch.isclose(total3, 2.0 * single["tv"] + 0.5 * single["kl_div"] + 1.5 * single["ce"], rtol=1e-6)
    assert set(terms3) == {"tv_loss", "kl_div_loss", "ce_loss"}
    # the gradient is the weighted sum of the terms' gradients (the terms dict carries none)
    gt, = torch.autograd.grad(total, a, retain_graph=True)
    gc, = torch.autograd.grad(single["ce"], a, retain_graph=True)
    gv, = torch.autograd.grad(single["tv"], a, retain_graph=True)
    assert torch.allclose(gt, 0.25 * gc + 0.75 * gv, atol=1e-7)
    # one term: the weight still applies, nothing is reported
    one, none = L.compound_loss(a, b, m, pos, L.resolve_loss_config({"tv": 0.3}), d)
    assert none == {} and torch.isclose(one, 0.3 * single["tv"], rtol=1e-6)
    plain, none = L.compound_loss(a, b, m, pos, L.resolve_loss_config("kl_div"), d)
    assert none == {} and torch.equal(plain, single["kl_div"])
