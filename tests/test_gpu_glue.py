"""HIP layer-glue kernels (RMSNorm, RoPE + relayout, SwiGLU) against the closed forms the
oracle uses (oracle/eagle3.py), forward and backward."""

import pytest
import torch

from oracle import eagle3 as OE

pytestmark = pytest.mark.gpu


def _close(got, want, rel=2e-2):
    err = (got.float().cpu() - want.float()).abs().max().item()
    assert err <= rel * want.float().abs().max().item() + 1e-6, (err, want.float().abs().max().item())


@pytest.mark.parametrize("rows,h", [(300, 4096), (77, 12288), (1000, 128), (64, 256), (5, 2048), (3, 64)])
def test_rmsnorm_forward_backward(rows, h):
    from speculators_amd.fused_ops import rms_norm

    g = torch.Generator().manual_seed(rows + h)
    x = (torch.randn(1, rows, h, generator=g) * 3).bfloat16()
    w = (1 + 0.2 * torch.randn(h, generator=g)).bfloat16()
    go = torch.randn(1, rows, h, generator=g).bfloat16()
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    y = rms_norm(xg, wg, 1e-5)
    y.backward(go.cuda())
    # forward: bit-exact against the same bf16 rounding points evaluated by PyTorch
    ref_bf16 = OE.rms_norm(x, w, 1e-5)
    mism = (y.cpu() != ref_bf16).float().mean().item()
    assert mism < 2e-3, mism  # rsqrt / reduction-order ulps may flip a rounding now and then
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    yr = OE.rms_norm(xr, wr, 1e-5)
    yr.backward(go.float())
    _close(y, yr.detach()); _close(xg.grad, xr.grad); _close(wg.grad, wr.grad)


@pytest.mark.parametrize("t,heads,d,offset", [(300, 8, 128, 0), (129, 2, 64, 3), (64, 32, 128, 6)])
def test_rope_relayout_forward_backward(t, heads, d, offset):
    from speculators_amd.fused_ops import rope_inv_freq, rope_relayout

    g = torch.Generator().manual_seed(t + d)
    x = torch.randn(1, t, heads * d, generator=g).bfloat16()
    pos = torch.randint(0, 5000, (t,), generator=g)
    go = torch.randn(1, heads, t, d, generator=g).bfloat16()
    inv = rope_inv_freq(d, 500000.0, "cuda")
    xg = x.cuda().requires_grad_(True)
    y = rope_relayout(xg, pos.cuda(), inv, heads, True, offset)
    y.backward(go.cuda())
    cos, sin = OE.rope_tables((pos + offset).unsqueeze(0), d, 500000.0, torch.bfloat16)
    ref_bf16 = OE.apply_rope(x.view(1, t, heads, d).transpose(1, 2), cos, sin)
    mism = (y.cpu() != ref_bf16).float().mean().item()
    assert mism < 5e-3, mism  # cos/sin ulps at bf16 rounding boundaries
    xr = x.float().requires_grad_(True)
    c32, s32 = OE.rope_tables((pos + offset).unsqueeze(0), d, 500000.0, torch.float32)
    yr = OE.apply_rope(xr.view(1, t, heads, d).transpose(1, 2), c32, s32)
    yr.backward(go.float())
    _close(y, yr.detach()); _close(xg.grad, xr.grad)
    # relayout only (V): exact
    v = rope_relayout(x.cuda(), pos.cuda(), inv, heads, False, 0)
    assert torch.equal(v.cpu(), x.view(1, t, heads, d).transpose(1, 2))


def test_swiglu_forward_backward():
    from speculators_amd.fused_ops import swiglu

    g = torch.Generator().manual_seed(0)
    a = (torch.randn(1, 100, 1024, generator=g) * 2).bfloat16()
    b = torch.randn(1, 100, 1024, generator=g).bfloat16()
    go = torch.randn(1, 100, 1024, generator=g).bfloat16()
    ag, bg = a.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    y = swiglu(ag, bg)
    y.backward(go.cuda())
    ref_bf16 = torch.nn.functional.silu(a) * b
    assert (y.cpu() != ref_bf16).float().mean().item() < 2e-3
    ar, br = a.float().requires_grad_(True), b.float().requires_grad_(True)
    yr = torch.nn.functional.silu(ar) * br
    yr.backward(go.float())
    _close(y, yr.detach()); _close(ag.grad, ar.grad); _close(bg.grad, br.grad)


@pytest.mark.parametrize("rows,h", [(300, 4096), (1500, 2048), (40, 256), (33, 8192)])
def test_add_rms_norm_matches_the_two_ops(rows, h):
    """``(a + b, rms_norm(a + b))`` fused, against the bf16 add followed by the norm."""
    from speculators_amd.fused_ops import add_rms_norm

    g = torch.Generator().manual_seed(rows + h)
    a = (torch.randn(1, rows, h, generator=g) * 2).bfloat16()
    b = (torch.randn(1, rows, h, generator=g) * 2).bfloat16()
    w = (1 + 0.2 * torch.randn(h, generator=g)).bfloat16()
    gs = torch.randn(1, rows, h, generator=g).bfloat16()
    gy = torch.randn(1, rows, h, generator=g).bfloat16()
    ag, bg, wg = (t.cuda().requires_grad_(True) for t in (a, b, w))
    s, y = add_rms_norm(ag, bg, wg, 1e-5)
    torch.autograd.backward((s, y), (gs.cuda(), gy.cuda()))
    assert torch.equal(s.cpu(), a + b)  # one bf16 rounding, like the tensor add
    ref_bf16 = OE.rms_norm(a + b, w, 1e-5)
    assert (y.cpu() != ref_bf16).float().mean().item() < 2e-3
    ar, br, wr = (t.float().requires_grad_(True) for t in (a, b, w))
    sr = (ar + br).bfloat16().float()  # the norm sees the rounded sum
    sr = ar + br + (sr - (ar + br)).detach()
    yr = OE.rms_norm(sr, wr, 1e-5)
    torch.autograd.backward((sr, yr), (gs.float(), gy.float()))
    _close(y, yr.detach()); _close(ag.grad, ar.grad); _close(bg.grad, br.grad); _close(wg.grad, wr.grad)
    assert torch.equal(ag.grad, bg.grad)
    # only one of the two outputs used
    ag.grad = bg.grad = wg.grad = None
    s, y = add_rms_norm(ag, bg, wg, 1e-5)
    s.backward(gs.cuda())
    assert torch.equal(ag.grad.cpu(), gs) and wg.grad is None
    ag.grad = bg.grad = None
    s, y = add_rms_norm(ag, bg, wg, 1e-5)
    y.backward(gy.cuda())
    ar.grad = br.grad = wr.grad = None
    OE.rms_norm(ar + br, wr, 1e-5).backward(gy.float())
    _close(ag.grad, ar.grad); _close(wg.grad, wr.grad)


@pytest.mark.parametrize("rows,h,embeds_grad", [(300, 4096, False), (129, 512, True), (64, 2048, False)])
def test_pair_norm_cat_matches_cat_of_norms(rows, h, embeds_grad):
    from speculators_amd.fused_ops import pair_norm_cat, rms_norm

    g = torch.Generator().manual_seed(rows + h)
    a = (torch.randn(1, rows, h, generator=g) * 2).bfloat16().cuda().requires_grad_(embeds_grad)
    b = (torch.randn(1, rows, h, generator=g) * 3).bfloat16().cuda().requires_grad_(True)
    wa = (1 + 0.2 * torch.randn(h, generator=g)).bfloat16().cuda().requires_grad_(True)
    wb = (1 + 0.2 * torch.randn(h, generator=g)).bfloat16().cuda().requires_grad_(True)
    go = torch.randn(1, rows, 2 * h, generator=g).bfloat16().cuda()
    out = pair_norm_cat(a, b, wa, wb, 1e-5)
    out.backward(go)
    got = [t.grad for t in (a, b, wa, wb)]
    for t in (a, b, wa, wb):
        t.grad = None
    ref = torch.cat([rms_norm(a, wa, 1e-5), rms_norm(b, wb, 1e-5)], dim=-1)
    ref.backward(go)
    assert torch.equal(out, ref)  # the same kernel, written in place
    for gt, t in zip(got, (a, b, wa, wb), strict=True):
        if t.grad is None:
            assert gt is None
        else:
            assert torch.equal(gt, t.grad)


@pytest.mark.parametrize("master", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("t,h_in,hq,hkv,d", [(300, 1024, 8, 2, 128), (129, 512, 4, 4, 64)])
def test_qkv_rope_matches_separate_projections(t, h_in, hq, hkv, d, master):
    """One merged q/k/v GEMM + fused relayouts == three projections + three relayouts; two uses of
    the staged weight in one graph (two TTT steps) sum their weight gradients in one fp32
    accumulator that reaches the parameters through autograd, in the parameters' dtype: bf16
    parameters, and fp32 master parameters under bf16 autocast."""
    from speculators_amd import gemm
    from speculators_amd.fused_ops import rope_inv_freq, rope_relayout
    from speculators_amd.weights import WeightStager

    g = torch.Generator().manual_seed(t)
    x = torch.randn(1, t, h_in, generator=g).bfloat16().cuda().requires_grad_(True)
    ws = [(torch.randn(n, h_in, generator=g) * 0.05).bfloat16().to(master).cuda().requires_grad_(True)
          for n in (hq * d, hkv * d, hkv * d)]
    pos = torch.randint(0, 4000, (t,), generator=g).cuda()
    inv = rope_inv_freq(d, 500000.0, "cuda")
    gos = [torch.randn(1, n, t, d, generator=g).bfloat16().cuda() for n in (hq, hkv, hkv)]
    stager = WeightStager()
    seen = []
    ws[1].register_hook(lambda gr: seen.append(gr.dtype))
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=master == torch.float32):
        stager.begin()
        st = stager.get(*ws)
        assert st.w.dtype == torch.bfloat16 and st.w.shape == ((hq + 2 * hkv) * d, h_in)
        outs = gemm.qkv_rope(x, st, pos, inv, hq, hkv, d, 3) + gemm.qkv_rope(x, st, pos, inv, hq, hkv, d, 3)
    via_grad = torch.autograd.grad(outs, [x, *ws], gos + gos, retain_graph=True)
    torch.autograd.backward(outs, gos + gos)  # a second pass over the retained graph starts afresh
    assert seen == [master, master]
    for got, t_ in zip(via_grad, [x, *ws], strict=True):
        assert got.dtype == t_.dtype and torch.equal(got, t_.grad)
    got_x, got_w = x.grad.clone(), [w.grad.clone() for w in ws]
    x.grad = None
    for w in ws:
        w.grad = None
    ref = []
    for w, heads, rot in zip(ws, (hq, hkv, hkv), (True, True, False), strict=True):
        ref.append(rope_relayout(torch.nn.functional.linear(x, w.bfloat16()), pos, inv, heads, rot,
                                 3 if rot else 0))
    for o, r in zip(outs[:3], ref, strict=True):
        _close(o, r.detach().cpu(), rel=1e-2)
    torch.autograd.backward(ref, gos)
    _close(got_x, 2 * x.grad.cpu())
    for gw, w in zip(got_w, ws, strict=True):
        assert gw.dtype == master
        _close(gw, 2 * w.grad.cpu())
    # existing gradients are added to, not replaced; a frozen member of the group gets none
    ws[2].requires_grad_(False)
    ws[2].grad = None
    for w in ws[:2]:
        w.grad = torch.ones_like(w)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=master == torch.float32):
        stager.begin()
        torch.autograd.backward(gemm.qkv_rope(x, stager.get(*ws), pos, inv, hq, hkv, d, 3), gos)
    assert ws[2].grad is None
    for gw, w in zip(got_w[:2], ws[:2], strict=True):
        _close(w.grad - 1, 0.5 * gw.cpu())


@pytest.mark.parametrize("t,h,f", [(300, 512, 1024), (129, 256, 640)])
def test_gate_up_swiglu_matches_separate_projections(t, h, f):
    """One merged gate/up GEMM + SwiGLU on its two halves == two projections + SwiGLU."""
    from speculators_amd import gemm
    from speculators_amd.fused_ops import swiglu
    from speculators_amd.weights import WeightStager

    g = torch.Generator().manual_seed(t + f)
    x = torch.randn(1, t, h, generator=g).bfloat16().cuda().requires_grad_(True)
    wg = (torch.randn(f, h, generator=g) * 0.05).bfloat16().cuda().requires_grad_(True)
    wu = (torch.randn(f, h, generator=g) * 0.05).bfloat16().cuda().requires_grad_(True)
    go = torch.randn(1, t, f, generator=g).bfloat16().cuda()
    stager = WeightStager()
    stager.begin()
    out = gemm.gate_up_swiglu(x, stager.get(wg, wu))
    out.backward(go)
    got = [x.grad.clone(), wg.grad.clone(), wu.grad.clone()]
    x.grad = wg.grad = wu.grad = None
    ref = swiglu(torch.nn.functional.linear(x, wg), torch.nn.functional.linear(x, wu))
    ref.backward(go)
    _close(out, ref.detach().cpu(), rel=1e-2)
    for a, b in zip(got, (x.grad, wg.grad, wu.grad), strict=True):
        _close(a, b.cpu())


def test_stager_refuses_fp32_outside_autocast_and_keeps_frozen_copies():
    from speculators_amd.weights import WeightStager, compute_input

    w = torch.randn(64, 32, device="cuda")
    stager = WeightStager()
    stager.begin()
    with pytest.raises(RuntimeError, match="autocast"):
        stager.get(w)
    with pytest.raises(RuntimeError, match="autocast"):
        compute_input(torch.randn(4, 4, device="cuda"))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        a = stager.get(w)
        assert a.w.dtype == torch.bfloat16 and torch.equal(a.w, w.bfloat16())
        assert torch.equal(a.wt, w.bfloat16().t().contiguous())
        stager.begin()
        assert stager.get(w) is a and not a.trainable   # a frozen weight is cast once and kept
        w.mul_(2)                            # an in-place change bumps the version counter
        stager.begin()
        b = stager.get(w)
        assert b is not a and torch.equal(b.w, w.bfloat16())
        w.data.add_(1)                       # a write through .data does not: invalidate() does
        stager.invalidate()
        assert torch.equal(stager.get(w).w, w.bfloat16())
        assert compute_input(torch.ones(2, 2, device="cuda")).dtype == torch.bfloat16


@pytest.mark.parametrize("master", [False, True])
def test_gain_gradient_over_several_uses_is_reduced_once(master):
    """A gain read through the weight stager and applied four times in one forward -- by all three
    norm nodes, three times over the same number of rows and once over another -- gets the sum of
    the per-use gradients: the uses with equal rows leave partial sums in one buffer that the
    staging node reduces, the odd one hands autograd a gradient of its own.  Against fp32 autograd
    of the same expression; a second backward over the retained graph gives the same result."""
    from speculators_amd import fused_ops as FO
    from speculators_amd.weights import WeightStager

    h, rows = 512, 300
    g = torch.Generator().manual_seed(3)
    p = (1 + 0.2 * torch.randn(h, generator=g))
    xs = [(torch.randn(1, r, h, generator=g) * 2).bfloat16() for r in (rows, rows, rows, 77)]
    gos = [torch.randn(1, r, h, generator=g).bfloat16() for r in (rows, rows, rows, 77)]
    extra = torch.randn(1, rows, h, generator=g).bfloat16()

    def expression(norm, add_norm, pair, gain, x):
        y0 = norm(x[0], gain)
        _, y1 = add_norm(x[1], extra_d, gain)
        y2 = pair(x[2], x[0], gain, gain)  # both halves of the pair use the gain
        y3 = norm(x[3], gain)
        return y0, y1, y2, y3

    param = p.cuda().to(torch.float32 if master else torch.bfloat16).requires_grad_(True)
    extra_d = extra.cuda()
    stager = WeightStager()
    stager.begin()
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=master):
        gain = stager.gain(param)
        assert stager.gain(param) is gain and gain.dtype == torch.bfloat16
        outs = expression(lambda x, w: FO.rms_norm(x, w, 1e-5),
                          lambda a, b, w: FO.add_rms_norm(a, b, w, 1e-5),
                          lambda a, b, wa, wb: FO.pair_norm_cat(a, b, wa, wb, 1e-5),
                          gain, [x.cuda() for x in xs])
    go2 = torch.cat([gos[2], gos[0]], -1)
    total = sum((o.float() * w.cuda().float()).sum() for o, w in zip(outs, (gos[0], gos[1], go2, gos[3])))
    total.backward(retain_graph=True)
    first = param.grad.clone()
    assert first.dtype == param.dtype
    param.grad = None
    total.backward()
    assert torch.equal(param.grad, first)

    pr = p.bfloat16().float().requires_grad_(True)
    extra_d = extra.float()
    ref = expression(lambda x, w: OE.rms_norm(x, w, 1e-5),
                     lambda a, b, w: (None, OE.rms_norm(a + b, w, 1e-5)),
                     lambda a, b, wa, wb: torch.cat([OE.rms_norm(a, wa, 1e-5), OE.rms_norm(b, wb, 1e-5)], -1),
                     pr, [x.float() for x in xs])
    sum((o * w.float()).sum() for o, w in zip(ref, (gos[0], gos[1], go2, gos[3]))).backward()
    _close(first, pr.grad, rel=1e-2)


@pytest.mark.parametrize("rows", [1, 63, 64, 1024, 1025, 5000])
@pytest.mark.parametrize("with_labels", [False, True])
def test_pack_row_map_and_unpack_rows(rows, with_labels):
    """Row map of the live rows (bit-exact against a running count) and the way back from packed rows."""
    from speculators_amd import _lib

    g = torch.Generator().manual_seed(rows)
    grad = torch.rand(rows, generator=g)
    grad[torch.rand(rows, generator=g) < 0.3] = 0.0
    labels = torch.randint(0, 50, (rows,), generator=g)
    labels[torch.rand(rows, generator=g) < 0.2] = -100
    live = grad != 0
    if with_labels:
        live &= labels != -100
    want = torch.where(live, torch.cumsum(live, 0) - 1, torch.full((rows,), -1)).to(torch.int32)

    gd, ld = grad.cuda(), labels.cuda()
    out = torch.empty(rows + 1, dtype=torch.int32, device="cuda")
    _lib.call("spx_pack_row_map", _lib.ptr(gd), _lib.ptr(ld) if with_labels else None, -100, rows,
              _lib.ptr(out), _lib.ptr(out[rows:]), _lib.stream_ptr(gd.device))
    assert torch.equal(out[:rows].cpu(), want) and int(out[rows]) == int(live.sum())

    cols, total = 72, rows + 3
    packed = torch.randn(rows, cols, generator=g).bfloat16().cuda()
    packed[int(live.sum()):] = float("nan")  # slots past the count must never be read
    back = torch.full((total, 80), 5.0, dtype=torch.bfloat16, device="cuda")
    _lib.call("spx_unpack_rows", _lib.ptr(packed), packed.stride(0), _lib.ptr(out), rows, total, cols,
              _lib.ptr(back), back.stride(0), _lib.stream_ptr(gd.device))
    ref = torch.zeros(total, cols, dtype=torch.bfloat16)
    ref[:rows][live] = packed.cpu()[want[live].long()]
    assert torch.equal(back[:, :cols].cpu(), ref) and (back[:, cols:] == 5).all()


@pytest.mark.parametrize("shape", [(64, 64), (8, 8), (72, 200), (3, 136, 72), (5, 64, 1024), (2, 8, 264)])
def test_transposed_copy_of_a_matrix_or_a_stack(shape):
    """Bit-exact against ``transpose(-1, -2).contiguous()``: tiles at and across the 64 x 64 edge."""
    from speculators_amd.weights import transposed_copy

    g = torch.Generator().manual_seed(sum(shape))
    w = torch.randn(*shape, generator=g).bfloat16().cuda()
    got = transposed_copy(w)
    assert got.is_contiguous() and torch.equal(got, w.transpose(-1, -2).contiguous())
