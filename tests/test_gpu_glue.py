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
