"""HIP TTT attention against the oracle's dense-mask attention (through the C ABI)."""

import pytest
import torch

from oracle import masks as OM
from oracle.attention import dense_attention

pytestmark = pytest.mark.gpu


def _docs(t, lengths):
    doc = torch.full((t,), -1, dtype=torch.long)
    o = 0
    for i, n in enumerate(lengths):
        doc[o:o + n] = i
        o += n
    return doc


CASES = [
    # (T, Hq, Hkv, D, docs, window, steps)
    (128, 4, 2, 128, None, None, 3),
    (256, 8, 2, 64, None, None, 2),
    (320, 4, 1, 128, [100, 150, 50], None, 3),   # 20 padding rows, ragged T
    (512, 4, 4, 128, [200, 300], 64, 2),
    (200, 2, 2, 64, [77], 16, 4),                # T not a tile multiple, padding tail
]


@pytest.mark.parametrize("t,hq,hkv,d,docs,window,steps", CASES)
def test_row_lo_bit_exact(t, hq, hkv, d, docs, window, steps):
    from speculators_amd.attention import create_ttt_mask

    doc = torch.zeros(t, dtype=torch.long) if docs is None else _docs(t, docs)
    for dt in (torch.int64, torch.int32):
        m = create_ttt_mask(doc.to(dt).cuda().unsqueeze(0), t, window)
        assert torch.equal(m.row_lo.cpu(), OM.ttt_row_lo(doc, window))


@pytest.mark.parametrize("t,hq,hkv,d,docs,window,steps", CASES)
def test_forward_matches_dense_oracle(t, hq, hkv, d, docs, window, steps):
    from speculators_amd.attention import create_ttt_mask, ttt_attention

    g = torch.Generator().manual_seed(t + d)
    doc = torch.zeros(t, dtype=torch.long) if docs is None else _docs(t, docs)
    mask = create_ttt_mask(doc.cuda(), t, window)
    ks, vs = [], []
    for step in range(steps):
        q = torch.randn(1, hq, t, d, generator=g).bfloat16()
        ks.append(torch.randn(1, hkv, t, d, generator=g).bfloat16())
        vs.append(torch.randn(1, hkv, t, d, generator=g).bfloat16())
        k, v = torch.cat(ks, 2), torch.cat(vs, 2)
        out = ttt_attention(q.cuda(), k.cuda(), v.cuda(), mask, d ** -0.5)
        ref = dense_attention(q.float(), k.float(), v.float(),
                              OM.ttt_mask_dense(doc, t, step, window), d ** -0.5)
        assert out.shape == (1, t, hq, d) and out.dtype == torch.bfloat16
        err = (out.float().cpu() - ref).abs().max().item()
        assert err <= 2e-2 * ref.abs().max().item(), (step, err)
        mask = mask.extended()


@pytest.mark.parametrize("t,hq,hkv,d,docs,window,steps", CASES)
def test_backward_matches_dense_oracle_autograd(t, hq, hkv, d, docs, window, steps):
    from speculators_amd.attention import create_ttt_mask, ttt_attention

    g = torch.Generator().manual_seed(7 * t + d)
    doc = torch.zeros(t, dtype=torch.long) if docs is None else _docs(t, docs)
    step = steps - 1
    mask = create_ttt_mask(doc.cuda(), t, window)
    for _ in range(step):
        mask = mask.extended()
    q = torch.randn(1, hq, t, d, generator=g).bfloat16()
    k = torch.randn(1, hkv, steps * t, d, generator=g).bfloat16()
    v = torch.randn(1, hkv, steps * t, d, generator=g).bfloat16()
    go = torch.randn(1, t, hq, d, generator=g).bfloat16()
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = ttt_attention(qg, kg, vg, mask, d ** -0.5)
    out.backward(go.cuda())
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = dense_attention(qr, kr, vr, OM.ttt_mask_dense(doc, t, step, window), d ** -0.5)
    ref.backward(go.float())
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        err = (got.float().cpu() - want).abs().max().item()
        assert err <= 2e-2 * want.abs().max().item(), (name, err, want.abs().max().item())
    # the diagonal rows of dk/dv are exactly the per-position gradients: check them apart
    if step > 0:
        err = (kg.grad.float().cpu()[:, :, t:] - kr.grad[:, :, t:]).abs().max().item()
        assert err <= 2e-2 * kr.grad[:, :, t:].abs().max().item()
