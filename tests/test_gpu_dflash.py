"""HIP anchored-block (DFlash) attention and model against the oracle."""

import pytest
import torch

from oracle import dflash as OD
from oracle import masks as OM
from oracle.attention import dense_attention
from oracle.eagle3 import DraftShape

pytestmark = pytest.mark.gpu


def _docs(t, lengths):
    doc = torch.full((t,), -1, dtype=torch.long)
    o = 0
    for i, n in enumerate(lengths):
        doc[o:o + n] = i
        o += n
    return doc


CASES = [
    # (T, Hq, Hkv, D, docs, anchors, block, window, non_causal_flag)
    (256, 4, 2, 128, [256], [3, 40, 41, 100, 200, 230], 16, None, False),
    (320, 4, 2, 64, [100, 150, 50], [0, 5, 99, 100, 180, 249, 251, 310], 8, None, False),
    (512, 8, 2, 128, [200, 300], [10, 150, 199, 205, 400, 490], 16, 64, False),
    (512, 4, 4, 64, [512], [17, 100, 333, 480, 0, 0], 16, 48, True),   # trailing padded anchors
    (200, 2, 1, 64, [77, 100], [5, 76, 80, 150, 190], 5, 16, False),   # block size not a power of 2, padding doc
]


@pytest.mark.parametrize("t,hq,hkv,d,docs,anchors,bs,window,ncf", CASES)
def test_row_ranges_bit_exact(t, hq, hkv, d, docs, anchors, bs, window, ncf):
    from speculators_amd.attention import create_dflash_mask

    doc = _docs(t, docs)
    a = torch.tensor(anchors)
    for dt in (torch.int64, torch.int32):
        m = create_dflash_mask(doc.to(dt).cuda(), t, a.to(dt).cuda(), bs, window, ncf)
        lo, hi = OM.dflash_row_range(doc, a, bs, window)
        assert torch.equal(m.ctx_lo.cpu(), lo) and torch.equal(m.ctx_hi.cpu(), hi)
        dense = OM.dflash_mask_dense(doc, t, a, bs, window, ncf)
        for r in range(dense.shape[0]):
            exp = torch.zeros(dense.shape[0], dtype=torch.bool)
            exp[int(m.blk_lo[r]): int(m.blk_hi[r])] = True
            assert torch.equal(dense[r, t:], exp), r


@pytest.mark.parametrize("t,hq,hkv,d,docs,anchors,bs,window,ncf", CASES)
def test_forward_backward_match_dense_oracle(t, hq, hkv, d, docs, anchors, bs, window, ncf):
    from speculators_amd.attention import create_dflash_mask, dflash_attention

    g = torch.Generator().manual_seed(t + d + bs)
    doc = _docs(t, docs)
    a = torch.tensor(anchors)
    nq = len(anchors) * bs
    q = torch.randn(1, hq, nq, d, generator=g).bfloat16()
    k = torch.randn(1, hkv, t + nq, d, generator=g).bfloat16()
    v = torch.randn(1, hkv, t + nq, d, generator=g).bfloat16()
    go = torch.randn(1, nq, hq, d, generator=g).bfloat16()
    mask = create_dflash_mask(doc.cuda(), t, a.cuda(), bs, window, ncf)
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = dflash_attention(qg, kg, vg, mask, d ** -0.5)
    out.backward(go.cuda())
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = dense_attention(qr, kr, vr, OM.dflash_mask_dense(doc, t, a, bs, window, ncf), d ** -0.5)
    ref.backward(go.float())
    err = (out.float().cpu() - ref.detach()).abs().max().item()
    assert err <= 2e-2 * ref.abs().max().item(), err
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        e = (got.float().cpu() - want).abs().max().item()
        assert e <= 2e-2 * want.abs().max().item() + 1e-5, (name, e, want.abs().max().item())


def _random_cases(n, seed):
    """Seeded anchored-block cases on the edges of the tiling: contexts shorter than one key tile or
    one row past it, block sizes 1 .. 16, a single anchor, padded anchor lists, windows shorter than a
    block, all three head sizes."""
    import random

    rnd = random.Random(seed)
    cases = []
    while len(cases) < n:
        d = rnd.choice([64, 128, 128, 256])
        bs = rnd.choice([1, 2, 5, 8, 16])
        t = rnd.choice([33, 64, 65, 130, 257, rnd.randint(bs + 2, 300)])
        if t <= bs + 1:
            continue
        hkv = rnd.choice([1, 2])
        hq = hkv * rnd.choice([1, 2, 4])
        cuts = sorted(rnd.sample(range(1, t), min(rnd.randint(0, 3), t - 1)))
        lengths = [b - a for a, b in zip([0] + cuts, cuts + [t])]
        if len(lengths) > 1 and rnd.random() < 0.4:
            lengths = lengths[:-1]  # the tail becomes padding
        live = min(sum(lengths), t - bs)
        anchors = sorted(rnd.sample(range(live), min(rnd.randint(1, 12), live)))
        if rnd.random() < 0.3:
            anchors += [0] * rnd.randint(1, 3)  # padded anchor slots
        window = rnd.choice([None, None, 1, 5, 64])
        cases.append((t, hq, hkv, d, lengths, anchors, bs, window, window is not None and rnd.random() < 0.5))
    return cases


@pytest.mark.parametrize("t,hq,hkv,d,docs,anchors,bs,window,ncf", _random_cases(20, 977))
def test_random_shapes(t, hq, hkv, d, docs, anchors, bs, window, ncf):
    test_row_ranges_bit_exact(t, hq, hkv, d, docs, anchors, bs, window, ncf)
    test_forward_backward_match_dense_oracle(t, hq, hkv, d, docs, anchors, bs, window, ncf)


@pytest.mark.parametrize("weighting,sliding,head_dim", [("fixed-exp-decay", False, 64), ("dpace", True, 64),
                                                        ("fixed-exp-decay", True, 96)])
def test_model_forward_backward_matches_oracle(weighting, sliding, head_dim):
    from speculators_amd import losses as L
    from speculators_amd.dflash import DFlashConfig, DFlashDraftModel

    kw = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=head_dim,
              intermediate_size=512, vocab_size=2000, draft_vocab_size=704, num_aux=2,
              num_hidden_layers=2, rms_norm_eps=1e-6, rope_theta=10000.0)
    sl = dict(sliding_window=40, sliding_layers=(1,)) if sliding else {}
    shape = DraftShape(qk_norm=True, **kw, **sl)
    w32 = OD.random_weights(shape, seed=4, std=0.05)
    g = torch.Generator().manual_seed(12)
    for k_ in w32:
        if "norm" in k_:
            w32[k_] = 1 + 0.1 * torch.randn(w32[k_].shape, generator=g)
    w = {k_: v.bfloat16() for k_, v in w32.items()}
    t, bs = 320, 8
    hs = torch.randn(1, t, 2 * 256, generator=g).bfloat16()
    ids = torch.randint(0, 2000, (1, t), generator=g)
    vl = torch.randn(1, t, 256, generator=g).bfloat16()
    mask = (torch.rand(1, t, generator=g) < 0.8).float()
    doc = _docs(t, [140, 160]).unsqueeze(0)
    mask[0, 300:] = 0
    pos = torch.cat([torch.arange(140), torch.arange(160), torch.zeros(20, dtype=torch.long)]).unsqueeze(0)
    anchors = OD.select_anchors(mask, 24, bs, g)
    loss_name = "ce" if weighting == "dpace" else "kl_div"

    model = DFlashDraftModel(DFlashConfig(block_size=bs, mask_token_id=7, **kw, **sl))
    missing, unexpected = model.load_state_dict(w, strict=False)
    assert not unexpected and set(missing) <= {"t2d", "d2t"}
    model = model.to(torch.bfloat16).cuda()
    _, loss, m = model(hs.cuda(), ids.cuda(), mask.cuda(), vl.cuda(), doc.cuda(), pos.cuda(),
                       loss_config=L.resolve_loss_config(loss_name), gamma=4.0,
                       per_position_loss_weight=weighting, dpace_alpha=0.5,
                       anchors=(anchors[0].cuda(), anchors[1].cuda()))
    loss.backward()

    from oracle import losses as OL
    wf = {k_: v.float().requires_grad_(True) for k_, v in w.items()}
    _, rloss, rm = OD.dflash_forward(wf, shape, hs.float(), ids, mask, vl.float(), doc, pos,
                                     block_size=bs, mask_token_id=7,
                                     loss_config=OL.resolve_loss_config(loss_name), gamma=4.0,
                                     per_position_loss_weight=weighting, dpace_alpha=0.5,
                                     anchors=anchors)
    rloss.backward()
    rel = abs(loss.item() - rloss.item()) / abs(rloss.item())
    print("dflash loss", loss.item(), rloss.item(), rel)
    assert rel < 2e-3
    assert set(m) == set(rm)
    for key in rm:
        if key.endswith("_total"):
            assert m[key].item() == rm[key].item(), key
    # the same oracle in bf16 on the CPU gives the rounding noise floor of this model
    wb = {k_: v.clone().requires_grad_(True) for k_, v in w.items()}
    _, bloss, _ = OD.dflash_forward(wb, shape, hs, ids, mask, vl, doc, pos, block_size=bs,
                                    mask_token_id=7, loss_config=OL.resolve_loss_config(loss_name),
                                    gamma=4.0, per_position_loss_weight=weighting, dpace_alpha=0.5,
                                    anchors=anchors)
    bloss.backward()
    for name, p in model.named_parameters():
        if not p.requires_grad:
            continue
        want = wf[name].grad
        scale = want.abs().max().item()
        err = (p.grad.float().cpu() - want).abs().max().item()
        floor = (wb[name].grad.float() - want).abs().max().item()
        # 2e-2 relative max-norm, or twice the error a bf16 PyTorch run of the oracle makes
        assert err <= max(2e-2 * scale, 2 * floor) + 1e-6, (name, err, floor, scale)


def test_full_size_sampled_rows():
    """configs[2] shape (seq 8192, 512 anchors x block 16 -> 8192 queries, 16384 keys, window
    2048, 32 q / 8 kv heads, head_dim 128): sampled rows (forward and dQ) against the explicit
    fp32 soft-max over the keys the mask rule of models/dflash/attention.py:7-100 lets each row
    see, and the dV column-sum identity."""
    from speculators_amd import attention as A
    from tests.test_gpu_attention import _check_dv_checksum, _check_sampled_rows

    t, bs, n_anchor, w, hq, hkv, d = 8192, 16, 512, 2048, 32, 8, 128
    g = torch.Generator().manual_seed(13)
    doc = torch.zeros(t, dtype=torch.long)
    doc[5000:] = 1
    anchors = (torch.arange(n_anchor) * ((t - bs) // n_anchor) + 1)
    n_q = n_anchor * bs
    q = torch.randn(1, hq, n_q, d, generator=g).bfloat16().cuda().requires_grad_(True)
    k = torch.randn(1, hkv, t + n_q, d, generator=g).bfloat16().cuda().requires_grad_(True)
    v = torch.randn(1, hkv, t + n_q, d, generator=g).bfloat16().cuda().requires_grad_(True)
    go = torch.randn(1, n_q, hq, d, generator=g).bfloat16().cuda()
    mask = A.create_dflash_mask(doc.cuda(), t, anchors.cuda(), bs, w, False)
    out = A.dflash_attention(q, k, v, mask)
    out.backward(go)
    rows = torch.cat([torch.tensor([0, 15, 16, n_q - 1]), torch.randint(0, n_q, (28,), generator=g)]).tolist()
    heads = torch.randint(0, hq, (len(rows),), generator=g).tolist()
    kv_idx = torch.arange(t + n_q)

    def visible(i):
        blk, a = i // bs, int(anchors[i // bs])
        ctx = (kv_idx < t) & (kv_idx < a) & (kv_idx >= a - w) & (doc[kv_idx.clamp(max=t - 1)] == doc[a])
        own = (kv_idx >= t) & ((kv_idx - t) // bs == blk) & (kv_idx - t <= i)  # windowed layer: causal block
        return ctx | own

    _check_sampled_rows(q, k, v, out, go, rows, heads, visible, d ** -0.5)
    _check_dv_checksum(v, go, hq)


@pytest.mark.parametrize("weighting,loss_name", [("fixed-exp-decay", "kl_div"), ("dpace", "ce")])
def test_head_and_loss_as_one_node_changes_nothing(weighting, loss_name):
    """lm_head + fused loss as one autograd node against the two-node form: loss, metrics and every
    parameter gradient bit for bit."""
    from speculators_amd import losses as L
    from speculators_amd.dflash import DFlashConfig, DFlashDraftModel

    kw = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
              intermediate_size=512, vocab_size=2000, draft_vocab_size=704, num_aux=2,
              num_hidden_layers=2, rms_norm_eps=1e-6, rope_theta=10000.0)
    shape = DraftShape(qk_norm=True, **kw)
    w = {k_: v.bfloat16() for k_, v in OD.random_weights(shape, seed=6, std=0.05).items()}
    g = torch.Generator().manual_seed(13)
    t, bs = 256, 8
    hs = torch.randn(1, t, 2 * 256, generator=g).bfloat16()
    ids = torch.randint(0, 2000, (1, t), generator=g)
    vl = torch.randn(1, t, 256, generator=g).bfloat16()
    mask = (torch.rand(1, t, generator=g) < 0.6).float()
    doc = _docs(t, [100, 156]).unsqueeze(0)
    pos = torch.cat([torch.arange(100), torch.arange(156)]).unsqueeze(0)
    anchors = OD.select_anchors(mask, 20, bs, g)
    got = []
    for fuse in (True, False):
        model = DFlashDraftModel(DFlashConfig(block_size=bs, mask_token_id=7, **kw))
        model.load_state_dict(w, strict=False)
        model = model.to(torch.bfloat16).cuda()
        model.fuse_head_loss = fuse
        _, loss, m = model(hs.cuda(), ids.cuda(), mask.cuda(), vl.cuda(), doc.cuda(), pos.cuda(),
                           loss_config=L.resolve_loss_config(loss_name), gamma=4.0,
                           per_position_loss_weight=weighting, dpace_alpha=0.5,
                           anchors=(anchors[0].cuda(), anchors[1].cuda()))
        loss.backward()
        got.append((loss.detach(), {k_: v.clone() for k_, v in m.items()},
                    {k_: p.grad.clone() for k_, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(got[0][0], got[1][0])
    for k_ in got[0][1]:
        assert torch.equal(got[0][1][k_], got[1][1][k_]), k_
    assert got[0][2].keys() == got[1][2].keys() and len(got[0][2]) > 5
    for k_ in got[0][2]:
        assert torch.equal(got[0][2][k_], got[1][2][k_]), k_
