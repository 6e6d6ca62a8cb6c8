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
    # eight and more query heads per key head with diagonal keys (the 70B shape is 64 : 8):
    # the diagonal-key backward keeps eight heads in registers, walks wider groups in passes
    (256, 8, 1, 128, [100, 140], None, 3),
    (192, 16, 2, 64, None, 32, 3),
    (160, 16, 1, 64, [150], None, 2),            # group 16: two passes of eight heads
    (130, 8, 1, 256, None, None, 3),             # head_dim 256: passes of four heads
    (96, 12, 1, 128, None, None, 2),             # a group that is not a multiple of the pass
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
        # the absolute floor covers gradients that are exactly zero in exact arithmetic (a query that
        # sees a single key has dq = 0; the kernel leaves rounding noise of the order of 1e-7 there)
        assert err <= 2e-2 * want.abs().max().item() + 1e-5, (name, err, want.abs().max().item())
    # the diagonal rows of dk/dv are exactly the per-position gradients: check them apart
    if step > 0:
        err = (kg.grad.float().cpu()[:, :, t:] - kr.grad[:, :, t:]).abs().max().item()
        assert err <= 2e-2 * kr.grad[:, :, t:].abs().max().item() + 1e-5


@pytest.mark.parametrize("d", [96, 80, 40, 192])
def test_head_sizes_between_the_kernels(d):
    """A head size the kernels are not built for runs through the next wider one (zero columns):
    forward and all three gradients against the dense oracle at the real width."""
    from speculators_amd.attention import create_ttt_mask, ttt_attention

    t, hq, hkv, steps, window = 160, 4, 2, 2, None
    g = torch.Generator().manual_seed(d)
    doc = _docs(t, [90, 60])
    mask = create_ttt_mask(doc.cuda(), t, window).extended()
    q = torch.randn(1, hq, t, d, generator=g).bfloat16()
    k = torch.randn(1, hkv, steps * t, d, generator=g).bfloat16()
    v = torch.randn(1, hkv, steps * t, d, generator=g).bfloat16()
    go = torch.randn(1, t, hq, d, generator=g).bfloat16()
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = ttt_attention(qg, kg, vg, mask)  # default scale: that of the real head size
    assert out.shape == (1, t, hq, d)
    out.backward(go.cuda())
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = dense_attention(qr, kr, vr, OM.ttt_mask_dense(doc, t, 1, window), d ** -0.5)
    ref.backward(go.float())
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        assert got.shape == want.shape
        err = (got.float().cpu() - want).abs().max().item()
        assert err <= 2e-2 * want.abs().max().item() + 1e-5, (name, err)
    with pytest.raises(ValueError):
        ttt_attention(torch.zeros(1, hq, t, 320, device="cuda", dtype=torch.bfloat16),
                      torch.zeros(1, hkv, 2 * t, 320, device="cuda", dtype=torch.bfloat16),
                      torch.zeros(1, hkv, 2 * t, 320, device="cuda", dtype=torch.bfloat16), mask)


class _Into(torch.autograd.Function):
    """Writes ``x`` into a window of the K / V cache and returns the window (what the q/k/v
    projection node of the models does with its ``kv_out``)."""

    @staticmethod
    def forward(ctx, x, window):
        # (through an alias with a version counter of its own: the models' kernels write the window
        # through its address, which autograd does not see either)
        torch.from_dlpack(window[0].detach()).copy_(x)
        return window[0]

    @staticmethod
    def backward(ctx, g):
        return g, None


@pytest.mark.parametrize("window", [None, 48])
def test_cache_gradients_shared_by_a_backward_pass_equal_autograds_sum(window):
    """Three chained TTT steps over one K / V cache: the attention nodes of a backward pass add
    their dK / dV into one buffer per layer and return their own step's rows only.  Against the
    same chain on concatenated tensors, where every node returns every step's rows and autograd
    adds them (itself checked against the dense oracle above).  Twice: the second pass must
    start from a fresh buffer."""
    from speculators_amd.attention import TTTKVCache, create_ttt_mask, ttt_attention, ttt_attention_cached

    t, hq, hkv, d, steps = 192, 4, 2, 64, 3
    g = torch.Generator().manual_seed(7)
    doc = _docs(t, [100, 92]).cuda()
    xs = [torch.randn(1, t, hq * d, generator=g).bfloat16().cuda() for _ in range(steps)]
    go = torch.randn(1, t, hq, d, generator=g).bfloat16().cuda()

    def heads(x, n):  # [1, T, n*D] -> [1, n, T, D]
        return x.view(1, t, n, d).transpose(1, 2).contiguous()

    def chain(cached):
        leaves = [x.clone().requires_grad_(True) for x in xs]
        mask = create_ttt_mask(doc, t, window)
        cache = TTTKVCache(hkv, t, d, steps, "cuda")
        ks, vs, h, total = [], [], None, 0
        for j in range(steps):
            h = leaves[j] if h is None else (leaves[j] + 0.5 * h)
            q = heads(h, hq)
            k_new, v_new = heads(h[..., :hkv * d], hkv), heads(h[..., hkv * d:2 * hkv * d] * 0.5, hkv)
            if cached:
                kw, vw = cache.window(j)
                out = ttt_attention_cached(q, _Into.apply(k_new, (kw,)), _Into.apply(v_new, (vw,)), cache, mask)
            else:
                ks.append(k_new)
                vs.append(v_new)
                out = ttt_attention(q, torch.cat(ks, 2), torch.cat(vs, 2), mask)
            total = total + (out.float() * go.float()).sum() * (j + 1)
            h = out.reshape(1, t, hq * d)
            mask = mask.extended()
        return leaves, total

    want_leaves, want = chain(False)
    want.backward()
    leaves, got = chain(True)
    assert (got - want).abs().item() <= 1e-3 * want.abs().item() + 1e-3
    for rep in range(2):
        for x in leaves:
            x.grad = None
        got.backward(retain_graph=rep == 0)
        for j, (a, b) in enumerate(zip(leaves, want_leaves)):
            err = (a.grad.float() - b.grad.float()).abs().max().item()
            assert err <= 2 ** -6 * b.grad.float().abs().max().item(), (rep, j, err)


def test_backward_refuses_more_rows_than_its_tile_list_holds():
    """The dK/dV kernel at head_dim <= 128 lists the query tiles that see a key block in LDS: a call
    with more rows than that list holds is refused before anything is launched (there is no
    second kernel behind it), and the forward of the same call still runs."""
    from speculators_amd._lib import SpxError
    from speculators_amd.attention import create_ttt_mask, ttt_attention

    t = 131072 + 64
    doc = torch.zeros(1, t, dtype=torch.long, device="cuda")
    mask = create_ttt_mask(doc, t, 256)
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.randn(1, 1, t, 64, device="cuda", generator=g).bfloat16().requires_grad_(True)
               for _ in range(3))
    out = ttt_attention(q, k, v, mask)
    assert torch.isfinite(out.float()).all()
    with pytest.raises(SpxError, match="query rows in one call"):
        out.backward(torch.ones_like(out))


def _random_cases(n, seed):
    """Seeded shapes that land on every edge of the tiling: sequences shorter than one key tile,
    one row past a tile, ragged document packs with and without padding, windows shorter and
    longer than a tile, all three head sizes, several query heads per key head."""
    import random

    rnd = random.Random(seed)
    cases = []
    for _ in range(n):
        d = rnd.choice([64, 128, 128, 256])
        t = rnd.choice([1, 2, 31, 33, 63, 64, 65, 127, 129, 191, 257, rnd.randint(3, 400)])
        hkv = rnd.choice([1, 2])
        hq = hkv * rnd.choice([1, 2, 4])
        docs = None
        if t >= 4 and rnd.random() < 0.6:
            cuts = sorted(rnd.sample(range(1, t), min(rnd.randint(1, 4), t - 1)))
            lengths = [b - a for a, b in zip([0] + cuts, cuts + [t])]
            if rnd.random() < 0.5:
                lengths = lengths[:-1]  # the tail becomes padding
            docs = lengths
        window = rnd.choice([None, None, 1, 5, 64, 100])
        cases.append((t, hq, hkv, d, docs, window, rnd.randint(1, 3)))
    return cases


@pytest.mark.parametrize("t,hq,hkv,d,docs,window,steps", _random_cases(24, 20240611))
def test_random_shapes_forward_and_backward(t, hq, hkv, d, docs, window, steps):
    test_forward_matches_dense_oracle(t, hq, hkv, d, docs, window, steps)
    test_backward_matches_dense_oracle_autograd(t, hq, hkv, d, docs, window, steps)


def _check_sampled_rows(q, k, v, out, go, rows, heads, visible, scale):
    """Forward output and dQ of single (row, head) pairs against the explicit fp32 soft-max over
    the keys ``visible(row)`` marks: both depend on that row only."""
    hq, hkv = q.shape[1], k.shape[1]
    for i, h in zip(rows, heads, strict=True):
        kvh = h // (hq // hkv)
        vis = visible(i).cuda()
        qi = q.detach()[0, h, i].float().cpu().requires_grad_(True)
        ks, vs = k.detach()[0, kvh, vis].float().cpu(), v.detach()[0, kvh, vis].float().cpu()
        p = torch.softmax((ks @ qi) * scale, dim=0)
        want = p @ vs
        (want * go[0, i, h].float().cpu()).sum().backward()
        got = out.detach()[0, i, h].float().cpu()
        assert (got - want.detach()).abs().max() <= 2e-2 * want.detach().abs().max() + 1e-3, (i, h)
        dq = q.grad[0, h, i].float().cpu()
        # delta = dO . O is taken from the bf16-rounded output (as in every flash-attention backward):
        # |d delta| <= 2^-9 sum_d |dO_d O_d|, and it reaches dQ through sum_j P_j k_j * scale.  That
        # floor matters for rows with very few keys, where dP - delta nearly cancels
        do = go[0, i, h].float().cpu()
        floor = 2.0 ** -9 * float(do.abs() @ want.detach().abs()) * scale * float(ks.abs().max())
        assert (dq - qi.grad).abs().max() <= 3e-2 * qi.grad.abs().max() + 1e-3 + floor, (i, h)


def _check_dv_checksum(v, go, hq):
    """Rows of P sum to one, so per K/V head: sum over keys of dV == sum over its query heads
    and rows of dO."""
    hkv, d, t = v.shape[1], v.shape[3], go.shape[1]
    dof = go[0].float().view(t, hkv, hq // hkv, d)
    want = dof.sum(dim=(0, 2)).cpu()
    got = v.grad[0].float().sum(dim=1).cpu()
    err = (got - want).abs()
    # what the identity can be off by: every probability enters the product rounded to bf16 (relative
    # 2^-9, and a row's probabilities sum to one), every dV element leaves rounded to bf16 (2^-9 again)
    bound = 2.0 ** -9 * (dof.abs().sum(dim=(0, 2)).cpu() + v.grad[0].float().abs().sum(dim=1).cpu())
    assert (err <= bound).all(), (err.max().item(), bound.min().item())


def _check_context_key_grads(q, k, v, go, keys, visible, scale):
    """dK and dV of single CONTEXT keys against the explicit fp32 soft-max of every (row, head) that sees
    them: ``dV_c = sum p_ic dO_i``, ``dK_c = scale sum p_ic (dP_ic - delta_i) q_i`` over the rows i whose
    visible set holds c and the query heads of the key's group.  (Keys near the end of a document keep
    that set small.)"""
    hq, hkv, t = q.shape[1], k.shape[1], q.shape[2]
    group = hq // hkv
    qf, kf, vf, gf = q.detach().float(), k.detach().float(), v.detach().float(), go.float()
    vis_rows = {}
    for c, kvh in keys:
        dk = torch.zeros(k.shape[3], device=q.device)
        dv = torch.zeros(k.shape[3], device=q.device)
        floor_k = 0.0
        rows = [i for i in range(c % t, t) if bool(visible(i)[c])] if c < t else [c % t]
        assert rows, c
        for i in rows:
            if i not in vis_rows:
                vis_rows[i] = visible(i).cuda()
            vis = vis_rows[i]
            at = int(vis[:c].sum().item())        # position of key c among the row's visible keys
            ks, vs = kf[0, kvh, vis], vf[0, kvh, vis]
            for h in range(kvh * group, (kvh + 1) * group):
                p = torch.softmax((ks @ qf[0, h, i]) * scale, dim=0)
                dp = vs @ gf[0, i, h]
                delta = (p * dp).sum()
                dv += p[at] * gf[0, i, h]
                dk += scale * p[at] * (dp[at] - delta) * qf[0, h, i]
                # delta comes from the bf16-rounded output in the kernel: 2^-9 sum_d |dO O|
                out_abs = (p.unsqueeze(1) * vs).sum(0).abs()
                floor_k += float(2.0 ** -9 * (gf[0, i, h].abs() @ out_abs) * scale * p[at] * qf[0, h, i].abs().max())
        gk, gv = k.grad[0, kvh, c].float(), v.grad[0, kvh, c].float()
        assert (gv - dv).abs().max() <= 3e-2 * dv.abs().max() + 1e-3, ("dV", c, kvh)
        assert (gk - dk).abs().max() <= 3e-2 * dk.abs().max() + 1e-3 + floor_k, ("dK", c, kvh, len(rows))


def test_full_size_sampled_rows_and_checksums():
    """The headline shape (T 4096, 32 q / 8 kv heads, head_dim 128, last TTT step of 7, three
    packed documents and a padded tail), checked through what does not need a dense T x 7T oracle:
    sampled query rows (forward and dQ) and the column-sum identity of dV."""
    from speculators_amd import attention as A

    t, hq, hkv, d, step = 4096, 32, 8, 128, 6
    g = torch.Generator().manual_seed(7)
    doc = torch.full((t,), -1, dtype=torch.long)
    doc[:1500], doc[1500:1501], doc[1501:4000] = 0, 1, 2  # a one-token document in the middle
    q = torch.randn(1, hq, t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    k = torch.randn(1, hkv, (step + 1) * t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    v = torch.randn(1, hkv, (step + 1) * t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    go = torch.randn(1, t, hq, d, generator=g).bfloat16().cuda()
    mask = A.create_ttt_mask(doc.cuda(), t, None)
    for _ in range(step):
        mask = mask.extended()
    out = A.ttt_attention(q, k, v, mask)
    out.backward(go)
    assert torch.isfinite(out).all() and torch.isfinite(q.grad).all() and torch.isfinite(k.grad).all()

    rows = torch.cat([torch.tensor([0, 1, 1499, 1500, 1501, 3999, 4000, 4095]),
                      torch.randint(0, t, (56,), generator=g)]).tolist()
    heads = torch.randint(0, hq, (len(rows),), generator=g).tolist()
    kv_idx = torch.arange((step + 1) * t)

    def visible(i):
        vis = (kv_idx % t) == i  # one key of every step at the row's own position
        if doc[i] != -1:
            vis = vis | ((kv_idx <= i) & (kv_idx < t) & (doc[kv_idx % t] == doc[i]))
        return vis

    _check_sampled_rows(q, k, v, out, go, rows, heads, visible, d ** -0.5)
    _check_dv_checksum(v, go, hq)
    # context keys, dK and dV: the last keys of each document (seen by 1 .. 10 rows), the one-token
    # document, keys further inside (200 and 600 rows, across tile and key-block boundaries) and the
    # first key of a document (seen by all of its rows would be 1500 rows: the 2300th, seen by 1700)
    keys = [(1499, 0), (1497, 3), (1490, 7), (1500, 2), (3999, 1), (3995, 6), (3990, 4), (1300, 5),
            (3400, 0), (2300, 2), (4 * t + 17, 3)]
    _check_context_key_grads(q, k, v, go, keys, visible, d ** -0.5)
    # a key of a later step is seen by exactly one row: its gradient is that row's, never zero
    assert (k.grad[0, :, t:2 * t].float().abs().sum(dim=-1) > 0).all()


def test_70b_shape_sampled_rows_and_checksums():
    """The Llama-3.3-70B draft shape: 64 query heads on 8 key heads (group 8), T 8192, head_dim 128,
    the last of 5 TTT steps; sampled rows (forward, dQ), the dV column-sum identity, and sampled
    diagonal-key gradients against their closed form (a diagonal key is seen by the eight heads of
    its group at its own position only)."""
    from speculators_amd import attention as A

    t, hq, hkv, d, step = 8192, 64, 8, 128, 4
    g = torch.Generator().manual_seed(11)
    doc = torch.full((t,), -1, dtype=torch.long)
    doc[:3000], doc[3000:8000] = 0, 1
    q = torch.randn(1, hq, t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    k = torch.randn(1, hkv, (step + 1) * t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    v = torch.randn(1, hkv, (step + 1) * t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    go = torch.randn(1, t, hq, d, generator=g).bfloat16().cuda()
    mask = A.create_ttt_mask(doc.cuda(), t, None)
    for _ in range(step):
        mask = mask.extended()
    out = A.ttt_attention(q, k, v, mask)
    out.backward(go)
    rows = torch.cat([torch.tensor([0, 2999, 3000, 7999, 8000, 8191]),
                      torch.randint(0, t, (26,), generator=g)]).tolist()
    heads = torch.randint(0, hq, (len(rows),), generator=g).tolist()
    kv_idx = torch.arange((step + 1) * t)

    def visible(i):
        vis = (kv_idx % t) == i
        if doc[i] != -1:
            vis = vis | ((kv_idx <= i) & (kv_idx < t) & (doc[kv_idx % t] == doc[i]))
        return vis

    _check_sampled_rows(q, k, v, out, go, rows, heads, visible, d ** -0.5)
    _check_dv_checksum(v, go, hq)
    # dK / dV of the diagonal key (j, i) of K/V head c: sum over the 8 heads h of its group of
    # p_h (dO_h . v - delta_h) scale q_h  and  p_h dO_h, with p_h from the explicit soft-max
    scale, grp = d ** -0.5, hq // hkv
    for i, c, j in [(5, 0, 1), (2999, 3, 4), (8100, 7, 2), (4096, 5, 3)]:
        vis = visible(i).cuda()
        want_k, want_v = torch.zeros(d), torch.zeros(d)
        for h in range(c * grp, (c + 1) * grp):
            qi = q.detach()[0, h, i].float().cpu()
            ks, vs = k.detach()[0, c, vis].float().cpu(), v.detach()[0, c, vis].float().cpu()
            p = torch.softmax((ks @ qi) * scale, dim=0)
            do = go[0, i, h].float().cpu()
            delta = (p @ vs) @ do
            pos = int((torch.nonzero(vis.cpu()).reshape(-1) == j * t + i).nonzero())
            want_k += p[pos] * (vs[pos] @ do - delta) * scale * qi
            want_v += p[pos] * do
        got_k, got_v = k.grad[0, c, j * t + i].float().cpu(), v.grad[0, c, j * t + i].float().cpu()
        assert (got_k - want_k).abs().max() <= 2e-2 * want_k.abs().max() + 1e-4, (i, c, j)
        assert (got_v - want_v).abs().max() <= 2e-2 * want_v.abs().max() + 1e-4, (i, c, j)


def test_full_size_head_dim_256_sampled_rows():
    """The MTP shape (two packed sequences of 16380, 16 q / 2 kv heads, head_dim 256, causal
    inside each sequence): sampled rows and the dV checksum."""
    from speculators_amd import attention as A

    n, b, hq, hkv, d = 16380, 2, 16, 2, 256
    t = n * b
    g = torch.Generator().manual_seed(9)
    seq = torch.arange(b).repeat_interleave(n)
    q = torch.randn(1, hq, t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    k = torch.randn(1, hkv, t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    v = torch.randn(1, hkv, t, d, generator=g).bfloat16().cuda().requires_grad_(True)
    go = torch.randn(1, t, hq, d, generator=g).bfloat16().cuda()
    out = A.ttt_attention(q, k, v, A.create_ttt_mask(seq.cuda(), t, None), d ** -0.5)
    out.backward(go)
    rows = torch.cat([torch.tensor([0, 1, n - 1, n, n + 1, t - 1]),
                      torch.randint(0, t, (26,), generator=g)]).tolist()
    heads = torch.randint(0, hq, (len(rows),), generator=g).tolist()
    kv_idx = torch.arange(t)
    _check_sampled_rows(q, k, v, out, go, rows, heads,
                        lambda i: (kv_idx <= i) & (seq == seq[i]), d ** -0.5)
    _check_dv_checksum(v, go, hq)
