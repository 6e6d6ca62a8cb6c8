"""HIP bf16 GEMM against an fp32 reference product (through the C ABI)."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (512, 768, 256), (300, 1000, 136),
                                   (1, 32000, 128), (4096, 512, 4096), (257, 255, 8)])
def test_gemm_nt_matches_fp32_reference(m, n, k):
    from speculators_amd.gemm import gemm_nt

    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    b = torch.randn(n, k, generator=g).bfloat16()
    got = gemm_nt(a.cuda(), b.cuda()).float().cpu()
    ref = a.float() @ b.float().T
    # bf16 output rounding: 2^-8 relative, plus fp32 accumulation noise
    torch.testing.assert_close(got, ref, rtol=1e-2, atol=1e-2 * ref.abs().max().item() * 0.05)


def test_gemm_strided_rows():
    from speculators_amd.gemm import gemm_nt

    g = torch.Generator().manual_seed(0)
    a_full = torch.randn(100, 512, generator=g).bfloat16().cuda()
    b = torch.randn(77, 256, generator=g).bfloat16().cuda()
    a = a_full[:, 128:384]  # lda 512, offset 256 B
    got = gemm_nt(a, b).float().cpu()
    ref = a.float().cpu() @ b.float().cpu().T
    torch.testing.assert_close(got, ref, rtol=1e-2, atol=0.1)


def test_linear_autograd_matches_fp32():
    from speculators_amd.gemm import linear

    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 300, 256, generator=g).bfloat16()
    w = (torch.randn(520, 256, generator=g) * 0.05).bfloat16()
    go = torch.randn(1, 300, 520, generator=g).bfloat16()
    for use_wt in (False, True):
        xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
        y = linear(xg, wg, wg.detach().t().contiguous() if use_wt else None)
        y.backward(go.cuda())
        xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
        yr = torch.nn.functional.linear(xr, wr)
        yr.backward(go.float())
        for got, want in ((y, yr), (xg.grad, xr.grad), (wg.grad, wr.grad)):
            err = (got.float().cpu() - want.detach()).abs().max().item()
            assert err <= 2e-2 * want.abs().max().item()


@pytest.mark.parametrize("m,k", [(4096, 4096), (8192, 8192)])
def test_full_size_lm_head_shape_sampled_and_linear(m, k):
    """The lm_head shapes of the 8B draft (4096 x 4096 x 32000) and of the 70B draft
    (8192 x 8192 x 32000): sampled output rows against an fp32 product of the same bf16 operands,
    and linearity in the first operand (bf16 rounding of each result aside)."""
    from speculators_amd.gemm import gemm_nt

    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randn(m, k, device="cuda", generator=g).bfloat16()
    a2 = torch.randn(m, k, device="cuda", generator=g).bfloat16()
    b = (torch.randn(32000, k, device="cuda", generator=g) * 0.02).bfloat16()
    c = gemm_nt(a, b)
    rows = torch.randint(0, m, (64,), device="cuda", generator=g)
    want = a[rows].float() @ b.float().t()
    assert (c[rows].float() - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-3
    # every tile edge of the 256 x 256 tiling is exercised: first / last rows and columns
    edge = torch.tensor([0, 255, 256, m - 1], device="cuda")
    want_e = a[edge].float() @ b.float().t()
    assert (c[edge].float() - want_e).abs().max() <= 2 ** -8 * want_e.abs().max() + 1e-3
    s = (a.float() + a2.float()).bfloat16()  # exact sums are not representable: compare against fp32
    c_sum = gemm_nt(s, b)
    want_s = s[rows].float() @ b.float().t()
    assert (c_sum[rows].float() - want_s).abs().max() <= 2 ** -8 * want_s.abs().max() + 1e-3
    # identical inputs give identical bits (fixed reduction order)
    assert torch.equal(c, gemm_nt(a, b))


@pytest.mark.parametrize("t,m,n", [(64, 256, 256), (72, 8, 8), (1, 16, 24), (200, 264, 520),
                                   (129, 40, 1000), (4096, 512, 256), (257, 776, 392)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_gemm_tn_matches_fp32_reference(t, m, n, accumulate):
    """The weight-gradient product dY^T X, plain and added to what the output holds: tile
    edges in all three dimensions, a contraction shorter than one slab, odd slab counts."""
    from speculators_amd.gemm import gemm_tn

    g = torch.Generator().manual_seed(t + m + n)
    a = torch.randn(t, m, generator=g).bfloat16()
    b = torch.randn(t, n, generator=g).bfloat16()
    ref = a.float().T @ b.float()
    if accumulate:
        c0 = (torch.randn(m, n, generator=g) * 30).bfloat16()
        ref = ref + c0.float()
        got = gemm_tn(a.cuda(), b.cuda(), c0.cuda(), accumulate=True).float().cpu()
    else:
        got = gemm_tn(a.cuda(), b.cuda()).float().cpu()
    # one rounding to bf16 of the fp32 result
    assert (got - ref).abs().max() <= 2 ** -8 * ref.abs().max() + 1e-3


@pytest.mark.parametrize("t,m,n", [(72, 8, 8), (200, 264, 520), (129, 40, 1000), (4096, 512, 256), (257, 776, 392)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_gemm_tn_fp32_result(t, m, n, accumulate):
    """The same product with an fp32 result: no rounding of the result at all, and accumulation
    over calls adds in fp32 (the gradient of an fp32 master weight summed over the TTT steps)."""
    from speculators_amd.gemm import gemm_tn

    g = torch.Generator().manual_seed(3 * t + m + n)
    a = torch.randn(t, m, generator=g).bfloat16()
    b = torch.randn(t, n, generator=g).bfloat16()
    ref = a.double().T @ b.double()
    if accumulate:
        c0 = torch.randn(m, n, generator=g) * 30
        out_full = torch.full((m, n + 12), 7.0, device="cuda")
        out = out_full[:, 4:4 + n]
        out.copy_(c0)
        got = gemm_tn(a.cuda(), b.cuda(), out, accumulate=True)
        assert got.data_ptr() == out.data_ptr()
        assert (out_full[:, :4] == 7).all() and (out_full[:, 4 + n:] == 7).all()
        ref = ref + c0.double()
    else:
        got = gemm_tn(a.cuda(), b.cuda(), out_dtype=torch.float32)
    assert got.dtype == torch.float32
    # fp32 accumulation of t products of bf16 values
    assert (got.double().cpu() - ref).abs().max() <= 2e-6 * t ** 0.5 * ref.abs().max() + 1e-5


def test_gemm_tn_fp32_accumulates_like_one_fp32_sum():
    """Seven calls into one fp32 accumulator (one per TTT step) equal the fp32 sum of the seven
    products to fp32 rounding, where a bf16 accumulator would lose 2^-8 per call."""
    from speculators_amd.gemm import gemm_tn

    g = torch.Generator(device="cuda").manual_seed(2)
    acc = torch.zeros(512, 768, device="cuda")
    want = torch.zeros(512, 768, device="cuda", dtype=torch.float64)
    for _ in range(7):
        dy = torch.randn(1024, 512, device="cuda", generator=g).bfloat16()
        x = torch.randn(1024, 768, device="cuda", generator=g).bfloat16()
        gemm_tn(dy, x, acc, accumulate=True)
        want += dy.double().t() @ x.double()
    assert (acc.double() - want).abs().max() <= 1e-5 * want.abs().max()


def test_gemm_tn_strided_operands_and_output():
    from speculators_amd.gemm import gemm_tn

    g = torch.Generator().manual_seed(5)
    a = torch.randn(300, 272, generator=g).bfloat16().cuda()[:, :264]
    b = torch.randn(300, 144, generator=g).bfloat16().cuda()[:, 8:144]
    out_full = torch.full((264, 200), 7.0, dtype=torch.bfloat16, device="cuda")
    out = out_full[:, 32:168]
    gemm_tn(a, b, out)
    ref = a.float().T @ b.float()
    assert (out.float() - ref).abs().max() <= 2 ** -8 * ref.abs().max() + 1e-3
    # nothing outside the view was touched
    assert (out_full[:, :32] == 7).all() and (out_full[:, 168:] == 7).all()


def test_gemm_tn_matches_library_on_a_layer_shape():
    """The o_proj weight gradient of the 8B draft layer (T = 4096, 4096 x 4096): sampled rows
    against fp32, repeatability, and accumulation over two calls against one fp32 sum."""
    from speculators_amd.gemm import gemm_tn

    g = torch.Generator(device="cuda").manual_seed(11)
    dy = torch.randn(4096, 4096, device="cuda", generator=g).bfloat16()
    x = torch.randn(4096, 4096, device="cuda", generator=g).bfloat16()
    c = gemm_tn(dy, x)
    rows = torch.tensor([0, 255, 256, 1000, 4095], device="cuda")
    want = dy[:, rows].float().t() @ x.float()
    assert (c[rows].float() - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-3
    assert torch.equal(c, gemm_tn(dy, x))
    acc = c.clone()
    gemm_tn(dy, x, acc, accumulate=True)
    want2 = c[rows].float() + want
    assert (acc[rows].float() - want2).abs().max() <= 2 ** -8 * want2.abs().max() + 1e-3


def test_gemm_tn_rejects_bad_arguments():
    from speculators_amd import _lib
    from speculators_amd.gemm import gemm_tn

    a = torch.zeros(16, 12, dtype=torch.bfloat16, device="cuda")  # M not a multiple of 8
    b = torch.zeros(16, 8, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.SpxError):
        gemm_tn(a, b)
    with pytest.raises(ValueError):
        gemm_tn(b, torch.zeros(8, 8, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        gemm_tn(b, b, accumulate=True)


@pytest.mark.parametrize("m,live", [(600, 0), (600, 1), (600, 256), (600, 257), (600, 599), (600, 600), (600, 900)])
def test_gemm_nt_with_a_row_count_on_the_device(m, live):
    """Rows from the device-side count on are neither read (they hold NaN here) nor written
    (the output keeps its fill value); the rows before it equal the plain product bit for bit."""
    from speculators_amd.gemm import gemm_nt

    g = torch.Generator().manual_seed(live)
    a = torch.randn(m, 136, generator=g).bfloat16().cuda()
    b = torch.randn(300, 136, generator=g).bfloat16().cuda()
    want = gemm_nt(a, b)
    n_live = min(live, m)
    a_dirty = a.clone()
    a_dirty[n_live:] = float("nan")
    out = torch.full((m, 300), 7.0, dtype=torch.bfloat16, device="cuda")
    count = torch.tensor([live], dtype=torch.int32, device="cuda")
    gemm_nt(a_dirty, b, out, m_live=count)
    assert torch.equal(out[:n_live], want[:n_live])
    assert (out[n_live:] == 7).all()


def _cu_rounds(tiles, parts, cus=256):
    return -(-tiles * parts // cus) / parts


@pytest.mark.parametrize("m,n,k,live,parts_expected", [
    (4096, 4096, 4096, 2860, 4),     # 12 x 16 = 192 tiles: three rounds of a quarter instead of one whole
    (4096, 4096, 4096, 2000, 2),     # 128 tiles: one round of a half
    (4096, 4096, 4096, 4096, 1),     # 256 tiles: nothing to gain, the direct store
    (4096, 4096, 4096, 0, 1),        # nothing counts, nothing is written
    (1200, 520, 6000, 700, 4),       # ragged: 3 x 3 tiles, N not a tile multiple, last part shorter
    (1200, 520, 1000, 700, 1),       # contraction too short to cut
])
def test_gemm_nt_rows_with_the_contraction_in_parts(m, n, k, live, parts_expected):
    """``gemm_nt(split=True)``: the kernel cuts the contraction when the live rows' tiles leave compute
    units idle (the count of parts follows from the row count on the device) and adds the fp32 partials
    in order.  Same rows written as by the plain live-rows product, equal to it up to the rounding of
    one bf16 value (and to the fp32 product), repeatable bit for bit; dead rows untouched."""
    from speculators_amd import gemm as G

    tiles = -(-min(live, m) // 256) * -(-n // 256)
    best = min(range(1, G.SPLIT_PARTS + 1), key=lambda s_: (_cu_rounds(tiles, s_), s_)) if tiles else 1
    if k // 64 // max(best, 1) < 16 or _cu_rounds(tiles, best) > 0.9 * _cu_rounds(tiles, 1):
        best = 1
    assert best == parts_expected  # (the rule the kernel applies, restated for the cases above)
    g = torch.Generator(device="cuda").manual_seed(m + live)
    a = torch.randn(m, k, device="cuda", generator=g).bfloat16()
    b = (torch.randn(n, k, device="cuda", generator=g) * 0.05).bfloat16()
    n_live = min(live, m)
    a[n_live:] = float("nan")
    count = torch.tensor([live], dtype=torch.int32, device="cuda")
    plain = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    G.gemm_nt(a, b, plain, m_live=count)
    outs = []
    for _ in range(2):
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
        G.gemm_nt(a, b, out, m_live=count, split=True)
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    assert (outs[0][n_live:] == 7).all()
    if n_live:
        ref = a[:n_live].float() @ b.float().t()
        scale = ref.abs().max().item()
        assert (outs[0][:n_live].float() - ref).abs().max().item() <= 1e-2 * scale
        assert (outs[0][:n_live].float() - plain[:n_live].float()).abs().max().item() <= 1e-2 * scale
        if parts_expected == 1:
            assert torch.equal(outs[0][:n_live], plain[:n_live])


def test_gemm_nt_rows_split_rejects_bad_arguments():
    from speculators_amd import _lib

    a = torch.zeros(256, 2048, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(264, 2048, dtype=torch.bfloat16, device="cuda")
    c = torch.zeros(256, 264, dtype=torch.bfloat16, device="cuda")
    cnt = torch.tensor([256], dtype=torch.int32, device="cuda")
    ws = torch.zeros(4 * 256 * 264, dtype=torch.float32, device="cuda")
    st = _lib.stream_ptr(a.device)

    def call(parts, ws_bytes, n=264, ldc=264):
        _lib.call("spx_gemm_bf16_nt_rows_split", _lib.ptr(a), 2048, _lib.ptr(b), 2048, _lib.ptr(c), ldc, 256, n,
                  2048, _lib.ptr(cnt), parts, _lib.ptr(ws), ws_bytes, st)

    call(4, ws.numel() * 4)
    assert _lib.load().spx_gemm_split_workspace_bytes(256, 264, 4) == 4 * 256 * 264 * 4
    for bad in (dict(parts=0, ws_bytes=ws.numel() * 4), dict(parts=9, ws_bytes=ws.numel() * 4),
                dict(parts=4, ws_bytes=ws.numel() * 4 - 1), dict(parts=4, ws_bytes=ws.numel() * 4, n=260)):
        with pytest.raises(_lib.SpxError):
            call(**bad)


@pytest.mark.parametrize("t,m,n", [(8192, 264, 136), (5000, 512, 512), (20000, 8, 1024)])
@pytest.mark.parametrize("fp32", [False, True])
def test_gemm_tn_small_result_long_contraction(t, m, n, fp32):
    """A result of a few tiles over a long contraction runs as row bands with fp32 partials summed
    in a fixed order: same answer as the fp32 product, repeatable bit for bit, and accumulation
    adds once."""
    from speculators_amd.gemm import _split_bands, gemm_tn

    assert _split_bands(t, m, n) > 1
    g = torch.Generator(device="cuda").manual_seed(t + m)
    a = torch.randn(t, m, device="cuda", generator=g).bfloat16()
    b = torch.randn(t, n, device="cuda", generator=g).bfloat16()
    want = a.double().t() @ b.double()
    dt = torch.float32 if fp32 else torch.bfloat16
    got = gemm_tn(a, b, out_dtype=dt)
    tol = 2e-6 * t ** 0.5 if fp32 else 2 ** -8
    assert got.dtype == dt and (got.double() - want).abs().max() <= tol * want.abs().max() + 1e-4
    assert torch.equal(got, gemm_tn(a, b, out_dtype=dt))
    acc = got.clone()
    gemm_tn(a, b, acc, accumulate=True)
    assert (acc.double() - 2 * want).abs().max() <= 2.5 * tol * want.abs().max() * 2 + 1e-4


@pytest.mark.parametrize("m,n", [(20, 13), (9, 64), (64, 1)])
def test_weight_gradient_of_unaligned_operands_takes_the_library_product(m, n):
    """``weights.wgrad_product`` hands operands the transposing MFMA kernel cannot take (a width that
    is no multiple of 8: a gate of width 1, an odd hidden size) to PyTorch's matmul: fp32 result,
    with and without a gradient to add to, against the fp64 product; aligned operands of the same
    size class take the kernel and agree with it."""
    from speculators_amd import weights

    g = torch.Generator().manual_seed(m * 100 + n)
    t = 300
    dy = torch.randn(t, m, generator=g).bfloat16().cuda()
    x = torch.randn(t, n, generator=g).bfloat16().cuda()
    assert not (weights._tn_ok(dy) and weights._tn_ok(x))
    want = dy.double().t() @ x.double()
    got = weights.wgrad_product(dy, x, None)
    assert got.dtype == torch.float32 and got.shape == (m, n)
    assert (got.double() - want).abs().max() <= 1e-5 * want.abs().max() + 1e-6
    acc0 = torch.randn(m, n, generator=g).cuda()
    acc = acc0.clone()
    got2 = weights.wgrad_product(dy, x, acc)
    assert got2 is acc
    assert (acc.double() - (acc0.double() + want)).abs().max() <= 1e-5 * want.abs().max() + 1e-6
    # the aligned neighbour runs on the kernel and gives the same kind of answer
    dy8, x8 = torch.nn.functional.pad(dy, (0, -m % 8)), torch.nn.functional.pad(x, (0, -n % 8))
    assert weights._tn_ok(dy8) and weights._tn_ok(x8)
    got8 = weights.wgrad_product(dy8, x8, None)
    assert (got8[:m, :n].double() - want).abs().max() <= 1e-5 * want.abs().max() + 1e-6


def _stats_reference(c):
    """(lse, first-index arg-max) of bf16 rows, the way the streaming loss kernels see them."""
    cf = c.float()
    return torch.logsumexp(cf.double(), -1), cf.argmax(-1)


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 1000, 136), (512, 32000, 256), (130, 2432, 512),
                                   (700, 151936, 64)])
def test_gemm_with_row_statistics_in_the_epilogue(m, n, k):
    """``spx_gemm_bf16_nt_stats``: the product is the plain product bit for bit; per row the
    log-sum-exp of the bf16-rounded results (1e-6 relative against float64 and against the
    streaming label-CE kernel's) and their first-index arg-max (exact, ``torch.argmax`` and the
    kernel's); with the product not stored the statistics are the same bits.  Shapes: one tile,
    ragged edges in both directions, a last tile whose right half lies past the last column
    (2432 = 9.5 tiles; 151936 = 593.5), the two vocabulary sizes."""
    from speculators_amd import _lib
    from speculators_amd.gemm import gemm_nt, gemm_nt_stats

    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16().cuda()
    b = (torch.randn(n, k, generator=g) * (4.0 / k ** 0.5)).bfloat16().cuda()
    plain = gemm_nt(a, b)
    c, lse, am = gemm_nt_stats(a, b)
    assert torch.equal(c.view(torch.int16), plain.view(torch.int16))
    want_lse, want_am = _stats_reference(c)
    assert torch.equal(am.long(), want_am)
    assert ((lse.double() - want_lse).abs() <= 1e-6 * want_lse.abs() + 1e-6).all()
    # the two-kernel path: the streaming kernel over the stored product
    labels = torch.zeros(m, dtype=torch.int64, device="cuda")
    out = torch.empty(2, m, device="cuda")
    am2 = torch.empty(m, device="cuda", dtype=torch.int32)
    _lib.call("spx_label_ce_fwd", _lib.ptr(c), c.stride(0), _lib.ptr(labels), m, n, _lib.dtype_code(c), -100,
              _lib.ptr(out[0]), _lib.ptr(out[1]), _lib.ptr(am2), _lib.stream_ptr(c.device))
    assert torch.equal(am, am2)
    assert ((lse - out[1]).abs() <= 1e-6 * out[1].abs() + 1e-6).all()
    none, lse3, am3 = gemm_nt_stats(a, b, store=False)
    assert none is None and torch.equal(lse3, lse) and torch.equal(am3, am)
    # only one of the two asked for: the same bits as when both are computed
    _, lse4, no_am = gemm_nt_stats(a, b, want_argmax=False)
    assert no_am is None and torch.equal(lse4, lse)
    _, no_lse, am5 = gemm_nt_stats(a, b, store=False, want_lse=False)
    assert no_lse is None and torch.equal(am5, am)


def test_row_statistics_break_ties_towards_the_first_column():
    """Equal maxima in one row -- inside a lane's columns, across the lanes of a wave, across the two
    waves of a tile and across tiles -- resolve to the lowest column; -0 and +0 are one value."""
    from speculators_amd.gemm import gemm_nt_stats

    g = torch.Generator().manual_seed(5)
    m, k, n = 64, 64, 1024
    a = torch.randn(m, k, generator=g).bfloat16().cuda()
    b = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    big = (torch.randn(k, generator=g) * 2).bfloat16()
    # duplicates of one strong column at distances that cross each of the boundaries
    for cols in ([5, 6], [40, 41 + 16], [100, 100 + 128], [200, 200 + 256, 900], [1023, 3]):
        bb = b.clone()
        bb[cols] = big
        c, _, am = gemm_nt_stats(a, bb.cuda())
        cf = c.float()
        assert torch.equal(am.long(), cf.argmax(-1))
        rows_won = (am.long() == min(cols)).sum().item()
        assert rows_won > 0  # the duplicated column wins some rows, and then always at its first copy
        assert not torch.isin(am.long(), torch.tensor(sorted(cols)[1:], device="cuda")).any()
    # an all-zero product: every element ties (and a sign of zero must not matter)
    c, lse, am = gemm_nt_stats(torch.zeros(m, k).bfloat16().cuda(), b.cuda())
    assert (am == 0).all() and torch.allclose(lse, torch.full_like(lse, float(torch.log(torch.tensor(float(n))))))
    neg = a.clone()
    bz = torch.zeros(n, k).bfloat16()
    bz[7, 0] = -0.0
    c, _, am = gemm_nt_stats(neg, bz.cuda())
    assert (am == 0).all()


def test_gemm_stats_rejects_bad_arguments():
    from speculators_amd import _lib

    lib = _lib.load()
    a = torch.zeros(256, 64, device="cuda", dtype=torch.bfloat16)
    lse = torch.empty(256, device="cuda")
    ws = torch.empty(16, device="cuda")
    assert lib.spx_gemm_stats_workspace_bytes(256, 300) == 3 * 2 * 256 * 4
    rc = lib.spx_gemm_bf16_nt_stats(_lib.ptr(a), 64, _lib.ptr(a), 64, None, 0, 256, 256, 64, _lib.ptr(lse), None,
                                    _lib.ptr(ws), 64, None)
    assert rc == 1 and b"workspace too small" in lib.spx_last_error()
    rc = lib.spx_gemm_bf16_nt_stats(_lib.ptr(a), 64, _lib.ptr(a), 64, None, 0, 256, 256, 64, None, None,
                                    _lib.ptr(ws), 1 << 20, None)
    assert rc == 1 and b"null lse and null argmax" in lib.spx_last_error()


@pytest.mark.parametrize("m,n,k,parts", [(512, 768, 4096, 4), (300, 1000, 8192, 4), (4096, 6144, 2048, 2),
                                         (512, 768, 1024, 1), (4096, 4096, 4096, 1), (1024, 1800, 2048 + 64, 2)])
def test_gemm_nt_with_the_last_round_of_tiles_cut_along_the_contraction(m, n, k, parts):
    """``spx_gemm_bf16_nt_tail``: a last round of tiles that leaves at least half of the 256 compute
    units idle is cut along the contraction (6 tiles -> 4 parts each; 384 tiles -> the last 128 in 2),
    every other tile -- and every tile when nothing is cut (short contraction, full rounds) -- is the plain
    kernel's bit for bit.  Ragged edges in both directions; against the float64 product."""
    from speculators_amd import _lib
    from speculators_amd import gemm

    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16().cuda()
    b = (torch.randn(n, k, generator=g) / k ** 0.5).bfloat16().cuda()
    plain = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    _lib.call("spx_gemm_bf16_nt", _lib.ptr(a), k, _lib.ptr(b), k, _lib.ptr(plain), n, m, n, k,
              _lib.stream_ptr(a.device))
    got = gemm.gemm_nt(a, b)     # takes the tail entry point whenever the tile count asks for it
    tiles = -(-m // 256) * -(-n // 256)
    rem = tiles % 256
    assert (0 < rem <= 128) or parts == 1
    if parts == 1:
        assert torch.equal(got.view(torch.int16), plain.view(torch.int16))
    else:
        assert not torch.equal(got.view(torch.int16), plain.view(torch.int16))  # another summation order
        # the tiles of the full rounds are untouched: tile index -> (row group of 8, column, row)
        if tiles > 256:
            assert torch.equal(got[:256, :256].view(torch.int16), plain[:256, :256].view(torch.int16))
    want = a.double() @ b.double().t()
    err = (got.double() - want).abs().max().item()
    assert err <= 1e-2 * want.abs().max().item(), err
    # run to run identical (fixed order of the parts)
    again = gemm.gemm_nt(a, b)
    assert torch.equal(again.view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("tiles", [(17, 20), (20, 17), (35, 3), (3, 35), (40, 33)])
def test_every_tile_of_a_ragged_tile_grid_is_computed_once(tiles):
    """Tile grids that are no multiple of the tile order's panels (16), groups (8) or rounds (256 tiles), in
    both orientations, with partial edge tiles: every element of the result of both GEMM kernels against an
    fp32 product (a tile left out or written twice by a wrong workgroup -> tile map shows up as a whole
    256 x 256 block of garbage)."""
    from speculators_amd.gemm import gemm_nt, gemm_tn

    tm, tn = tiles
    m, n, k = tm * 256 - 8, tn * 256 - 248, 64
    g = torch.Generator(device="cuda").manual_seed(tm * 100 + tn)
    a = torch.randn(m, k, generator=g, device="cuda").bfloat16()
    b = torch.randn(n, k, generator=g, device="cuda").bfloat16()
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    gemm_nt(a, b, out=out)
    ref = a.float() @ b.float().T
    torch.testing.assert_close(out.float(), ref, rtol=1e-2, atol=0.1)
    # the weight-gradient orientation: a^T b over 64 rows, fp32 result
    at = torch.randn(k, m, generator=g, device="cuda").bfloat16()
    bt = torch.randn(k, n, generator=g, device="cuda").bfloat16()
    out32 = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    gemm_tn(at, bt, out=out32)
    torch.testing.assert_close(out32, at.float().T @ bt.float(), rtol=1e-4, atol=1e-3)
