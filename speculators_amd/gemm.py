"""bf16 Linear products on the MFMA GEMM kernel.

``linear(x, weight)`` is ``torch.nn.functional.linear`` without bias
(``x @ weight.T``) for bf16 tensors.  The backward computes the input gradient
with the same NT kernel against a transposed copy of the weight
(``weight_t``, ``[K, N]`` contiguous) -- kept by the caller for frozen weights
such as ``lm_head`` (model.py:70-71) so it is made once.  The weight gradient is the
transposed-operand product ``gemm_tn``.
The models call the ``*_staged`` forms below with the compute weights of ``weights.WeightStager``.
"""

from __future__ import annotations

import os

import torch

from . import _lib
from . import fused_ops as FO

_MAX_SPAN = 0x7ffffff0 - 64  # bytes an operand of the weight-gradient product (gemm_tn) may span per call


_CUS = 256  # workgroups the chip runs at a time (one per compute unit for the GEMM kernels)

# parts the contraction of a live-rows product may be cut into (gemm_nt(split=True)); 1 = never cut
SPLIT_PARTS = int(os.environ.get("SPX_GEMM_SPLIT_PARTS", "4"))
if not 1 <= SPLIT_PARTS <= 8:
    raise ValueError(f"SPX_GEMM_SPLIT_PARTS must be 1 .. 8, got {SPLIT_PARTS}")


# parts the tiles of a mostly empty last round of a product may be cut into (spx_gemm_bf16_nt_tail); 1 = never
TAIL_PARTS = int(os.environ.get("SPX_GEMM_TAIL_PARTS", "4"))
if not 1 <= TAIL_PARTS <= 8:
    raise ValueError(f"SPX_GEMM_TAIL_PARTS must be 1 .. 8, got {TAIL_PARTS}")

_split_ws: dict = {}


def _split_workspace(device, numel: int) -> torch.Tensor:
    """The fp32 partials of a product cut along its contraction: one buffer per (device, stream), kept
    and grown on demand, so a TTT loop does not allocate hundreds of MB per step for a workspace the
    kernel leaves untouched whenever the device-side row count asks for one part.  Launches of one
    stream are ordered, so consecutive products may share it."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _split_ws.get(key)
    if ws is None or ws.numel() < numel:
        ws = torch.empty(numel, device=device, dtype=torch.float32)
        _split_ws[key] = ws
    return ws


def gemm_nt(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None,
            m_live: torch.Tensor | None = None, split: bool = False) -> torch.Tensor:
    """``a[M, K] @ b[N, K].T -> [M, N]`` (bf16, fp32 accumulation).

    ``m_live`` (a one-element int32 device tensor) says how many leading rows of ``a`` count:
    the rows from there on are neither read nor written, and the host never learns the
    number (no synchronisation).  ``split``: the kernel may cut the contraction into up to
    ``SPLIT_PARTS`` parts when the tiles of the rows that count would leave compute units idle
    (decided on the device from the row count; fp32 partials in a workspace, added in a fixed
    order)."""
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise _lib.SpxError("gemm_nt takes bf16 operands")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"shape mismatch: a {tuple(a.shape)} b {tuple(b.shape)}")
    if a.stride(1) != 1:
        a = a.contiguous()
    if b.stride(1) != 1:
        b = b.contiguous()
    m, k = a.shape
    n = b.shape[0]
    if out is None:
        out = torch.empty(m, n, device=a.device, dtype=torch.bfloat16)
    # (operands of any size go in one launch: the kernel's 32-bit offsets are relative to a tile)
    st = _lib.stream_ptr(a.device)
    if m_live is None:
        # a last round of tiles that fills at most half the chip is cut along the contraction
        # (the kernel decides from the same numbers; here only whether the workspace is handed over)
        rem = (-(-m // 256) * -(-n // 256)) % _CUS
        if TAIL_PARTS > 1 and 0 < rem <= _CUS // 2 and k >= 64 * 16 * 2 and a.is_cuda:
            nbytes = _lib.load().spx_gemm_tail_workspace_bytes()
            ws = _split_workspace(a.device, nbytes // 4)
            _lib.call("spx_gemm_bf16_nt_tail", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
                      _lib.ptr(out), out.stride(0), m, n, k, TAIL_PARTS, _lib.ptr(ws), nbytes, st)
            return out
        _lib.call("spx_gemm_bf16_nt", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
                  _lib.ptr(out), out.stride(0), m, n, k, st)
    else:
        if m_live.dtype != torch.int32 or m_live.numel() != 1 or m_live.device != a.device:
            raise ValueError("m_live must be a one-element int32 tensor on the operands' device")
        # (a product of many rounds of tiles has little to gain from cutting: at most 1 / rounds)
        few_tiles = -(-m // 256) * -(-n // 256) <= 2 * 256
        if split and SPLIT_PARTS > 1 and few_tiles and n % 8 == 0 and out.stride(0) % 8 == 0 and k >= 64 * 16 * 2:
            ws = _split_workspace(a.device, SPLIT_PARTS * m * n)
            _lib.call("spx_gemm_bf16_nt_rows_split", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
                      _lib.ptr(out), out.stride(0), m, n, k, _lib.ptr(m_live), SPLIT_PARTS, _lib.ptr(ws),
                      SPLIT_PARTS * m * n * 4, st)
        else:
            _lib.call("spx_gemm_bf16_nt_rows", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
                      _lib.ptr(out), out.stride(0), m, n, k, _lib.ptr(m_live), st)
    return out


def gemm_nt_stats(a: torch.Tensor, b: torch.Tensor, store: bool = True, want_argmax: bool = True,
                  want_lse: bool = True):
    """``gemm_nt(a, b)`` whose epilogue also reduces every row of the (bf16-rounded) product to its
    soft-max statistics: returns ``(c [M, N] bf16 or None, lse [M] f32, argmax [M] i32 or None)``.
    ``store=False``: the product is not written at all (``c`` is None) -- the statistics are all a
    cross-entropy against arg-max targets needs of the verifier's logits."""
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise _lib.SpxError("gemm_nt_stats takes bf16 operands")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"shape mismatch: a {tuple(a.shape)} b {tuple(b.shape)}")
    if a.stride(1) != 1:
        a = a.contiguous()
    if b.stride(1) != 1:
        b = b.contiguous()
    m, k = a.shape
    n = b.shape[0]
    dev = a.device
    out = torch.empty(m, n, device=dev, dtype=torch.bfloat16) if store else None
    if not (want_lse or want_argmax):
        raise ValueError("gemm_nt_stats: ask for the log-sum-exp, the arg-max or both")
    lse = torch.empty(m, device=dev, dtype=torch.float32) if want_lse else None
    am = torch.empty(m, device=dev, dtype=torch.int32) if want_argmax else None
    nbytes = _lib.load().spx_gemm_stats_workspace_bytes(m, n)
    ws = torch.empty(nbytes // 4, device=dev, dtype=torch.float32)
    _lib.call("spx_gemm_bf16_nt_stats", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
              _lib.ptr(out), out.stride(0) if store else 0, m, n, k, _lib.ptr(lse), _lib.ptr(am), _lib.ptr(ws),
              nbytes, _lib.stream_ptr(dev))
    return out, lse, am




def _split_bands(t: int, m: int, n: int) -> int:
    """How many row bands the contraction of a ``[t, m]^T [t, n]`` product is cut into: enough to
    give every compute unit a workgroup, every band at least 1024 rows long; 1 = no split."""
    tiles = -(-m // 256) * -(-n // 256)
    if tiles * 2 > _CUS or t < 2048:
        return 1
    return max(1, min(_CUS // tiles, t // 1024))


_band_cache: dict = {}


def _band_offsets(t: int, step: int, bands: int, device) -> torch.Tensor:
    key = (t, step, bands, str(device))
    off = _band_cache.get(key)
    if off is None:
        off = torch.tensor([min(i * step, t) for i in range(bands + 1)], dtype=torch.int32, device=device)
        _band_cache[key] = off
    return off


def gemm_tn(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None,
            accumulate: bool = False, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``a[T, M].T @ b[T, N] -> [M, N]`` (bf16 operands, fp32 accumulation): the weight gradient
    ``dY.T @ X`` of a Linear.  ``accumulate`` adds the product to ``out``.  The result is bf16 or,
    with ``out_dtype=torch.float32`` (or an fp32 ``out``), fp32."""
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise _lib.SpxError("gemm_tn takes bf16 operands")
    if a.dim() != 2 or b.dim() != 2 or a.shape[0] != b.shape[0]:
        raise ValueError(f"shape mismatch: a {tuple(a.shape)} b {tuple(b.shape)}")
    if a.stride(1) != 1:
        a = a.contiguous()
    if b.stride(1) != 1:
        b = b.contiguous()
    t, m = a.shape
    n = b.shape[1]
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs the tensor to add to")
        if out_dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("out_dtype must be bfloat16 or float32")
        out = torch.empty(m, n, device=a.device, dtype=out_dtype)
    elif out.shape != (m, n) or out.dtype not in (torch.bfloat16, torch.float32) or out.stride(1) != 1:
        raise ValueError(f"out must be a bf16 or fp32 [{m}, {n}] tensor with unit column stride")
    # A small result with a long contraction leaves most of the chip idle (one workgroup per
    # 256 x 256 tile of the result): the contraction is then cut into row bands, every band's
    # product goes to an fp32 partial of its own (the grouped kernel with the bands as groups) and
    # the partials are summed in a fixed order
    bands = _split_bands(t, m, n)
    if bands > 1 and max(a.stride(0), b.stride(0)) * 2 * (t + 256) < _MAX_SPAN:
        step = -(-t // bands)
        off = _band_offsets(t, step, bands, a.device)
        part = torch.empty(bands, m, n, device=a.device, dtype=torch.float32)
        _lib.call("spx_gemm_bf16_tn_grouped", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0), _lib.ptr(part),
                  n, m * n, m, n, t, _lib.ptr(off), bands, 1, 0, _lib.stream_ptr(a.device))
        total = part.sum(0)
        if accumulate:
            total += out  # in fp32: what the result holds is added before the one rounding
        out.copy_(total)
        return out
    entry = "spx_gemm_bf16_tn_f32" if out.dtype == torch.float32 else "spx_gemm_bf16_tn"
    # 32-bit byte offsets inside the kernel: a contraction that spans 2 GiB or more of an
    # operand is fed in bands of rows, every band after the first added to the result
    rows = max(_MAX_SPAN // (2 * max(a.stride(0), b.stride(0))) - 256, 1)
    st = _lib.stream_ptr(a.device)
    for t0 in range(0, t, rows):
        at, bt = a[t0:t0 + rows], b[t0:t0 + rows]
        _lib.call(entry, _lib.ptr(at), at.stride(0), _lib.ptr(bt), bt.stride(0),
                  _lib.ptr(out), out.stride(0), m, n, at.shape[0], int(accumulate or t0 > 0), st)
    return out


class _Linear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, weight_t):
        x2 = x.reshape(-1, x.shape[-1])
        y = gemm_nt(x2, weight)
        ctx.save_for_backward(x2, weight, weight_t)
        ctx.x_shape = x.shape
        return y.view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x2, weight, weight_t = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1]).to(torch.bfloat16)
        dx = dw = None
        if ctx.needs_input_grad[0]:
            wt = weight_t if weight_t is not None else weight.t().contiguous()
            dx = gemm_nt(dy2, wt).view(ctx.x_shape)
        if ctx.needs_input_grad[1]:
            from .weights import wgrad_product

            dw = wgrad_product(dy2 if dy2.stride(1) == 1 else dy2.contiguous(), x2, None).to(weight.dtype)
        return dx, dw, None


def linear(x: torch.Tensor, weight: torch.Tensor, weight_t: torch.Tensor | None = None):
    """``x[..., K] @ weight[N, K].T`` on the HIP GEMM; ``weight_t`` optionally holds
    ``weight.T`` contiguous for the backward."""
    return _Linear.apply(x, weight, weight_t)


# Which GEMM runs the decoder-layer projections (q/k/v, o, gate/up, down and their input
# gradients): "hipblaslt" = PyTorch's matmul (the library GEMM), "spx" = this library's MFMA kernel
# (the input gradients then run against the transposed copy of the staged weight), "mixed" = each
# where it is faster on these shapes: the forward products on hipBLASLt (6 - 12 % ahead there) except
# those whose tile count leaves the last round of workgroups mostly idle, which this library's kernel
# cuts along the contraction (the merged q/k/v projection: 10 % ahead of the library), the input
# gradients on this library's kernel (8 - 20 % ahead of the library's NN product).  The fc /
# lm_head / verifier-head products and every weight gradient always run on this library's kernels.
DECODER_GEMM = os.environ.get("SPX_DECODER_GEMM", "mixed")
if DECODER_GEMM not in ("hipblaslt", "spx", "mixed"):
    raise ValueError(f"SPX_DECODER_GEMM must be 'hipblaslt', 'spx' or 'mixed', got {DECODER_GEMM!r}")


def _tail_cut_applies(m: int, n: int, k: int) -> bool:
    """Whether ``gemm_nt`` cuts the last round of tiles of an ``[m, k] x [n, k]^T`` product (the rule of
    ``spx_gemm_bf16_nt_tail``): the shapes on which a 256 x 256 tiling loses most to tile quantisation
    and the cut wins it back (the merged q/k/v projection of the 8B shape: 384 tiles)."""
    rem = (-(-m // 256) * -(-n // 256)) % _CUS
    return TAIL_PARTS > 1 and 0 < rem <= _CUS // 2 and k >= 64 * 16 * 2 and (-(-m // 256) * -(-n // 256)) < 2 * _CUS


def _project(x2: torch.Tensor, staged) -> torch.Tensor:
    """``x2 @ staged.w.T`` of a decoder-layer projection."""
    if DECODER_GEMM == "spx":
        return gemm_nt(x2, staged.w)
    if (DECODER_GEMM == "mixed" and x2.dtype == torch.bfloat16
            and _tail_cut_applies(x2.shape[0], staged.w.shape[0], x2.shape[1])):
        # (measured at [4096, 8192] x [6144, 8192]^T: 322 us here, 357 us on the library)
        return gemm_nt(x2, staged.w)
    return torch.nn.functional.linear(x2, staged.w)


def _project_back(dy2: torch.Tensor, staged) -> torch.Tensor:
    """``dy2 @ staged.w``: the input gradient of a decoder-layer projection ("mixed": this one on the
    library's kernel against the transposed copy, the forward product on hipBLASLt)."""
    # (the kernel contracts in chunks of 8: a projection a few columns wide -- a gate of width 1 --
    # stays with the library)
    if DECODER_GEMM != "hipblaslt" and dy2.shape[1] % 8 == 0 and dy2.stride(0) % 8 == 0 and dy2.stride(1) == 1:
        return gemm_nt(dy2, staged.wt)
    return torch.matmul(dy2, staged.w)


class _StagedLinear(torch.autograd.Function):
    """``x @ w.T`` against a staged weight (``weights.Staged``): on the MFMA kernel of this library
    (``hip``) or on PyTorch's hipBLASLt matmul.  The weight gradient is left to the staged weight,
    which computes it over all of its uses at once (``weights.Staged.defer``)."""

    @staticmethod
    def forward(ctx, x, _token, staged, hip: bool):
        if x.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP layer kernels take bf16 tensors")
        w = staged.w
        x2 = x.reshape(-1, x.shape[-1])
        y = gemm_nt(x2, w) if hip else _project(x2, staged)
        ctx.save_for_backward(x2, w)
        ctx.staged, ctx.hip, ctx.x_shape = staged, hip, x.shape
        ctx.slot = staged.take(x2) if ctx.needs_input_grad[1] else -1
        ctx.rows = x2.shape[0]
        return y.view(*x.shape[:-1], w.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x2, w = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1]).to(torch.bfloat16)
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = (gemm_nt(dy2, ctx.staged.wt) if ctx.hip else _project_back(dy2, ctx.staged)).view(ctx.x_shape)
        if ctx.needs_input_grad[1]:
            dw = ctx.staged.defer(ctx.slot, dy2, x2)
        return dx, dw, None, None


def linear_staged(x: torch.Tensor, staged, hip: bool = False) -> torch.Tensor:
    """``x[..., K] @ staged.w[N, K].T``; see ``_StagedLinear``."""
    if not torch.is_grad_enabled() or not (x.requires_grad or staged.trainable):
        x2 = x.reshape(-1, x.shape[-1])
        y = gemm_nt(x2, staged.w) if hip else _project(x2, staged)
        return y.view(*x.shape[:-1], staged.w.shape[0])
    y = _StagedLinear.apply(x, staged.token, staged, hip)
    node = y.grad_fn
    if node is not None and getattr(node, "slot", -1) >= 0:
        # where the gradient of `y` belongs, for the backward that produces it (fused_ops._AddRMSNorm):
        # written there, it is not copied into the weight's output-gradient buffer afterwards
        y.spx_grad_slot = (staged, node.slot, node.rows)
    return y


class _QKVRope(torch.autograd.Function):
    """q/k/v projections of one input as ONE GEMM against the staged concatenation of the three
    weights, followed by the rotary embedding + head-major relayout of each part.  The backward
    undoes the relayout into the three column blocks of one ``[T, Nq + 2 Nkv]`` buffer, so the
    input gradient is one GEMM (no per-projection partial results to add up); that buffer is the
    step's slot of the staged weight's output-gradient buffer, from which the weight gradient of
    all TTT steps comes as one product."""

    @staticmethod
    def forward(ctx, x, _token, staged, position_ids, inv_freq, hq, hkv, d, offset, kv_out=None):
        if x.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP layer kernels take bf16 tensors")
        wcat = staged.w
        t = x.shape[-2]
        x2 = x.reshape(t, x.shape[-1])
        qkv = _project(x2, staged)
        n = qkv.shape[1]
        st = _lib.stream_ptr(x.device)
        scale = FO.table_scale_of(inv_freq)
        outs, col = [], 0
        for idx, (heads, rotate) in enumerate(((hq, 1), (hkv, 1), (hkv, 0))):
            if idx and kv_out is not None:
                # a [1, Hkv, T, D] window of the preallocated K / V cache: written in place
                out = kv_out[idx - 1]
                head_stride = out.stride(1)
            else:
                out = torch.empty(1, heads, t, d, device=x.device, dtype=torch.bfloat16)
                head_stride = 0
            part = qkv[:, col:]
            FO.rope_call(_lib.ptr(part), n, d, position_ids, inv_freq, _lib.ptr(out), head_stride, t, heads, d,
                         rotate, 0, offset, scale, st)
            outs.append(out)
            col += heads * d
        ctx.save_for_backward(x2, wcat, position_ids, inv_freq)
        ctx.meta = (x.shape, hq, hkv, d, offset, n, staged, scale)
        ctx.slot = staged.take(x2) if ctx.needs_input_grad[1] else -1
        ctx.set_materialize_grads(False)
        return tuple(outs)

    @staticmethod
    def backward(ctx, dq, dk, dv):
        x2, wcat, position_ids, inv_freq = ctx.saved_tensors
        shape, hq, hkv, d, offset, n, staged, scale = ctx.meta
        t = x2.shape[0]
        st = _lib.stream_ptr(x2.device)
        dqkv = staged.dy_slot(ctx.slot, t) if ctx.needs_input_grad[1] else None
        if dqkv is None:
            dqkv = torch.empty(t, n, device=x2.device, dtype=torch.bfloat16)
        col = 0
        for g, heads, rotate in ((dq, hq, 1), (dk, hkv, 1), (dv, hkv, 0)):
            part = dqkv[:, col:]
            if g is None:
                dqkv[:, col:col + heads * d].zero_()
            else:
                g = g.to(torch.bfloat16)
                # a window of a longer gradient tensor is read in place through its head stride
                if not (g.stride(3) == 1 and g.stride(2) == d and g.stride(1) % 8 == 0
                        and g.stride(1) >= t * d and g.data_ptr() % 16 == 0):
                    g = g.contiguous()
                FO.rope_call(_lib.ptr(g), g.stride(1), d, position_ids, inv_freq, _lib.ptr(part), n, t, heads, d,
                             rotate, 1, offset, scale, st)
            col += heads * d
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = _project_back(dqkv, staged).view(shape)
        if ctx.needs_input_grad[1]:
            dw = staged.defer(ctx.slot, dqkv, x2)
        return (dx, dw) + (None,) * 8


def qkv_rope(x, staged, position_ids, inv_freq, hq: int, hkv: int, d: int, offset: int, kv_out=None):
    """``(q [1,Hq,T,D], k [1,Hkv,T,D], v [1,Hkv,T,D])`` with the rotary embedding at
    ``position_ids + offset`` applied to q and k; ``staged`` holds the row-wise concatenation of
    the q, k and v weights.  ``kv_out = (k_window, v_window)``: write k and v straight into these
    ``[1, Hkv, T, D]`` windows of a K / V cache and return them."""
    return _QKVRope.apply(x, staged.token, staged, position_ids, inv_freq, hq, hkv, d, offset, kv_out)


class _GateUpSwiGLU(torch.autograd.Function):
    """``silu(x @ Wg.T) * (x @ Wu.T)`` with the two projections as ONE GEMM against the staged
    concatenation of the two weights; the SwiGLU kernels read (and, in the backward, write) the two
    column halves of the merged ``[T, 2F]`` buffer in place, so the input gradient is one GEMM; the
    backward's ``[T, 2F]`` buffer is the step's slot of the staged weight's output-gradient buffer,
    from which the weight gradient of all TTT steps comes as one product.  ``out``: where the
    result goes (the input slot of the down projection's staged weight)."""

    @staticmethod
    def forward(ctx, x, _token, staged, out=None):
        if x.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP layer kernels take bf16 tensors")
        wcat = staged.w
        x2 = x.reshape(-1, x.shape[-1])
        f = wcat.shape[0] // 2
        gu = _project(x2, staged)  # [T, 2F]
        rows = x2.shape[0]
        if out is None or out.shape != (rows, f) or not out.is_contiguous():
            out = torch.empty(rows, f, device=x.device, dtype=torch.bfloat16)
        _lib.call("spx_swiglu_rows_fwd", _lib.ptr(gu), 2 * f, _lib.ptr(gu[:, f:]), 2 * f, _lib.ptr(out), f,
                  rows, f, _lib.stream_ptr(x.device))
        ctx.save_for_backward(x2, gu, wcat)
        ctx.meta = (x.shape, f, staged)
        ctx.slot = staged.take(x2) if ctx.needs_input_grad[1] else -1
        return out.view(*x.shape[:-1], f)

    @staticmethod
    def backward(ctx, dout):
        x2, gu, wcat = ctx.saved_tensors
        shape, f, staged = ctx.meta
        rows = x2.shape[0]
        d2 = dout.reshape(rows, f).to(torch.bfloat16)
        if d2.stride(1) != 1 or d2.stride(0) % 8:
            d2 = d2.contiguous()
        dgu = staged.dy_slot(ctx.slot, rows) if ctx.needs_input_grad[1] else None
        if dgu is None:
            dgu = torch.empty(rows, 2 * f, device=x2.device, dtype=torch.bfloat16)
        _lib.call("spx_swiglu_rows_bwd", _lib.ptr(gu), 2 * f, _lib.ptr(gu[:, f:]), 2 * f, _lib.ptr(d2),
                  d2.stride(0), _lib.ptr(dgu), 2 * f, _lib.ptr(dgu[:, f:]), 2 * f, rows, f,
                  _lib.stream_ptr(x2.device))
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = _project_back(dgu, staged).view(shape)
        if ctx.needs_input_grad[1]:
            dw = staged.defer(ctx.slot, dgu, x2)
        return dx, dw, None, None


def gate_up_swiglu(x, staged, out=None):
    """See ``_GateUpSwiGLU``; ``staged`` holds the row-wise concatenation of the gate and up
    weights."""
    return _GateUpSwiGLU.apply(x, staged.token, staged, out)
