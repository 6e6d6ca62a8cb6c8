"""bf16 Linear products on the MFMA GEMM kernel.

``linear(x, weight)`` is ``torch.nn.functional.linear`` without bias
(``x @ weight.T``) for bf16 tensors.  The backward computes the input gradient
with the same NT kernel against a transposed copy of the weight
(``weight_t``, ``[K, N]`` contiguous) -- kept by the caller for frozen weights
such as ``lm_head`` (model.py:70-71) so it is made once -- and leaves the
weight gradient (a TN product) to the rocBLAS/hipBLASLt matmul of PyTorch.
"""

from __future__ import annotations

import os

import torch

from . import _lib

_MAX_SPAN = 0x7ffffff0 - 64  # bytes an operand of the weight-gradient product (gemm_tn) may span per call


def gemm_nt(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None,
            m_live: torch.Tensor | None = None) -> torch.Tensor:
    """``a[M, K] @ b[N, K].T -> [M, N]`` (bf16, fp32 accumulation).

    ``m_live`` (a one-element int32 device tensor) says how many leading rows of ``a`` count:
    the rows from there on are neither read nor written, and the host never learns the
    number (no synchronisation)."""
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
        _lib.call("spx_gemm_bf16_nt", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
                  _lib.ptr(out), out.stride(0), m, n, k, st)
    else:
        if m_live.dtype != torch.int32 or m_live.numel() != 1 or m_live.device != a.device:
            raise ValueError("m_live must be a one-element int32 tensor on the operands' device")
        _lib.call("spx_gemm_bf16_nt_rows", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0),
                  _lib.ptr(out), out.stride(0), m, n, k, _lib.ptr(m_live), st)
    return out


def gemm_tn(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None,
            accumulate: bool = False) -> torch.Tensor:
    """``a[T, M].T @ b[T, N] -> [M, N]`` (bf16, fp32 accumulation): the weight gradient
    ``dY.T @ X`` of a Linear.  ``accumulate`` adds the product to ``out``."""
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
        out = torch.empty(m, n, device=a.device, dtype=torch.bfloat16)
    elif out.shape != (m, n) or out.dtype != torch.bfloat16 or out.stride(1) != 1:
        raise ValueError(f"out must be a bf16 [{m}, {n}] tensor with unit column stride")
    # 32-bit byte offsets inside the kernel: a contraction that spans 2 GiB or more of an
    # operand is fed in bands of rows, every band after the first added to the result
    rows = max(_MAX_SPAN // (2 * max(a.stride(0), b.stride(0))) - 256, 1)
    st = _lib.stream_ptr(a.device)
    for t0 in range(0, t, rows):
        at, bt = a[t0:t0 + rows], b[t0:t0 + rows]
        _lib.call("spx_gemm_bf16_tn", _lib.ptr(at), at.stride(0), _lib.ptr(bt), bt.stride(0),
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
            dw = torch.matmul(dy2.t(), x2)
        return dx, dw, None


def linear(x: torch.Tensor, weight: torch.Tensor, weight_t: torch.Tensor | None = None):
    """``x[..., K] @ weight[N, K].T`` on the HIP GEMM; ``weight_t`` optionally holds
    ``weight.T`` contiguous for the backward."""
    return _Linear.apply(x, weight, weight_t)


FUSE_WGRAD_ACCUMULATION = os.environ.get("SPX_FUSE_WGRAD", "1") != "0"


class _LinearAccumulate(torch.autograd.Function):
    """``x @ weight.T`` on PyTorch's (hipBLASLt) matmul whose backward ADDS the weight
    gradient into ``weight.grad`` inside the GEMM (beta = 1) instead of returning a fresh
    tensor for autograd to add.  A weight that is applied once per TTT step otherwise costs
    one full read-modify-write pass over a weight-sized tensor per step after the first."""

    @staticmethod
    def forward(ctx, x, weight):
        ctx.save_for_backward(x, weight)
        return torch.nn.functional.linear(x, weight)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dx = None
        if ctx.needs_input_grad[0]:
            dx = torch.matmul(dy, weight)
        if weight.requires_grad:
            dy2 = dy.reshape(-1, dy.shape[-1])
            x2 = x.reshape(-1, x.shape[-1])
            if weight.grad is None:
                weight.grad = torch.matmul(dy2.t(), x2)
            else:
                torch.addmm(weight.grad, dy2.t(), x2, out=weight.grad)
        return dx, None


def linear_accumulate(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """See ``_LinearAccumulate``.  The weight gradient lands in ``weight.grad`` during
    ``backward()`` (it is not visible to ``torch.autograd.grad``)."""
    if not FUSE_WGRAD_ACCUMULATION or not torch.is_grad_enabled() or not (
            x.requires_grad or weight.requires_grad):
        return torch.nn.functional.linear(x, weight)
    # autograd must see a differentiable input even when only the weight needs a gradient
    return _LinearAccumulate.apply(x, weight)


class _MergedWeights:
    """Per-module state of a merged projection (q/k/v, or gate/up): the concatenated weight of the
    current weight versions, and the merged gradient buffer the ``.grad`` tensors are views of."""

    def __init__(self):
        self.key = None
        self.weight = None
        self.grad = None

    def merged_weight(self, ws):
        key = tuple((w.data_ptr(), w._version) for w in ws)
        if key != self.key:
            self.weight = torch.cat([w.detach() for w in ws], dim=0)
            self.key = key
        return self.weight

    def accumulate(self, ws, dy2, x2):
        """``grad(w_i) += dy2[:, rows_i].T @ x2`` for all the weights with one GEMM.  While their
        ``.grad`` are the views this object handed out, the GEMM adds into the shared buffer
        (beta = 1); otherwise (gradients that came from elsewhere) it falls back to one add each."""
        sizes = [w.shape[0] for w in ws]
        views = None
        if self.grad is not None:
            views = self.grad.split(sizes, dim=0)
            if not all(w.grad is not None and w.grad.data_ptr() == v.data_ptr()
                       and w.grad.shape == v.shape for w, v in zip(ws, views, strict=True)):
                views = None
        if views is not None:
            torch.addmm(self.grad, dy2.t(), x2, out=self.grad)
            return
        fresh = torch.matmul(dy2.t(), x2)
        parts = fresh.split(sizes, dim=0)
        if all(w.grad is None for w in ws):
            self.grad = fresh
            for w, v in zip(ws, parts, strict=True):
                w.grad = v
        else:
            self.grad = None
            for w, v in zip(ws, parts, strict=True):
                if w.requires_grad:
                    w.grad = v.clone() if w.grad is None else w.grad.add_(v)


class _QKVRope(torch.autograd.Function):
    """q/k/v projections of one input as ONE GEMM against the concatenated weight, followed by
    the rotary embedding + head-major relayout of each part.  The backward undoes the relayout
    into the three column blocks of one ``[T, Nq + 2 Nkv]`` buffer, so the input gradient is one
    GEMM (no per-projection partial results to add up) and the weight gradient one GEMM that
    accumulates across TTT steps."""

    @staticmethod
    def forward(ctx, x, wq, wk, wv, position_ids, inv_freq, hq, hkv, d, offset, state, kv_out=None):
        t = x.shape[-2]
        x2 = x.reshape(t, x.shape[-1])
        wcat = state.merged_weight((wq, wk, wv))
        qkv = torch.nn.functional.linear(x2, wcat)
        n = qkv.shape[1]
        st = _lib.stream_ptr(x.device)
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
            _lib.call("spx_rope_relayout", _lib.ptr(part), n, _lib.ptr(position_ids), _lib.ptr(inv_freq),
                      _lib.ptr(out), head_stride, t, heads, d, rotate, 0, int(offset), st)
            outs.append(out)
            col += heads * d
        ctx.save_for_backward(x2, wq, wk, wv, position_ids, inv_freq)
        ctx.meta = (x.shape, hq, hkv, d, offset, n, state, wcat)
        ctx.set_materialize_grads(False)
        return tuple(outs)

    @staticmethod
    def backward(ctx, dq, dk, dv):
        x2, wq, wk, wv, position_ids, inv_freq = ctx.saved_tensors
        shape, hq, hkv, d, offset, n, state, wcat = ctx.meta
        t = x2.shape[0]
        st = _lib.stream_ptr(x2.device)
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
                _lib.call("spx_rope_relayout", _lib.ptr(g), g.stride(1), _lib.ptr(position_ids),
                          _lib.ptr(inv_freq), _lib.ptr(part), n, t, heads, d, rotate, 1, int(offset), st)
            col += heads * d
        dx = None
        if ctx.needs_input_grad[0]:
            dx = torch.matmul(dqkv, wcat).view(shape)
        if any(w.requires_grad for w in (wq, wk, wv)):
            state.accumulate((wq, wk, wv), dqkv, x2)
        return (dx,) + (None,) * 11


def qkv_rope(x, wq, wk, wv, position_ids, inv_freq, hq: int, hkv: int, d: int, offset: int,
             state: _MergedWeights, kv_out=None):
    """``(q [1,Hq,T,D], k [1,Hkv,T,D], v [1,Hkv,T,D])`` with the rotary embedding at
    ``position_ids + offset`` applied to q and k.  Weight gradients land in ``.grad`` during
    ``backward()`` (like ``linear_accumulate``).  ``kv_out = (k_window, v_window)``: write k and v
    straight into these ``[1, Hkv, T, D]`` windows of a K / V cache and return them."""
    return _QKVRope.apply(x, wq, wk, wv, position_ids, inv_freq, hq, hkv, d, offset, state, kv_out)


_MergedQKV = _MergedWeights


class _GateUpSwiGLU(torch.autograd.Function):
    """``silu(x @ Wg.T) * (x @ Wu.T)`` with the two projections as ONE GEMM against the
    concatenated weight; the SwiGLU kernels read (and, in the backward, write) the two column
    halves of the merged ``[T, 2F]`` buffer in place, so the input gradient is one GEMM and the
    weight gradient one GEMM that accumulates across TTT steps."""

    @staticmethod
    def forward(ctx, x, wg, wu, state):
        if x.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP layer kernels take bf16 tensors")
        x2 = x.reshape(-1, x.shape[-1])
        f = wg.shape[0]
        wcat = state.merged_weight((wg, wu))
        gu = torch.nn.functional.linear(x2, wcat)  # [T, 2F]
        rows = x2.shape[0]
        out = torch.empty(rows, f, device=x.device, dtype=torch.bfloat16)
        _lib.call("spx_swiglu_rows_fwd", _lib.ptr(gu), 2 * f, _lib.ptr(gu[:, f:]), 2 * f, _lib.ptr(out), f,
                  rows, f, _lib.stream_ptr(x.device))
        ctx.save_for_backward(x2, gu, wg, wu)
        ctx.meta = (x.shape, f, state, wcat)
        return out.view(*x.shape[:-1], f)

    @staticmethod
    def backward(ctx, dout):
        x2, gu, wg, wu = ctx.saved_tensors
        shape, f, state, wcat = ctx.meta
        rows = x2.shape[0]
        d2 = dout.reshape(rows, f).to(torch.bfloat16)
        if d2.stride(1) != 1 or d2.stride(0) % 8:
            d2 = d2.contiguous()
        dgu = torch.empty(rows, 2 * f, device=x2.device, dtype=torch.bfloat16)
        _lib.call("spx_swiglu_rows_bwd", _lib.ptr(gu), 2 * f, _lib.ptr(gu[:, f:]), 2 * f, _lib.ptr(d2),
                  d2.stride(0), _lib.ptr(dgu), 2 * f, _lib.ptr(dgu[:, f:]), 2 * f, rows, f,
                  _lib.stream_ptr(x2.device))
        dx = None
        if ctx.needs_input_grad[0]:
            dx = torch.matmul(dgu, wcat).view(shape)
        if wg.requires_grad or wu.requires_grad:
            state.accumulate((wg, wu), dgu, x2)
        return dx, None, None, None


def gate_up_swiglu(x, w_gate, w_up, state: _MergedWeights):
    """See ``_GateUpSwiGLU``.  Weight gradients land in ``.grad`` during ``backward()``."""
    return _GateUpSwiGLU.apply(x, w_gate, w_up, state)
