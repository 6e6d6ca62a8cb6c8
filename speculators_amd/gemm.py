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

_MAX_SPAN = 0x7ffffff0 - 64  # bytes one GEMM operand may span


def gemm_nt(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``a[M, K] @ b[N, K].T -> [M, N]`` (bf16, fp32 accumulation)."""
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
    # the kernel addresses each operand with 32-bit byte offsets: an operand that spans
    # 2 GiB or more is fed in row bands (full-vocabulary logits gradients are that large)
    rows_a = max(_MAX_SPAN // (2 * a.stride(0)), 1) if m > 1 else 1
    rows_b = max(_MAX_SPAN // (2 * b.stride(0)), 1) if n > 1 else 1
    st = _lib.stream_ptr(a.device)
    for m0 in range(0, m, max(rows_a, 1)):
        am = a[m0:m0 + rows_a]
        for n0 in range(0, n, max(rows_b, 1)):
            bn = b[n0:n0 + rows_b]
            o = out[m0:m0 + rows_a, n0:n0 + rows_b]
            _lib.call("spx_gemm_bf16_nt", _lib.ptr(am), am.stride(0), _lib.ptr(bn), bn.stride(0),
                      _lib.ptr(o), o.stride(0), am.shape[0], bn.shape[0], k, st)
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
