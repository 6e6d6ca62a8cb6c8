"""Sparse MoE MLP of the hybrid MTP flavours on the HIP path.

The layer is the library's ``Qwen3NextSparseMoeBlock`` (``modeling_qwen3_next.py``; the
``qwen3_5_moe`` block is the same with the renormalisation always on), which the reference
reaches by wrapping ``Qwen3NextDecoderLayer`` / ``Qwen3_5MoeDecoderLayer``
(models/mtp/model_definitions.py:159-205).  The library walks over the experts that were hit and
gathers each one's tokens; here the ``(token, slot)`` pairs are sorted by expert once per call and
every product -- gate/up, down, their input gradients and their weight gradients -- is ONE grouped
launch over all experts (``spx_gemm_bf16_nt_grouped`` / ``spx_gemm_bf16_tn_grouped``), with the
group boundaries kept on the device: the host never learns how many tokens an expert received.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from . import _lib
from .weights import Staged


def gemm_nt_grouped(a: torch.Tensor, b: torch.Tensor, offsets: torch.Tensor,
                    out: torch.Tensor | None = None) -> torch.Tensor:
    """``out[r] = a[r] @ b[e].T`` for the rows ``offsets[e] <= r < offsets[e + 1]``: ``a [rows, K]``
    sorted by group, ``b [groups, N, K]``, ``offsets`` int32 ``[groups + 1]`` on the device."""
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise _lib.SpxError("gemm_nt_grouped takes bf16 operands")
    if a.dim() != 2 or b.dim() != 3 or a.shape[1] != b.shape[2] or not b.is_contiguous():
        raise ValueError(f"shape mismatch: a {tuple(a.shape)} b {tuple(b.shape)} (b contiguous)")
    groups, n, k = b.shape
    if offsets.dtype != torch.int32 or offsets.numel() != groups + 1 or offsets.device != a.device:
        raise ValueError("offsets must be an int32 [groups + 1] tensor on the operands' device")
    if a.stride(1) != 1:
        a = a.contiguous()
    rows = a.shape[0]
    if out is None:
        out = torch.empty(rows, n, device=a.device, dtype=torch.bfloat16)
    nbytes = int(_lib.load().spx_gemm_grouped_workspace_bytes(rows, groups))
    ws = torch.empty(nbytes // 4, device=a.device, dtype=torch.int32)
    _lib.call("spx_gemm_bf16_nt_grouped", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(1), b.stride(0),
              _lib.ptr(out), out.stride(0), rows, n, k, _lib.ptr(offsets), groups, _lib.ptr(ws), nbytes,
              _lib.stream_ptr(a.device))
    return out


def gemm_tn_grouped(a: torch.Tensor, b: torch.Tensor, offsets: torch.Tensor, out: torch.Tensor,
                    accumulate: bool = False) -> torch.Tensor:
    """``out[e] (+)= a[rows of e].T @ b[rows of e]``: ``a [rows, M]``, ``b [rows, N]`` sorted by
    group, ``out [groups, M, N]`` bf16 or fp32 -- the weight gradients of all experts."""
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise _lib.SpxError("gemm_tn_grouped takes bf16 operands")
    if a.dim() != 2 or b.dim() != 2 or a.shape[0] != b.shape[0]:
        raise ValueError(f"shape mismatch: a {tuple(a.shape)} b {tuple(b.shape)}")
    groups = offsets.numel() - 1
    m, n = a.shape[1], b.shape[1]
    if out.shape != (groups, m, n) or not out.is_contiguous() or out.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"out must be a contiguous bf16 or fp32 [{groups}, {m}, {n}] tensor")
    if offsets.dtype != torch.int32 or offsets.device != a.device:
        raise ValueError("offsets must be an int32 tensor on the operands' device")
    if a.stride(1) != 1:
        a = a.contiguous()
    if b.stride(1) != 1:
        b = b.contiguous()
    _lib.call("spx_gemm_bf16_tn_grouped", _lib.ptr(a), a.stride(0), _lib.ptr(b), b.stride(0), _lib.ptr(out),
              out.stride(1), out.stride(0), m, n, a.shape[0], _lib.ptr(offsets), groups,
              int(out.dtype == torch.float32), int(accumulate), _lib.stream_ptr(a.device))
    return out


def gemm_tn_grouped_multi(a: torch.Tensor, b: torch.Tensor, offsets: torch.Tensor, out: torch.Tensor,
                          accumulate: bool = False) -> torch.Tensor:
    """The grouped weight gradient over several uses at once: ``a [S * rows, M]`` and
    ``b [S * rows, N]`` are S segments of ``rows`` sorted rows each, ``offsets [S, groups + 1]``
    holds every segment's group boundaries (a row of zeros: that segment has nothing), and
    ``out[e] (+)= sum_s a[rows of e in s].T @ b[rows of e in s]``."""
    segments, g1 = offsets.shape
    rows = a.shape[0] // segments
    m, n = a.shape[1], b.shape[1]
    if (a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16 or a.shape[0] != segments * rows
            or b.shape[0] != a.shape[0] or not a.is_contiguous() or not b.is_contiguous()):
        raise ValueError("a and b must be contiguous bf16 stacks of equally long segments")
    if out.shape != (g1 - 1, m, n) or not out.is_contiguous() or out.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"out must be a contiguous bf16 or fp32 [{g1 - 1}, {m}, {n}] tensor")
    if offsets.dtype != torch.int32 or not offsets.is_contiguous() or offsets.device != a.device:
        raise ValueError("offsets must be a contiguous int32 tensor on the operands' device")
    _lib.call("spx_gemm_bf16_tn_grouped_multi", _lib.ptr(a), m, _lib.ptr(b), n, _lib.ptr(out), n, m * n, m, n,
              rows, segments, _lib.ptr(offsets), g1 - 1, int(out.dtype == torch.float32), int(accumulate),
              _lib.stream_ptr(a.device))
    return out


class _ExpertStacks:
    """Inputs, output gradients and group boundaries of all uses of one expert weight stack in one
    forward / backward, one use below the other, so that the stack's weight gradient is ONE
    multi-segment grouped product when autograd reaches its staging node (the sum over the uses
    happens in the MFMA accumulators and the gradient is written once)."""

    def __init__(self, staged: Staged, rows: int, x_cols: int, dy_cols: int):
        w = staged.w
        # (no reference back to `staged`: it owns this object and its hook, and the buffers go
        # with it as soon as the graph is dropped)
        self.w_shape, self.rows, self.dy_cols = w.shape, rows, dy_cols
        self.x = torch.empty(staged.uses * rows, x_cols, device=w.device, dtype=torch.bfloat16)
        self.dy = None
        self.off = torch.zeros(staged.uses, w.shape[0] + 1, device=w.device, dtype=torch.int32)
        self.fill = 0
        self.live = False
        staged._finishers.append(self.add_gradient)

    @staticmethod
    def use(staged: Staged, rows: int, x_cols: int, dy_cols: int):
        """``(stacks, use index)`` for the next product against ``staged``, or ``(None, -1)`` when
        there is nothing to gain (frozen, one use, no graph) or no room."""
        if staged.token is None or staged.uses <= 1 or not torch.is_grad_enabled():
            return None, -1
        st = staged.aux
        if st is None:
            st = staged.aux = _ExpertStacks(staged, rows, x_cols, dy_cols)
        if st.rows != rows or st.fill >= staged.uses:
            return None, -1
        st.fill += 1
        return st, st.fill - 1

    def x_slot(self, u: int) -> torch.Tensor:
        return self.x[u * self.rows:(u + 1) * self.rows]

    def dy_slot(self, u: int) -> torch.Tensor:
        if self.dy is None:
            self.dy = torch.empty(self.x.shape[0], self.dy_cols, device=self.x.device, dtype=torch.bfloat16)
        return self.dy[u * self.rows:(u + 1) * self.rows]

    def record(self, u: int, offsets: torch.Tensor):
        self.off[u].copy_(offsets)
        self.live = True

    def add_gradient(self, acc):
        if not self.live:
            return acc
        fresh = acc is None
        if fresh:
            acc = torch.empty(self.w_shape, device=self.x.device, dtype=torch.float32)
        gemm_tn_grouped_multi(self.dy, self.x, self.off, acc, accumulate=not fresh)
        self.off.zero_()  # uses whose backward does not run next time contribute nothing
        self.live = False
        return acc


def gather_rows(x2: torch.Tensor, src_row: torch.Tensor, scale: torch.Tensor | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor:
    """``out[p] = scale[p] * x2[src_row[p]]`` (bf16 rows, ``src_row`` int32, ``scale`` fp32)."""
    rows, h = src_row.numel(), x2.shape[1]
    if out is None:
        out = torch.empty(rows, h, device=x2.device, dtype=torch.bfloat16)
    _lib.call("spx_moe_gather_rows", _lib.ptr(x2), x2.stride(0), x2.shape[0], _lib.ptr(src_row),
              _lib.ptr(scale), _lib.ptr(out), h, rows, h, _lib.stream_ptr(x2.device))
    return out


def combine_rows(sorted_rows: torch.Tensor, pos: torch.Tensor, weight: torch.Tensor | None) -> torch.Tensor:
    """``out[t] = sum_j weight[t, j] * sorted_rows[pos[t, j]]`` (``pos`` int32 ``[T, k]``)."""
    tokens, k = pos.shape
    h = sorted_rows.shape[1]
    out = torch.empty(tokens, h, device=sorted_rows.device, dtype=torch.bfloat16)
    _lib.call("spx_moe_combine_rows", _lib.ptr(sorted_rows), sorted_rows.stride(0), sorted_rows.shape[0],
              _lib.ptr(pos), _lib.ptr(weight), _lib.ptr(out), h, tokens, k, h,
              _lib.stream_ptr(sorted_rows.device))
    return out


def pair_dot(a: torch.Tensor, sorted_rows: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """``out[t, j] = <a[t], sorted_rows[pos[t, j]]>`` in fp32."""
    tokens, k = pos.shape
    out = torch.empty(tokens, k, device=a.device, dtype=torch.float32)
    _lib.call("spx_moe_pair_dot", _lib.ptr(a), a.stride(0), _lib.ptr(sorted_rows), sorted_rows.stride(0),
              sorted_rows.shape[0], _lib.ptr(pos), _lib.ptr(out), tokens, k, a.shape[1],
              _lib.stream_ptr(a.device))
    return out


def route(logits: torch.Tensor, top_k: int, renormalise: bool):
    """``Qwen3NextTopKRouter.forward`` after the router product: soft-max over all experts in
    fp32, the ``top_k`` largest, optionally renormalised, cast to the logits' dtype.
    -> (scores ``[T, k]``, expert ids ``[T, k]``)."""
    probs = F.softmax(logits, dtype=torch.float, dim=-1)
    top, idx = torch.topk(probs, top_k, dim=-1)
    if renormalise:
        top = top / top.sum(dim=-1, keepdim=True)
    return top.to(logits.dtype), idx


def sort_pairs(idx: torch.Tensor, num_experts: int):
    """The ``(token, slot)`` pairs of ``idx [T, k]`` sorted by expert (stable: token order inside an
    expert).  -> ``order`` (pair of every sorted row, int64), ``src_row`` (its token, int32),
    ``pos`` (sorted row of every pair, int32 ``[T, k]``), ``offsets`` (int32 ``[E + 1]``).  All on
    the device; nothing is read back."""
    t, k = idx.shape
    flat = idx.reshape(-1)
    order = torch.argsort(flat, stable=True)
    counts = torch.zeros(num_experts, device=idx.device, dtype=torch.int32)
    counts.index_add_(0, flat, torch.ones_like(flat, dtype=torch.int32))
    offsets = torch.zeros(num_experts + 1, device=idx.device, dtype=torch.int32)
    offsets[1:] = counts.cumsum(0)
    src_row = (order // k).to(torch.int32)
    pos = torch.empty(t * k, device=idx.device, dtype=torch.int32)
    pos[order] = torch.arange(t * k, device=idx.device, dtype=torch.int32)
    return order, src_row, pos.view(t, k), offsets


class _ExpertsMLP(torch.autograd.Function):
    """``Qwen3NextExperts.forward``: ``out[t] = sum_j scores[t, j] * down_e(silu(gate_e x_t) * up_e x_t)``,
    ``e = idx[t, j]``, on expert-sorted rows.  The weight gradients of the uses of one forward add
    up in one fp32 buffer per weight (``Staged.grad_buffer``), which the staging node hands to
    autograd once."""

    @staticmethod
    def forward(ctx, x2, scores, idx, _tok_gu, _tok_dn, st_gu: Staged, st_dn: Staged):
        if x2.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP layer kernels take bf16 tensors")
        w_gu, w_dn = st_gu.w, st_dn.w  # [E, 2I, H], [E, H, I]
        e, i2, h = w_gu.shape
        inter = i2 // 2
        order, src_row, pos, off = sort_pairs(idx, e)
        rows = src_row.numel()
        st = _lib.stream_ptr(x2.device)
        # with several uses per forward the inputs of the two products go straight into the stacks
        # that the one weight-gradient product over all uses reads
        stack_gu, use_gu = _ExpertStacks.use(st_gu, rows, h, i2)
        stack_dn, use_dn = _ExpertStacks.use(st_dn, rows, inter, h)
        xs = gather_rows(x2, src_row, out=None if stack_gu is None else stack_gu.x_slot(use_gu))
        hid = gemm_nt_grouped(xs, w_gu, off)
        act = (torch.empty(rows, inter, device=x2.device, dtype=torch.bfloat16) if stack_dn is None
               else stack_dn.x_slot(use_dn))
        up = hid[:, inter:]
        _lib.call("spx_swiglu_rows_fwd", _lib.ptr(hid), i2, _lib.ptr(up), i2, _lib.ptr(act), inter, rows,
                  inter, st)
        ys = gemm_nt_grouped(act, w_dn, off)
        wts = scores.float().contiguous()
        out = combine_rows(ys, pos, wts)
        ctx.save_for_backward(xs, hid, act, ys, pos, src_row, off, order, wts)
        ctx.staged = (st_gu, st_dn)
        ctx.stacks = ((stack_gu, use_gu), (stack_dn, use_dn))
        ctx.score_dtype = scores.dtype
        return out

    @staticmethod
    def backward(ctx, dout):
        xs, hid, act, ys, pos, src_row, off, order, wts = ctx.saved_tensors
        st_gu, st_dn = ctx.staged
        rows, inter = act.shape
        i2 = 2 * inter
        dout = dout.to(torch.bfloat16).contiguous()
        st = _lib.stream_ptr(dout.device)
        dscores = None
        if ctx.needs_input_grad[1]:
            dscores = pair_dot(dout, ys, pos).to(ctx.score_dtype)
        (stack_gu, use_gu), (stack_dn, use_dn) = ctx.stacks
        want_gu, want_dn = ctx.needs_input_grad[3], ctx.needs_input_grad[4]
        dys = gather_rows(dout, src_row, wts.reshape(-1)[order].contiguous(),
                          out=stack_dn.dy_slot(use_dn) if stack_dn is not None and want_dn else None)
        dact = gemm_nt_grouped(dys, st_dn.wt, off)
        dh = (stack_gu.dy_slot(use_gu) if stack_gu is not None and want_gu
              else torch.empty(rows, i2, device=dout.device, dtype=torch.bfloat16))
        _lib.call("spx_swiglu_rows_bwd", _lib.ptr(hid), i2, _lib.ptr(hid[:, inter:]), i2, _lib.ptr(dact), inter,
                  _lib.ptr(dh), i2, _lib.ptr(dh[:, inter:]), i2, rows, inter, st)
        dx = None
        if ctx.needs_input_grad[0]:
            dx = combine_rows(gemm_nt_grouped(dh, st_gu.wt, off), pos, None)
        marks = []
        for need, staged, dy2, x2, stack, use in ((want_gu, st_gu, dh, xs, stack_gu, use_gu),
                                                 (want_dn, st_dn, dys, act, stack_dn, use_dn)):
            if not need:
                marks.append(None)
                continue
            if stack is not None:
                stack.record(use, off)  # the product runs once, over all uses, in the staging node
            else:
                buf, holds = staged.grad_buffer()
                gemm_tn_grouped(dy2, x2, off, buf, accumulate=holds)
            marks.append(staged.mark())
        return dx, dscores, None, marks[0], marks[1], None, None


def experts_mlp(x2, scores, idx, st_gu: Staged, st_dn: Staged):
    """``[T, H]`` tokens through their ``idx [T, k]`` experts, weighted by ``scores [T, k]``."""
    return _ExpertsMLP.apply(x2, scores, idx, st_gu.token, st_dn.token, st_gu, st_dn)
