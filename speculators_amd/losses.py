"""Loss-function registry backed by the HIP fused vocabulary loss.

Mirror of the reference's loss plug-in (``speculators/losses/utils.py``): a
``LossConfig`` is ``{name: (fn(logits, targets) -> [B, T] float32, weight)}``
(losses/utils.py:12-14) and ``resolve_loss_config(spec, implementation)``
(losses/utils.py:184-230) turns ``"kl_div"`` or a JSON dict of weights into
one.  The implementation name registered here is ``"hip"``; its functions are
differentiable with respect to ``logits`` only, like the reference's fused
losses (losses/fused.py:238-291).
"""

from __future__ import annotations

import json
from collections.abc import Callable
from dataclasses import dataclass

import torch

from . import _lib

LossConfig = dict[str, tuple[Callable[[torch.Tensor, torch.Tensor], torch.Tensor], float]]

OP_KL, OP_RKL, OP_JSD, OP_CE, OP_TV = 0, 1, 2, 3, 4
_NLA_EPS = 1e-5  # losses/fused.py:294


def _rows_2d(t: torch.Tensor) -> torch.Tensor:
    """[B, T, V] -> [B*T, V] view with unit inner stride (copies only if the
    vocabulary axis itself is strided or the rows are not equally spaced)."""
    v = t.shape[-1]
    if t.stride(-1) != 1:
        t = t.contiguous()
    try:
        return t.view(-1, v)
    except RuntimeError:
        return t.reshape(-1, v)


@dataclass
class StepPass:
    """What one TTT step adds to the row pass of the loss kernel (``spx_vocab_loss_step_fwd``).

    ``d2t`` (int64 ``[Vd]``): the targets are FULL-vocabulary verifier rows and target element i
    is read at column ``i + d2t[i]`` while streaming; the draft-vocabulary rows come back in
    ``gathered`` (``[rows, Vd]``) for the later steps and the backward.
    ``counts`` (int32 ``[3]``, zeroed): the acceptance chain is done row by row in the same pass
    (``mask`` / ``prev`` are the step's 1-D views, ``prev`` is updated in place).
    ``grad_in_pass``: a promise of the caller that the reduction behind the row losses gives a row
    whose ``mask`` entry is zero the weight zero (the masked mean of ``compute_metrics`` does).  The
    head + loss node may then leave the gradient of the logits behind in the same row pass
    (``spx_vocab_loss_step_fwd_grad``) instead of reading both rows again in its backward; masked
    rows get no gradient whatever arrives for them."""

    d2t: torch.Tensor | None = None
    gathered: torch.Tensor | None = None
    mask: torch.Tensor | None = None
    prev: torch.Tensor | None = None
    counts: torch.Tensor | None = None
    grad_in_pass: bool = False


def fused_loss_forward(op: int, logits: torch.Tensor, targets: torch.Tensor, target_stats=None,
                       step: StepPass | None = None):
    """Run the forward kernel.  Returns (loss [R] f32, lse_d, lse_t, extra,
    argmax_draft [R] i32, argmax_target [R] i32, logits2d, targets2d).

    ``target_stats = (lse_target [R] f32, argmax_target [R] i32)`` from an earlier call on
    the same target rows lets kl / ce skip the target row statistics (ce then does not
    read the targets at all).  ``step``: see ``StepPass``; with ``step.d2t`` the returned
    ``targets2d`` are the gathered draft-vocabulary rows."""
    gather = step is not None and step.d2t is not None
    if targets is None:
        # cross-entropy against arg-max targets whose arg-max is known: no target row is read
        if op != OP_CE or target_stats is None or gather:
            raise ValueError("only ce with known target statistics runs without the target rows")
        return _ce_without_targets(logits, target_stats, step)
    if not gather and logits.shape != targets.shape:
        raise ValueError(f"logits {tuple(logits.shape)} and targets {tuple(targets.shape)} differ")
    if gather and logits.shape[:-1] != targets.shape[:-1]:
        raise ValueError(f"logits {tuple(logits.shape)} and full-vocabulary targets "
                         f"{tuple(targets.shape)} differ in their rows")
    if logits.dtype != targets.dtype:
        targets = targets.to(logits.dtype)
    x, y = _rows_2d(logits), _rows_2d(targets)
    rows, vocab = x.shape
    dev = x.device
    if step is not None:
        if gather:
            if target_stats is not None:
                raise ValueError("the gather form computes the target statistics itself")
            if step.d2t.dtype != torch.int64 or step.d2t.numel() != vocab or not step.d2t.is_contiguous():
                raise ValueError("d2t must be a contiguous int64 [draft vocabulary] tensor")
            step.gathered = torch.empty(rows, vocab, device=dev, dtype=x.dtype)
        stats = torch.empty(4, rows, device=dev, dtype=torch.float32)
        arg = torch.empty(2, rows, device=dev, dtype=torch.int32)
        reuse = target_stats is not None and op in (OP_KL, OP_CE)
        lse_t, am_t = stats[2], arg[1]
        if reuse:
            lse_t, am_t = target_stats[0].reshape(-1), target_stats[1].reshape(-1)
        g = step.gathered
        _lib.call(
            "spx_vocab_loss_step_fwd", op, _lib.ptr(x), x.stride(0), _lib.ptr(y), y.stride(0),
            _lib.ptr(step.d2t), y.shape[1] if gather else 0, _lib.ptr(g) if gather else None,
            g.stride(0) if gather else 0, rows, vocab, _lib.dtype_code(x), _lib.ptr(stats[0]),
            _lib.ptr(stats[1]), _lib.ptr(lse_t), _lib.ptr(stats[3]), _lib.ptr(arg[0]), _lib.ptr(am_t),
            int(reuse), _lib.ptr(step.mask), _lib.kind_code(step.mask) if step.mask is not None else 0,
            _lib.ptr(step.prev), _lib.kind_code(step.prev) if step.prev is not None else 0,
            _lib.ptr(step.counts), _lib.stream_ptr(dev),
        )
        return stats[0], stats[1], lse_t, stats[3], arg[0], am_t, x, (g if gather else y)
    reuse = target_stats is not None and op in (OP_KL, OP_CE)
    stats = torch.empty(4, rows, device=dev, dtype=torch.float32)
    arg = torch.empty(2, rows, device=dev, dtype=torch.int32)
    lse_t, am_t = stats[2], arg[1]
    if reuse:
        lse_t = target_stats[0].reshape(-1)
        am_t = target_stats[1].reshape(-1)
        if lse_t.numel() != rows or am_t.numel() != rows or lse_t.stride(0) != 1 or am_t.stride(0) != 1:
            raise ValueError("target_stats must be contiguous [rows] tensors")
    _lib.call(
        "spx_fused_vocab_loss_fwd", op, _lib.ptr(x), x.stride(0), _lib.ptr(y), y.stride(0),
        rows, vocab, _lib.dtype_code(x), _lib.ptr(stats[0]), _lib.ptr(stats[1]),
        _lib.ptr(lse_t), _lib.ptr(stats[3]), _lib.ptr(arg[0]), _lib.ptr(am_t), int(reuse),
        _lib.stream_ptr(dev),
    )
    return stats[0], stats[1], lse_t, stats[3], arg[0], am_t, x, y


def _ce_without_targets(logits, target_stats, step):
    x = _rows_2d(logits)
    rows, vocab = x.shape
    dev = x.device
    stats = torch.empty(4, rows, device=dev, dtype=torch.float32)
    arg = torch.empty(1, rows, device=dev, dtype=torch.int32)
    lse_t, am_t = target_stats[0].reshape(-1), target_stats[1].reshape(-1)
    if lse_t.numel() != rows or am_t.numel() != rows or lse_t.stride(0) != 1 or am_t.stride(0) != 1:
        raise ValueError("target_stats must be contiguous [rows] tensors")
    if step is not None:
        _lib.call(
            "spx_vocab_loss_step_fwd", OP_CE, _lib.ptr(x), x.stride(0), None, 0, None, 0, None, 0, rows, vocab,
            _lib.dtype_code(x), _lib.ptr(stats[0]), _lib.ptr(stats[1]), _lib.ptr(lse_t), _lib.ptr(stats[3]),
            _lib.ptr(arg[0]), _lib.ptr(am_t), 1, _lib.ptr(step.mask),
            _lib.kind_code(step.mask) if step.mask is not None else 0, _lib.ptr(step.prev),
            _lib.kind_code(step.prev) if step.prev is not None else 0, _lib.ptr(step.counts),
            _lib.stream_ptr(dev))
    else:
        _lib.call(
            "spx_fused_vocab_loss_fwd", OP_CE, _lib.ptr(x), x.stride(0), None, 0, rows, vocab,
            _lib.dtype_code(x), _lib.ptr(stats[0]), _lib.ptr(stats[1]), _lib.ptr(lse_t), _lib.ptr(stats[3]),
            _lib.ptr(arg[0]), _lib.ptr(am_t), 1, _lib.stream_ptr(dev))
    return stats[0], stats[1], lse_t, stats[3], arg[0], am_t, x, None


class _FusedLoss(torch.autograd.Function):
    """``(logits, targets, op[, lse_t, am_t]) -> (row_loss [B, T] f32, argmax_draft,
    argmax_target, lse_target)``; the autograd counterpart of ``_FusedLoss`` in
    losses/fused.py:238-291.  Targets get no gradient."""

    @staticmethod
    def forward(ctx, logits, targets, op, known_lse_t=None, known_am_t=None, n_rows=None, step=None):
        known = (known_lse_t, known_am_t) if known_lse_t is not None else None
        # n_rows: only the first n_rows rows of ``logits`` (a [1, T, V] tensor) take part, the
        # rest get a zero gradient.  Doing the cut here instead of slicing outside keeps
        # autograd from materialising a zero-padded copy of the whole gradient.
        ctx.full_shape = logits.shape
        used = logits if n_rows is None else logits[:, :n_rows]
        loss, lse_d, lse_t, extra, am_d, am_t, x, y = fused_loss_forward(op, used, targets, known, step)
        ctx.save_for_backward(x, None if op == OP_CE else y, lse_d, lse_t, extra, am_t)
        ctx.op = op
        lead = used.shape[:-1]
        am_d, am_t, lse_t = am_d.view(lead), am_t.view(lead), lse_t.view(lead)
        ctx.mark_non_differentiable(am_d, am_t, lse_t)
        ctx.set_materialize_grads(False)  # no zero tensors for the outputs that carry no gradient
        return loss.view(lead), am_d, am_t, lse_t

    @staticmethod
    def backward(ctx, grad_rows, _gd, _gt, _gl):
        if grad_rows is None:
            return (None,) * 7
        x, y, lse_d, lse_t, extra, am_t = ctx.saved_tensors
        rows, vocab = x.shape
        full_rows = 1
        for d in ctx.full_shape[:-1]:
            full_rows *= d
        g = grad_rows.reshape(-1).to(torch.float32).contiguous()
        grad = torch.empty(full_rows, vocab, device=x.device, dtype=x.dtype)
        _lib.call(
            "spx_fused_vocab_loss_bwd", ctx.op, _lib.ptr(x), x.stride(0), _lib.ptr(y),
            y.stride(0) if y is not None else 0, rows, vocab, _lib.dtype_code(x),
            _lib.ptr(lse_d), _lib.ptr(lse_t), _lib.ptr(extra), _lib.ptr(am_t), _lib.ptr(g), None,
            _lib.ptr(grad), grad.stride(0), _lib.stream_ptr(x.device),
        )
        if full_rows > rows:
            grad[rows:].zero_()
        return grad.view(ctx.full_shape), None, None, None, None, None, None


def _packed_row_map(row_grad: torch.Tensor, labels: torch.Tensor | None = None, ignore_index: int = -100):
    """(row map int32 [rows], live-row count int32 [1]): a row is live when its incoming gradient is
    non-zero (and its label is not the ignored one); live row r goes to slot ``#live rows before
    r``, the others to -1.  One small kernel; the count stays on the device."""
    rows = row_grad.numel()
    out = torch.empty(rows + 1, device=row_grad.device, dtype=torch.int32)
    _lib.call("spx_pack_row_map", _lib.ptr(row_grad), _lib.ptr(labels), int(ignore_index), rows,
              _lib.ptr(out), _lib.ptr(out[rows:]), _lib.stream_ptr(row_grad.device))
    return out[:rows], out[rows:]


def _unpack_rows_scaled(packed: torch.Tensor, row_map: torch.Tensor, row_scale: torch.Tensor, total_rows: int):
    """``_unpack_rows`` with live row r multiplied by ``row_scale[r]`` (fp32) on its way."""
    out = torch.empty(total_rows, packed.shape[1], device=packed.device, dtype=packed.dtype)
    _lib.call("spx_unpack_rows_scaled", _lib.ptr(packed), packed.stride(0), _lib.ptr(row_map), _lib.ptr(row_scale),
              row_map.numel(), total_rows, packed.shape[1], _lib.ptr(out), out.stride(0),
              _lib.stream_ptr(packed.device))
    return out


# The head + loss node writes the logits gradient in its forward row pass where it can (see StepPass)
HEAD_LOSS_ONE_PASS = True


def _one_pass_ok(op, x, y, step) -> bool:
    if not (HEAD_LOSS_ONE_PASS and step is not None and step.grad_in_pass and step.d2t is None
            and step.mask is not None and op in (OP_KL, OP_CE) and x.dtype == torch.bfloat16):
        return False
    rows, vocab = x.shape
    if rows == 0 or vocab % 8 or vocab > 32768 or x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        return False
    if step.mask.numel() != rows or (y is None and op != OP_CE):
        return False
    return y is None or (y.dtype == torch.bfloat16 and y.stride(1) == 1 and y.stride(0) % 8 == 0
                         and y.data_ptr() % 16 == 0)


def _loss_forward_with_grad(op, x, y, known, step):
    """The row pass that also writes the unit-weight logits gradient of the unmasked rows, packed to
    the front.  Returns ``(loss, lse_t, am_d, am_t, packed, row_map, count)``."""
    rows, vocab = x.shape
    dev = x.device
    mask_f = step.mask if step.mask.dtype == torch.float32 else step.mask.to(torch.float32)
    row_map, count = _packed_row_map(mask_f.contiguous())
    packed = torch.empty(rows, vocab, device=dev, dtype=torch.bfloat16)
    stats = torch.empty(4, rows, device=dev, dtype=torch.float32)
    arg = torch.empty(2, rows, device=dev, dtype=torch.int32)
    lse_t, am_t = stats[2], arg[1]
    if known is not None:
        lse_t, am_t = known[0].reshape(-1), known[1].reshape(-1)
        if lse_t.numel() != rows or am_t.numel() != rows or lse_t.stride(0) != 1 or am_t.stride(0) != 1:
            raise ValueError("target_stats must be contiguous [rows] tensors")
    _lib.call(
        "spx_vocab_loss_step_fwd_grad", op, _lib.ptr(x), x.stride(0), _lib.ptr(y),
        y.stride(0) if y is not None else 0, rows, vocab, _lib.ptr(stats[0]), _lib.ptr(stats[1]),
        _lib.ptr(lse_t), _lib.ptr(stats[3]), _lib.ptr(arg[0]), _lib.ptr(am_t), int(known is not None),
        _lib.ptr(step.mask), _lib.kind_code(step.mask), _lib.ptr(step.prev),
        _lib.kind_code(step.prev) if step.prev is not None else 0, _lib.ptr(step.counts),
        _lib.ptr(row_map), _lib.ptr(packed), packed.stride(0), _lib.stream_ptr(dev))
    return stats[0], lse_t, arg[0], am_t, packed, row_map, count


def _unpack_rows(packed: torch.Tensor, row_map: torch.Tensor, total_rows: int):
    """One row per position again: live rows from their packed slot, the others (and the rows past
    the map, up to ``total_rows``) zero.  Slots past the count are never read."""
    out = torch.empty(total_rows, packed.shape[1], device=packed.device, dtype=packed.dtype)
    _lib.call("spx_unpack_rows", _lib.ptr(packed), packed.stride(0), _lib.ptr(row_map), row_map.numel(),
              total_rows, packed.shape[1], _lib.ptr(out), out.stride(0), _lib.stream_ptr(packed.device))
    return out


class _HeadFusedLoss(torch.autograd.Function):
    """A frozen ``lm_head`` and the fused vocabulary loss behind it as ONE autograd node:
    ``(x [T, H], weight [Vd, H], weight_t [H, Vd], targets [n_rows, Vd], op, ...) ->
    (row loss [n_rows], argmax_draft, argmax_target, lse_target, logits [T, Vd])``.

    Rows the loss mask removes (and the rows past ``n_rows``) have an all-zero logits gradient.
    With both steps in one node the backward packs the live rows to the front
    (``spx_fused_vocab_loss_bwd_packed``) and the input-gradient product of the head runs over
    them only (``spx_gemm_bf16_nt_rows``, count read on the device); dead rows of the result are
    exact zeros, as they are when the product runs over all rows.  The logits come back for the
    metrics and the draft tokens and carry no gradient of their own."""

    @staticmethod
    def forward(ctx, x2, weight, weight_t, targets, op, known_lse_t, known_am_t, n_rows, step=None):
        from .gemm import gemm_nt

        logits = gemm_nt(x2, weight)
        known = (known_lse_t, known_am_t) if known_lse_t is not None else None
        ctx.op, ctx.total_rows = op, logits.shape[0]
        xs = logits[:n_rows]
        ys = None if targets is None else _rows_2d(targets)
        ctx.one_pass = (known is not None or ys is not None) and _one_pass_ok(op, xs, ys, step)
        if ctx.one_pass:
            # the rows are read once: loss, statistics, chain and the (unit-weight) logits gradient
            loss, lse_t, am_d, am_t, packed, row_map, count = _loss_forward_with_grad(op, xs, ys, known, step)
            ctx.save_for_backward(packed, row_map, count, weight_t)
        else:
            loss, lse_d, lse_t, extra, am_d, am_t, x, y = fused_loss_forward(op, xs, targets, known, step)
            ctx.save_for_backward(x, None if op == OP_CE else y, lse_d, lse_t, extra, am_t, weight_t)
        ctx.mark_non_differentiable(am_d, am_t, lse_t, logits)
        ctx.set_materialize_grads(False)  # no [T, Vd] zeros for the logits, which carry no gradient
        return loss, am_d, am_t, lse_t, logits

    @staticmethod
    def backward(ctx, grad_rows, _gd, _gt, _gl, _glogits):
        from .gemm import gemm_nt

        if grad_rows is None:
            return (None,) * 9
        if ctx.one_pass:
            packed, row_map, count, weight_t = ctx.saved_tensors
            g = grad_rows.reshape(-1).to(torch.float32).contiguous()
            dx_packed = gemm_nt(packed, weight_t, m_live=count, split=True)
            return (_unpack_rows_scaled(dx_packed, row_map, g, ctx.total_rows), None, None, None, None, None,
                    None, None, None)

        x, y, lse_d, lse_t, extra, am_t, weight_t = ctx.saved_tensors
        rows, vocab = x.shape
        g = grad_rows.reshape(-1).to(torch.float32).contiguous()
        row_map, count = _packed_row_map(g)
        packed = torch.empty(rows, vocab, device=x.device, dtype=x.dtype)
        _lib.call(
            "spx_fused_vocab_loss_bwd_packed", ctx.op, _lib.ptr(x), x.stride(0), _lib.ptr(y),
            y.stride(0) if y is not None else 0, rows, vocab, _lib.dtype_code(x),
            _lib.ptr(lse_d), _lib.ptr(lse_t), _lib.ptr(extra), _lib.ptr(am_t), _lib.ptr(g), None,
            _lib.ptr(row_map), _lib.ptr(packed), packed.stride(0), _lib.stream_ptr(x.device),
        )
        dx_packed = gemm_nt(packed, weight_t, m_live=count, split=True)
        return (_unpack_rows(dx_packed, row_map, ctx.total_rows), None, None, None, None, None,
                None, None, None)


def head_fused_rows(op: int, x, weight, weight_t, targets, target_stats=None, n_rows=None, step=None):
    """``fused_rows`` with the frozen head in front: ``x [1, T, H]`` instead of logits.  Returns
    ``(row_loss [1, n_rows], argmax_draft, argmax_target, lse_target, logits [1, T, Vd])``."""
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise _lib.SpxError("head_fused_rows takes bf16 operands")
    if weight.requires_grad:
        raise ValueError("head_fused_rows is for a frozen head (no weight gradient is produced)")
    if x.dim() != 3 or x.shape[0] != 1:
        raise ValueError("x must be [1, T, H] (the packed batch layout)")
    t = x.shape[1]
    n = t if n_rows is None else int(n_rows)
    y = None if targets is None else _rows_2d(targets)
    if y is not None and y.shape[0] != n:
        raise ValueError(f"targets have {y.shape[0]} rows, expected {n}")
    ks = (None, None) if target_stats is None else (target_stats[0], target_stats[1])
    # (a view, not x[0]: the backward of a select writes the gradient into a zero-filled copy)
    loss, am_d, am_t, lse_t, logits = _HeadFusedLoss.apply(x.reshape(t, x.shape[2]), weight, weight_t, y, op,
                                                           ks[0], ks[1], n, step)
    lead = (1, n)
    return (loss.view(lead), am_d.view(lead), am_t.view(lead), lse_t.view(lead),
            logits.view(1, t, weight.shape[0]))


def fused_rows(op: int, logits, targets, target_stats=None, n_rows=None, step: StepPass | None = None):
    """(row_loss, argmax_draft, argmax_target, lse_target) of one primitive reduction;
    ``n_rows`` restricts ``logits [1, T, V]`` to its first ``n_rows`` rows (``targets`` already
    has that many) without slicing it under autograd; ``step``: see ``StepPass``."""
    if target_stats is None:
        return _FusedLoss.apply(logits, targets, op, None, None, n_rows, step)
    return _FusedLoss.apply(logits, targets, op, target_stats[0], target_stats[1], n_rows, step)


def kl_div_loss(logits, targets):
    return fused_rows(OP_KL, logits, targets)[0]


def reverse_kl_div_loss(logits, targets):
    return fused_rows(OP_RKL, logits, targets)[0]


def js_div_loss(logits, targets):
    return fused_rows(OP_JSD, logits, targets)[0]


def ce_loss(logits, targets):
    return fused_rows(OP_CE, logits, targets)[0]


def tv_loss(logits, targets):
    return fused_rows(OP_TV, logits, targets)[0]


def neg_log_acceptance_loss(logits, targets):
    """-log(max(1 - tv, 1e-5)) composed on the [B, T] tv rows (losses/fused.py:322-324)."""
    return -torch.log((1.0 - tv_loss(logits, targets)).clamp_min(_NLA_EPS))


def lk_hybrid_loss(logits, targets, eta: float = 3.0):
    """lam*kl + (1-lam)*tv with lam = exp(-eta*stopgrad(1-tv)) (losses/fused.py:327-334)."""
    kl = kl_div_loss(logits, targets)
    tv = tv_loss(logits, targets)
    lam = torch.exp(-eta * (1.0 - tv).detach())
    return lam * kl + (1.0 - lam) * tv


_HIP_LOSS_FN_MAP: dict[str, Callable] = {
    "kl_div": kl_div_loss,
    "rkl": reverse_kl_div_loss,
    "jsd": js_div_loss,
    "ce": ce_loss,
    "tv": tv_loss,
    "nla": neg_log_acceptance_loss,
    "lk_hybrid": lk_hybrid_loss,
}

# which primitive kernel reduction also yields the arg-maxes for a named loss
PRIMITIVE_OP = {"kl_div": OP_KL, "rkl": OP_RKL, "jsd": OP_JSD, "ce": OP_CE, "tv": OP_TV}

_LOSS_FN_MAPS = {"hip": _HIP_LOSS_FN_MAP}


def resolve_loss_config(spec: str, implementation: str = "hip") -> LossConfig:
    """``"kl_div"`` or ``'{"ce": 0.1, "tv": 0.9}'`` -> ``{name: (fn, weight)}`` with the
    error behaviour of losses/utils.py:184-230."""
    try:
        table = _LOSS_FN_MAPS[implementation]
    except KeyError:
        raise ValueError(
            f"Unknown loss implementation '{implementation}'. Choose from: {sorted(_LOSS_FN_MAPS)}"
        ) from None
    if spec in table:
        return {spec: (table[spec], 1.0)}
    try:
        parsed = json.loads(spec)
    except json.JSONDecodeError:
        raise ValueError(
            f"Unknown loss function '{spec}'. Pass a known name ({sorted(table)}) or a JSON dict, "
            'e.g. \'{"ce": 0.1, "tv": 0.9}\'.'
        ) from None
    if not isinstance(parsed, dict) or not parsed:
        raise ValueError(
            "Loss config must be a non-empty JSON dict mapping loss names to weights, "
            f'e.g. \'{{"ce": 0.1, "tv": 0.9}}\'. Got: {spec}'
        )
    out: LossConfig = {}
    for name, weight in parsed.items():
        if name not in table:
            raise ValueError(
                f"Unknown loss function '{name}' in loss config. Choose from: {sorted(table)}"
            )
        if isinstance(weight, bool) or not isinstance(weight, (int, float)):
            raise ValueError(
                f"Loss weight for '{name}' must be a number, got {type(weight).__name__}"
            )
        out[name] = (table[name], float(weight))
    return out


class _LabelCE(torch.autograd.Function):
    """Per-row cross-entropy of ``logits [R, V]`` against integer ``labels [R]`` with an
    ignore index, on the HIP label-CE kernels (one read of the logits in the forward, one
    read + one write in the backward)."""

    @staticmethod
    def forward(ctx, logits2d, labels, ignore_index):
        rows, vocab = logits2d.shape
        dev = logits2d.device
        out = torch.empty(2, rows, device=dev, dtype=torch.float32)
        _lib.call("spx_label_ce_fwd", _lib.ptr(logits2d), logits2d.stride(0), _lib.ptr(labels), rows,
                  vocab, _lib.dtype_code(logits2d), int(ignore_index), _lib.ptr(out[0]),
                  _lib.ptr(out[1]), None, _lib.stream_ptr(dev))
        ctx.save_for_backward(logits2d, labels, out[1])
        ctx.ignore_index = int(ignore_index)
        return out[0]

    @staticmethod
    def backward(ctx, grad_rows):
        logits2d, labels, lse = ctx.saved_tensors
        rows, vocab = logits2d.shape
        g = grad_rows.to(torch.float32).contiguous()
        dlogits = torch.empty(rows, vocab, device=logits2d.device, dtype=logits2d.dtype)
        _lib.call("spx_label_ce_bwd", _lib.ptr(logits2d), logits2d.stride(0), _lib.ptr(labels),
                  _lib.ptr(lse), _lib.ptr(g), rows, vocab, _lib.dtype_code(logits2d),
                  ctx.ignore_index, _lib.ptr(dlogits), dlogits.stride(0),
                  _lib.stream_ptr(logits2d.device))
        return dlogits, None, None


def label_cross_entropy(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int = -100):
    """``F.cross_entropy(logits.permute(0, 2, 1), labels, ignore_index=..., reduction="none")``
    (models/mtp/core.py:204-216) for ``logits [..., V]`` (bf16 or fp32) and integer ``labels
    [...]``: returns float32 losses of the shape of ``labels``, 0 at ignored positions."""
    if logits.shape[:-1] != labels.shape:
        raise ValueError(f"logits {tuple(logits.shape)} and labels {tuple(labels.shape)} do not match")
    if logits.dtype not in (torch.bfloat16, torch.float32):
        raise _lib.SpxError("label_cross_entropy takes bf16 or fp32 logits")
    x = _rows_2d(logits)
    lab = labels.reshape(-1).to(torch.int64).contiguous()
    return _LabelCE.apply(x, lab, ignore_index).view(labels.shape)


class _HeadLabelCE(torch.autograd.Function):
    """A frozen output head and the label cross-entropy behind it as ONE autograd node:
    ``(x [R, H], weight [V, H], weight_t [H, V], labels [R]) -> (row loss [R] f32, logits [R, V])``.

    What the single node buys is the backward: a position with an ignored label (or a zero
    incoming gradient) has an all-zero logits-gradient row, so the loss backward packs the live
    rows to the front (``spx_label_ce_bwd_packed``) and the input-gradient product runs over
    those rows only (``spx_gemm_bf16_nt_rows``, row count read on the device, no host
    synchronisation); the dead rows of ``dx`` are exact zeros, as they are when the product
    runs over all rows.  The logits come back for the caller's metrics / return value but carry
    no gradient of their own."""

    @staticmethod
    def forward(ctx, x2, weight, weight_t, labels, ignore_index, epilogue_stats=False):
        from .gemm import gemm_nt, gemm_nt_stats

        if epilogue_stats:
            # the head product's epilogue leaves every row's log-sum-exp; the loss then reads one
            # element of each row instead of streaming the [rows, V] logits a second time
            logits, lse, _ = gemm_nt_stats(x2, weight, want_argmax=False)
            rows, vocab = logits.shape
            out = torch.empty(2, rows, device=logits.device, dtype=torch.float32)
            out[1] = lse
            _lib.call("spx_label_ce_from_lse", _lib.ptr(logits), logits.stride(0), _lib.ptr(labels), rows,
                      vocab, _lib.dtype_code(logits), int(ignore_index), _lib.ptr(out[1]), _lib.ptr(out[0]),
                      _lib.stream_ptr(logits.device))
        else:
            logits = gemm_nt(x2, weight)
            rows, vocab = logits.shape
            out = torch.empty(2, rows, device=logits.device, dtype=torch.float32)
            _lib.call("spx_label_ce_fwd", _lib.ptr(logits), logits.stride(0), _lib.ptr(labels), rows,
                      vocab, _lib.dtype_code(logits), int(ignore_index), _lib.ptr(out[0]),
                      _lib.ptr(out[1]), None, _lib.stream_ptr(logits.device))
        ctx.save_for_backward(logits, labels, out[1], weight_t)
        ctx.ignore_index = int(ignore_index)
        ctx.mark_non_differentiable(logits)
        ctx.set_materialize_grads(False)  # no [rows, V] zeros for the logits, which carry no gradient
        return out[0], logits

    @staticmethod
    def backward(ctx, grad_rows, _grad_logits):
        from .gemm import gemm_nt

        if grad_rows is None:
            return (None,) * 6

        logits, labels, lse, weight_t = ctx.saved_tensors
        rows, vocab = logits.shape
        g = grad_rows.to(torch.float32).contiguous()
        row_map, count = _packed_row_map(g, labels, ctx.ignore_index)
        packed = torch.empty(rows, vocab, device=logits.device, dtype=logits.dtype)
        _lib.call("spx_label_ce_bwd_packed", _lib.ptr(logits), logits.stride(0), _lib.ptr(labels),
                  _lib.ptr(lse), _lib.ptr(g), rows, vocab, _lib.dtype_code(logits), ctx.ignore_index,
                  _lib.ptr(row_map), _lib.ptr(packed), packed.stride(0),
                  _lib.stream_ptr(logits.device))
        dx_packed = gemm_nt(packed, weight_t, m_live=count, split=True)
        return _unpack_rows(dx_packed, row_map, rows), None, None, None, None, None


# Whether the frozen-head cross-entropy takes its row statistics from the head product's epilogue
# (spx_gemm_bf16_nt_stats, log-sum-exp only) instead of a streaming pass over the logits
# (spx_label_ce_fwd).  Measured at the MTP head shape (32760 rows x 2048 -> 151936, 70 % live rows):
# product + epilogue statistics + their reduction + one element per row 16.7 ms, product 15.9 ms +
# streaming pass 1.25 ms = 17.2 ms; the iteration 199.1 against 200.4 ms.  (With the arg-max computed
# too and a reduction of one thread per row the epilogue form LOST 1 ms per step: two compares per
# element more on every row, with the matrix pipe idle, cost what the streaming pass costs.)
HEAD_CE_EPILOGUE_STATS = True


def head_label_cross_entropy(x: torch.Tensor, weight: torch.Tensor, weight_t: torch.Tensor,
                             labels: torch.Tensor, ignore_index: int = -100,
                             epilogue_stats: bool | None = None):
    """``logits = x @ weight.T`` and ``F.cross_entropy(logits, labels, ignore_index=...,
    reduction="none")`` (models/mtp/core.py:190-216) for a FROZEN ``weight [V, H]`` whose
    transpose ``weight_t [H, V]`` the caller keeps: returns ``(loss [...] f32, logits [..., V])``.
    Gradient flows to ``x`` through the loss only; the returned logits are detached."""
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight_t.dtype != torch.bfloat16:
        raise _lib.SpxError("head_label_cross_entropy takes bf16 operands")
    if weight.requires_grad:
        raise ValueError("head_label_cross_entropy is for a frozen head (no weight gradient is produced)")
    if x.shape[:-1] != labels.shape:
        raise ValueError(f"x {tuple(x.shape)} and labels {tuple(labels.shape)} do not match")
    if weight_t.shape != (weight.shape[1], weight.shape[0]) or not weight_t.is_contiguous():
        raise ValueError("weight_t must be the contiguous transpose of weight")
    x2 = x.reshape(-1, x.shape[-1])
    lab = labels.reshape(-1).to(torch.int64).contiguous()
    if epilogue_stats is None:
        epilogue_stats = HEAD_CE_EPILOGUE_STATS
    loss, logits = _HeadLabelCE.apply(x2, weight, weight_t, lab, ignore_index, bool(epilogue_stats))
    return loss.view(labels.shape), logits.view(*labels.shape, weight.shape[0])


def vocab_gather(full_logits: torch.Tensor, d2t: torch.Tensor) -> torch.Tensor:
    """``full_logits[..., i + d2t[i]]`` on the device: verifier logits over the target
    vocabulary restricted to the draft vocabulary (the gather form of the t2d row-slice,
    model.py:161-169, with the offset table of train/vocab_mapping.py:86-96)."""
    x = _rows_2d(full_logits)
    rows, vt = x.shape
    vd = d2t.numel()
    d2t = d2t.to(device=x.device, dtype=torch.int64).contiguous()
    out = torch.empty(rows, vd, device=x.device, dtype=x.dtype)
    done = 0
    while done < rows:  # the gather grid carries rows in its y dimension
        n = min(rows - done, 65535)
        xs, os_ = x[done:done + n], out[done:done + n]
        _lib.call("spx_vocab_gather", _lib.ptr(xs), x.stride(0), _lib.ptr(d2t), _lib.ptr(os_),
                  out.stride(0), n, vd, vt, _lib.dtype_code(x), _lib.stream_ptr(x.device))
        done += n
    return out.view(*full_logits.shape[:-1], vd)
