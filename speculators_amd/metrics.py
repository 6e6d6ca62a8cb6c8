"""Per-step loss and acceptance metrics on the device.

Drop-in replacements, with identical metric keys and the identical in-place
mutation of ``prev_correct``, for
  * ``compute_metrics`` of EAGLE3 (models/eagle3/metrics.py:51-119) and
  * ``compute_metrics`` of DFlash (models/dflash/metrics.py:20-108).
The row losses and both arg-maxes come out of one pass of the fused loss
kernel; the masked mean, the acceptance chain and the counts are one more
single-workgroup kernel.  Nothing of size ``[T, V]`` is ever created here.
"""

from __future__ import annotations

import numpy as np
import torch

from . import _lib
from . import losses as L


def _as_mask(t: torch.Tensor) -> torch.Tensor:
    """1-D unit-stride view of a ``[1, n]`` mask (its dtype is kept)."""
    t = t.reshape(-1)
    return t if t.stride(0) == 1 else t.contiguous()


class _StepReduce(torch.autograd.Function):
    """(row_loss [n] f32) -> weighted masked mean (0-d); also fills ``out`` (6 floats)
    and updates ``prev_correct`` in place.  d/d row_loss = row_weight.  With ``counts`` (int32
    ``[3]``) the acceptance chain was already done by the loss pass (``losses.StepPass``): only
    the mean is reduced here and the counts are copied into ``out``."""

    @staticmethod
    def forward(ctx, row_loss, am_d, am_t, mask, prev, weight, out, counts=None):
        n = row_loss.numel()
        row_loss = row_loss.reshape(-1).contiguous()
        row_weight = torch.empty(n, device=row_loss.device, dtype=torch.float32)
        if counts is not None:
            _lib.call(
                "spx_ttt_step_mean", _lib.ptr(row_loss), _lib.ptr(mask),
                _lib.kind_code(mask) if mask is not None else 0, n, float(weight), _lib.ptr(counts),
                _lib.ptr(out), _lib.ptr(row_weight), _lib.stream_ptr(row_loss.device),
            )
        else:
            _lib.call(
                "spx_ttt_step_reduce", _lib.ptr(row_loss), _lib.ptr(am_d), _lib.ptr(am_t),
                _lib.ptr(mask), _lib.kind_code(mask) if mask is not None else 0,
                _lib.ptr(prev), _lib.kind_code(prev) if prev is not None else 0,
                n, float(weight), _lib.ptr(out), _lib.ptr(row_weight),
                _lib.stream_ptr(row_loss.device),
            )
        ctx.save_for_backward(row_weight)
        ctx.shape = row_loss.shape
        return out[0].clone()

    @staticmethod
    def backward(ctx, g):
        (row_weight,) = ctx.saved_tensors
        return (row_weight * g).view(ctx.shape), None, None, None, None, None, None, None


class TargetGather:
    """Full-vocabulary verifier logits (``[1, T, Vt]``) with the ``d2t`` offset table, standing
    where ``compute_metrics`` takes the targets.  The first TTT step reads its target rows
    THROUGH the table inside the loss pass (no gather kernel, no ``[T, Vd]`` copy made first) and
    leaves the draft-vocabulary rows in ``compact`` (``[1, T, Vd]``), which the later steps and the
    backward stream."""

    def __init__(self, full_logits: torch.Tensor, d2t: torch.Tensor):
        if full_logits.dim() != 3 or full_logits.shape[0] != 1:
            raise ValueError("verifier logits must be [1, T, Vt] (the packed batch layout)")
        self.full = full_logits
        self.d2t = d2t.to(torch.int64).contiguous()
        self.compact = None

    def materialize(self) -> torch.Tensor:
        if self.compact is None:
            self.compact = L.vocab_gather(self.full, self.d2t)
        return self.compact


class VerifierHead:
    """The frozen verifier head (``verifier_lm_head(verifier_norm(h))``, models/eagle3/core.py:250-253)
    applied lazily, standing where ``compute_metrics`` takes the targets.  A cross-entropy loss needs
    nothing of the target logits but their row arg-max (losses/eager.py ``ce_loss``), and the acceptance
    metrics need the same: with that loss alone the head product is reduced to per-row statistics in its
    own epilogue (``gemm.gemm_nt_stats(store=False)``) and the ``[T, Vd]`` target logits are never
    written or read.  Any other loss gets them the ordinary way (``materialize``)."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor):
        if x.dim() != 3 or x.shape[0] != 1:
            raise ValueError("verifier hidden states must be [1, T, H] (the packed batch layout)")
        self.x, self.weight = x, weight
        self.logits = None

    def materialize(self) -> torch.Tensor:
        from . import gemm

        if self.logits is None:
            self.logits = gemm.gemm_nt(self.x[0], self.weight).view(1, self.x.shape[1], self.weight.shape[0])
        return self.logits

    def stats(self):
        """(lse [T] f32, argmax [T] i32) of the target rows; the rows themselves are not stored.  The
        cross-entropy reads the arg-max only: the log-sum-exp is not computed (zeros stand in)."""
        from . import gemm

        _, _, am = gemm.gemm_nt_stats(self.x[0], self.weight, store=False, want_lse=False)
        return torch.zeros(am.shape, device=am.device, dtype=torch.float32), am


def _step_views(logits, targets, loss_mask, prev_correct, ttt_step):
    """align_for_step (models/eagle3/metrics.py:16-48): views only."""
    n = logits.shape[1] - ttt_step
    return (
        logits[:, :n],
        None if targets is None else targets[:, ttt_step:],
        None if loss_mask is None else loss_mask[:, ttt_step:],
        None if prev_correct is None else prev_correct[:, :n],
    )


class Head:
    """The frozen ``lm_head`` applied lazily: ``compute_metrics`` takes this in place of the logits
    and, when the loss is a single fused HIP reduction, runs head and loss as ONE autograd node (the
    backward then skips the rows the loss mask removes in the head's input-gradient product,
    ``losses.head_fused_rows``); otherwise the logits are made the ordinary way.  Either way
    ``.logits`` holds them afterwards (``[1, T, Vd]``)."""

    def __init__(self, x, weight, weight_t):
        self.x, self.weight, self.weight_t = x, weight, weight_t
        self.logits = None

    def materialize(self):
        from . import gemm

        if self.logits is None:
            self.logits = gemm.linear(self.x, self.weight, self.weight_t)
        return self.logits


def compute_metrics(logits, targets, loss_mask, prev_correct, ttt_step: int,
                    ttt_step_loss_decay: float, loss_config: L.LossConfig | None = None,
                    target_stats_cache: dict | None = None, return_pred: bool = False):
    """EAGLE3 per-step loss + metrics; same contract as models/eagle3/metrics.py:51-119.

    ``prev_correct`` (any mask dtype) is updated in place.  Returns
    ``(loss 0-d, metrics dict of 0-d tensors)``.

    Two optional extras beyond the reference contract: ``target_stats_cache`` (a dict the
    caller keeps across the TTT steps of ONE forward) lets steps >= 1 reuse the verifier
    rows' log-sum-exp / arg-max computed at step 0 (``targets`` is the same tensor at every
    step, only shifted); ``return_pred=True`` also returns the draft arg-max of the aligned
    rows (int32 ``[T - ttt_step]``).
    """
    if loss_config is None:
        loss_config = {"kl_div": (L.kl_div_loss, 1.0)}
    head = None
    if isinstance(logits, Head):
        # one node for head + loss only when the whole loss is one fused reduction
        (name0, (fn0, _w0)), = list(loss_config.items())[:1]
        single = (len(loss_config) == 1 and name0 in L.PRIMITIVE_OP and fn0 is L._HIP_LOSS_FN_MAP.get(name0)
                  and logits.x.requires_grad and not logits.weight.requires_grad
                  and logits.weight_t is not None)
        if single:
            head = logits
            logits = torch.empty(1, head.x.shape[1], 0, device=head.x.device)  # shape carrier only
        else:
            logits = logits.materialize()
    if logits.shape[0] != 1:
        raise ValueError("the packed batch layout has batch size 1 (train/data.py:306-393)")
    gather = None
    if isinstance(targets, TargetGather):
        name0, (fn0, _) = next(iter(loss_config.items()))
        if (targets.compact is None and ttt_step == 0 and name0 in L.PRIMITIVE_OP
                and fn0 is L._HIP_LOSS_FN_MAP.get(name0)):
            gather, targets = targets, targets.full  # read through d2t inside the first loss pass
        else:
            targets = targets.materialize()
    if isinstance(targets, VerifierHead):
        (name0, (fn0, _w0)), = list(loss_config.items())[:1]
        ce_only = (len(loss_config) == 1 and name0 == "ce" and fn0 is L._HIP_LOSS_FN_MAP.get("ce")
                   and target_stats_cache is not None and targets.logits is None)
        if ce_only:
            if "ce" not in target_stats_cache:
                target_stats_cache["ce"] = targets.stats()
            targets = None  # every step reads the statistics; no target row exists
        else:
            targets = targets.materialize()
    s_logits, s_targets, s_mask, s_prev = _step_views(
        logits, targets, loss_mask, prev_correct, ttt_step)
    dev = logits.device
    # gamma ** step evaluated in fp32 like exp_loss_decay on a float tensor
    # (losses/utils.py:51-61)
    weight = float(np.float32(ttt_step_loss_decay) ** np.float32(ttt_step))

    mask1 = None if s_mask is None else _as_mask(s_mask)
    prev1 = None
    if s_prev is not None:
        prev1 = s_prev.reshape(-1)
        if prev1.stride(0) != 1:
            raise ValueError("prev_correct must be contiguous (it is updated in place)")

    total = None
    terms = {}
    multi = len(loss_config) > 1
    first_out = None
    counts = None
    for ti, (name, (fn, w)) in enumerate(loss_config.items()):
        out = torch.empty(6, device=dev, dtype=torch.float32)
        op = L.PRIMITIVE_OP.get(name)
        step = None
        if ti == 0:
            # the first term's row pass also gathers the targets (first step of a TargetGather)
            # and advances the acceptance chain
            counts = torch.zeros(3, device=dev, dtype=torch.int32)
            # (a row the mask removes has weight zero in the masked mean below: the head + loss node may
            # write the logits gradient of the other rows in the same pass)
            step = L.StepPass(d2t=gather.d2t if gather is not None else None, mask=mask1, prev=prev1,
                              counts=counts, grad_in_pass=head is not None and mask1 is not None)
        elif gather is not None:
            s_targets = gather.compact
        if fn is L._HIP_LOSS_FN_MAP.get(name) and op is not None:
            known = None
            if target_stats_cache is not None and op in (L.OP_KL, L.OP_CE) and gather is None:
                full = target_stats_cache.get("kl" if op == L.OP_KL else "ce")
                if full is None and op == L.OP_CE:
                    full = target_stats_cache.get("kl")  # the arg-max is all ce needs
                if full is not None:
                    known = (full[0][ttt_step:], full[1][ttt_step:])
            # the full logits go in with a row count: see _FusedLoss.forward
            if head is not None:
                rows, am_d, am_t, lse_t, head.logits = L.head_fused_rows(
                    op, head.x, head.weight, head.weight_t, s_targets, known, n_rows=s_logits.shape[1],
                    step=step)
            else:
                rows, am_d, am_t, lse_t = L.fused_rows(op, logits, s_targets, known,
                                                       n_rows=s_logits.shape[1], step=step)
            if step is not None and step.gathered is not None:
                gather.compact = step.gathered.view(1, -1, step.gathered.shape[-1])
            if (target_stats_cache is not None and known is None and ttt_step == 0
                    and op in (L.OP_KL, L.OP_CE)):
                target_stats_cache["kl" if op == L.OP_KL else "ce"] = (
                    lse_t.reshape(-1), am_t.reshape(-1))
        else:
            rows = fn(s_logits, s_targets)
            _, am_d, am_t, _ = L.fused_rows(L.OP_CE, s_logits.detach(), s_targets, step=step)
        if ti == 0:
            pred = am_d.reshape(-1)
        # only the first term advances the acceptance chain (inside its row pass)
        term = _StepReduce.apply(rows.reshape(-1), am_d.reshape(-1), am_t.reshape(-1), mask1,
                                 None, weight, out, counts if ti == 0 else None)
        if ti == 0:
            first_out = out
        if multi:
            terms[f"{name}_loss"] = term.detach()
        total = w * term if total is None else total + w * term

    one = torch.ones((), device=dev)
    m = {f"loss_{ttt_step}_sum": total.detach().clone(), f"loss_{ttt_step}_total": one}
    for tname, tval in terms.items():
        m[f"{tname}_{ttt_step}_sum"] = tval
        m[f"{tname}_{ttt_step}_total"] = one.clone()
    m[f"full_acc_{ttt_step}_sum"] = first_out[1]
    m[f"full_acc_{ttt_step}_total"] = first_out[2]
    m[f"cond_acc_{ttt_step}_sum"] = first_out[3]
    m[f"cond_acc_{ttt_step}_total"] = first_out[4]
    if return_pred:
        return total, m, pred
    return total, m


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    """First-index arg-max over the last axis as int64, through the loss kernel's
    arg-max path (pairs every row with itself)."""
    x = L._rows_2d(logits)
    rows, vocab = x.shape
    dev = x.device
    scratch = torch.empty(4, max(rows, 1), device=dev, dtype=torch.float32)
    out = torch.empty(max(rows, 1), device=dev, dtype=torch.int32)
    if rows:
        _lib.call(
            "spx_fused_vocab_loss_fwd", L.OP_CE, _lib.ptr(x), x.stride(0), _lib.ptr(x),
            x.stride(0), rows, vocab, _lib.dtype_code(x), _lib.ptr(scratch[0]),
            _lib.ptr(scratch[1]), _lib.ptr(scratch[2]), _lib.ptr(scratch[3]), _lib.ptr(out),
            None, 0, _lib.stream_ptr(dev),
        )
    return out[:rows].to(torch.int64).view(logits.shape[:-1])


class _BlockReduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, row_loss, am_d, am_t, mask, pos_weight, block_size, out, correct, total):
        n = row_loss.numel()
        row_loss = row_loss.reshape(-1).contiguous()
        row_weight = torch.empty(n, device=row_loss.device, dtype=torch.float32)
        _lib.call(
            "spx_block_reduce", _lib.ptr(row_loss), _lib.ptr(am_d), _lib.ptr(am_t), _lib.ptr(mask),
            _lib.kind_code(mask), _lib.ptr(pos_weight), n, int(block_size), _lib.ptr(out),
            _lib.ptr(correct), _lib.ptr(total), _lib.ptr(row_weight),
            _lib.stream_ptr(row_loss.device),
        )
        ctx.save_for_backward(row_weight)
        ctx.shape = row_loss.shape
        return out[0].clone()

    @staticmethod
    def backward(ctx, g):
        (row_weight,) = ctx.saved_tensors
        return (row_weight * g).view(ctx.shape), None, None, None, None, None, None, None, None


def dflash_loss_decay(pos_idx: torch.Tensor, gamma: float, sample_from_anchor: bool = False):
    """Per-slot weight of losses/utils.py:17-48 (a [block_size]-periodic vector)."""
    pos = pos_idx.to(torch.float32)
    if sample_from_anchor:
        return torch.exp(-pos / gamma)
    w = torch.exp(-(pos - 1.0).clamp_min(0.0) / gamma)
    return torch.where(pos == 0, torch.zeros_like(w), w)


def dpace_loss_decay(row_ce: torch.Tensor, loss_mask: torch.Tensor, block_size: int,
                     dpace_alpha: float) -> torch.Tensor:
    """D-PACE weight from masked CE row losses (losses/utils.py:64-112); no gradient."""
    with torch.no_grad():
        n = row_ce.numel()
        if n % block_size != 0:
            raise ValueError(f"q.shape[1] ({n}) must be divisible by block_size ({block_size})")
        conf = torch.exp(-row_ce.float()).reshape(n // block_size, block_size)
        m = loss_mask.reshape(n // block_size, block_size).to(conf.dtype)
        s = torch.where(m > 0, (1.0 - dpace_alpha) * conf + dpace_alpha, torch.ones_like(conf))
        prefix = torch.cumprod(s, dim=-1) * m
        suffix = torch.flip(torch.cumsum(torch.flip(prefix, dims=[-1]), dim=-1), dims=[-1])
        return (suffix * m).reshape(-1)


def dflash_compute_metrics(logits, targets, loss_mask, block_size: int = 1, gamma: float = 4.0,
                           loss_config: L.LossConfig | None = None,
                           per_position_loss_weight: str = "fixed-exp-decay",
                           dpace_alpha: float = 0.5, sample_from_anchor: bool = False):
    """DFlash loss + per-slot accuracy + EAL; contract of models/dflash/metrics.py:20-108.
    ``logits`` may be a ``Head`` (see ``compute_metrics``)."""
    if loss_config is None:
        loss_config = {"kl_div": (L.kl_div_loss, 1.0)}
    head = None
    if isinstance(logits, Head):
        (name0, (fn0, _w0)), = list(loss_config.items())[:1]
        if (len(loss_config) == 1 and name0 in L.PRIMITIVE_OP and fn0 is L._HIP_LOSS_FN_MAP.get(name0)
                and logits.x.requires_grad and not logits.weight.requires_grad
                and logits.weight_t is not None):
            head = logits
            logits = torch.empty(1, head.x.shape[1], 0, device=head.x.device)  # shape carrier only
        else:
            logits = logits.materialize()
    dev = logits.device
    n = logits.shape[1]
    mask1 = _as_mask(loss_mask)
    pos = torch.arange(n, device=dev) % block_size
    total_loss = None
    terms = {}
    multi = len(loss_config) > 1
    correct = total = None
    for ti, (name, (fn, w)) in enumerate(loss_config.items()):
        op = L.PRIMITIVE_OP.get(name)
        if head is not None:
            rows, am_d, am_t, _, head.logits = L.head_fused_rows(
                op, head.x, head.weight, head.weight_t, targets)
        elif fn is L._HIP_LOSS_FN_MAP.get(name) and op is not None:
            rows, am_d, am_t, _ = L.fused_rows(op, logits, targets)
        else:
            rows = fn(logits, targets)
            _, am_d, am_t, _ = L.fused_rows(L.OP_CE, logits.detach(), targets)
        if per_position_loss_weight == "dpace":
            masked = rows.detach().reshape(-1) * mask1.to(torch.float32)
            pw = dpace_loss_decay(masked, mask1, block_size, dpace_alpha)
        else:
            pw = dflash_loss_decay(pos, gamma, sample_from_anchor)
        out = torch.empty(2, device=dev, dtype=torch.float32)
        c = torch.empty(block_size, device=dev, dtype=torch.float32)
        t = torch.empty(block_size, device=dev, dtype=torch.float32)
        term = _BlockReduce.apply(rows.reshape(-1), am_d.reshape(-1), am_t.reshape(-1), mask1,
                                  pw.contiguous(), block_size, out, c, t)
        if ti == 0:
            correct, total = c, t
        if multi:
            terms[f"{name}_loss"] = term.detach()
        total_loss = w * term if total_loss is None else total_loss + w * term

    one = torch.ones((), device=dev)
    m = {"loss_sum": total_loss.detach().clone(), "loss_total": one}
    for tname, tval in terms.items():
        m[f"{tname}_sum"] = tval
        m[f"{tname}_total"] = one.clone()
    first = 0 if sample_from_anchor else 1
    m["full_acc_sum"] = correct[first:].sum()
    m["full_acc_total"] = total[first:].sum()
    acc = correct[first:] / total[first:].clamp(min=1.0)
    m["eal_sum"] = torch.cumprod(acc, dim=0).sum() if acc.numel() else torch.zeros((), device=dev)
    m["eal_total"] = one.clone()
    for s in range(first, block_size):
        m[f"position_{s}_acc_sum"] = correct[s]
        m[f"position_{s}_acc_total"] = total[s]
    return total_loss, m
