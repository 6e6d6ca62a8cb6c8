"""Step alignment, acceptance counts and per-step metric dictionaries
(oracle, CPU).

Pinned by the hand-worked two-step ``prev_correct`` chain with its four
expected counts (tests/unit/models/test_metrics.py:326-370), the per-position
count cases of tests/unit/models/test_dflash_metrics.py:25-161, and brute force
on tiny inputs (tests/test_oracle_metrics.py).
"""

from __future__ import annotations

from functools import partial

import torch

from . import losses as L


def align_for_step(logits, targets, loss_mask, prev_correct, ttt_step: int):
    """Views for TTT step k: logits rows [0, T-k), targets / loss_mask rows
    [k, T), prev_correct rows [0, T-k); models/eagle3/metrics.py:16-48."""
    t = logits.shape[1]
    n = t - ttt_step
    return (
        logits[:, :n],
        targets[:, ttt_step:],
        None if loss_mask is None else loss_mask[:, ttt_step:],
        None if prev_correct is None else prev_correct[:, :n],
    )


def accuracy_single_step(pred_ids, target_ids, loss_mask, prev_correct):
    """(full_correct, full_total, cond_correct, cond_total) as fp32 0-d tensors;
    models/metrics.py:6-36.  ``prev_correct`` (a view) is AND-ed in place with
    this step's match, ``cond_total`` is its sum BEFORE the update, and the
    AND-ed tensor -- not the raw match -- is what gets counted under the mask."""
    match = pred_ids == target_ids
    if prev_correct is not None:
        cond_total = prev_correct.sum().float()
        merged = prev_correct.to(torch.bool) & match
        prev_correct.copy_(merged.to(prev_correct.dtype))
        counted = merged
    else:
        cond_total = torch.tensor(float(match.numel()))
        counted = match
    if loss_mask is not None:
        counted = counted[loss_mask.to(torch.bool)]
    correct = counted.float().sum()
    total = torch.tensor(float(counted.numel()))
    return correct, total, correct.clone(), cond_total


def accuracy_multi_step(pred_ids, target_ids, loss_mask, pos_idx, num_pos: int):
    """Per-slot (correct, total) fp32 ``[num_pos]`` over masked rows;
    models/metrics.py:39-69."""
    keep = loss_mask.to(torch.bool).reshape(-1)
    match = (pred_ids == target_ids).reshape(-1)[keep]
    pos = pos_idx.reshape(-1)[keep].long()
    correct = torch.zeros(num_pos).index_add_(0, pos, match.float())
    total = torch.zeros(num_pos).index_add_(0, pos, torch.ones_like(match, dtype=torch.float))
    return correct, total


def eagle3_compute_metrics(logits, targets, loss_mask, prev_correct, ttt_step: int,
                           ttt_step_loss_decay: float, loss_config=None):
    """One TTT step's loss and metric dict; models/eagle3/metrics.py:51-119."""
    if loss_config is None:
        loss_config = L.resolve_loss_config("kl_div")
    s_logits, s_targets, s_mask, s_prev = align_for_step(
        logits, targets, loss_mask, prev_correct, ttt_step
    )
    n = s_logits.shape[1]
    if s_mask is None:
        s_mask = torch.ones(1, n, dtype=torch.bool)
    pos_idx = torch.full((1, n), ttt_step, dtype=torch.long)
    loss, terms = L.compound_loss(
        s_logits, s_targets, s_mask, pos_idx, loss_config,
        decay_fn=partial(L.exp_loss_decay, gamma=ttt_step_loss_decay),
    )
    pred = s_logits.argmax(-1)
    tgt = s_targets.argmax(-1)
    fc, ft, cc, ct = accuracy_single_step(pred, tgt, s_mask, s_prev)
    one = torch.tensor(1.0)
    m = {f"loss_{ttt_step}_sum": loss.detach().clone(), f"loss_{ttt_step}_total": one}
    for name, val in terms.items():
        m[f"{name}_{ttt_step}_sum"] = val
        m[f"{name}_{ttt_step}_total"] = one.clone()
    m[f"full_acc_{ttt_step}_sum"] = fc
    m[f"full_acc_{ttt_step}_total"] = ft
    m[f"cond_acc_{ttt_step}_sum"] = cc
    m[f"cond_acc_{ttt_step}_total"] = ct
    return loss, m


def dflash_compute_metrics(logits, targets, loss_mask, block_size: int = 1,
                           gamma: float = 4.0, loss_config=None,
                           per_position_loss_weight: str = "fixed-exp-decay",
                           dpace_alpha: float = 0.5, sample_from_anchor: bool = False):
    """DFlash loss, per-slot accuracy and expected accepted length;
    models/dflash/metrics.py:20-108."""
    if loss_config is None:
        loss_config = L.resolve_loss_config("kl_div")
    n = logits.shape[1]
    pos_idx = (torch.arange(n) % block_size).unsqueeze(0)
    if per_position_loss_weight == "dpace":
        decay = partial(L.dpace_loss_decay, loss_mask=loss_mask,
                        block_size=block_size, dpace_alpha=dpace_alpha)
    else:
        decay = partial(L.dflash_loss_decay, gamma=gamma,
                        sample_from_anchor=sample_from_anchor)
    loss, terms = L.compound_loss(logits, targets, loss_mask, pos_idx, loss_config, decay)
    correct, total = accuracy_multi_step(
        logits.argmax(-1), targets.argmax(-1), loss_mask, pos_idx, block_size
    )
    one = torch.tensor(1.0)
    m = {"loss_sum": loss.detach().clone(), "loss_total": one}
    for name, val in terms.items():
        m[f"{name}_sum"] = val
        m[f"{name}_total"] = one.clone()
    first = 0 if sample_from_anchor else 1
    m["full_acc_sum"] = correct[first:].sum()
    m["full_acc_total"] = total[first:].sum()
    eal = torch.zeros(())
    run = torch.ones(())
    for s in range(first, block_size):
        m[f"position_{s}_acc_sum"] = correct[s]
        m[f"position_{s}_acc_total"] = total[s]
        run = run * (correct[s] / total[s].clamp(min=1.0))
        eal = eal + run
    m["eal_sum"] = eal
    m["eal_total"] = one.clone()
    return loss, m
