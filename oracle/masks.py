"""Dense boolean masks of the two draft-attention patterns (oracle, CPU).

Pinned by: the literal 6x6 matrix and the ``kv % N == q`` diagonal rule of the
reference's tests (tests/unit/models/test_eagle3_attention.py:14-65), the
dense-extension known answer (:122-152), and for DFlash the pure-Python brute
force of tests/integration/models/test_dflash_vllm_parity.py:29-61 restated in
``tests/test_oracle_masks.py``.
"""

from __future__ import annotations

import numpy as np
import torch


def ttt_mask_dense(
    document_ids: torch.Tensor,
    total_seq_len: int,
    ttt_step: int,
    sliding_window: int | None = None,
) -> torch.Tensor:
    """Mask seen by the queries of TTT step ``ttt_step`` (0-based).

    Follows ``create_combined_mask_mod`` (models/eagle3/attention.py:11-34)
    evaluated over Q = T rows and KV = (ttt_step + 1) * T columns, which is
    also what ``extend_dense_mask_for_draft_tokens`` (:115-132) builds step by
    step:  (q >= kv  and  [kv > q - W]  and  doc[q] != -1  and
    doc[q] == doc[kv % T])  or  (kv % T == q).

    Returns bool ``[T, (ttt_step + 1) * T]``.
    """
    doc = np.asarray(document_ids.cpu().numpy()).reshape(-1).astype(np.int64)
    t = int(total_seq_len)
    assert doc.shape[0] == t
    q = np.arange(t, dtype=np.int64)[:, None]
    kv = np.arange((ttt_step + 1) * t, dtype=np.int64)[None, :]
    causal = q >= kv
    if sliding_window is not None:
        causal &= kv > q - int(sliding_window)
    same_doc = (doc[q] != -1) & (doc[q] == doc[kv % t])
    diagonal = (kv % t) == q
    return torch.from_numpy((causal & same_doc) | diagonal)


def ttt_row_lo(
    document_ids: torch.Tensor, sliding_window: int | None = None
) -> torch.Tensor:
    """Lowest visible context key of every query row, as the interval form
    ``row_lo[i] <= c <= i`` of the step-0 part of ``ttt_mask_dense``.

    Derived (not in the reference): for run-contiguous ``document_ids`` -- what
    ``CollateFn`` produces (train/data.py:323-393) -- the predicate above
    restricted to kv < T is an interval; padding rows (doc == -1) see only
    themselves.  Checked against ``ttt_mask_dense`` by brute force in the tests.
    """
    doc = np.asarray(document_ids.cpu().numpy()).reshape(-1).astype(np.int64)
    t = doc.shape[0]
    lo = np.zeros(t, dtype=np.int32)
    start = 0
    for i in range(t):
        if i > 0 and doc[i] != doc[i - 1]:
            start = i
        if doc[i] == -1:
            lo[i] = i
        else:
            lo[i] = start
            if sliding_window is not None:
                lo[i] = max(lo[i], i - int(sliding_window) + 1)
    return torch.from_numpy(lo)


def dflash_mask_dense(
    document_ids: torch.Tensor,
    total_seq_len: int,
    anchor_positions: torch.Tensor,
    block_size: int,
    sliding_window: int | None = None,
    sliding_window_non_causal: bool = False,
) -> torch.Tensor:
    """Anchored-block mask, bool ``[A*bs, T + A*bs]``.

    Follows ``create_anchor_block_mask_mod`` (models/dflash/attention.py:7-100):
    a query of block j (anchor a_j) sees base keys kv < T with
    doc[kv] == doc[a_j] != -1, kv < a_j and (window) kv >= a_j - W; and the
    synthetic keys of its own block, all of them when the layer is full
    attention or ``sliding_window_non_causal``, otherwise only kv <= q + T.
    """
    doc = np.asarray(document_ids.cpu().numpy()).reshape(-1).astype(np.int64)
    t = int(total_seq_len)
    anchors = np.asarray(anchor_positions.cpu().numpy()).reshape(-1).astype(np.int64)
    bs = int(block_size)
    q_len = anchors.shape[0] * bs
    non_causal = sliding_window is None or sliding_window_non_causal

    q = np.arange(q_len, dtype=np.int64)[:, None]
    kv = np.arange(t + q_len, dtype=np.int64)[None, :]
    q_anchor = np.repeat(anchors, bs)[:, None]
    q_doc = doc[q_anchor]
    kv_base = kv % t
    base = (kv < t) & (q_doc == doc[kv_base]) & (q_doc != -1) & (kv_base < q_anchor)
    if sliding_window is not None:
        base &= kv_base >= q_anchor - int(sliding_window)
    block = (kv >= t) & ((q // bs) == ((kv - t) // bs))
    if not non_causal:
        block &= kv <= q + t
    return torch.from_numpy(base | block)


def dflash_row_range(
    document_ids: torch.Tensor,
    anchor_positions: torch.Tensor,
    block_size: int,
    sliding_window: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Interval form ``lo[r] <= c < hi[r]`` of the base-key part of
    ``dflash_mask_dense`` for run-contiguous ``document_ids`` (derived; checked
    against the dense mask by brute force in the tests)."""
    doc = np.asarray(document_ids.cpu().numpy()).reshape(-1).astype(np.int64)
    t = doc.shape[0]
    run_start = np.zeros(t, dtype=np.int64)
    for i in range(1, t):
        run_start[i] = run_start[i - 1] if doc[i] == doc[i - 1] else i
    anchors = np.asarray(anchor_positions.cpu().numpy()).reshape(-1).astype(np.int64)
    lo = np.zeros(anchors.shape[0], dtype=np.int32)
    hi = np.zeros(anchors.shape[0], dtype=np.int32)
    for j, a in enumerate(anchors):
        if doc[a] == -1:
            lo[j] = hi[j] = 0
            continue
        lo[j] = run_start[a]
        if sliding_window is not None:
            lo[j] = max(lo[j], a - int(sliding_window))
        hi[j] = a
        if hi[j] < lo[j]:
            hi[j] = lo[j]
    return (
        torch.from_numpy(np.repeat(lo, block_size)),
        torch.from_numpy(np.repeat(hi, block_size)),
    )
