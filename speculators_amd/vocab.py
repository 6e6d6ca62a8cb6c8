"""Draft vocabulary selection: which target-vocabulary ids the draft predicts.

Host-side counterpart of train/vocab_mapping.py:17-96.  The tables it returns are the
ones ``load_vocab_mappings`` installs and the kernels consume: ``d2t`` (int64 ``[Vd]``
OFFSETS, ``target_id = i + d2t[i]``, ascending) and ``t2d`` (bool ``[Vt]`` with exactly
``Vd`` ones).  Everything is tensor arithmetic (``bincount`` / stable sort), so it runs
on the device the token ids live on; it is set-up work, done once per run.
"""

from __future__ import annotations

import torch


def count_token_frequencies(samples, target_vocab_size: int, device=None) -> torch.Tensor:
    """int64 ``[Vt]`` counts of the tokens under the loss mask, over an iterable of
    ``{"input_ids", "loss_mask"}`` items (what ``save_token_frequency_distribution``,
    train/vocab_mapping.py:17-46, stores as a dict of the non-zero entries)."""
    counts = torch.zeros(target_vocab_size, dtype=torch.int64, device=device)
    for item in samples:
        ids = torch.as_tensor(item["input_ids"], device=counts.device).reshape(-1)
        keep = torch.as_tensor(item["loss_mask"], device=counts.device).reshape(-1).to(torch.bool)
        ids = ids[keep].to(torch.int64)
        if ids.numel() and (int(ids.min()) < 0 or int(ids.max()) >= target_vocab_size):
            raise ValueError(f"token id outside [0, {target_vocab_size})")
        counts += torch.bincount(ids, minlength=target_vocab_size)
    return counts


def build_vocab_mappings_from_distribution(token_freq, draft_vocab_size: int, target_vocab_size: int):
    """``(d2t, t2d)`` from token frequencies (train/vocab_mapping.py:64-96): the
    ``draft_vocab_size`` most frequent ids, ties broken towards the smaller id; when fewer
    ids were seen, the smallest unseen ids fill up.  ``token_freq``: the reference's
    ``{token_id: count}`` dict, or a count tensor ``[Vt]`` (ids with count 0 are unseen)."""
    if draft_vocab_size > target_vocab_size:
        raise ValueError("draft_vocab_size exceeds target_vocab_size")
    if isinstance(token_freq, dict):
        seen_ids = torch.tensor(sorted(token_freq), dtype=torch.int64)
        if seen_ids.numel() and (int(seen_ids[0]) < 0 or int(seen_ids[-1]) >= target_vocab_size):
            raise ValueError(f"token id outside [0, {target_vocab_size})")
        freq = torch.tensor([token_freq[int(i)] for i in seen_ids], dtype=torch.int64)
    else:
        counts = torch.as_tensor(token_freq).reshape(-1).to(torch.int64)
        if counts.numel() != target_vocab_size:
            raise ValueError("count tensor must have target_vocab_size entries")
        seen_ids = torch.nonzero(counts, as_tuple=False).reshape(-1)
        freq = counts[seen_ids]
    device = seen_ids.device
    # seen_ids is ascending: a stable descending sort on the count keeps smaller ids first in a tie
    order = torch.sort(freq, descending=True, stable=True).indices
    selected = seen_ids[order[:draft_vocab_size]]
    t2d = torch.zeros(target_vocab_size, dtype=torch.bool, device=device)
    t2d[selected] = True
    missing = draft_vocab_size - selected.numel()
    if missing > 0:
        # the smallest ids below draft_vocab_size that are not selected yet
        free = torch.nonzero(~t2d[:draft_vocab_size], as_tuple=False).reshape(-1)[:missing]
        t2d[free] = True
    selected = torch.nonzero(t2d, as_tuple=False).reshape(-1)
    d2t = selected - torch.arange(draft_vocab_size, dtype=torch.int64, device=device)
    return d2t, t2d
