"""Draft <-> target vocabulary tables (oracle, CPU, integer-exact).

Pinned by the closed form of train/vocab_mapping.py:86-96 -- ``d2t[i] = sel[i]
- i`` with ``sel`` ascending and ``t2d[sel] = True``, hence ``nonzero(t2d) ==
arange(Vd) + d2t`` -- and by the linear-algebra identity ``(W h)[t2d] ==
W[t2d] h`` that makes a gather of full-vocab verifier logits equal to the
reference's row-sliced verifier head (model.py:161-169).
"""

from __future__ import annotations

import torch


def build_vocab_mappings(selected_token_ids, target_vocab_size: int):
    """(d2t int64 ``[Vd]`` offsets, t2d bool ``[Vt]``) from a set of target ids;
    train/vocab_mapping.py:64-96 (the part after the frequency ranking)."""
    sel = torch.as_tensor(sorted(int(x) for x in selected_token_ids), dtype=torch.long)
    d2t = sel - torch.arange(sel.numel(), dtype=torch.long)
    t2d = torch.zeros(target_vocab_size, dtype=torch.bool)
    t2d[sel] = True
    return d2t, t2d


def validate_vocab_mappings(t2d, d2t, draft_vocab_size: int, target_vocab_size: int):
    """The shape / population rules of model.py:104-119."""
    if t2d.shape[0] != target_vocab_size:
        raise ValueError("t2d length must equal the target vocabulary size")
    if int(t2d.sum(dtype=torch.long)) != draft_vocab_size:
        raise ValueError("t2d must select exactly draft_vocab_size ids")
    if d2t.shape[0] != draft_vocab_size:
        raise ValueError("d2t length must equal the draft vocabulary size")


def gather_targets(full_logits: torch.Tensor, d2t: torch.Tensor) -> torch.Tensor:
    """``full_logits[..., i + d2t[i]]`` -- verifier logits restricted to the
    draft vocabulary, equal to ``verifier_lm_head`` built from ``W[t2d]``
    (model.py:161-169)."""
    idx = torch.arange(d2t.numel(), dtype=torch.long) + d2t.long()
    return full_logits.index_select(-1, idx)


def build_vocab_mappings_from_distribution(token_freq: dict, draft_vocab_size: int, target_vocab_size: int):
    """train/vocab_mapping.py:64-96 in full: rank ids by (count descending, id ascending), keep
    the first ``draft_vocab_size``; if fewer were seen, walk ids 0, 1, 2, ... below
    ``draft_vocab_size`` and add the ones not yet chosen."""
    ranked = sorted(token_freq.items(), key=lambda kv: (-kv[1], kv[0]))
    chosen = [tid for tid, _ in ranked[:draft_vocab_size]]
    have = set(chosen)
    tid = 0
    while len(chosen) < draft_vocab_size and tid < draft_vocab_size:
        if tid not in have:
            chosen.append(tid)
            have.add(tid)
        tid += 1
    return build_vocab_mappings(chosen, target_vocab_size)
