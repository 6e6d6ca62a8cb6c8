"""CPU restatement of the batch layout the draft models are trained on.

TEST INFRASTRUCTURE ONLY: nothing under ``speculators_amd`` may import this.

Follows:
  * the layer split of a hidden-state file      train/data.py:293-303
    (``hs_{idx}.safetensors`` = {"hidden_states": [seq, layers + 1, H], "token_ids": [seq]},
    hs_connectors/src/hs_connectors/transfer.py:136-155)
  * ``BaseDataset.__getitem__``                  train/data.py:110-149 (lengths, position_ids)
  * ``shift_batch``                              models/eagle3/data.py:8-44
  * ``shift_batch_mtp``                          models/mtp/data.py:6-18
  * ``create_empty_sample``                      train/data.py:25-48
  * ``CollateFn.__call__``                       train/data.py:323-393

Pinned by the reference's own known-answer tests, restated as data in
tests/test_oracle_data.py: tests/unit/train/test_data.py:16-51 (shift), :54-131 (two
documents packed into 10 rows), :134-152 (dtype cast), :155-200 (truncation, document
ids [0]*5 + [1]*6).
"""

from __future__ import annotations

import torch


def sample_from_file(loaded: dict, loss_mask: torch.Tensor) -> dict:
    """One dataset item from the tensors of a hidden-state file: all layers but the last,
    flattened, feed the draft model; the last layer is the verifier's final state."""
    hs = loaded["hidden_states"]
    seq = hs.shape[0]
    return {
        "hidden_states": hs[:, :-1].flatten(1),
        "input_ids": loaded["token_ids"],
        "verifier_last_hidden_states": hs[:, -1],
        "loss_mask": loss_mask,
        "lengths": torch.tensor([seq], dtype=torch.long),
        "position_ids": torch.arange(seq, dtype=torch.long),
    }


def empty_sample(hidden_size: int, num_target_layers: int = 3, dtype=torch.bfloat16) -> dict:
    return {
        "hidden_states": torch.empty(0, num_target_layers * hidden_size, dtype=dtype),
        "input_ids": torch.empty(0, dtype=torch.long),
        "verifier_last_hidden_states": torch.empty(0, hidden_size, dtype=dtype),
        "loss_mask": torch.empty(0, dtype=torch.bool),
        "lengths": torch.tensor([0], dtype=torch.long),
        "position_ids": torch.arange(0, dtype=torch.long),
    }


def shift_eagle3(sample: dict) -> dict:
    """Aligns (x[i+1], g[i], y[i+1], mask[i+1]): one row shorter, positions start at 1."""
    return {
        "input_ids": sample["input_ids"][1:],
        "hidden_states": sample["hidden_states"][:-1],
        "verifier_last_hidden_states": sample["verifier_last_hidden_states"][1:],
        "loss_mask": sample["loss_mask"][1:],
        "lengths": (sample["lengths"] - 1).clamp(min=0),
        "position_ids": sample["position_ids"][1:],
    }


def shift_mtp(sample: dict) -> dict:
    """No token shift: the verifier's final state becomes ``hidden_states``."""
    return {
        "input_ids": sample["input_ids"],
        "hidden_states": sample["verifier_last_hidden_states"],
        "loss_mask": sample["loss_mask"],
        "lengths": sample["lengths"],
        "position_ids": sample["position_ids"],
    }


def kept_lengths(lengths, max_len: int) -> list[int]:
    """Document lengths that fit: the document that reaches ``max_len`` is cut there and
    every later one is dropped."""
    kept, used = [], 0
    for n in (int(x) for x in lengths):
        if used + n >= max_len:
            kept.append(max_len - used)
            break
        kept.append(n)
        used += n
    return kept


def collate(samples, max_len: int, hidden_size: int, num_target_layers: int = 3,
            dtype=torch.bfloat16, preprocess=None) -> dict:
    """``[1, max_len, ...]`` per key: the samples' rows back to back, cut at ``max_len``,
    zero padded; hidden-state keys cast to ``dtype``; ``document_ids`` = index of the
    sample each row came from, -1 on padding."""
    items = [preprocess(s) if preprocess else s for s in samples if s is not None]
    if not items:
        e = empty_sample(hidden_size, num_target_layers, dtype)
        items = [preprocess(e) if preprocess else e]
    out = {}
    for key in items[0]:
        if key == "lengths":
            continue
        joined = torch.cat([it[key] for it in items], dim=0)[:max_len]
        want = dtype if "hidden_states" in key else joined.dtype
        full = torch.zeros((max_len, *joined.shape[1:]), dtype=want)
        full[:joined.shape[0]] = joined.to(want)
        out[key] = full.unsqueeze(0)
    kept = kept_lengths(torch.cat([it["lengths"] for it in items]), max_len)
    doc = torch.full((max_len,), -1, dtype=torch.long)
    at = 0
    for d, n in enumerate(kept):
        doc[at:at + n] = d
        at += n
    out["document_ids"] = doc.unsqueeze(0)
    return out
