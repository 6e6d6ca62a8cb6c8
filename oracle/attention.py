"""Dense masked attention (oracle, CPU).

Textbook ``softmax(scale * Q K^T + mask) V`` with fp32 scores, GQA by
repeating each K/V head over its query group -- the arithmetic that both torch
``flex_attention`` with a BlockMask (call site models/attention.py:20-66) and
the HF eager path compute.  Pinned by agreement with the library routine
``torch.nn.functional.scaled_dot_product_attention`` under a dense bool mask
(tests/test_oracle_attention.py) and by hand-sized brute force.
"""

from __future__ import annotations

import torch


def dense_attention(
    q: torch.Tensor,  # [B, Hq, Q, D]
    k: torch.Tensor,  # [B, Hkv, KV, D]
    v: torch.Tensor,  # [B, Hkv, KV, D]
    mask: torch.Tensor,  # bool [Q, KV], True = attend
    scaling: float | None = None,
) -> torch.Tensor:
    """Returns ``[B, Q, Hq, D]`` (the layout ``flex_attention_forward`` hands
    back, models/attention.py:64-66) in q's dtype.  Fully masked rows give 0,
    as flex_attention does."""
    b, hq, ql, d = q.shape
    hkv = k.shape[1]
    group = hq // hkv
    scale = d**-0.5 if scaling is None else scaling
    kk = k.repeat_interleave(group, dim=1)
    vv = v.repeat_interleave(group, dim=1)
    s = torch.matmul(q.float(), kk.float().transpose(-1, -2)) * scale
    s = s.masked_fill(~mask[None, None], float("-inf"))
    row_max = s.amax(dim=-1, keepdim=True)
    row_max = torch.where(torch.isinf(row_max), torch.zeros_like(row_max), row_max)
    p = torch.exp(s - row_max)
    denom = p.sum(dim=-1, keepdim=True)
    p = torch.where(denom > 0, p / denom.clamp_min(1e-38), torch.zeros_like(p))
    out = torch.matmul(p, vv.float())
    return out.to(q.dtype).transpose(1, 2).contiguous()
