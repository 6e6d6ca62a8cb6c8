"""Per-row draft/target losses, position weights and the masked reduction
(oracle, CPU, fp32).

q = softmax(logits) is the draft distribution, p = softmax(targets) the
verifier's.  Row formulas follow losses/eager.py:11-213; the closed-form
gradients used by ``row_loss_grad`` follow the table at losses/fused.py:11-18
and the backward kernel at losses/fused.py:177-235.

Pinned by the identities the reference tests assert
(tests/unit/models/test_metrics.py:44-319, 373-439): KL(x,x)=0 and >=0,
RKL(a,b)=KL(b,a), JSD symmetric / <= log 2 / manual formula, TV = L1/2 in
[0,1], NLA = -log(1-TV) with the 1e-5 clamp and -> CE at a point mass,
LK-hybrid eta=0 -> KL and eta->inf -> TV with a detached blend weight, the
masked-mean and gamma**step rules; by the library routines
``F.kl_div`` / ``F.cross_entropy``; and by autograd == closed-form gradient.
``dpace_loss_decay`` (no reference test): per-element float64 double loop over random masks.
"""

from __future__ import annotations

import math
from collections.abc import Callable

import torch

LOSS_NAMES = ("kl_div", "rkl", "jsd", "ce", "tv", "nla", "lk_hybrid")
_NLA_FLOOR = 1e-5  # losses/eager.py:8
_REDUCTION_EPS = 1e-5  # losses/utils.py:10


def _logp(x: torch.Tensor) -> torch.Tensor:
    return torch.log_softmax(x.float(), dim=-1)


def kl_div(logits, targets):
    """sum_v p (log p - log q); losses/eager.py:11-31."""
    lq, lp = _logp(logits), _logp(targets)
    p = lp.exp()
    return torch.where(p > 0, p * (lp - lq), torch.zeros_like(p)).sum(-1)


def rkl(logits, targets):
    """sum_v q (log q - log p); losses/eager.py:34-55."""
    lq, lp = _logp(logits), _logp(targets)
    q = lq.exp()
    return torch.where(q > 0, q * (lq - lp), torch.zeros_like(q)).sum(-1)


def _log_mix(lq, lp):
    return torch.logaddexp(lq, lp) - math.log(2.0)


def jsd(logits, targets):
    """(KL(p||m) + KL(q||m)) / 2 with m = (p+q)/2 in log space;
    losses/eager.py:58-95."""
    lq, lp = _logp(logits), _logp(targets)
    lm = _log_mix(lq, lp)
    q, p = lq.exp(), lp.exp()
    return 0.5 * ((p * (lp - lm)).sum(-1) + (q * (lq - lm)).sum(-1))


def ce(logits, targets):
    """lse(logits) - logits[argmax targets], first index on ties;
    losses/eager.py:98-121.  (The reference runs this one in the logits' dtype;
    the oracle and the fused kernels run it in fp32, as losses/fused.py does.)"""
    lq = _logp(logits)
    idx = torch.argmax(targets, dim=-1, keepdim=True)
    return -lq.gather(-1, idx).squeeze(-1)


def tv(logits, targets):
    """1 - sum_v min(p, q); losses/eager.py:124-147."""
    q, p = _logp(logits).exp(), _logp(targets).exp()
    return 1.0 - torch.minimum(q, p).sum(-1)


def nla(logits, targets):
    """-log(max(overlap, 1e-5)); losses/eager.py:150-177."""
    overlap = 1.0 - tv(logits, targets)
    return -torch.log(overlap.clamp_min(_NLA_FLOOR))


def lk_hybrid(logits, targets, eta: float = 3.0):
    """lam*KL + (1-lam)*TV, lam = exp(-eta*stopgrad(overlap));
    losses/eager.py:180-213."""
    t = tv(logits, targets)
    lam = torch.exp(-eta * (1.0 - t).detach())
    return lam * kl_div(logits, targets) + (1.0 - lam) * t


LOSS_FNS: dict[str, Callable] = {
    "kl_div": kl_div,
    "rkl": rkl,
    "jsd": jsd,
    "ce": ce,
    "tv": tv,
    "nla": nla,
    "lk_hybrid": lk_hybrid,
}


def row_loss_grad(name: str, logits, targets) -> torch.Tensor:
    """d(row loss)/d(logits) in closed form (targets constant), fp32.

    kl_div: q - p;  rkl: q (log q - log p - L);  jsd: q/2 (log q - log m -
    KL(q||m));  ce: q - onehot(argmax p);  tv: -q (1[q <= p] - s), s = sum of
    q where q <= p  (losses/fused.py:11-18, 221-234)."""
    lq, lp = _logp(logits), _logp(targets)
    q, p = lq.exp(), lp.exp()
    if name == "kl_div":
        return q - p
    if name == "rkl":
        big_l = (q * (lq - lp)).sum(-1, keepdim=True)
        return q * (lq - lp - big_l)
    if name == "jsd":
        lm = _log_mix(lq, lp)
        kl_qm = (q * (lq - lm)).sum(-1, keepdim=True)
        return 0.5 * q * (lq - lm - kl_qm)
    if name == "ce":
        idx = torch.argmax(targets, dim=-1, keepdim=True)
        return q - torch.zeros_like(q).scatter_(-1, idx, 1.0)
    if name == "tv":
        le = (q <= p).float()
        s = (q * le).sum(-1, keepdim=True)
        return -q * (le - s)
    raise KeyError(name)


# ---------------------------------------------------------------- weights


def exp_loss_decay(pos_idx, gamma: float, **_):
    """gamma ** pos_idx; losses/utils.py:51-61."""
    return gamma**pos_idx


def dflash_loss_decay(pos_idx, gamma: float, sample_from_anchor: bool = False, **_):
    """losses/utils.py:17-48: slot 0 (the anchor) weighs 0, slot s>=1 weighs
    exp(-(s-1)/gamma); with ``sample_from_anchor`` slot s weighs exp(-s/gamma)."""
    pos = pos_idx.float()
    if sample_from_anchor:
        return torch.exp(-pos / gamma)
    w = torch.exp(-(pos - 1.0).clamp_min(0.0) / gamma)
    return torch.where(pos == 0, torch.zeros_like(w), w)


def dpace_loss_decay(pos_idx, loss_mask, block_size: int, dpace_alpha: float,
                     elementwise_loss, **_):
    """D-PACE weight (losses/utils.py:64-112; the reference holds no test of it: pinned by a
    per-element float64 double loop over random masks and a hand-worked example).  Per block:
    c = exp(-CE), s = (1-a)c + a (1 where the mask is 0), prefix = cumprod(s),
    w_i = m_i * sum_{j>=i} prefix_j m_j.  No gradient flows through it."""
    with torch.no_grad():
        conf = torch.exp(-elementwise_loss.float())
        n = conf.shape[1]
        if n % block_size:
            raise ValueError("row count must be a multiple of block_size")
        conf = conf.reshape(n // block_size, block_size)
        m = loss_mask.reshape(n // block_size, block_size).float()
        s = torch.where(m > 0, (1.0 - dpace_alpha) * conf + dpace_alpha,
                        torch.ones_like(conf))
        prefix = torch.cumprod(s, dim=-1) * m
        suffix = prefix.flip(-1).cumsum(-1).flip(-1)
        return (suffix * m).reshape(1, -1)


# ---------------------------------------------------------------- reduction


def loss_function(logits, targets, loss_mask, pos_idx, loss_fn=kl_div,
                  decay_fn=None):
    """mean_b [ sum_i l_i m_i w_i / (sum_i m_i + 1e-5) ]; losses/utils.py:269-304.
    The weight multiplies the numerator only."""
    row = loss_fn(logits, targets)
    m = loss_mask.to(row.dtype)
    row = row * m
    if decay_fn is not None:
        row = row * decay_fn(pos_idx.to(row.dtype), elementwise_loss=row)
    return (row.sum(dim=1) / (m.sum(dim=1) + _REDUCTION_EPS)).mean()


def compound_loss(logits, targets, loss_mask, pos_idx, loss_config, decay_fn=None):
    """sum_terms weight * loss_function(term); per-term values are reported
    only when there is more than one term; losses/utils.py:233-266."""
    total = torch.zeros((), dtype=torch.float32)
    terms: dict[str, torch.Tensor] = {}
    for name, (fn, weight) in loss_config.items():
        val = loss_function(logits, targets, loss_mask, pos_idx, fn, decay_fn)
        if len(loss_config) > 1:
            terms[f"{name}_loss"] = val.detach()
        total = total + weight * val
    return total, terms


def resolve_loss_config(spec: str | dict):
    """``"kl_div"`` or ``{"ce": 0.1, "tv": 0.9}`` -> {name: (fn, weight)};
    the oracle's counterpart of losses/utils.py:184-230."""
    if isinstance(spec, str):
        return {spec: (LOSS_FNS[spec], 1.0)}
    return {k: (LOSS_FNS[k], float(w)) for k, w in spec.items()}
