"""Attention plug-in: the HIP TTT / anchored-block attention behind the
reference's attention-function interface.

The reference selects an attention function by name from an
``AttentionInterface`` registry (models/attention.py:107-108) and calls it as
``fn(module, q[B,Hq,Q,D], k[B,Hkv,KV,D], v, attention_mask, scaling=..., **kw)
-> (out[B,Q,Hq,D], None)`` (models/attention.py:20-66).  ``attention_mask`` is
whatever the model's mask builder returned; for the HIP kernels it is a small
descriptor (``TTTMask``) instead of a BlockMask or a dense tensor, and the
model's "extend the mask for the next TTT step" operation just bumps a counter.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib

ATTN_IMPL_TTT = "ttt_hip"
ATTN_IMPL_DFLASH = "dflash_hip"


def _workspace_bytes(t, hq, hkv, d, backward):
    return int(_lib.load().spx_ttt_attn_workspace_bytes(t, hq, hkv, d, int(backward)))


@dataclass
class TTTMask:
    """Descriptor of the EAGLE3 mask of one layer: ``row_lo`` (int32 ``[T]``, lowest
    visible context key per query), the sequence length and the current TTT step.
    Stands where the reference passes a BlockMask / dense mask
    (models/eagle3/core.py:149-162, 341-356)."""

    row_lo: torch.Tensor
    total_seq_len: int
    ttt_step: int = 0
    sliding_window: int | None = None

    def extended(self) -> "TTTMask":
        """The mask of the next TTT step (one more diagonal of keys); the
        counterpart of extend_mask_for_draft_tokens (models/eagle3/attention.py:37-132)."""
        return TTTMask(self.row_lo, self.total_seq_len, self.ttt_step + 1, self.sliding_window)


def create_ttt_mask(document_ids: torch.Tensor, total_seq_len: int,
                    sliding_window: int | None = None) -> TTTMask:
    """Build the step-0 descriptor from ``document_ids`` (``[T]`` or ``[1, T]``, -1 =
    padding); the counterpart of ``_build_attn_mask`` (models/eagle3/core.py:149-162).
    ``document_ids`` must be run-contiguous, as the packing collate produces them."""
    doc = document_ids.reshape(-1)
    if doc.numel() != total_seq_len:
        raise ValueError(f"document_ids has {doc.numel()} entries, expected {total_seq_len}")
    if doc.dtype not in (torch.int32, torch.int64):
        doc = doc.to(torch.int64)
    doc = doc.contiguous()
    row_lo = torch.empty(total_seq_len, device=doc.device, dtype=torch.int32)
    _lib.call("spx_ttt_row_lo", _lib.ptr(doc), _lib.kind_code(doc), total_seq_len,
              int(sliding_window) if sliding_window else 0, _lib.ptr(row_lo),
              _lib.stream_ptr(doc.device))
    return TTTMask(row_lo, total_seq_len, 0, sliding_window)


def _check_qkv(q, k, v, mask: TTTMask):
    if q.dim() != 4 or q.shape[0] != 1:
        raise ValueError("the packed batch layout has batch size 1: q must be [1, Hq, T, D]")
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise _lib.SpxError("the HIP attention kernels take bf16 q/k/v")
    _, hq, t, d = q.shape
    hkv, kv_len = k.shape[1], k.shape[2]
    if t != mask.total_seq_len or kv_len != (mask.ttt_step + 1) * t or v.shape != k.shape:
        raise ValueError(
            f"q {tuple(q.shape)} / k {tuple(k.shape)} do not match TTT step {mask.ttt_step} "
            f"of a length-{mask.total_seq_len} sequence")
    return hq, hkv, t, d


class _TTTAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask: TTTMask, scaling: float):
        hq, hkv, t, d = _check_qkv(q, k, v, mask)
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        dev = q.device
        out = torch.empty(1, t, hq, d, device=dev, dtype=torch.bfloat16)
        lse = torch.empty(hq, t, device=dev, dtype=torch.float32)
        ws = torch.empty(_workspace_bytes(t, hq, hkv, d, False), device=dev, dtype=torch.uint8)
        _lib.call("spx_ttt_attn_fwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1),
                  _lib.ptr(v), v.stride(1), _lib.ptr(mask.row_lo), t, mask.ttt_step, hq, hkv, d,
                  float(scaling), _lib.ptr(out), _lib.ptr(lse), _lib.ptr(ws), ws.numel(),
                  _lib.stream_ptr(dev))
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mask, ctx.scaling = mask, float(scaling)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        mask = ctx.mask
        _, hq, t, d = q.shape
        hkv = k.shape[1]
        dev = q.device
        dout = dout.to(torch.bfloat16).contiguous()
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        ws = torch.empty(_workspace_bytes(t, hq, hkv, d, True), device=dev, dtype=torch.uint8)
        _lib.call("spx_ttt_attn_bwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1),
                  _lib.ptr(v), v.stride(1), _lib.ptr(out), _lib.ptr(dout), _lib.ptr(lse),
                  _lib.ptr(mask.row_lo), t, mask.ttt_step, hq, hkv, d, ctx.scaling,
                  _lib.ptr(dq), dq.stride(1), _lib.ptr(dk), dk.stride(1), _lib.ptr(dv),
                  dv.stride(1), _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
        return dq, dk, dv, None, None


class TTTKVCache:
    """K / V of all TTT steps of one layer in ONE preallocated buffer ``[1, Hkv, steps * T, D]``
    (step j's keys are rows ``j*T .. j*T+T-1``: the layout ``DynamicCache.update`` builds by
    concatenation, models/eagle3/core.py:283-300, without the growing copies).  ``window(j)``
    is where step j's projection writes; the kernels read rows ``[0, (j+1) * T)``."""

    def __init__(self, hkv: int, t: int, d: int, steps: int, device):
        self.t, self.steps = t, steps
        self.k = torch.empty(1, hkv, steps * t, d, device=device, dtype=torch.bfloat16)
        self.v = torch.empty(1, hkv, steps * t, d, device=device, dtype=torch.bfloat16)
        self.k_parts: list = []
        self.v_parts: list = []
        self.grads = _CacheGrads()

    def window(self, j: int):
        lo = j * self.t
        return self.k[:, :, lo:lo + self.t], self.v[:, :, lo:lo + self.t]


class _CacheGrads:
    """dK / dV of one layer's cache during ONE backward pass: a ``[1, Hkv, n * T, D]`` buffer each,
    allocated by the first attention node the pass reaches (the latest step in it, ``n`` steps of
    keys), added to by the nodes of the earlier steps.  Holds no tensor of the graph."""

    def __init__(self):
        self.task, self.dk, self.dv, self.low = -1, None, None, 0


class _TTTAttentionCached(torch.autograd.Function):
    """TTT attention over a ``TTTKVCache``: the per-step key / value tensors (windows of the
    cache, already written) are the differentiable inputs, the kernels read the cache in place.
    The keys of step j are seen by every step from j on, so their gradient is a sum over those steps'
    backwards.  Autograd would form it with one add per tensor and step; here the nodes of one
    backward pass share one dK / dV buffer per layer (``_CacheGrads``): the node of the latest step
    writes it, every earlier one adds to it inside its kernels, and a node returns the gradient of
    its OWN step's keys only -- complete by then, because the nodes of all later steps depend on
    this node's output and have run."""

    @staticmethod
    def forward(ctx, q, mask: TTTMask, scaling: float, cache: TTTKVCache, n_parts: int, out, *parts):
        t = cache.t
        k = cache.k[:, :, :n_parts * t]
        v = cache.v[:, :, :n_parts * t]
        hq, hkv, t, d = _check_qkv(q, k, v, mask)
        q = q.contiguous()
        dev = q.device
        if out is not None and out.numel() == t * hq * d and out.is_contiguous() and out.dtype == torch.bfloat16:
            out = out.view(1, t, hq, d)
        else:
            out = torch.empty(1, t, hq, d, device=dev, dtype=torch.bfloat16)
        lse = torch.empty(hq, t, device=dev, dtype=torch.float32)
        ws = torch.empty(_workspace_bytes(t, hq, hkv, d, False), device=dev, dtype=torch.uint8)
        _lib.call("spx_ttt_attn_fwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1),
                  _lib.ptr(v), v.stride(1), _lib.ptr(mask.row_lo), t, mask.ttt_step, hq, hkv, d,
                  float(scaling), _lib.ptr(out), _lib.ptr(lse), _lib.ptr(ws), ws.numel(),
                  _lib.stream_ptr(dev))
        ctx.save_for_backward(q, out, lse)
        ctx.kv = (k, v)  # windows of the cache: later steps only write rows beyond them
        ctx.mask, ctx.scaling, ctx.n_parts = mask, float(scaling), n_parts
        ctx.grads = cache.grads  # (not the cache: its per-step tensors belong to the graph)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, out, lse = ctx.saved_tensors
        k, v = ctx.kv
        mask, n = ctx.mask, ctx.n_parts
        _, hq, t, d = q.shape
        hkv = k.shape[1]
        dev = q.device
        dout = dout.to(torch.bfloat16).contiguous()
        dq = torch.empty_like(q)
        g = ctx.grads
        task = torch._C._current_graph_task_id()
        shared = task >= 0
        if shared and g.task == task:
            if n > g.low:
                raise RuntimeError("the attention node of a later TTT step ran after an earlier step's "
                                   "in one backward pass")
            entry = "spx_ttt_attn_bwd_accumulate"
            dk, dv = g.dk[:, :, :n * t], g.dv[:, :, :n * t]
        else:
            entry = "spx_ttt_attn_bwd"
            dk = torch.empty(1, hkv, n * t, d, device=dev, dtype=torch.bfloat16)
            dv = torch.empty(1, hkv, n * t, d, device=dev, dtype=torch.bfloat16)
            if shared:
                g.task, g.dk, g.dv = task, dk, dv
        ws = torch.empty(_workspace_bytes(t, hq, hkv, d, True), device=dev, dtype=torch.uint8)
        _lib.call(entry, _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1),
                  _lib.ptr(v), v.stride(1), _lib.ptr(out), _lib.ptr(dout), _lib.ptr(lse),
                  _lib.ptr(mask.row_lo), t, mask.ttt_step, hq, hkv, d, ctx.scaling,
                  _lib.ptr(dq), dq.stride(1), _lib.ptr(dk), dk.stride(1), _lib.ptr(dv),
                  dv.stride(1), _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
        if not shared:  # outside a backward pass of the engine: every step's window, to be summed by the caller
            dks = [dk[:, :, i * t:(i + 1) * t] for i in range(n)]
            dvs = [dv[:, :, i * t:(i + 1) * t] for i in range(n)]
            return (dq, None, None, None, None, None, *dks, *dvs)
        g.low = n
        own = slice((n - 1) * t, n * t)
        dks, dvs = [None] * n, [None] * n
        dks[-1], dvs[-1] = dk[:, :, own], dv[:, :, own]
        if n == 1:  # the first step's node is the last to run: the pass is done with the buffers
            g.task, g.dk, g.dv = -1, None, None
        return (dq, None, None, None, None, None, *dks, *dvs)


def ttt_attention_cached(q, k_new, v_new, cache: TTTKVCache, mask: TTTMask,
                         scaling: float | None = None, out=None) -> torch.Tensor:
    """TTT attention of the step whose keys / values ``k_new`` / ``v_new`` (the windows
    ``cache.window(step)``, already written) were just appended; ``[1, T, Hq, D]`` (bf16),
    written into ``out`` (a contiguous bf16 buffer of ``T * Hq * D`` elements) if given."""
    if scaling is None:
        scaling = q.shape[-1] ** -0.5
    cache.k_parts.append(k_new)
    cache.v_parts.append(v_new)
    n = len(cache.k_parts)
    if n != mask.ttt_step + 1:
        raise ValueError(f"the cache holds {n} steps but the mask is at TTT step {mask.ttt_step}")
    return _TTTAttentionCached.apply(q, mask, scaling, cache, n, out, *cache.k_parts, *cache.v_parts)


KERNEL_HEAD_DIMS = (64, 128, 256)


def _at_kernel_head_dim(fn, q, k, v, mask, scaling):
    """Run ``fn`` at a head size the kernels are built for.  Any other ``D <= 256`` (96 and 80 occur
    among the verifiers the reference lists) is widened with zero columns to the next one: zero
    columns of q / k add nothing to a score, zero columns of v give zero output columns, which are
    cut off again; the soft-max scale stays that of the real ``D``.  The copies make this the slow
    way round, and the result is exactly that of a kernel of the real width."""
    d = q.shape[-1]
    if scaling is None:
        scaling = d ** -0.5
    if d in KERNEL_HEAD_DIMS:
        return fn(q, k, v, mask, scaling)
    wide = next((s for s in KERNEL_HEAD_DIMS if s >= d), None)
    if wide is None or k.shape[-1] != d or v.shape[-1] != d:
        raise ValueError(f"head_dim {d}: q, k and v must share one head size of at most {KERNEL_HEAD_DIMS[-1]}")
    pad = (0, wide - d)
    F = torch.nn.functional
    return fn(F.pad(q, pad), F.pad(k, pad), F.pad(v, pad), mask, scaling)[..., :d]


def ttt_attention(q, k, v, mask: TTTMask, scaling: float | None = None) -> torch.Tensor:
    """``[1, Hq, T, D]`` x ``[1, Hkv, (step+1)*T, D]`` -> ``[1, T, Hq, D]`` (bf16)."""
    return _at_kernel_head_dim(_TTTAttention.apply, q, k, v, mask, scaling)


@dataclass
class SpanMask:
    """One interval ``[row_lo, row_hi)`` of visible keys per query (int32 ``[T]`` each) over the
    ``T`` keys of a packed row: what ``transformers.masking_utils.create_causal_mask`` yields for a
    2-D padding mask whose non-padding positions are contiguous in every batch row (the way the
    MTP forward passes ``attention_mask``, models/mtp/core.py:180-186)."""

    row_lo: torch.Tensor
    row_hi: torch.Tensor
    total_seq_len: int


def create_padding_span_mask(attention_mask: torch.Tensor) -> SpanMask:
    """``attention_mask [B, L]`` (non-zero = token, zero = padding) -> the ``SpanMask`` of the packed
    row ``[1, B * L]``: query ``i`` of batch row ``b`` sees the keys ``j <= i`` of its own row with
    ``attention_mask[b, j] != 0``.  Those must form one run per row (left or right padding); a row
    with holes raises.  A query in front of its row's first token sees nothing and yields zeros."""
    if attention_mask.dim() != 2:
        raise ValueError(f"attention_mask must be [batch, seq_len], got {tuple(attention_mask.shape)}")
    if not attention_mask.is_cuda:
        raise _lib.SpxError("libspx_hip works on HIP device tensors only (got a CPU tensor)")
    keep = attention_mask != 0
    b, n = keep.shape
    idx = torch.arange(n, device=keep.device, dtype=torch.int64)
    count = keep.sum(-1)
    first = torch.where(keep, idx, n).amin(-1)
    last = torch.where(keep, idx, -1).amax(-1)
    if bool(((last - first + 1 != count) & (count > 0)).any()):
        raise ValueError("attention_mask must mark one contiguous run of tokens per row "
                         "(left or right padding)")
    first = torch.where(count > 0, first, torch.zeros_like(first))
    end = torch.where(count > 0, last + 1, torch.zeros_like(last))
    base = (torch.arange(b, device=keep.device, dtype=torch.int64) * n).unsqueeze(1)
    lo = (base + first.unsqueeze(1)).expand(b, n)
    hi = base + torch.minimum(idx.unsqueeze(0) + 1, end.unsqueeze(1))
    hi = torch.maximum(hi, lo)  # empty, never negative
    return SpanMask(lo.reshape(-1).to(torch.int32).contiguous(), hi.reshape(-1).to(torch.int32).contiguous(),
                    b * n)


class _SpanAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask: SpanMask, scaling: float):
        if q.dim() != 4 or q.shape[0] != 1:
            raise ValueError("the packed batch layout has batch size 1: q must be [1, Hq, T, D]")
        if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP attention kernels take bf16 q/k/v")
        _, hq, t, d = q.shape
        hkv = k.shape[1]
        if t != mask.total_seq_len or k.shape[2] != t or v.shape != k.shape:
            raise ValueError(f"q {tuple(q.shape)} / k {tuple(k.shape)} do not match a span mask over "
                             f"{mask.total_seq_len} positions")
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        dev = q.device
        out = torch.empty(1, t, hq, d, device=dev, dtype=torch.bfloat16)
        lse = torch.empty(hq, t, device=dev, dtype=torch.float32)
        ws = torch.empty(_workspace_bytes(t, hq, hkv, d, False), device=dev, dtype=torch.uint8)
        _lib.call("spx_span_attn_fwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1), _lib.ptr(v),
                  v.stride(1), _lib.ptr(mask.row_lo), _lib.ptr(mask.row_hi), t, hq, hkv, d, float(scaling),
                  _lib.ptr(out), _lib.ptr(lse), _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mask, ctx.scaling = mask, float(scaling)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        mask = ctx.mask
        _, hq, t, d = q.shape
        hkv = k.shape[1]
        dev = q.device
        dout = dout.to(torch.bfloat16).contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        ws = torch.empty(_workspace_bytes(t, hq, hkv, d, True), device=dev, dtype=torch.uint8)
        _lib.call("spx_span_attn_bwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1), _lib.ptr(v),
                  v.stride(1), _lib.ptr(out), _lib.ptr(dout), _lib.ptr(lse), _lib.ptr(mask.row_lo),
                  _lib.ptr(mask.row_hi), t, hq, hkv, d, ctx.scaling, _lib.ptr(dq), dq.stride(1),
                  _lib.ptr(dk), dk.stride(1), _lib.ptr(dv), dv.stride(1), _lib.ptr(ws), ws.numel(),
                  _lib.stream_ptr(dev))
        return dq, dk, dv, None, None


def span_attention(q, k, v, mask: SpanMask, scaling: float | None = None) -> torch.Tensor:
    """``[1, Hq, T, D]`` x ``[1, Hkv, T, D]`` -> ``[1, T, Hq, D]`` (bf16) under a ``SpanMask``."""
    return _at_kernel_head_dim(_SpanAttention.apply, q, k, v, mask, scaling)


def ttt_hip_attention_forward(module, query, key, value, attention_mask, scaling=None, **_kwargs):
    """The attention-function signature of the reference registry
    (models/attention.py:20-66); ``attention_mask`` must be a ``TTTMask``."""
    if isinstance(attention_mask, SpanMask):
        return span_attention(query, key, value, attention_mask, scaling), None
    if not isinstance(attention_mask, TTTMask):
        raise TypeError(
            f"attention impl '{ATTN_IMPL_TTT}' needs a TTTMask descriptor as attention_mask, "
            f"got {type(attention_mask).__name__}")
    return ttt_attention(query, key, value, attention_mask, scaling), None


# ---------------------------------------------------------------------- DFlash
@dataclass
class DFlashMask:
    """Descriptor of the anchored-block mask of one layer: per query row the visible
    interval of context keys ``[ctx_lo, ctx_hi)`` and of its own block's keys
    ``[blk_lo, blk_hi)`` (all int32 ``[A * block_size]``).  Stands where the reference
    passes the BlockMask built from create_anchor_block_mask_mod
    (models/dflash/attention.py:7-100, models/dflash/core.py:273-328)."""

    ctx_lo: torch.Tensor
    ctx_hi: torch.Tensor
    blk_lo: torch.Tensor
    blk_hi: torch.Tensor
    total_seq_len: int
    q_len: int


def create_dflash_mask(document_ids: torch.Tensor, total_seq_len: int,
                       anchor_positions: torch.Tensor, block_size: int,
                       sliding_window: int | None = None,
                       sliding_window_non_causal: bool = False) -> DFlashMask:
    """Counterpart of ``_create_attention_mask`` (models/dflash/core.py:273-297): block
    keys are non-causal for full-attention layers and for ``sliding_window_non_causal``,
    causal otherwise.  ``document_ids`` must be run-contiguous."""
    doc = document_ids.reshape(-1)
    if doc.numel() != total_seq_len:
        raise ValueError(f"document_ids has {doc.numel()} entries, expected {total_seq_len}")
    if anchor_positions.dim() != 1:
        raise ValueError(f"anchor_positions must be 1D, got shape {tuple(anchor_positions.shape)}")
    if doc.dtype not in (torch.int32, torch.int64):
        doc = doc.to(torch.int64)
    doc = doc.contiguous()
    anchors = anchor_positions.to(device=doc.device)
    if anchors.dtype not in (torch.int32, torch.int64):
        anchors = anchors.to(torch.int64)
    anchors = anchors.contiguous()
    n_q = anchors.numel() * block_size
    dev = doc.device
    bounds = torch.empty(4, n_q, device=dev, dtype=torch.int32)
    scratch = torch.empty(total_seq_len, device=dev, dtype=torch.int32)
    causal_block = sliding_window is not None and not sliding_window_non_causal
    _lib.call("spx_dflash_row_ranges", _lib.ptr(doc), _lib.kind_code(doc), total_seq_len,
              _lib.ptr(anchors), _lib.kind_code(anchors), anchors.numel(), int(block_size),
              int(sliding_window) if sliding_window else 0, int(causal_block),
              _lib.ptr(bounds[0]), _lib.ptr(bounds[1]), _lib.ptr(bounds[2]), _lib.ptr(bounds[3]),
              _lib.ptr(scratch), _lib.stream_ptr(dev))
    return DFlashMask(bounds[0], bounds[1], bounds[2], bounds[3], total_seq_len, n_q)


class _DFlashAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask: DFlashMask, scaling: float):
        if q.dim() != 4 or q.shape[0] != 1:
            raise ValueError("the packed batch layout has batch size 1: q must be [1, Hq, NQ, D]")
        if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP attention kernels take bf16 q/k/v")
        _, hq, nq, d = q.shape
        hkv = k.shape[1]
        t = mask.total_seq_len
        if nq != mask.q_len or k.shape[2] != t + nq or v.shape != k.shape:
            raise ValueError(f"q {tuple(q.shape)} / k {tuple(k.shape)} do not match the mask "
                             f"(T {t}, {mask.q_len} block rows)")
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        dev = q.device
        out = torch.empty(1, nq, hq, d, device=dev, dtype=torch.bfloat16)
        lse = torch.empty(hq, nq, device=dev, dtype=torch.float32)
        nbytes = int(_lib.load().spx_dflash_attn_workspace_bytes(t, nq, hq, hkv, d, 0))
        ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
        _lib.call("spx_dflash_attn_fwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1),
                  _lib.ptr(v), v.stride(1), _lib.ptr(mask.ctx_lo), _lib.ptr(mask.ctx_hi),
                  _lib.ptr(mask.blk_lo), _lib.ptr(mask.blk_hi), t, nq, hq, hkv, d, float(scaling),
                  _lib.ptr(out), _lib.ptr(lse), _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mask, ctx.scaling = mask, float(scaling)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        mask = ctx.mask
        _, hq, nq, d = q.shape
        hkv = k.shape[1]
        t = mask.total_seq_len
        dev = q.device
        dout = dout.to(torch.bfloat16).contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = int(_lib.load().spx_dflash_attn_workspace_bytes(t, nq, hq, hkv, d, 1))
        ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
        _lib.call("spx_dflash_attn_bwd", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1),
                  _lib.ptr(v), v.stride(1), _lib.ptr(out), _lib.ptr(dout), _lib.ptr(lse),
                  _lib.ptr(mask.ctx_lo), _lib.ptr(mask.ctx_hi), _lib.ptr(mask.blk_lo),
                  _lib.ptr(mask.blk_hi), t, nq, hq, hkv, d, ctx.scaling, _lib.ptr(dq), dq.stride(1),
                  _lib.ptr(dk), dk.stride(1), _lib.ptr(dv), dv.stride(1), _lib.ptr(ws), ws.numel(),
                  _lib.stream_ptr(dev))
        return dq, dk, dv, None, None


def dflash_attention(q, k, v, mask: DFlashMask, scaling: float | None = None) -> torch.Tensor:
    """``[1, Hq, NQ, D]`` x ``[1, Hkv, T + NQ, D]`` -> ``[1, NQ, Hq, D]`` (bf16)."""
    return _at_kernel_head_dim(_DFlashAttention.apply, q, k, v, mask, scaling)


def dflash_hip_attention_forward(module, query, key, value, attention_mask, scaling=None, **_kwargs):
    """Attention-function signature of the reference registry (models/attention.py:20-66,
    called from models/dflash/model_definitions.py:134-152); the mask is a ``DFlashMask``."""
    if not isinstance(attention_mask, DFlashMask):
        raise TypeError(
            f"attention impl '{ATTN_IMPL_DFLASH}' needs a DFlashMask descriptor as attention_mask, "
            f"got {type(attention_mask).__name__}")
    return dflash_attention(query, key, value, attention_mask, scaling), None


class AttentionRegistry(dict):
    """Name -> attention function; the local mirror of the reference's
    ``ALL_ATTENTION_FUNCTIONS`` (models/attention.py:107-108)."""

    def register(self, name, fn):
        self[name] = fn


ALL_ATTENTION_FUNCTIONS = AttentionRegistry()
ALL_ATTENTION_FUNCTIONS.register(ATTN_IMPL_TTT, ttt_hip_attention_forward)
ALL_ATTENTION_FUNCTIONS.register(ATTN_IMPL_DFLASH, dflash_hip_attention_forward)


def register_with_transformers() -> None:
    """Also register the HIP attention functions in HF's global ``AttentionInterface`` so a
    ``LlamaAttention`` / ``Qwen3Attention`` whose config says
    ``_attn_implementation = "ttt_hip"`` dispatches to them."""
    from transformers.modeling_utils import AttentionInterface

    for name, fn in ALL_ATTENTION_FUNCTIONS.items():
        AttentionInterface.register(name, fn)
