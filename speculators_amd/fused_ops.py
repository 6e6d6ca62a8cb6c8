"""Autograd wrappers of the HBM-bound layer glue kernels: RMSNorm, rotary embedding
fused with the head-major relayout, SwiGLU.  bf16 HIP tensors only."""

from __future__ import annotations

import math

import torch

from . import _lib


def _need_bf16(*ts):
    for t in ts:
        if t.dtype != torch.bfloat16:
            raise _lib.SpxError("the HIP layer kernels take bf16 tensors: cast the model and its "
                                "inputs to bfloat16")


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        _need_bf16(x, weight)
        h = x.shape[-1]
        x2 = x.reshape(-1, h)
        if x2.stride(1) != 1:
            x2 = x2.contiguous()
        rows = x2.shape[0]
        y = torch.empty(rows, h, device=x.device, dtype=torch.bfloat16)
        rstd = torch.empty(rows, device=x.device, dtype=torch.float32)
        w = weight.contiguous()
        _lib.call("spx_rmsnorm_fwd", _lib.ptr(x2), x2.stride(0), _lib.ptr(w), _lib.ptr(y), h,
                  _lib.ptr(rstd), rows, h, float(eps), _lib.stream_ptr(x.device))
        ctx.save_for_backward(x2, w, rstd)
        ctx.shape = x.shape
        ctx.gain_grads = getattr(weight, "spx_gain_grads", None)
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x2, w, rstd = ctx.saved_tensors
        rows, h = x2.shape
        dy2 = dy.reshape(rows, h).to(torch.bfloat16)
        if dy2.stride(1) != 1:
            dy2 = dy2.contiguous()
        dx = torch.empty(rows, h, device=x2.device, dtype=torch.bfloat16)
        dw = _norm_backward(ctx.gain_grads, ctx.needs_input_grad[1], x2, w, dy2, None, rstd, dx, rows, h)
        return dx.view(ctx.shape), dw, None


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return _RMSNorm.apply(x, weight, eps)


def _dw_buffers(rows: int, h: int, device):
    slots = int(_lib.load().spx_rmsnorm_bwd_slots(rows, h))
    return (torch.empty(slots * h, device=device, dtype=torch.float32),
            torch.empty(h, device=device, dtype=torch.bfloat16))


class GainGrads:
    """The gradient of one RMSNorm gain over ALL of its uses in one backward pass (a draft layer's
    norms run once per TTT step): the uses leave their partial column sums in one fp32 buffer --
    the first writes it, the others add to it inside their kernels -- and the node that staged
    the gain (``weights._StageGain``), which autograd runs after every use, reduces it once.
    A staged gain carries its ``GainGrads`` as the attribute ``spx_gain_grads``."""

    def __init__(self):
        self.scratch, self.slots, self.h, self.marked, self.task = None, 0, 0, False, None

    def target(self, rows: int, h: int, device):
        """``(scratch, accumulate)`` for a use over ``rows`` rows, None if it cannot share the buffer
        (another row count lays the partial sums out differently): it then returns a gradient of
        its own, which autograd adds."""
        task = torch._C._current_graph_task_id()
        if task != self.task:  # a pass that never reached the staging node leaves nothing behind
            self.scratch, self.marked, self.task = None, False, task
        slots = int(_lib.load().spx_rmsnorm_bwd_slots(rows, h))
        if self.scratch is None:
            self.scratch = torch.empty(slots * h, device=device, dtype=torch.float32)
            self.slots, self.h = slots, h
            return self.scratch, 0
        if (slots, h) != (self.slots, self.h) or self.scratch.device != device:
            return None
        return self.scratch, 1

    def mark(self, device):
        """What a use returns as the gain's gradient: an empty marker that makes autograd reach the
        staging node, once per backward pass; None afterwards."""
        if self.marked:
            return None
        self.marked = True
        return torch.zeros(1, device=device, dtype=torch.bfloat16).expand(self.h)

    def finish(self):
        """The summed gradient (bf16 ``[H]``) of the uses recorded since the last call, or None."""
        scratch, self.scratch, self.marked = self.scratch, None, False
        if scratch is None:
            return None
        dw = torch.empty(self.h, device=scratch.device, dtype=torch.bfloat16)
        _lib.call("spx_rmsnorm_dweight", _lib.ptr(scratch), self.slots, self.h, _lib.ptr(dw),
                  _lib.stream_ptr(scratch.device))
        return dw


def _norm_backward(grads, need_dw, x, w, dy, dres, rstd, dx, rows, h):
    """One launch of the norm's backward; returns the gradient to hand autograd for the gain."""
    dev = x.device
    st = _lib.stream_ptr(dev)
    ld_dres = dres.stride(0) if dres is not None else 0
    if need_dw and grads is not None:
        tgt = grads.target(rows, h, dev)
        if tgt is not None:
            _lib.call("spx_rmsnorm_bwd_partial", _lib.ptr(x), x.stride(0), _lib.ptr(w), _lib.ptr(dy),
                      dy.stride(0), _lib.ptr(dres), ld_dres, _lib.ptr(rstd), _lib.ptr(dx), h,
                      _lib.ptr(tgt[0]), tgt[1], rows, h, st)
            return grads.mark(dev)
    scratch = dw = None
    if need_dw:
        scratch, dw = _dw_buffers(rows, h, dev)
    if dres is not None:
        _lib.call("spx_add_rmsnorm_bwd", _lib.ptr(x), x.stride(0), _lib.ptr(w), _lib.ptr(dy), dy.stride(0),
                  _lib.ptr(dres), ld_dres, _lib.ptr(rstd), _lib.ptr(dx), h, _lib.ptr(dw), _lib.ptr(scratch),
                  rows, h, st)
    else:
        _lib.call("spx_rmsnorm_bwd", _lib.ptr(x), x.stride(0), _lib.ptr(w), _lib.ptr(dy), dy.stride(0),
                  _lib.ptr(rstd), _lib.ptr(dx), h, _lib.ptr(dw), _lib.ptr(scratch), rows, h, st)
    return dw


class _AddRMSNorm(torch.autograd.Function):
    """``s = a + b; y = rms_norm(s)`` in one pass; returns ``(s, y)``.  The backward folds the
    gradient that reaches ``s`` along the residual stream into the norm's input gradient."""

    @staticmethod
    def forward(ctx, a, b, weight, eps, out=None):
        _need_bf16(a, b, weight)
        h = a.shape[-1]
        a2, b2 = a.reshape(-1, h), b.reshape(-1, h)
        if a2.stride(1) != 1:
            a2 = a2.contiguous()
        if b2.stride(1) != 1:
            b2 = b2.contiguous()
        rows = a2.shape[0]
        s = torch.empty(rows, h, device=a.device, dtype=torch.bfloat16)
        y = out if out is not None and out.shape == (rows, h) and out.is_contiguous() else \
            torch.empty(rows, h, device=a.device, dtype=torch.bfloat16)
        rstd = torch.empty(rows, device=a.device, dtype=torch.float32)
        w = weight.contiguous()
        _lib.call("spx_add_rmsnorm_fwd", _lib.ptr(a2), a2.stride(0), _lib.ptr(b2), b2.stride(0),
                  _lib.ptr(s), h, _lib.ptr(w), _lib.ptr(y), h, _lib.ptr(rstd), rows, h, float(eps),
                  _lib.stream_ptr(a.device))
        ctx.save_for_backward(s, w, rstd)
        ctx.shape = a.shape
        # (a product of gemm.linear_staged says where its output gradient belongs; the sum's gradient
        # IS that gradient)
        ctx.grad_slot = getattr(b, "spx_grad_slot", None)
        ctx.gain_grads = getattr(weight, "spx_gain_grads", None)
        ctx.set_materialize_grads(False)  # an unused output arrives as None, not as zeros
        return s.view(a.shape), y.view(a.shape)

    @staticmethod
    def backward(ctx, ds, dy):
        s, w, rstd = ctx.saved_tensors
        rows, h = s.shape
        if dy is None:  # the normalised output was not used
            return ds, ds, None, None, None
        dy2 = dy.reshape(rows, h).to(torch.bfloat16)
        if dy2.stride(1) != 1:
            dy2 = dy2.contiguous()
        ds2 = None
        if ds is not None:
            ds2 = ds.reshape(rows, h).to(torch.bfloat16)
            if ds2.stride(1) != 1:
                ds2 = ds2.contiguous()
        dx = None
        if ctx.grad_slot is not None and ctx.needs_input_grad[1]:
            staged, r0, n = ctx.grad_slot
            if n == rows:
                dx = staged.dy_slot(r0, rows)
                if dx.shape != (rows, h) or not dx.is_contiguous():
                    dx = None
        if dx is None:
            dx = torch.empty(rows, h, device=s.device, dtype=torch.bfloat16)
        dw = _norm_backward(ctx.gain_grads, ctx.needs_input_grad[2], s, w, dy2, ds2, rstd, dx, rows, h)
        dx = dx.view(ctx.shape)
        return dx, dx, dw, None, None


def add_rms_norm(a: torch.Tensor, b: torch.Tensor, weight: torch.Tensor, eps: float, out=None):
    """``(a + b, rms_norm(a + b))``: the residual add in front of a norm, fused into it.  ``out``:
    a contiguous ``[rows, H]`` bf16 buffer for the normalised result."""
    return _AddRMSNorm.apply(a, b, weight, eps, out)


class _PairNormCat(torch.autograd.Function):
    """``cat([rms_norm(a, wa), rms_norm(b, wb)], -1)`` written straight into the halves of one
    ``[rows, 2H]`` buffer (the input of the first EAGLE3 layer's q/k/v projections,
    models/eagle3/model_definitions.py:70-94).  With ``residual`` the node also hands ``b`` through
    as a second output -- the layer's residual stream -- so that the gradient arriving along it is
    folded into the norm's input gradient by the same kernel instead of being added afterwards."""

    @staticmethod
    def forward(ctx, a, b, wa, wb, eps, out=None, residual=False):
        _need_bf16(a, b, wa, wb)
        h = a.shape[-1]
        a2, b2 = a.reshape(-1, h), b.reshape(-1, h)
        if a2.stride(1) != 1:
            a2 = a2.contiguous()
        if b2.stride(1) != 1:
            b2 = b2.contiguous()
        rows = a2.shape[0]
        if out is None or out.shape != (rows, 2 * h) or not out.is_contiguous():
            out = torch.empty(rows, 2 * h, device=a.device, dtype=torch.bfloat16)
        rstd = torch.empty(2, rows, device=a.device, dtype=torch.float32)
        ctx.gain_grads = (getattr(wa, "spx_gain_grads", None), getattr(wb, "spx_gain_grads", None))
        wa, wb = wa.contiguous(), wb.contiguous()
        st = _lib.stream_ptr(a.device)
        _lib.call("spx_rmsnorm_fwd", _lib.ptr(a2), a2.stride(0), _lib.ptr(wa), _lib.ptr(out), 2 * h,
                  _lib.ptr(rstd[0]), rows, h, float(eps), st)
        _lib.call("spx_rmsnorm_fwd", _lib.ptr(b2), b2.stride(0), _lib.ptr(wb), _lib.ptr(out[:, h:]), 2 * h,
                  _lib.ptr(rstd[1]), rows, h, float(eps), st)
        ctx.save_for_backward(a2, b2, wa, wb, rstd)
        ctx.shapes = (a.shape, b.shape)
        cat = out.view(*a.shape[:-1], 2 * h)
        if not residual:
            return cat
        ctx.set_materialize_grads(False)  # an unused output arrives as None, not as zeros
        return cat, b.view_as(b)

    @staticmethod
    def backward(ctx, dy, dres=None):
        a2, b2, wa, wb, rstd = ctx.saved_tensors
        rows, h = a2.shape
        if dy is None:  # only the handed-through residual was used
            return None, dres, None, None, None, None, None
        dy2 = dy.reshape(rows, 2 * h).to(torch.bfloat16)
        if dy2.stride(1) != 1:
            dy2 = dy2.contiguous()
        if dres is not None:
            dres = dres.reshape(rows, h).to(torch.bfloat16)
            if dres.stride(1) != 1:
                dres = dres.contiguous()
        grads = []
        for i, (x, w) in enumerate(((a2, wa), (b2, wb))):
            need_dx, need_dw = ctx.needs_input_grad[i], ctx.needs_input_grad[2 + i]
            dx = dw = None
            if need_dx:
                dx = torch.empty(rows, h, device=x.device, dtype=torch.bfloat16)
            if need_dx or need_dw:
                # (the residual's gradient rides along with b's: dx = rms_norm_bwd(half) + dres)
                dw = _norm_backward(ctx.gain_grads[i], need_dw, x, w, dy2[:, i * h:],
                                    dres if i == 1 and need_dx else None, rstd[i], dx, rows, h)
            grads.append((dx.view(ctx.shapes[i]) if dx is not None else None, dw))
        if dres is not None and not ctx.needs_input_grad[1]:
            raise RuntimeError("the handed-through residual received a gradient but b needs none")
        return grads[0][0], grads[1][0], grads[0][1], grads[1][1], None, None, None


def pair_norm_cat(a, b, weight_a, weight_b, eps: float, out=None, residual: bool = False):
    """See ``_PairNormCat``.  ``out``: a contiguous ``[rows, 2H]`` bf16 buffer for the result;
    ``residual``: return ``(cat, b)`` with ``b`` handed through the node."""
    return _PairNormCat.apply(a, b, weight_a, weight_b, eps, out, residual)


def rope_call(x_ptr, ld_x, x_head_stride, position_ids, inv_freq, out_ptr, ld_out, t, heads, d, rotate,
              inverse, offset, table_scale, stream):
    """One launch of the rotary relayout kernel; the rotated part of a head is what the frequency
    table covers (all of it, or its first ``2 * len(inv_freq)`` elements)."""
    rot = 2 * inv_freq.numel() if rotate else d
    _lib.call("spx_rope_relayout_partial", x_ptr, ld_x, x_head_stride, _lib.ptr(position_ids), _lib.ptr(inv_freq),
              out_ptr, ld_out, t, heads, d, rot, int(rotate), int(inverse), int(offset), float(table_scale),
              stream)


def table_scale_of(inv_freq) -> float:
    """The attention factor ``rope_inv_freq`` attached to the table (1 for most scalings)."""
    return float(getattr(inv_freq, "attention_scaling", 1.0))


class _RopeRelayout(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, position_ids, inv_freq, heads, rotate, offset):
        _need_bf16(x)
        t = x.shape[-2]
        d = x.shape[-1] // heads
        x2 = x.reshape(t, heads * d)
        if x2.stride(1) != 1:
            x2 = x2.contiguous()
        scale = table_scale_of(inv_freq)
        out = torch.empty(1, heads, t, d, device=x.device, dtype=torch.bfloat16)
        rope_call(_lib.ptr(x2), x2.stride(0), d, position_ids, inv_freq, _lib.ptr(out), 0, t, heads, d, rotate,
                  0, offset, scale, _lib.stream_ptr(x.device))
        ctx.save_for_backward(position_ids, inv_freq)
        ctx.meta = (x.shape, heads, d, t, rotate, offset, scale)
        return out

    @staticmethod
    def backward(ctx, dout):
        position_ids, inv_freq = ctx.saved_tensors
        shape, heads, d, t, rotate, offset, scale = ctx.meta
        dout = dout.to(torch.bfloat16).contiguous()
        dx = torch.empty(t, heads * d, device=dout.device, dtype=torch.bfloat16)
        rope_call(_lib.ptr(dout), 0, d, position_ids, inv_freq, _lib.ptr(dx), heads * d, t, heads, d, rotate, 1,
                  offset, scale, _lib.stream_ptr(dout.device))
        return dx.view(shape), None, None, None, None, None


class _SplitQueryGate(torch.autograd.Function):
    """``[T, heads * 2 D]`` (the widened q projection of the gated attention: per head the query,
    then its output gate) -> the two ``[T, heads, D]`` halves as strided views; the backward writes
    both gradients into one buffer of the input's layout."""

    @staticmethod
    def forward(ctx, y, heads):
        t = y.shape[-2]
        d = y.shape[-1] // (2 * heads)
        y4 = y.reshape(t, heads, 2, d)
        ctx.meta = (y.shape, t, heads, d)
        return y4[:, :, 0], y4[:, :, 1]

    @staticmethod
    def backward(ctx, dq, dgate):
        shape, t, heads, d = ctx.meta
        dy = torch.empty(t, heads, 2, d, device=(dq if dq is not None else dgate).device, dtype=torch.bfloat16)
        for half, g in ((0, dq), (1, dgate)):
            if g is None:
                dy[:, :, half].zero_()
            else:
                dy[:, :, half].copy_(g.reshape(t, heads, d))
        return dy.view(shape), None


def split_query_gate(y: torch.Tensor, heads: int):
    return _SplitQueryGate.apply(y, heads)


class _SigmoidGate(torch.autograd.Function):
    """``o * sigmoid(gate)`` with the rounding points of the bf16 eager form; ``o [.., T, heads * D]``
    contiguous rows, ``gate [T, heads, D]`` with any row and head stride."""

    @staticmethod
    def forward(ctx, o, gate):
        _need_bf16(o, gate)
        t, heads, d = gate.shape
        o2 = o.reshape(t, heads * d)
        if o2.stride(1) != 1:
            o2 = o2.contiguous()
        if gate.stride(2) != 1:
            gate = gate.contiguous()
        y = torch.empty(t, heads * d, device=o.device, dtype=torch.bfloat16)
        _lib.call("spx_sigmoid_gate_fwd", _lib.ptr(o2), o2.stride(0), _lib.ptr(gate), gate.stride(0),
                  gate.stride(1), _lib.ptr(y), heads * d, t, heads, d, _lib.stream_ptr(o.device))
        ctx.save_for_backward(o2, gate)
        ctx.o_shape = o.shape
        return y.view(o.shape)

    @staticmethod
    def backward(ctx, dy):
        o2, gate = ctx.saved_tensors
        t, heads, d = gate.shape
        dy2 = dy.reshape(t, heads * d).to(torch.bfloat16)
        if dy2.stride(1) != 1:
            dy2 = dy2.contiguous()
        d_o = torch.empty(t, heads * d, device=dy.device, dtype=torch.bfloat16)
        dgate = torch.empty(t, heads, d, device=dy.device, dtype=torch.bfloat16)
        _lib.call("spx_sigmoid_gate_bwd", _lib.ptr(o2), o2.stride(0), _lib.ptr(gate), gate.stride(0),
                  gate.stride(1), _lib.ptr(dy2), dy2.stride(0), _lib.ptr(d_o), heads * d, _lib.ptr(dgate),
                  heads * d, d, t, heads, d, _lib.stream_ptr(dy.device))
        return d_o.view(ctx.o_shape), dgate


def sigmoid_gate(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    return _SigmoidGate.apply(o, gate)


def rope_relayout(x, position_ids, inv_freq, heads: int, rotate: bool = True, offset: int = 0):
    """``[1, T, heads*D]`` -> ``[1, heads, T, D]`` with (``rotate``) the rotary embedding of
    position ``position_ids[t] + offset`` applied; ``position_ids`` int64 ``[T]``."""
    pos = position_ids.reshape(-1)
    if pos.dtype != torch.int64:
        pos = pos.to(torch.int64)
    return _RopeRelayout.apply(x, pos.contiguous(), inv_freq, heads, rotate, offset)


def _rope_kind(scaling) -> str:
    return (scaling or {}).get("rope_type", (scaling or {}).get("type", "default"))


def rope_inv_freq(head_dim: int, theta: float, device, scaling: dict | None = None,
                  seq_len: int | None = None) -> torch.Tensor:
    """fp32 inverse frequencies, evaluated like the HF rotary initialisation the draft layer
    inherits from its verifier config: ``scaling`` is the HF rope-parameter dict (``rope_type``
    "default", "linear", "llama3", "yarn", "dynamic" or "longrope"; Llama-3.1 verifiers use
    "llama3").  ``head_dim`` is the number of rotated elements per head (all of them, or the first
    ``int(head_dim * partial_rotary_factor)`` for a partial rotary embedding).  The factor yarn and
    longrope put on the cos / sin tables rides on the returned tensor as ``attention_scaling`` (read
    by the rotary kernels' wrappers through ``table_scale_of``).  "dynamic" and "longrope" depend on
    the length ``seq_len`` of the running sequence (``max_position_embeddings`` travels in
    ``scaling`` for them); which length applies from call to call is ``RotaryFrequencies``."""
    steps = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    inv = 1.0 / (theta ** steps)
    kind = _rope_kind(scaling)
    table_scale = 1.0
    if kind == "linear":
        inv = inv / float(scaling["factor"])
    elif kind == "llama3":
        factor = float(scaling["factor"])
        low, high = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
        old_len = float(scaling["original_max_position_embeddings"])
        wavelen = 2 * math.pi / inv
        # long wavelengths are stretched by `factor`, short ones kept, the band between blended
        scaled = torch.where(wavelen > old_len / low, inv / factor, inv)
        smooth = (old_len / wavelen - low) / (high - low)
        blended = (1 - smooth) * scaled / factor + smooth * scaled
        medium = (wavelen >= old_len / high) & (wavelen <= old_len / low)
        inv = torch.where(medium, blended, scaled)
    elif kind == "yarn":
        inv, table_scale = _yarn(inv, head_dim, theta, scaling)
    elif kind == "dynamic":
        # NTK-aware: the base grows once the sequence is longer than the trained context
        # (_compute_dynamic_ntk_parameters of transformers' modeling_rope_utils.py, whose forward-time
        # update passes the length as an int64 tensor: the new base is an fp32 value)
        factor, ctx = float(scaling["factor"]), int(scaling["max_position_embeddings"])
        if seq_len is None or int(seq_len) <= ctx:
            grow = (factor * ctx / ctx) - (factor - 1) if seq_len is None else \
                (factor * torch.tensor(ctx, dtype=torch.int64) / ctx) - (factor - 1)
        else:
            grow = (factor * torch.tensor(int(seq_len), dtype=torch.int64) / ctx) - (factor - 1)
        base = theta * grow ** (head_dim / (head_dim - 2))
        inv = 1.0 / (base ** steps)
    elif kind == "longrope":
        # per-frequency divisors (_compute_longrope_parameters): the long set beyond the original context
        ctx0 = int(scaling["original_max_position_embeddings"])
        long = seq_len is not None and int(seq_len) > ctx0
        ext = torch.tensor(scaling["long_factor" if long else "short_factor"], dtype=torch.float32)
        inv = 1.0 / (ext * theta ** steps)
        table_scale = scaling.get("attention_factor")
        if table_scale is None:
            factor = scaling.get("factor")
            if factor is None:
                factor = int(scaling["max_position_embeddings"]) / ctx0
            table_scale = 1.0 if factor <= 1.0 else math.sqrt(1 + math.log(factor) / math.log(ctx0))
    elif kind != "default":
        raise NotImplementedError(f"rope_type '{kind}' is not one of default, linear, llama3, yarn, dynamic, longrope")
    inv = inv.to(device)
    inv.attention_scaling = float(table_scale)
    return inv


class RotaryFrequencies:
    """The inverse frequencies a model's rotary embedding runs with from call to call: fixed for most
    types; "longrope" switches to its long divisors when the highest position of the call is beyond
    the original context, "dynamic" recomputes them whenever a call is longer than every call before
    it (and than ``max_position_embeddings``) and goes back to the original ones on a call shorter
    than ``max_position_embeddings`` -- the behaviour of ``dynamic_rope_update``, which wraps the
    forward of every HF rotary module (the reference builds the verifier's, models/eagle3/core.py:112).
    Only those two types look at the positions (one device-to-host read per forward pass)."""

    def __init__(self, head_dim: int, theta: float, scaling: dict | None = None):
        self.head_dim, self.theta, self.scaling = head_dim, theta, scaling
        self.kind = _rope_kind(scaling)
        self.by_length = self.kind in ("dynamic", "longrope")
        self._made: dict = {}
        if self.kind == "dynamic":
            self._ctx = int(scaling["max_position_embeddings"])
            self._seen = self._ctx
            self._length = None

    def top(self, position_ids) -> int | None:
        """Highest position of the call (``None`` where the frequencies do not depend on it)."""
        return int(position_ids.max()) if self.by_length else None

    def _get(self, device, length):
        key = (str(device), length)
        if key not in self._made:
            self._made[key] = rope_inv_freq(self.head_dim, self.theta, device, self.scaling, length)
        return self._made[key]

    def select(self, device, top: int | None = None, offset: int = 0) -> torch.Tensor:
        """Frequencies of a call whose highest position is ``top + offset``."""
        if not self.by_length:
            return self._get(device, None)
        n = top + offset + 1
        if self.kind == "longrope":
            ctx0 = int(self.scaling["original_max_position_embeddings"])
            return self._get(device, ctx0 + 1 if n > ctx0 else None)
        if n > self._seen:
            self._seen, self._length = n, n
        if n < self._ctx and self._seen > self._ctx:
            self._seen, self._length = self._ctx, None
        if len(self._made) > 64:
            self._made.clear()
        return self._get(device, self._length)


def _yarn(inv, dim: int, theta: float, scaling: dict):
    """YaRN (``_compute_yarn_parameters`` of transformers' ``modeling_rope_utils.py``): frequencies
    whose wavelength fits the original context ``beta_fast`` times or more are kept, those that fit
    it ``beta_slow`` times or less are divided by ``factor``, a linear ramp over the frequency index
    blends between; both tables are scaled by ``0.1 ln(factor) + 1`` unless the config says
    otherwise."""
    factor = float(scaling["factor"])
    old_len = float(scaling["original_max_position_embeddings"])
    mscale, mscale_all = scaling.get("mscale"), scaling.get("mscale_all_dim")

    def get_mscale(scale, m=1.0):
        return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0

    table_scale = scaling.get("attention_factor")
    if table_scale is None:
        if mscale and mscale_all:
            table_scale = get_mscale(factor, mscale) / get_mscale(factor, mscale_all)
        else:
            table_scale = get_mscale(factor)
    beta_fast = scaling.get("beta_fast") or 32
    beta_slow = scaling.get("beta_slow") or 1

    def correction_dim(rotations):
        return dim * math.log(old_len / (rotations * 2 * math.pi)) / (2 * math.log(theta))

    low, high = correction_dim(beta_fast), correction_dim(beta_slow)
    if scaling.get("truncate", True):
        low, high = math.floor(low), math.ceil(high)
    low, high = max(low, 0), min(high, dim - 1)
    if low == high:
        high += 0.001
    ramp = torch.clamp((torch.arange(dim // 2, dtype=torch.float32) - low) / (high - low), 0, 1)
    keep = 1 - ramp
    freqs = theta ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim)
    return (1.0 / (factor * freqs)) * (1 - keep) + (1.0 / freqs) * keep, float(table_scale)


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate, up):
        _need_bf16(gate, up)
        gate, up = gate.contiguous(), up.contiguous()
        out = torch.empty_like(gate)
        _lib.call("spx_swiglu_fwd", _lib.ptr(gate), _lib.ptr(up), _lib.ptr(out), gate.numel(),
                  _lib.stream_ptr(gate.device))
        ctx.save_for_backward(gate, up)
        return out

    @staticmethod
    def backward(ctx, dout):
        gate, up = ctx.saved_tensors
        dout = dout.to(torch.bfloat16).contiguous()
        dg, du = torch.empty_like(gate), torch.empty_like(up)
        _lib.call("spx_swiglu_bwd", _lib.ptr(gate), _lib.ptr(up), _lib.ptr(dout), _lib.ptr(dg),
                  _lib.ptr(du), gate.numel(), _lib.stream_ptr(gate.device))
        return dg, du


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` (bf16)."""
    return _SwiGLU.apply(gate, up)
