"""Compute copies of the parameters for one forward / backward.

The kernels compute in bf16.  The parameters may be bf16 (the whole model cast, the regime of
the reference's integration tests, tests/integration/conftest.py:130,165) or fp32 master weights
under ``torch.autocast(dtype=torch.bfloat16)`` (the regime of the reference's trainer,
train/trainer.py:459-465, train/config/schema.py:221-226).  Either way every weight the forward
touches is *staged* once per forward:

  * trainable weights go through one autograd node (``_Stage``) that casts to bf16 and, for
    projections that share their input (q/k/v, gate/up), concatenates them row-wise so they run as
    one product.  The weight gradient comes back through that node, so ``torch.autograd.grad``,
    tensor hooks and post-accumulate-grad hooks see it like any other gradient, and it is cast to
    the parameter's dtype there (fp32 for master weights);
  * a weight that is applied several times in one forward (once per TTT step) does not hand
    autograd one weight-sized gradient per use: the uses add their products into ONE fp32
    accumulator inside the GEMM (``out_dtype=float32``, beta = 1), the use whose backward runs
    first returns that accumulator to autograd and the others return nothing.  No rounding happens
    between the uses.  Autograd casts a gradient to the dtype of the tensor it belongs to (and
    would copy the accumulator, half filled, into bf16), so the accumulator does not travel as
    the gradient of the bf16 weight: the staging node has a second, fp32 output of the weight's
    shape that occupies no memory (``Staged.token``, one element expanded), the products take
    it as their differentiable input and return the accumulator as ITS gradient;
  * frozen weights (``lm_head``, ``verifier_lm_head``, ``embed_tokens``, ``verifier_norm``) are
    cast (and transposed where the backward needs it) once and kept until the parameter changes:
    the key is ``(data_ptr, _version, dtype)``; ``WeightStager.invalidate()`` drops every kept
    copy, and the models call it from ``train()`` / ``eval()`` and ``load_state_dict`` so that a
    write through ``param.data`` (which does not bump ``_version``) is picked up at those points.
"""

from __future__ import annotations

import torch

from . import _lib


def _autocast_bf16(device_type: str = "cuda") -> bool:
    return torch.is_autocast_enabled(device_type) and torch.get_autocast_dtype(device_type) == torch.bfloat16


def compute_input(x: torch.Tensor) -> torch.Tensor:
    """An activation input in the compute dtype: bf16 as is; fp32 cast to bf16 under bf16 autocast
    (what the first ``nn.Linear`` of the reference does to it there); anything else is refused."""
    if x.dtype == torch.bfloat16:
        return x
    if x.dtype == torch.float32 and _autocast_bf16(x.device.type):
        return x.to(torch.bfloat16)
    raise RuntimeError(
        "the HIP draft path computes in bf16: cast the model and its inputs to bfloat16, or keep "
        "fp32 master weights and run the forward under torch.autocast(dtype=torch.bfloat16)")


def _check_param_dtype(p: torch.Tensor):
    if p.dtype == torch.bfloat16:
        return
    if p.dtype == torch.float32 and _autocast_bf16(p.device.type):
        return
    raise RuntimeError(
        "the HIP draft path computes in bf16: cast the model to bfloat16, or keep fp32 master "
        "weights and run the forward under torch.autocast(dtype=torch.bfloat16)")


def _cat_bf16(params) -> torch.Tensor:
    """Row-wise concatenation of the parameters as one bf16 tensor (one pass: the copies cast)."""
    if len(params) == 1:
        return params[0].detach().to(torch.bfloat16)
    rows = sum(p.shape[0] for p in params)
    out = torch.empty(rows, *params[0].shape[1:], device=params[0].device, dtype=torch.bfloat16)
    r = 0
    for p in params:
        out[r:r + p.shape[0]].copy_(p.detach())
        r += p.shape[0]
    return out


class Staged:
    """One compute weight of this forward.  ``w``: bf16 ``[rows, cols]`` (or 1-D for a norm gain);
    ``rows_of``: the row count of every parameter in it; ``acc``: the fp32 gradient accumulator of
    the running backward (None outside one)."""

    __slots__ = ("w", "token", "rows_of", "acc", "_wt")

    def __init__(self, w, rows_of):
        self.w = w
        self.token = None  # fp32 stand-in of w's shape that carries the gradient edge (trainable only)
        self.rows_of = rows_of
        self.acc = None
        self._wt = None

    @property
    def trainable(self) -> bool:
        return self.token is not None

    @property
    def wt(self) -> torch.Tensor:
        """``w.T`` contiguous (made on first use, kept with the staged weight)."""
        if self._wt is None:
            self._wt = self.w.detach().t().contiguous()
        return self._wt

    def add_wgrad(self, dy2: torch.Tensor, x2: torch.Tensor):
        """``acc += dy2.T @ x2`` in fp32 inside the GEMM.  Returns the accumulator if this call
        created it (the caller returns it to autograd as the gradient of ``token``), else None."""
        if self.acc is None:
            self.acc = torch.mm(dy2.t(), x2, out_dtype=torch.float32)
            return self.acc
        torch.addmm(self.acc, dy2.t(), x2, out_dtype=torch.float32, out=self.acc)
        return None


class _Stage(torch.autograd.Function):
    """params -> (their bf16 row-wise concatenation, the fp32 token that carries its gradient);
    backward: split the token's gradient, cast to each parameter's dtype.  That gradient is
    normally the fp32 accumulator of ``Staged.add_wgrad``."""

    @staticmethod
    def forward(ctx, staged: Staged, *params):
        ctx.staged = staged
        ctx.rows = [p.shape[0] for p in params]
        ctx.dtypes = [p.dtype for p in params]
        if len(params) == 1 and params[0].dtype == torch.bfloat16:
            w = params[0].detach()
        else:
            w = _cat_bf16(params)
        token = torch.zeros(1, device=w.device, dtype=torch.float32).expand(w.shape)
        ctx.mark_non_differentiable(w)
        return w, token

    @staticmethod
    def backward(ctx, _gw, g):
        ctx.staged.acc = None  # consumed: a later backward through a retained graph starts afresh
        if g is None:
            return (None,) * (1 + len(ctx.rows))
        parts = g.split(ctx.rows, dim=0) if len(ctx.rows) > 1 else (g,)
        grads = []
        for i, (part, dt) in enumerate(zip(parts, ctx.dtypes, strict=True)):
            if not ctx.needs_input_grad[1 + i]:
                grads.append(None)
            elif part.dtype == dt and len(parts) == 1:
                grads.append(part)
            else:
                grads.append(part.to(dt))  # a copy: the parts of a merged buffer become independent
        return (None, *grads)


class WeightStager:
    """Hands out the ``Staged`` compute weights of one model.  ``begin()`` starts a forward."""

    def __init__(self):
        self._fwd: dict = {}
        self._frozen: dict = {}

    def begin(self):
        self._fwd = {}

    def invalidate(self):
        """Forget every kept copy of a frozen weight (they are rebuilt on the next forward)."""
        self._frozen = {}
        self._fwd = {}

    def get(self, *params) -> Staged:
        """The staged row-wise concatenation of ``params`` for the running forward."""
        key = tuple(id(p) for p in params)
        hit = self._fwd.get(key)
        if hit is not None:
            return hit
        for p in params:
            _check_param_dtype(p)
            if not p.is_cuda:
                raise _lib.SpxError("libspx_hip works on HIP device tensors only (got a CPU parameter)")
        rows_of = [p.shape[0] for p in params]
        if torch.is_grad_enabled() and any(p.requires_grad for p in params):
            st = Staged(None, rows_of)
            st.w, st.token = _Stage.apply(st, *params)
        else:
            fkey = tuple((p.data_ptr(), p._version, p.dtype) for p in params)
            kept = self._frozen.get(key)
            if kept is None or kept[0] != fkey:
                w = params[0].detach() if len(params) == 1 and params[0].dtype == torch.bfloat16 \
                    else _cat_bf16(params)
                kept = (fkey, Staged(w, rows_of))
                if not any(p.requires_grad for p in params):
                    self._frozen[key] = kept  # trainable weights seen under no_grad are not kept
            st = kept[1]
        self._fwd[key] = st
        return st

    def gain(self, p: torch.Tensor) -> torch.Tensor:
        """A small 1-D weight (an RMSNorm gain) in bf16 for the running forward: the parameter
        itself, or an ordinary differentiable cast of an fp32 master (its per-use gradients are
        tiny; autograd sums them and casts the sum back)."""
        key = ("gain", id(p))
        hit = self._fwd.get(key)
        if hit is None:
            _check_param_dtype(p)
            hit = p if p.dtype == torch.bfloat16 else p.to(torch.bfloat16)
            self._fwd[key] = hit
        return hit
