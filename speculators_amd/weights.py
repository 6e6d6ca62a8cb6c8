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
    autograd one weight-sized gradient per use, and its gradient is not summed over the uses in
    memory either: the inputs ``X_j`` of its uses lie one after the other in ONE buffer
    (``Staged.x_slot``: the kernel that produces an input writes it there) and so do the output
    gradients ``dY_j`` of the backward, so that the weight gradient of all uses is ONE product
    ``[dY_0; dY_1; ...]^T [X_0; X_1; ...]`` with the contraction running over ``uses * T`` rows
    (``spx_gemm_bf16_tn_f32``): the sum over the uses happens in the MFMA accumulators, in fp32,
    and the gradient is written once.  That product runs in the staging node's backward, which
    autograd calls after every use has run its own.  The node has a second, fp32 output of the
    weight's shape that occupies no memory (``Staged.token``, one element expanded); the
    products take it as their differentiable input, and the first one to run its backward
    returns an equally empty marker for it so that the node is reached.  A use whose input
    is not in the buffer (nobody asked for the slot, or it was full) is added by a product of
    its own (accumulating in fp32);
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


def transposed_copy(w: torch.Tensor) -> torch.Tensor:
    """``w.transpose(-1, -2)`` as a new contiguous tensor; a stack ``[E, N, K]`` is transposed
    matrix by matrix.  On the library's kernel where its alignment rules hold."""
    if (w.dtype == torch.bfloat16 and w.is_cuda and w.dim() in (2, 3) and w.is_contiguous()
            and w.shape[-1] % 8 == 0 and w.shape[-2] % 8 == 0 and w.data_ptr() % 16 == 0):
        r, c = w.shape[-2], w.shape[-1]
        batches = w.shape[0] if w.dim() == 3 else 1
        out = torch.empty(*w.shape[:-2], c, r, device=w.device, dtype=w.dtype)
        _lib.call("spx_transpose_bf16", _lib.ptr(w), c, r * c, _lib.ptr(out), r, r * c, r, c, batches,
                  _lib.stream_ptr(w.device))
        return out
    return w.transpose(-1, -2).contiguous()


def _tn_ok(t: torch.Tensor) -> bool:
    return (t.dtype == torch.bfloat16 and t.stride(1) == 1 and t.shape[1] % 8 == 0
            and t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0)


def wgrad_product(dy: torch.Tensor, x: torch.Tensor, acc: torch.Tensor | None) -> torch.Tensor:
    """``acc (+)= dy.T @ x`` with an fp32 result: on the transposing MFMA kernel of this library
    where its alignment rules hold, else on PyTorch's matmul."""
    if _tn_ok(dy) and _tn_ok(x):
        from .gemm import gemm_tn

        if acc is None:
            return gemm_tn(dy, x, out_dtype=torch.float32)
        return gemm_tn(dy, x, acc, accumulate=True)
    if acc is None:
        return torch.mm(dy.t(), x, out_dtype=torch.float32)
    return torch.addmm(acc, dy.t(), x, out_dtype=torch.float32, out=acc)


class Staged:
    """One compute weight of this forward.  ``w``: bf16 ``[rows, cols]`` (or 1-D for a norm gain);
    ``rows_of``: the row count of every parameter in it; ``uses``: how many products the forward
    is expected to run against it (the size of the input / output-gradient buffers)."""

    __slots__ = ("w", "token", "rows_of", "uses", "_wt", "_xs", "_fill", "_dys", "_live", "_extras",
                 "_marked", "_acc", "aux", "_finishers", "_task")

    def __init__(self, w, rows_of, uses: int = 1):
        self.w = w
        self.token = None  # fp32 stand-in of w's shape that carries the gradient edge (trainable only)
        self.rows_of = rows_of
        self.uses = uses
        self._wt = None
        self._xs = None    # [uses * T, cols]: the inputs of the uses, one after the other
        self._fill = 0     # rows of _xs taken by products so far
        self._dys = None   # [uses * T, rows]: the output gradients, same row positions (backward only)
        self._live = []    # (first row, rows) of the uses whose backward has run
        self._extras = []  # (dy, x) of uses outside the buffers
        self._marked = False
        self._acc = None   # fp32 gradient buffer of uses that add their gradient themselves
        self.aux = None    # whatever a family of products keeps per staged weight (the expert stacks)
        self._finishers = []  # callables acc -> acc that add deferred gradients when the node runs
        self._task = None     # the backward pass (autograd graph task) the recorded uses belong to

    @property
    def trainable(self) -> bool:
        return self.token is not None

    @property
    def wt(self) -> torch.Tensor:
        """``w.T`` contiguous (made on first use, kept with the staged weight)."""
        if self._wt is None:
            self._wt = transposed_copy(self.w.detach())
        return self._wt

    # ---- forward side
    def x_slot(self, rows: int):
        """Where the input ``[rows, cols]`` of the next product against this weight should be
        written so that its weight gradient joins the one product over all uses; None when
        there is nothing to gain (frozen weight, no graph, a single use) or no room."""
        if self.token is None or self.uses <= 1 or not torch.is_grad_enabled():
            return None
        if self._xs is None:
            self._xs = torch.empty(self.uses * rows, self.w.shape[1], device=self.w.device,
                                   dtype=torch.bfloat16)
        if self._fill + rows > self._xs.shape[0]:
            return None
        return self._xs[self._fill:self._fill + rows]

    def take(self, x2: torch.Tensor) -> int:
        """Called by a product's forward with its input: the first row of ``x2`` in the input
        buffer if it is the slot ``x_slot`` handed out (the slot is then taken), else -1."""
        xs = self._xs
        if xs is None:
            return -1
        rows = x2.shape[0]
        if (x2.data_ptr() == xs.data_ptr() + self._fill * xs.stride(0) * 2 and x2.is_contiguous()
                and x2.shape[1] == xs.shape[1] and self._fill + rows <= xs.shape[0]):
            self._fill += rows
            return self._fill - rows
        return -1

    # ---- backward side
    def _enter_pass(self):
        """What the uses record belongs to ONE backward pass, which ends in ``finish`` when autograd
        reaches the staging node.  A pass that never got there (``autograd.grad`` for other inputs
        over a retained graph) must not leak its records into the next one."""
        task = torch._C._current_graph_task_id()
        if task != self._task:
            self._dys, self._live, self._extras, self._marked, self._acc = None, [], [], False, None
            self._task = task

    def dy_slot(self, r0: int, rows: int):
        """Where the output gradient of the use at rows ``r0`` belongs (None for a use outside the
        buffers): a backward that allocates its own result writes it here."""
        if r0 < 0:
            return None
        self._enter_pass()
        if self._dys is None:
            self._dys = torch.empty(self._xs.shape[0], self.w.shape[0], device=self.w.device,
                                    dtype=torch.bfloat16)
        return self._dys[r0:r0 + rows]

    def defer(self, r0: int, dy2: torch.Tensor, x2: torch.Tensor):
        """Record one use's ``(dy, x)`` for the weight-gradient product the staging node runs.
        Returns what the calling backward returns as the gradient of ``token``."""
        self._enter_pass()
        if r0 >= 0:
            slot = self.dy_slot(r0, dy2.shape[0])
            if dy2.data_ptr() != slot.data_ptr():
                slot.copy_(dy2)
            self._live.append((r0, dy2.shape[0]))
        else:
            self._extras.append((dy2, x2))
        return self.mark()

    def mark(self):
        """What a use's backward returns as the gradient of ``token``: the empty marker that makes
        autograd reach the staging node, once per backward; None afterwards."""
        self._enter_pass()
        if self._marked:
            return None
        self._marked = True
        return torch.zeros(1, device=self.w.device, dtype=torch.float32).expand(self.w.shape)

    def grad_buffer(self):
        """``(buffer, holds)``: the fp32 buffer of ``w``'s shape that uses which compute their weight
        gradient themselves (the grouped expert products) add it to, and whether an earlier use of
        this backward has written it already (the first one overwrites)."""
        self._enter_pass()
        holds = self._acc is not None
        if not holds:
            self._acc = torch.empty(self.w.shape, device=self.w.device, dtype=torch.float32)
        return self._acc, holds

    def finish(self, bf16_ok: bool = False):
        """The fp32 weight gradient of every recorded use (None if there is none): one product
        per run of adjacent uses in the buffers -- normally one -- plus one per outside use.
        ``bf16_ok``: the parameters are bf16, so when ONE product is all there is, it writes bf16
        itself (the same fp32 accumulation and the same one rounding as a cast of its fp32 result)."""
        acc = self._acc
        runs: list = []
        for r0, n in sorted(self._live):
            if runs and runs[-1][0] + runs[-1][1] == r0:
                runs[-1][1] += n
            else:
                runs.append([r0, n])
        if bf16_ok and acc is None and len(runs) == 1 and not self._extras and not self._finishers:
            r0, n = runs[0]
            dy, x = self._dys[r0:r0 + n], self._xs[r0:r0 + n]
            if _tn_ok(dy) and _tn_ok(x):
                from .gemm import gemm_tn

                self._dys, self._live, self._marked = None, [], False
                return gemm_tn(dy, x, out_dtype=torch.bfloat16)
        for r0, n in runs:
            acc = wgrad_product(self._dys[r0:r0 + n], self._xs[r0:r0 + n], acc)
        for dy2, x2 in self._extras:
            acc = wgrad_product(dy2, x2, acc)
        for add_deferred in self._finishers:
            acc = add_deferred(acc)
        self._dys, self._live, self._extras, self._marked, self._acc = None, [], [], False, None
        return acc


class _Stage(torch.autograd.Function):
    """params -> (their bf16 row-wise concatenation, the fp32 token that carries its gradient);
    backward: the weight-gradient product over all recorded uses (``Staged.finish``), split and
    cast to each parameter's dtype."""

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
        ctx.set_materialize_grads(False)
        return w, token

    @staticmethod
    def backward(ctx, _gw, g):
        # g is the marker of ``Staged.defer`` (no memory behind it): the gradient is computed here,
        # now that every use has run its backward
        acc = ctx.staged.finish(bf16_ok=all(dt == torch.bfloat16 for dt in ctx.dtypes))
        if acc is not None:
            g = acc
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


class _StageGain(torch.autograd.Function):
    """bf16 compute copy of an RMSNorm gain (``1 + p`` for the zero-centred form).  Its backward
    adds what the uses left in the gain's ``GainGrads`` (reduced here, once) to whatever gradient
    arrives the ordinary way, and casts to the parameter's dtype."""

    @staticmethod
    def forward(ctx, p, plus_one, grads):
        ctx.grads, ctx.dtype = grads, p.dtype
        if plus_one:
            return (1.0 + p.detach().float()).to(torch.bfloat16)
        return p.detach().to(torch.bfloat16) if p.dtype != torch.bfloat16 else p.detach().clone()

    @staticmethod
    def backward(ctx, g):
        total = ctx.grads.finish()
        if total is None:
            out = g
        elif g is None or g.stride(0) == 0:  # nothing but the empty marker arrived
            out = total
        else:
            out = (total.float() + g.float())
        return (out.to(ctx.dtype) if out is not None else None), None, None


class WeightStager:
    """Hands out the ``Staged`` compute weights of one model.  ``begin()`` starts a forward."""

    def __init__(self):
        self._fwd: dict = {}
        self._frozen: dict = {}
        self._uses = 1

    def begin(self, uses: int = 1):
        """``uses``: how often the forward applies each trainable layer weight (the TTT / MTP
        step count)."""
        self._fwd = {}
        self._uses = max(int(uses), 1)

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
            st = Staged(None, rows_of, self._uses)
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

    def gain(self, p: torch.Tensor, plus_one: bool = False) -> torch.Tensor:
        """A small 1-D weight (an RMSNorm gain) in bf16 for the running forward.  ``plus_one``: the
        gain is ``1 + p`` (evaluated in fp32), the form of the Qwen3-Next norms.  A trainable gain
        goes through one autograd node (``_StageGain``) and carries a ``fused_ops.GainGrads``: the
        norm kernels of all its uses leave their partial sums there, and the node reduces them
        once, after the last use's backward."""
        key = ("gain", id(p), plus_one)
        hit = self._fwd.get(key)
        if hit is None:
            _check_param_dtype(p)
            if p.requires_grad and torch.is_grad_enabled():
                from .fused_ops import GainGrads

                grads = GainGrads()
                hit = _StageGain.apply(p, plus_one, grads)
                hit.spx_gain_grads = grads
            elif plus_one:
                hit = (1.0 + p.float()).to(torch.bfloat16)
            else:
                hit = p if p.dtype == torch.bfloat16 else p.to(torch.bfloat16)
            self._fwd[key] = hit
        return hit
