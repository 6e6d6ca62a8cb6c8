#!/usr/bin/env python
"""Headline benchmark: EAGLE3 draft train tokens/s (forward + backward) at the
Llama-3.1-8B shape, seq 4096, TTT 7, bf16, on one MI355X.

A "step" is one forward + backward of the draft over one packed synthetic row
(inputs already resident in HBM).  Prints ONE JSON line.  Besides the whole-job
throughput it times every hand-written kernel at its real shape with HIP
events on the launch stream and reports the fraction of the roofline that
bounds it, and times the CPU oracle (the restatement of the reference path) on
a bounded sample of the same workload on the host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# HBM traffic per launch (bytes): read at import from the committed rocprofv3 --pmc summary
# (FETCH_SIZE / WRITE_SIZE in KiB per dispatch, one counter per run, at the default shapes), scaled
# by what the same counters read for a plain copy of known size (the factor is stated in that
# file).  Only valid for the default --seq-len / --ttt-steps; other shapes, and kernels the
# summary does not list, report null.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "kernels_config1_hbm_traffic_pmc.txt")
# bench key -> (substring of the kernel name, launch grid in threads or None = any)
TRAFFIC_ROWS = {
    "gemm_fwd": ("gemm_bf16_nt_kernel<true, 0>", 512000),
    "gemm_dx": ("gemm_bf16_nt_kernel<true, 0>", 65536),
    "loss_fwd": ("loss_fwd_kernel<unsigned short, 0, true, false, false", None),
    "loss_fwd_reuse": ("loss_fwd_kernel<unsigned short, 0, true, true, false", None),
    "gemm_tn": ("gemm_bf16_tn_kernel<2, false>", None),
    "loss_fwd_grad_step0": ("loss_fwd_grad_kernel<0, false>", None),
    "loss_fwd_grad": ("loss_fwd_grad_kernel<0, true>", None),
    # (the summary averages the loss backward over its full and packed launches: no per-launch figure)
}
# The attention kernels are listed per timed call in lines that start with "[attn_step<k>]" or
# "[attn_step<k>_w<window>]": a forward call is the V^T transpose + attn_fwd_kernel, a backward call every
# other kernel of the section (one launch of each per call); their sums are the keys "<section>_fwd|_bwd"
ATTN_FWD_KERNELS = ("attn_fwd_kernel", "transpose_bf16_kernel<false>")


def load_measured_traffic(path=TRAFFIC_SUMMARY):
    import re

    try:
        text = open(path).read()
    except OSError:
        return {}
    m = re.search(r"FETCH_SIZE under-reads by\s+a factor ([0-9.]+)", text.replace("\n#", " "))
    fetch_scale = float(m.group(1)) if m else 1.0
    rows = []
    out = {}
    calls = {}
    for line in text.splitlines():
        m = re.match(r"^(?!#)(.*?) grid=(\d+)\s+n=\s*\d+\s+FETCH_KiB avg\s+([0-9.]+)\s+WRITE_KiB avg\s+([0-9.]+)", line)
        if not m:
            continue
        name, kib = m.group(1), fetch_scale * float(m.group(3)) + float(m.group(4))
        sec = re.match(r"^\[(attn_step\w+)\] (.*)$", name)
        if sec:
            side = "_fwd" if any(k in sec.group(2) for k in ATTN_FWD_KERNELS) else "_bwd"
            calls[sec.group(1) + side] = calls.get(sec.group(1) + side, 0.0) + kib
        else:
            rows.append((name, int(m.group(2)), float(m.group(3)), float(m.group(4))))
    for key, kib in calls.items():
        out[key] = int(kib * 1024)
    for key, (name, grid) in TRAFFIC_ROWS.items():
        hit = [r for r in rows if name in r[0] and (grid is None or r[1] == grid)]
        if len(hit) == 1:
            out[key] = int((fetch_scale * hit[0][2] + hit[0][3]) * 1024)
    return out


MEASURED_TRAFFIC = load_measured_traffic()

CONFIG1 = dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=14336, vocab_size=128256, draft_vocab_size=32000,
               rope_theta=500000.0, rms_norm_eps=1e-5,
               # the rotary frequency scaling Llama-3.1 ships with (the draft layer inherits it)
               rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                             "high_freq_factor": 4.0, "original_max_position_embeddings": 8192})
SEQ_LEN, TTT_STEPS = 4096, 7
# configs[3]: the Llama-3.1-70B shape (seq 8192, TTT 5), same code path as configs[1]
CONFIG3 = dict(CONFIG1, hidden_size=8192, num_attention_heads=64, intermediate_size=28672)
SEQ_LEN3, TTT_STEPS3 = 8192, 5


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", choices=["eagle3", "eagle3-70b", "mtp", "mtp-next", "dflash"],
                    default="eagle3",
                    help="eagle3 = configs[1], the headline; eagle3-70b = configs[3]; mtp = configs[4] (MTP "
                         "head, full-vocab CE); mtp-next = the same shape with the qwen3_next layer (gated "
                         "attention, partial rotary, 512-expert MoE); dflash = configs[2] (anchored blocks, "
                         "5 layers)")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seq-len", type=int, default=SEQ_LEN)
    ap.add_argument("--ttt-steps", type=int, default=TTT_STEPS)
    ap.add_argument("--targets", choices=["hidden", "logits"], default="hidden",
                    help="hidden: verifier_last_hidden_states through the frozen verifier head "
                         "(the reference's forward contract); logits: full-vocab verifier "
                         "logits gathered through d2t")
    ap.add_argument("--loss", default="kl_div",
                    help="loss spec of the EAGLE3 workloads (losses/utils.py:184-230): kl_div (the reference "
                         "default, the headline), ce, tv, ... or a JSON weighting such as '{\"ce\": 0.1, \"tv\": 0.9}'")
    ap.add_argument("--regime", choices=["autocast", "bf16"], default="autocast",
                    help="autocast: fp32 master weights, forward under torch.autocast(bf16), fp32 "
                         "gradients (the regime of the reference's Trainer, train/trainer.py:459-465); "
                         "bf16: the whole model cast to bf16 (the reference's integration tests)")
    ap.add_argument("--window", type=int, default=0,
                    help="sliding window of every draft layer for the HEADLINE figure (0 = full attention, what "
                         "BASELINE's configs[1] names).  The reference's scripts/train.py makes every EAGLE3 draft "
                         "layer sliding-window with W = 2048 unless --full-attention-indices is given "
                         "(scripts/train.py:176-179,498-506; train/config/schema.py:172-183): the default run "
                         "times that configuration as a second figure, `reference_default_config`")
    ap.add_argument("--cpu-baseline", choices=["sample", "off"], default="sample")
    ap.add_argument("--cpu-seq-len", type=int, default=1024)
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel roofline timing")
    ap.add_argument("--only-kernels", action="store_true",
                    help="run only the per-kernel timing loops (for rocprofv3 counter runs)")
    return ap.parse_args()


def make_inputs(torch, cfg, t, device, with_logits):
    g = torch.Generator(device=device).manual_seed(0)
    h, vt, vd = cfg["hidden_size"], cfg["vocab_size"], cfg["draft_vocab_size"]
    batch = {
        "hidden_states": (torch.randn(1, t, 3 * h, device=device, generator=g) * 4).bfloat16(),
        "input_ids": torch.randint(0, vt, (1, t), device=device, generator=g),
        "document_ids": torch.zeros(1, t, dtype=torch.long, device=device),
        "loss_mask": (torch.rand(1, t, device=device, generator=g) < 0.7).float(),
        "position_ids": 1 + torch.arange(t, device=device).unsqueeze(0),
    }
    sel = torch.randperm(vt, device=device, generator=g)[:vd].sort().values
    d2t = sel - torch.arange(vd, device=device)
    t2d = torch.zeros(vt, dtype=torch.bool, device=device)
    t2d[sel] = True
    if with_logits:
        batch["verifier_logits"] = (torch.randn(1, t, vt, device=device, generator=g) * 2).bfloat16()
    else:
        batch["verifier_last_hidden_states"] = torch.randn(1, t, h, device=device, generator=g).bfloat16()
    return batch, d2t, t2d


def make_model(torch, cfg, device, d2t, t2d, param_dtype=None):
    """Random-init draft of the given shape; the same bf16-representable values in either
    parameter dtype, so the two regimes start from identical weights."""
    from speculators_amd.eagle3 import Eagle3Config, Eagle3DraftModel

    model = Eagle3DraftModel(Eagle3Config(**cfg))
    g = torch.Generator(device=device).manual_seed(1)
    model = model.to(param_dtype or torch.bfloat16).to(device)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("norm.weight") or "layernorm" in name:
                p.fill_(1.0)
            else:
                p.copy_((torch.randn(p.shape, device=device, generator=g) * 0.02).bfloat16().to(p.dtype))
    model.load_vocab_mappings(t2d, d2t)
    return model


class quiet_gc:
    """The timed region runs without the cyclic garbage collector: one of its full passes in
    the middle of a forward (tens of milliseconds of host time) drains the GPU's launch queue and
    shows up as one slow step."""

    def __enter__(self):
        import gc

        gc.collect()
        self.was = gc.isenabled()
        gc.disable()

    def __exit__(self, *exc):
        import gc

        if self.was:
            gc.enable()


def time_events(torch, fn, iters, warmup=2):
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters  # ms per launch


class GemmProbe:
    """HIP events around the launches of ONE GEMM shape (``[m, k] x [n, k]^T``) that the model
    makes through ``speculators_amd.gemm.gemm_nt`` while the probe is active: the kernel's
    duration inside the timed iterations, where its neighbours are other kernels and not its
    own repetitions.  The events are recorded on the stream the GEMM is launched on."""

    def __init__(self, torch, m, n, k):
        from speculators_amd import gemm
        self.torch, self.gemm, self.shape = torch, gemm, ((m, k), (n, k))
        self.pairs = []

    def __enter__(self):
        self.orig = self.gemm.gemm_nt
        ev = self.torch.cuda.Event

        def probed(a, b, out=None, **kw):
            if (tuple(a.shape), tuple(b.shape)) != self.shape:
                return self.orig(a, b, out, **kw)
            e0, e1 = ev(enable_timing=True), ev(enable_timing=True)
            e0.record()
            r = self.orig(a, b, out, **kw)
            e1.record()
            self.pairs.append((e0, e1))
            return r

        self.gemm.gemm_nt = probed
        return self

    def __exit__(self, *exc):
        self.gemm.gemm_nt = self.orig
        return False

    def mean_ms(self):
        """after a device synchronisation"""
        if not self.pairs:
            return None
        return sum(a.elapsed_time(b) for a, b in self.pairs) / len(self.pairs)


def windowed_pairs(t, window):
    """Live (query, context key) pairs of one document of ``t`` rows under a causal mask with a
    sliding window (``kv > q - window``); no window = all ``t (t + 1) / 2``."""
    if not window or window >= t:
        return t * (t + 1) / 2
    return window * (window + 1) / 2 + (t - window) * window


def kernel_rooflines(torch, cfg, t, k_steps, device, windows=(None,)):
    """Per-kernel average launch time (HIP events on the launch stream) against the
    algorithmic flops / bytes of that launch.  ``windows``: the sliding windows (None = full
    attention) the attention kernels are timed with."""
    from speculators_amd import _lib
    from speculators_amd import attention as A
    from speculators_amd import losses as L
    from speculators_amd.gemm import gemm_nt, gemm_tn
    from speculators_amd.data import plan_rows

    h, vd = cfg["hidden_size"], cfg["draft_vocab_size"]
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    g = torch.Generator(device=device).manual_seed(2)
    out = []

    default_shape = (t == SEQ_LEN and k_steps == TTT_STEPS)

    def traffic_of(key):
        return MEASURED_TRAFFIC.get(key) if (default_shape and key) else None

    def mfma(name, flops, ms, launches, key=None):
        tf = flops / (ms * 1e-3) / 1e12
        out.append({"kernel": name, "bound": "mfma", "achieved": round(tf, 1),
                    "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4),
                    "traffic": traffic_of(key), "algorithmic_flops": flops,
                    "ms_per_launch": round(ms, 4), "launches_per_step": launches})

    def hbm(name, nbytes, ms, launches, key=None):
        gbs = nbytes / (ms * 1e-3) / 1e9
        out.append({"kernel": name, "bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": traffic_of(key),
                    "algorithmic_bytes": nbytes,
                    "ms_per_launch": round(ms, 4), "launches_per_step": launches})

    # a plain copy of known size (T x Vd bf16 read + written once): the yardstick the
    # FETCH_SIZE / WRITE_SIZE counters of the other kernels are scaled by
    src = torch.randn(t, vd, device=device, generator=g).bfloat16()
    dst = torch.empty_like(src)
    ms = time_events(torch, lambda: dst.copy_(src), 20)
    hbm("reference copy[T x Vd bf16, torch copy_]", 2.0 * t * vd * 2, ms, 0)
    del src, dst

    # lm_head GEMM (forward shape; the input-gradient product has the same flops)
    x = torch.randn(t, h, device=device, generator=g).bfloat16()
    w = (torch.randn(vd, h, device=device, generator=g) * 0.02).bfloat16()
    y = torch.empty(t, vd, device=device, dtype=torch.bfloat16)
    ms = time_events(torch, lambda: gemm_nt(x, w, y), 20)
    mfma("gemm_bf16_nt_kernel[lm_head fwd T x H x Vd]", 2.0 * t * h * vd, ms, k_steps + 1, "gemm_fwd")
    # the vendor library on the same product: a yardstick beside the kernel above, not part of the step
    ms = time_events(torch, lambda: torch.nn.functional.linear(x, w), 20)
    mfma("hipBLASLt through torch.nn.functional.linear[lm_head fwd T x H x Vd, yardstick]",
         2.0 * t * h * vd, ms, 0)
    # the same product with per-row soft-max statistics (log-sum-exp, first-index arg-max of the bf16 results)
    # out of its epilogue: with the product stored (what a KL loss would still need of the verifier head) and
    # without (all a cross-entropy loss needs: the verifier's logits never exist in memory)
    from speculators_amd.gemm import gemm_nt_stats
    ms = time_events(torch, lambda: gemm_nt_stats(x, w, store=True), 20)
    mfma("gemm_bf16_nt_kernel<statistics epilogue> + reduce[verifier head T x H x Vd, product stored]",
         2.0 * t * h * vd, ms, 0)
    ms = time_events(torch, lambda: gemm_nt_stats(x, w, store=False, want_lse=False), 20)
    mfma("gemm_bf16_nt_kernel<statistics epilogue> + reduce[verifier head T x H x Vd, statistics only: ce targets]",
         2.0 * t * h * vd, ms, 0)
    wt = w.t().contiguous()
    dx = torch.empty(t, h, device=device, dtype=torch.bfloat16)
    ms = time_events(torch, lambda: gemm_nt(y, wt, dx), 20)
    mfma("gemm_bf16_nt_kernel[lm_head dX T x Vd x H]", 2.0 * t * h * vd, ms, k_steps, "gemm_dx")
    del wt, dx

    # fused loss forward / backward over T rows (step 0 shape)
    tg = (torch.randn(t, vd, device=device, generator=g) * 2).bfloat16()
    lg = (torch.randn(t, vd, device=device, generator=g) * 2).bfloat16()
    stats = torch.empty(4, t, device=device)
    arg = torch.empty(2, t, device=device, dtype=torch.int32)
    st = _lib.stream_ptr(device)

    def loss_fwd():
        _lib.call("spx_fused_vocab_loss_fwd", L.OP_KL, _lib.ptr(lg), vd, _lib.ptr(tg), vd, t, vd, 0,
                  _lib.ptr(stats[0]), _lib.ptr(stats[1]), _lib.ptr(stats[2]), _lib.ptr(stats[3]),
                  _lib.ptr(arg[0]), _lib.ptr(arg[1]), 0, st)

    def loss_fwd_reuse():  # steps >= 1: the target rows' statistics come from step 0
        _lib.call("spx_fused_vocab_loss_fwd", L.OP_KL, _lib.ptr(lg), vd, _lib.ptr(tg), vd, t, vd, 0,
                  _lib.ptr(stats[0]), _lib.ptr(stats[1]), _lib.ptr(stats[2]), _lib.ptr(stats[3]),
                  _lib.ptr(arg[0]), _lib.ptr(arg[1]), 1, st)

    # (what the timed step launches is the one-pass form further down; these two are the streaming forward of
    # the validation pass and of every configuration the one-pass form does not cover)
    ms = time_events(torch, loss_fwd, 20)
    hbm("loss_fwd_kernel[KL, T rows x Vd, step 0]", 2.0 * t * vd * 2, ms, 0, "loss_fwd")
    ms = time_events(torch, loss_fwd_reuse, 20)
    hbm("loss_fwd_kernel[KL, T rows x Vd, steps >= 1 (target statistics reused)]", 2.0 * t * vd * 2,
        ms, 0, "loss_fwd_reuse")
    rg = torch.full((t,), 1.0 / t, device=device)
    grad = torch.empty(t, vd, device=device, dtype=torch.bfloat16)

    def loss_bwd():
        _lib.call("spx_fused_vocab_loss_bwd", L.OP_KL, _lib.ptr(lg), vd, _lib.ptr(tg), vd, t, vd, 0,
                  _lib.ptr(stats[1]), _lib.ptr(stats[2]), _lib.ptr(stats[3]), _lib.ptr(arg[1]),
                  _lib.ptr(rg), None, _lib.ptr(grad), vd, st)

    ms = time_events(torch, loss_bwd, 20)
    hbm("loss_bwd_kernel[KL, T rows x Vd]", 3.0 * t * vd * 2, ms, 0)

    # what the model launches while lm_head is frozen: the same gradient with the live rows (loss
    # mask Bernoulli(0.7), as in the timed step) packed to the front; dead rows are neither read
    # nor written
    live_mask = torch.rand(t, device=device, generator=g) < 0.7
    rg_live = torch.where(live_mask, rg, torch.zeros_like(rg))
    row_map, _count = L._packed_row_map(rg_live)
    n_live = int(live_mask.sum().item())

    def loss_bwd_packed():
        _lib.call("spx_fused_vocab_loss_bwd_packed", L.OP_KL, _lib.ptr(lg), vd, _lib.ptr(tg), vd, t, vd, 0,
                  _lib.ptr(stats[1]), _lib.ptr(stats[2]), _lib.ptr(stats[3]), _lib.ptr(arg[1]),
                  _lib.ptr(rg_live), None, _lib.ptr(row_map), _lib.ptr(grad), vd, st)

    ms = time_events(torch, loss_bwd_packed, 20)
    hbm(f"loss_bwd_kernel[KL, packed: {n_live} live of T rows x Vd]", 3.0 * n_live * vd * 2, ms, 0)
    # what the timed step launches while lm_head is frozen: loss, statistics, acceptance chain AND the
    # unit-weight logits gradient of the live rows in one read of the row pair.  Step 0 reads every target row
    # (their statistics are made there), the later steps only those of the live rows.
    mask_f = live_mask.float()
    prev_fg = live_mask.clone()
    cnt_fg = torch.zeros(3, device=device, dtype=torch.int32)
    step_fg = L.StepPass(mask=mask_f, prev=prev_fg, counts=cnt_fg, grad_in_pass=True)
    fg0 = L._loss_forward_with_grad(L.OP_KL, lg, tg, None, step_fg)
    known_fg = (fg0[1].clone(), fg0[3].clone())
    ms = time_events(torch, lambda: L._loss_forward_with_grad(L.OP_KL, lg, tg, None, step_fg), 20)
    hbm(f"loss_fwd_grad_kernel[KL forward + logits gradient of {n_live} live rows, step 0, + row map]",
        (2.0 * t + n_live) * vd * 2, ms, 1, "loss_fwd_grad_step0")
    ms = time_events(torch, lambda: L._loss_forward_with_grad(L.OP_KL, lg, tg, known_fg, step_fg), 20)
    hbm(f"loss_fwd_grad_kernel[KL forward + logits gradient of {n_live} live rows, steps >= 1, + row map]",
        (1.0 * t + 2.0 * n_live) * vd * 2, ms, k_steps - 1, "loss_fwd_grad")
    del fg0
    # the yardstick of that launch's size: a plain copy of n_live rows (one read + one write per element;
    # the kernel above reads two rows for every row it writes)
    src = lg[:n_live]
    dst = torch.empty_like(src)
    ms = time_events(torch, lambda: dst.copy_(src), 20)
    hbm(f"reference copy[{n_live} x Vd bf16, torch copy_]", 2.0 * n_live * vd * 2, ms, 0)
    del src, dst

    # the first step of the verifier-logits entry point: target rows read THROUGH d2t from the
    # full-vocabulary logits, draft-vocabulary rows written out for the later steps, acceptance
    # chain in the same pass.  Algorithmic bytes per row: the draft row, the 64-byte sectors of the
    # full row that hold a selected id, the gathered row written.
    vt = cfg["vocab_size"]
    sel = torch.randperm(vt, device=device, generator=g)[:vd].sort().values
    d2t = (sel - torch.arange(vd, device=device)).contiguous()
    touched = int(torch.unique(sel // 32).numel()) * 64
    full = (torch.randn(t, vt, device=device, generator=g) * 2).bfloat16()
    gathered = torch.empty(t, vd, device=device, dtype=torch.bfloat16)
    mask_f = live_mask.float()
    prev = live_mask.clone()
    counts = torch.zeros(3, device=device, dtype=torch.int32)

    def loss_step_gather():
        _lib.call("spx_vocab_loss_step_fwd", L.OP_KL, _lib.ptr(lg), vd, _lib.ptr(full), vt, _lib.ptr(d2t),
                  vt, _lib.ptr(gathered), vd, t, vd, 0, _lib.ptr(stats[0]), _lib.ptr(stats[1]),
                  _lib.ptr(stats[2]), _lib.ptr(stats[3]), _lib.ptr(arg[0]), _lib.ptr(arg[1]), 0,
                  _lib.ptr(mask_f), _lib.kind_code(mask_f), _lib.ptr(prev), _lib.kind_code(prev),
                  _lib.ptr(counts), st)

    ms = time_events(torch, loss_step_gather, 20)
    hbm("loss_fwd_gather_pipe_kernel[KL + d2t gather from T x Vt + acceptance chain, step 0 of --targets logits]",
        float(t) * (vd * 2 + touched + vd * 2), ms, 0)
    del tg, lg, grad, y, full, gathered

    # batch producer: 8 documents of (T + 8) / 8 rows, 3 auxiliary layers + the last one, bf16 ->
    # the packed [1, T, ...] row (outside the timed step: it runs on a side stream ahead of it)
    n_docs = 8
    rows = t + n_docs
    hs = torch.randn(rows, 4, h, device=device, generator=g).bfloat16()
    ids = torch.randint(0, 1000, (rows,), device=device, generator=g)
    lm = torch.ones(rows, device=device, dtype=torch.int64)
    lens = [rows // n_docs] * n_docs
    src_s, out_s = plan_rows(lens, t, 1)
    plan = torch.tensor([src_s, out_s], device=device, dtype=torch.int64)
    p_aux = torch.empty(t, 3 * h, device=device, dtype=torch.bfloat16)
    p_last = torch.empty(t, h, device=device, dtype=torch.bfloat16)
    p_i64 = torch.empty(4, t, device=device, dtype=torch.int64)

    def pack():
        _lib.call("spx_pack_batch", _lib.ptr(hs), _lib.dtype_code(hs), rows, 3, h, _lib.ptr(ids),
                  _lib.ptr(lm), 8, None, _lib.ptr(plan[0]), _lib.ptr(plan[1]), n_docs, t, 1,
                  _lib.ptr(p_aux), _lib.ptr(p_last), _lib.ptr(p_i64[0]), _lib.ptr(p_i64[1]),
                  _lib.ptr(p_i64[2]), _lib.ptr(p_i64[3]), st)

    ms = time_events(torch, pack, 20)
    hbm("pack_batch_kernel[8 documents -> T x (3H + H) bf16, ids, mask, positions, document ids]",
        2.0 * t * 4 * h * 2 + t * 7 * 8, ms, 0)
    del hs, p_aux, p_last

    # TTT attention, forward and backward, at the first step (no diagonal keys) and at the last one
    # (K - 1 diagonal keys per row), full and -- where asked -- with every layer's sliding window
    def attn_rows(step, window):
        mask = A.create_ttt_mask(torch.zeros(t, dtype=torch.long, device=device), t, window)
        for _ in range(step):
            mask = mask.extended()
        q = torch.randn(1, hq, t, d, device=device, generator=g).bfloat16().requires_grad_(True)
        kk = torch.randn(1, hkv, (step + 1) * t, d, device=device, generator=g).bfloat16().requires_grad_(True)
        vv = torch.randn(1, hkv, (step + 1) * t, d, device=device, generator=g).bfloat16().requires_grad_(True)
        pairs = windowed_pairs(t, window) + step * t
        tag = f"TTT step {step}" + (f", window {window}" if window else "")
        key = f"attn_step{step}" + (f"_w{window}" if window else "")
        ms_f = time_events(torch, lambda: A.ttt_attention(q.detach(), kk.detach(), vv.detach(), mask), 10)
        mfma(f"attn_fwd_kernel[{tag}]", 4.0 * pairs * d * hq, ms_f, 1, key + "_fwd")
        o = A.ttt_attention(q, kk, vv, mask)
        go = torch.randn_like(o)
        ms_b = time_events(torch, lambda: torch.autograd.grad(o, (q, kk, vv), go, retain_graph=True), 10)
        names = "dq + dkv + diag kernels" if step else "dq + dkv kernels"
        mfma(f"attn_bwd[{names}, {tag}]", 10.0 * pairs * d * hq, ms_b, 1, key + "_bwd")

    for window in windows:
        attn_rows(k_steps - 1, window)
        attn_rows(0, window)

    # weight gradient of the merged gate / up projection over all TTT steps in one product: the steps'
    # output gradients [K T, 2F] and inputs [K T, H] lie one after the other, the contraction runs over
    # K T rows, the fp32 result is written once
    f2 = 2 * cfg["intermediate_size"]
    dys = torch.randn(k_steps * t, f2, device=device, generator=g).bfloat16()
    xs = torch.randn(k_steps * t, h, device=device, generator=g).bfloat16()
    acc = torch.empty(f2, h, device=device, dtype=torch.float32)
    ms = time_events(torch, lambda: gemm_tn(dys, xs, acc), 5)
    mfma(f"gemm_bf16_tn_kernel[gate+up weight gradient, all {k_steps} steps: (K T x 2F)^T (K T x H) -> fp32]",
         2.0 * k_steps * t * f2 * h, ms, 1, "gemm_tn")
    return out


CONFIG0 = dict(hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               intermediate_size=8192, vocab_size=128256, draft_vocab_size=32000,
               rope_theta=500000.0, rms_norm_eps=1e-5)
SEQ_LEN0, TTT_STEPS0 = 512, 3


def _cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _oracle_case(torch, cfg, t, scale):
    """Seeded weights and one packed row of the given shape, on the host (fp32)."""
    from oracle import eagle3 as OE

    shape = OE.DraftShape(**cfg)
    w = OE.random_weights(shape, seed=0)
    g = torch.Generator().manual_seed(0)
    hs = (torch.randn(1, t, 3 * shape.hidden_size, generator=g) * scale).bfloat16().float()
    ids = torch.randint(0, shape.vocab_size, (1, t), generator=g)
    vl = torch.randn(1, t, shape.hidden_size, generator=g).bfloat16().float()
    mask = (torch.rand(1, t, generator=g) < 0.7).float()
    doc = torch.zeros(1, t, dtype=torch.long)
    return shape, w, (hs, ids, doc, mask, None, vl)


def _oracle_step(torch, shape, w, case, k_steps):
    from oracle import eagle3 as OE

    frozen = ("embed_tokens.weight", "lm_head.weight", "verifier_lm_head.weight", "verifier_norm.weight")
    for name, p in w.items():
        p.grad = None
        p.requires_grad_(name not in frozen)
    t0 = time.perf_counter()
    _, loss, metrics = OE.eagle3_forward(w, shape, *case, ttt_steps=k_steps, attn="sdpa")
    loss.backward()
    return time.perf_counter() - t0, float(loss.detach()), metrics


def _hip_same_case(torch, device, cfg, w, case, k_steps):
    """The HIP model (fp32 master weights under bf16 autocast) on the oracle's weights and inputs."""
    from speculators_amd.eagle3 import Eagle3Config, Eagle3DraftModel

    model = Eagle3DraftModel(Eagle3Config(**cfg))
    model.load_state_dict({k: v.detach() for k, v in w.items()}, strict=False)
    model = model.to(device)
    hs, ids, doc, mask, _pos, vl = case
    with torch.autocast("cuda", dtype=torch.bfloat16):
        _, loss, metrics = model(hs.bfloat16().to(device), ids.to(device), doc.to(device), mask.to(device),
                                 None, vl.bfloat16().to(device), ttt_steps=k_steps)
    loss.backward()
    out = float(loss.detach()), {k: float(v) for k, v in metrics.items()}
    del model
    torch.cuda.empty_cache()
    return out


def cpu_baseline(torch, device, cfg, t, k_steps):
    """The oracle (CPU restatement of the reference eager path, fp32) timed on the host cores:
    configs[0] in full (1 warm-up + 3 timed forward + backward), and one forward + backward of
    the headline shape on a shortened sequence.  Both cases also go through the HIP model with the
    same weights and inputs: an in-run parity check (loss, exact mask counts)."""
    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(threads)

    def parity(gpu, cpu_loss, cpu_metrics):
        gl, gm = gpu
        totals = [k for k in cpu_metrics if k.endswith("_total")]
        return {"loss_gpu": round(gl, 6), "loss_cpu": round(cpu_loss, 6),
                "rel": round(abs(gl - cpu_loss) / abs(cpu_loss), 7),
                "counts_equal": all(gm[k] == float(cpu_metrics[k]) for k in totals)}

    # configs[0]: the reference's own CPU-runnable case, in full
    shape0, w0, case0 = _oracle_case(torch, CONFIG0, SEQ_LEN0, 1.0)
    _oracle_step(torch, shape0, w0, case0, TTT_STEPS0)
    times = []
    for _ in range(3):
        dt, loss0, m0 = _oracle_step(torch, shape0, w0, case0, TTT_STEPS0)
        times.append(dt)
    mean0 = sum(times) / len(times)
    std0 = (sum((x - mean0) ** 2 for x in times) / len(times)) ** 0.5
    cfg0 = {"workload": f"configs[0]: Llama-3.2-1B shape, seq {SEQ_LEN0}, TTT {TTT_STEPS0}, fp32, in full",
            "value": round(SEQ_LEN0 / mean0, 2), "unit": "tokens/s",
            "s_per_iteration": round(mean0, 3), "s_std": round(std0, 3), "iterations": "1 warm-up + 3 timed",
            "parity": parity(_hip_same_case(torch, device, CONFIG0, w0, case0, TTT_STEPS0), loss0, m0)}
    del w0, case0

    # the headline shape on a shortened sequence
    shape, w, case = _oracle_case(torch, cfg, t, 4.0)
    dt, loss, m = _oracle_step(torch, shape, w, case, k_steps)
    par = parity(_hip_same_case(torch, device, cfg, w, case, k_steps), loss, m)
    return {"value": round(t / dt, 2), "unit": "tokens/s", "cores": threads, "kind": "port",
            "cpu_model": _cpu_model_name(), "host_cpus": cores,
            "sample": f"config[1] shape (Llama-3.1-8B draft, TTT {k_steps}, fp32 oracle), sequence "
                      f"shortened to {t} tokens, 1 forward+backward, no warm-up, {dt:.1f} s",
            "parity": par, "configs0": cfg0}


# configs[4]: MTP head finetune, Qwen3-Next-like shape.  The FFN width is not stated there;
# 3 x hidden is assumed.  The layer built is the Qwen3 flavour of the MTP layer.
CONFIG4 = dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=2, head_dim=256,
               intermediate_size=6144, vocab_size=151936, rms_norm_eps=1e-6, rope_theta=1000000.0)
MTP_SEQ_LEN, MTP_BATCH, MTP_STEPS = 16384, 2, 3
# the hybrid flavour of the same shape: the MTP layer of Qwen3-Next-80B-A3B (its model card's sizes)
NEXT_EXTRA = dict(model_type="qwen3_next", partial_rotary_factor=0.25, num_experts=512, num_experts_per_tok=10,
                  moe_intermediate_size=512, shared_expert_intermediate_size=512, norm_topk_prob=True)


def run_mtp(args):
    """configs[4]: MTP forward + backward, tokens/s over all B x T positions, and the roofline of
    the label cross-entropy kernels, the full-vocabulary lm_head GEMMs and the attention."""
    import torch

    from speculators_amd import _lib, gemm
    from speculators_amd.attention import create_ttt_mask, ttt_attention
    from speculators_amd.losses import label_cross_entropy
    from speculators_amd.mtp import MTPConfig, MTPDraftModel, compute_step_weights

    _lib.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    n = args.seq_len if args.seq_len != SEQ_LEN else MTP_SEQ_LEN
    b, k_steps = MTP_BATCH, MTP_STEPS
    hybrid = args.workload == "mtp-next"
    cfg = MTPConfig(num_speculative_steps=k_steps, **CONFIG4, **(NEXT_EXTRA if hybrid else {}))
    torch.manual_seed(0)
    model = MTPDraftModel(cfg)
    with torch.no_grad():
        for name, p_ in model.named_parameters():
            if name.endswith("norm.weight"):
                p_.fill_(0.0 if hybrid else 1.0)  # the hybrid flavour's gain is 1 + weight
            else:
                p_.normal_(0.0, 0.02)
    model = model.to(torch.bfloat16).to(device)
    g = torch.Generator(device="cpu").manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size, (b, n), generator=g).to(device)
    hs = torch.randn(b, n, cfg.hidden_size, generator=g).bfloat16().to(device)
    lm = (torch.rand(b, n, generator=g) < 0.7).float().to(device)
    pos = torch.arange(n, device=device).unsqueeze(0).expand(b, -1).contiguous()
    sw = compute_step_weights(0.6, k_steps)

    def step():
        model.zero_grad(set_to_none=True)
        _, loss, _ = model(ids, hs, position_ids=pos, loss_mask=lm, step_weights=sw)
        loss.backward()
        return loss

    for _ in range(args.warmup):
        step()
    with quiet_gc():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = step()
        torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    tokens = b * n
    final_loss = float(loss.detach())
    # the same iteration with the row log-sum-exp streamed by the label cross-entropy kernel instead of
    # taken from the head product's epilogue (the default): what that fusion is worth on this workload
    from speculators_amd import losses as losses_mod
    epi_default = losses_mod.HEAD_CE_EPILOGUE_STATS
    losses_mod.HEAD_CE_EPILOGUE_STATS = not epi_default
    try:
        for _ in range(2):
            step()
        with quiet_gc():
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                loss = step()
            torch.cuda.synchronize()
        other_ms = (time.perf_counter() - t0) / args.steps * 1e3
    finally:
        losses_mod.HEAD_CE_EPILOGUE_STATS = epi_default
    head_stats = {"epilogue_statistics" if epi_default else "streamed_statistics": round(ms_per_step, 3),
                  "streamed_statistics" if epi_default else "epilogue_statistics": round(other_ms, 3),
                  "unit": "ms_per_step", "default": "epilogue_statistics" if epi_default else "streamed_statistics"}
    del loss
    model.zero_grad(set_to_none=True)
    torch.cuda.empty_cache()

    rows, v, h = b * (n - k_steps - 1), cfg.vocab_size, cfg.hidden_size
    kernels = []

    def rec(name, bound, work, ms, launches):
        peak = PEAK_BF16_TFLOPS if bound == "mfma" else PEAK_HBM_GBS
        ach = work / (ms * 1e-3) / (1e12 if bound == "mfma" else 1e9)
        kernels.append({"kernel": name, "bound": bound, "achieved": round(ach, 1), "peak": peak,
                        "unit": "TFLOP/s" if bound == "mfma" else "GB/s", "frac": round(ach / peak, 4),
                        "traffic": None, "ms_per_launch": round(ms, 4), "launches_per_step": launches,
                        ("algorithmic_flops" if bound == "mfma" else "algorithmic_bytes"): float(work)})

    x = torch.randn(rows, h, device=device).bfloat16()
    w = model.lm_head.weight
    logits = gemm.gemm_nt(x, w)
    rec("gemm_bf16_nt_kernel[lm_head fwd rows x H x V]", "mfma", 2.0 * rows * h * v,
        time_events(torch, lambda: gemm.gemm_nt(x, w, out=logits), 5), 0 if epi_default else k_steps)
    lab = torch.randint(0, v, (rows,), device=device)
    lab[torch.rand(rows, device=device) > 0.7] = -100
    live = int((lab != -100).sum())
    lg = logits.detach().requires_grad_(True)
    out = label_cross_entropy(lg, lab)
    rec("label_ce_fwd_kernel[rows x V, 70% live rows]", "hbm", live * v * 2.0,
        time_events(torch, lambda: label_cross_entropy(logits, lab), 5), 0 if epi_default else k_steps)
    # the head product with every row's log-sum-exp out of its epilogue + one element per row for the loss:
    # what replaces the two launches above in the model
    lse_buf = torch.empty(rows, device=device)
    st_ws = torch.empty(_lib.load().spx_gemm_stats_workspace_bytes(rows, v) // 4, device=device)
    loss_buf = torch.empty(rows, device=device)
    stp = _lib.stream_ptr(device)

    def head_stats_ce():
        _lib.call("spx_gemm_bf16_nt_stats", _lib.ptr(x), x.stride(0), _lib.ptr(w), w.stride(0), _lib.ptr(logits),
                  logits.stride(0), rows, v, h, _lib.ptr(lse_buf), None, _lib.ptr(st_ws), st_ws.numel() * 4, stp)
        _lib.call("spx_label_ce_from_lse", _lib.ptr(logits), logits.stride(0), _lib.ptr(lab), rows, v,
                  _lib.dtype_code(logits), -100, _lib.ptr(lse_buf), _lib.ptr(loss_buf), stp)

    rec("gemm_bf16_nt_kernel<statistics epilogue> + reduce + label_ce_pick[lm_head fwd + CE rows x H x V]", "mfma",
        2.0 * rows * h * v, time_events(torch, head_stats_ce, 5), k_steps if epi_default else 0)
    del st_ws
    go = torch.ones_like(out)

    def ce_bwd():
        lg.grad = None
        out.backward(go, retain_graph=True)

    # live rows: one read + one write; dead rows: one write of zeros
    rec("label_ce_bwd_kernel[rows x V, 70% live rows]", "hbm", (2 * live + (rows - live)) * v * 2.0,
        time_events(torch, ce_bwd, 5), k_steps)
    dl = lg.grad
    del lg, out
    wt = w.detach().t().contiguous()
    rec("gemm_bf16_nt_kernel[lm_head dX rows x V x H, all rows]", "mfma",
        2.0 * rows * h * v, time_events(torch, lambda: gemm.gemm_nt(dl, wt), 3), k_steps)
    del dl, logits, wt
    torch.cuda.empty_cache()
    hq, hkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    t_row = n - k_steps - 1
    doc = torch.arange(b, device=device).repeat_interleave(t_row)
    mask = create_ttt_mask(doc, b * t_row, None)
    q = torch.randn(1, hq, b * t_row, d, device=device).bfloat16().requires_grad_(True)
    kk = torch.randn(1, hkv, b * t_row, d, device=device).bfloat16().requires_grad_(True)
    vv = torch.randn(1, hkv, b * t_row, d, device=device).bfloat16().requires_grad_(True)
    pairs = b * t_row * (t_row + 1) / 2
    rec("attn_fwd_kernel[head_dim 256, causal per row]", "mfma", 4.0 * pairs * d * hq,
        time_events(torch, lambda: ttt_attention(q.detach(), kk.detach(), vv.detach(), mask, d ** -0.5), 3),
        k_steps)
    o = ttt_attention(q, kk, vv, mask, d ** -0.5)
    gd = torch.randn_like(o)

    def attn_bwd():
        q.grad = kk.grad = vv.grad = None
        o.backward(gd, retain_graph=True)

    rec("attn_bwd[head_dim 256, causal per row]", "mfma", 10.0 * pairs * d * hq,
        time_events(torch, attn_bwd, 3), k_steps)
    del q, kk, vv, o, gd
    if hybrid:
        from speculators_amd import moe

        e, topk, inter = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size
        tok = b * t_row
        idx = torch.stack([torch.randperm(e, device=device)[:topk] for _ in range(64)]).repeat(tok // 64 + 1, 1)[:tok]
        _, src_row, _, off = moe.sort_pairs(idx, e)
        pairs_n = tok * topk
        xs = torch.randn(pairs_n, h, device=device).bfloat16()
        w_gu = (torch.randn(e, 2 * inter, h, device=device) * 0.02).bfloat16()
        hid = moe.gemm_nt_grouped(xs, w_gu, off)
        rec("gemm_bf16_nt_kernel[grouped: experts' gate+up, T*k rows x H x 2I, 512 groups]", "mfma",
            2.0 * pairs_n * h * 2 * inter, time_events(torch, lambda: moe.gemm_nt_grouped(xs, w_gu, off, out=hid), 3),
            k_steps)
        dw = torch.empty(e, 2 * inter, h, device=device, dtype=torch.float32)
        rec("gemm_bf16_tn_kernel[grouped: experts' gate+up weight gradient, fp32]", "mfma",
            2.0 * pairs_n * h * 2 * inter, time_events(torch, lambda: moe.gemm_tn_grouped(hid, xs, off, dw), 3),
            k_steps)
        xt = torch.randn(tok, h, device=device).bfloat16()
        rec("gather_rows_kernel[T*k rows of H]", "hbm", 2.0 * pairs_n * h * 2,
            time_events(torch, lambda: moe.gather_rows(xt, src_row), 3), 2 * k_steps)
        del xs, w_gu, hid, dw, xt
    dominant = max(kernels, key=lambda r: r["ms_per_launch"] * r["launches_per_step"])

    cpu = None
    if args.cpu_baseline != "off":
        from oracle import mtp as OM
        from oracle.eagle3 import DraftShape

        if hybrid:
            shape = OM.HybridShape(draft_vocab_size=CONFIG4["vocab_size"], **CONFIG4, **NEXT_EXTRA)
        else:
            shape = DraftShape(draft_vocab_size=CONFIG4["vocab_size"], qk_norm=True, **CONFIG4)
        tn = args.cpu_seq_len
        torch.set_num_threads(os.cpu_count() or 1)
        if hybrid:
            # 512 expert stacks in fp32 with their gradients: one short row pair bounds the time (the
            # experts' weight-gradient stacks cost the same whatever the length); eight random experts
            # tiled 64 times (the values do not matter for the time, drawing 1.6 G normals does)
            tn = min(tn, 128)
            few = OM.random_weights(OM.HybridShape(draft_vocab_size=CONFIG4["vocab_size"], **CONFIG4,
                                                   **dict(NEXT_EXTRA, num_experts=8)), 0)
            reps = NEXT_EXTRA["num_experts"] // 8
            raw = {k_: (v_.repeat(reps, *([1] * (v_.dim() - 1))) if ".mlp.gate.weight" in k_ or ".experts." in k_
                        else v_) for k_, v_ in few.items()}
        else:
            raw = OM.random_weights(shape, 0)
        wts = {k_: v_.requires_grad_(k_ not in ("embed_tokens.weight", "lm_head.weight")) for k_, v_ in raw.items()}
        cg = torch.Generator().manual_seed(0)
        cids = torch.randint(0, shape.vocab_size, (b, tn), generator=cg)
        chs = torch.randn(b, tn, shape.hidden_size, generator=cg)

        def cpu_step():
            for v_ in wts.values():
                v_.grad = None
            _, l_, _ = OM.mtp_forward(wts, shape, cids, chs, step_weights=sw, num_steps=k_steps, attn="sdpa")
            l_.backward()

        if not hybrid:
            cpu_step()
        c0 = time.perf_counter()
        cpu_step()
        cdt = time.perf_counter() - c0
        cpu = {"value": round(b * tn / cdt, 2), "unit": "tokens/s", "cores": torch.get_num_threads(),
               "kind": "port", "sample": f"oracle MTP forward+backward, configs[4] shape at batch {b} x seq {tn}, "
                                         + ("fp32, qwen3_next layer with 512 experts (8 random ones tiled), one timed "
                                            "iteration, no warm-up" if hybrid else
                                            "fp32, 1 warm-up + 1 timed iteration")}
    print(json.dumps({
        "metric": "MTP train tokens/sec (fwd+bwd) @Qwen3-Next-like MTP head, full-vocab CE",
        "value": round(tokens / (ms_per_step * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": (f"configs[4] shape with the qwen3_next layer: gated attention, rotary on 64 of 256, "
                                f"512 experts top-10 of width 512 + shared expert 512, hidden 2048, 16 q / 2 kv "
                                f"heads, head_dim 256, vocab 151936, batch {b}, seq {n}, {k_steps} prediction "
                                f"steps, label cross-entropy, loss_mask Bernoulli(0.7)") if hybrid else
                               f"configs[4]: MTP head, one Qwen3 decoder layer, hidden 2048, 16 q / 2 kv heads, "
                               f"head_dim 256, FFN 6144 (assumed), vocab 151936, batch {b}, seq {n}, "
                               f"{k_steps} prediction steps, label cross-entropy, loss_mask Bernoulli(0.7)",
                   "seq_len": n, "batch": b, "steps": k_steps, "tokens_per_step": tokens,
                   "final_loss": round(final_loss, 6)},
        "roofline": {k_: dominant[k_] for k_ in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
                    | {"kernel": dominant["kernel"]},
        "head_cross_entropy_statistics": head_stats,
        "kernels": kernels, "cpu_baseline": cpu}))


# configs[2]: DFlash on a Qwen3-8B shaped verifier.  5 draft layers (the reference default for
# dflash), every layer windowed; 512 anchors on a uniform non-overlapping grid.
CONFIG2 = dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=12288, vocab_size=151936, draft_vocab_size=32000, num_aux=5,
               num_hidden_layers=5, rms_norm_eps=1e-6, rope_theta=1000000.0, block_size=16,
               mask_token_id=151935, sliding_window=2048, sliding_layers=(0, 1, 2, 3, 4))
DFLASH_SEQ_LEN, DFLASH_ANCHORS = 8192, 512


def run_dflash(args):
    """configs[2]: DFlash forward + backward, tokens/s over the T context positions, and the
    roofline of the anchored-block attention."""
    import torch

    from speculators_amd import _lib
    from speculators_amd import attention as A
    from speculators_amd.dflash import DFlashConfig, DFlashDraftModel
    from speculators_amd.losses import resolve_loss_config

    _lib.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    t = args.seq_len if args.seq_len != SEQ_LEN else DFLASH_SEQ_LEN
    cfg = DFlashConfig(**CONFIG2)
    bs, n_anchor = cfg.block_size, DFLASH_ANCHORS
    torch.manual_seed(0)
    model = DFlashDraftModel(cfg)
    with torch.no_grad():
        for name, p_ in model.named_parameters():
            if name.endswith("norm.weight") or "layernorm" in name:
                p_.fill_(1.0)
            else:
                p_.normal_(0.0, 0.02)
    g = torch.Generator().manual_seed(0)
    sel = torch.randperm(cfg.vocab_size, generator=g)[:cfg.draft_vocab_size].sort().values
    t2d = torch.zeros(cfg.vocab_size, dtype=torch.bool)
    t2d[sel] = True
    model.t2d.copy_(t2d)
    model.d2t.copy_(sel - torch.arange(cfg.draft_vocab_size))
    model = model.to(torch.bfloat16).to(device)
    hs = (torch.randn(1, t, cfg.num_aux * cfg.hidden_size, generator=g) * 4).bfloat16().to(device)
    vl = torch.randn(1, t, cfg.hidden_size, generator=g).bfloat16().to(device)
    ids = torch.randint(0, cfg.vocab_size, (1, t), generator=g).to(device)
    lm = (torch.rand(1, t, generator=g) < 0.7).float().to(device)
    doc = torch.zeros(1, t, dtype=torch.long, device=device)
    stride = (t - bs) // n_anchor
    anchor_pos = (torch.arange(n_anchor) * stride + 1).to(device)
    anchors = (anchor_pos, torch.ones(n_anchor, dtype=torch.bool, device=device))
    loss_config = resolve_loss_config("kl_div", "hip")

    def step():
        model.zero_grad(set_to_none=True)
        _, loss, _ = model(hs, ids, lm, vl, doc, loss_config=loss_config, anchors=anchors)
        loss.backward()
        return loss

    for _ in range(args.warmup):
        step()
    with quiet_gc():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = step()
        torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    final_loss = float(loss.detach())
    del loss
    model.zero_grad(set_to_none=True)

    kernels = []
    hq, hkv, d, w = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.sliding_window
    n_q = n_anchor * bs
    # live (query, key) pairs: the context window in front of the anchor + the causal part of the block
    pairs = float((torch.clamp(anchor_pos.cpu(), max=w) * bs).sum() + n_anchor * bs * (bs + 1) // 2)
    mask = A.create_dflash_mask(doc.reshape(-1), t, anchor_pos, bs, w, False)
    gq = torch.Generator(device=device).manual_seed(1)
    q = torch.randn(1, hq, n_q, d, device=device, generator=gq).bfloat16().requires_grad_(True)
    kk = torch.randn(1, hkv, t + n_q, d, device=device, generator=gq).bfloat16().requires_grad_(True)
    vv = torch.randn(1, hkv, t + n_q, d, device=device, generator=gq).bfloat16().requires_grad_(True)

    def rec(name, flops, ms, launches):
        tf = flops / (ms * 1e-3) / 1e12
        kernels.append({"kernel": name, "bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                        "algorithmic_flops": flops, "ms_per_launch": round(ms, 4),
                        "launches_per_step": launches})

    ms_f = time_events(torch, lambda: A.dflash_attention(q.detach(), kk.detach(), vv.detach(), mask), 10)
    rec(f"attn_fwd_kernel[DFlash, {n_anchor} anchors x block {bs}, window {w}]", 4.0 * pairs * d * hq, ms_f,
        cfg.num_hidden_layers)
    o = A.dflash_attention(q, kk, vv, mask)
    go = torch.randn_like(o)
    ms_b = time_events(torch, lambda: torch.autograd.grad(o, (q, kk, vv), go, retain_graph=True), 10)
    rec(f"attn_bwd[DFlash, {n_anchor} anchors x block {bs}, window {w}]", 10.0 * pairs * d * hq, ms_b,
        cfg.num_hidden_layers)
    dominant = max(kernels, key=lambda r: r["ms_per_launch"] * r["launches_per_step"])
    print(json.dumps({
        "metric": "draft train tokens/sec (fwd+bwd) @Qwen3-8B DFlash", "value": round(t / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"configs[2]: DFlash draft, Qwen3-8B shape, {cfg.num_hidden_layers} layers, seq {t}, "
                               f"{n_anchor} anchors x block {bs} (queries {n_q}, keys {t + n_q}), window {w} on "
                               "every layer, 5 auxiliary layers, vocab 151936 -> draft 32000, kl_div loss",
                   "seq_len": t, "anchors": n_anchor, "block_size": bs, "tokens_per_step": t,
                   "final_loss": round(final_loss, 6)},
        "roofline": {k_: dominant[k_] for k_ in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
                    | {"kernel": dominant["kernel"]},
        "kernels": kernels, "cpu_baseline": None}))


def _decoder_gemm_mode():
    """Whose GEMM ran the decoder-layer projections (SPX_DECODER_GEMM, see speculators_amd/gemm.py)."""
    from speculators_amd import gemm

    return gemm.DECODER_GEMM


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (no collectives are built); got --gpus {args.gpus}",
              file=sys.stderr)
        sys.exit(2)
    if args.workload in ("mtp", "mtp-next"):
        run_mtp(args)
        return
    if args.workload == "dflash":
        run_dflash(args)
        return
    import torch

    from speculators_amd import _lib

    _lib.load()  # fail loudly if the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    t, k_steps = args.seq_len, args.ttt_steps
    big = args.workload == "eagle3-70b"
    CONFIG1 = CONFIG3 if big else globals()["CONFIG1"]  # noqa: N806 - the config of this run
    if big:
        t = SEQ_LEN3 if t == SEQ_LEN else t
        k_steps = TTT_STEPS3 if k_steps == TTT_STEPS else k_steps
    REF_WINDOW = 2048  # noqa: N806 - the reference's default sliding window (train/config/schema.py:172-183)
    head_window = args.window or None
    # the attention kernels are timed with the headline's mask and with the reference default's
    kernel_windows = (head_window,) if head_window else (None, REF_WINDOW)
    if args.only_kernels:
        print(json.dumps({"kernels": kernel_rooflines(torch, CONFIG1, t, k_steps, device, kernel_windows)}))
        return
    batch, d2t, t2d = make_inputs(torch, CONFIG1, t, device, args.targets == "logits")
    from speculators_amd import losses as losses_mod
    loss_cfg = None if args.loss == "kl_div" else losses_mod.resolve_loss_config(args.loss)  # None = kl_div
    autocast = args.regime == "autocast"

    def build(auto, window=head_window):
        cfg = dict(CONFIG1)
        if window:  # every draft layer sliding-window, as scripts/train.py builds them by default
            cfg.update(sliding_window=window, sliding_layers=(0,))
        mdl = make_model(torch, cfg, device, d2t, t2d, torch.float32 if auto else torch.bfloat16)

        def one_step():
            mdl.zero_grad(set_to_none=True)
            with torch.autocast("cuda", dtype=torch.bfloat16, enabled=auto):
                _, loss_, _ = mdl(**batch, ttt_steps=k_steps, ttt_step_loss_decay=1.0, loss_config=loss_cfg)
            loss_.backward()
            return loss_
        return mdl, one_step

    # the other regime first, timed the same way (reported beside the headline, not as `value`)
    model, step = build(not autocast)
    for _ in range(args.warmup):
        step()
    with quiet_gc():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = step()
        torch.cuda.synchronize()
    other_ms = (time.perf_counter() - t0) / args.steps * 1e3
    other_loss = float(loss.detach())
    del model, step, loss
    torch.cuda.empty_cache()

    # the reference's default training configuration beside the headline: the same step with every
    # draft layer sliding-window (W = 2048), same regime, same inputs
    ref_default = None
    if not head_window and t > REF_WINDOW:
        model, step = build(autocast, REF_WINDOW)
        for _ in range(args.warmup):
            step()
        with quiet_gc():
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                loss = step()
            torch.cuda.synchronize()
        w_ms = (time.perf_counter() - t0) / args.steps * 1e3
        ref_default = {"sliding_window": REF_WINDOW, "sliding_layers": "all", "regime": args.regime,
                       "ms_per_step": round(w_ms, 3), "value": round(t / (w_ms * 1e-3), 1), "unit": "tokens/s",
                       "final_loss": round(float(loss.detach()), 6),
                       "note": "what scripts/train.py trains by default (scripts/train.py:176-179,498-506); "
                               "BASELINE's configs[1] names no window, so the headline above is full attention"}
        del model, step, loss
        torch.cuda.empty_cache()

    # the other entry point beside the headline: targets handed over as full-vocabulary verifier logits, whose
    # first TTT step gathers through d2t inside the loss pass (spx_vocab_loss_step_fwd)
    other_entry = None
    if not head_window:
        alt = "hidden" if args.targets == "logits" else "logits"
        saved = batch
        batch, _d2t, _t2d = make_inputs(torch, CONFIG1, t, device, alt == "logits")
        model, step = build(autocast)
        for _ in range(args.warmup):
            step()
        with quiet_gc():
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                loss = step()
            torch.cuda.synchronize()
        a_ms = (time.perf_counter() - t0) / args.steps * 1e3
        other_entry = {"targets": alt, "regime": args.regime, "ms_per_step": round(a_ms, 3),
                       "value": round(t / (a_ms * 1e-3), 1), "unit": "tokens/s",
                       "final_loss": round(float(loss.detach()), 6),
                       "note": ("full-vocabulary verifier logits gathered through d2t in the first step's loss pass "
                                "(no verifier-head product)" if alt == "logits" else
                                "verifier hidden states through the frozen verifier head")}
        del model, step, loss
        batch = saved
        torch.cuda.empty_cache()

    model, step = build(autocast)
    for _ in range(args.warmup):
        step()
    # the lm_head forward product (and the verifier head, the same shape) is timed where it runs:
    # two events around each of its launches inside the timed steps
    probe = GemmProbe(torch, t, CONFIG1["draft_vocab_size"], CONFIG1["hidden_size"])
    with quiet_gc(), probe:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = step()
        torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tokens = int((batch["document_ids"] != -1).sum().item())
    value = tokens / (ms_per_step * 1e-3)

    kernels = [] if args.no_kernels else kernel_rooflines(torch, CONFIG1, t, k_steps, device, kernel_windows)
    in_step = probe.mean_ms()
    for rec in kernels:
        if rec["kernel"].startswith("gemm_bf16_nt_kernel[lm_head fwd") and in_step:
            # the figure of record is the one from the timed steps; the back-to-back one stays beside it
            rec["ms_per_launch_back_to_back"] = rec["ms_per_launch"]
            rec["ms_per_launch"] = round(in_step, 4)
            tf = rec["algorithmic_flops"] / (in_step * 1e-3) / 1e12
            rec["achieved"], rec["frac"] = round(tf, 1), round(tf / PEAK_BF16_TFLOPS, 4)
            rec["timed"] = (f"HIP events around each of the {len(probe.pairs)} launches of this shape "
                            f"inside the {args.steps} timed steps")
    dominant = None
    if kernels:
        dominant = max(kernels, key=lambda r: r["ms_per_launch"] * r["launches_per_step"])
        kernels = [k for k in kernels if k["launches_per_step"] > 0] + \
                  [k for k in kernels if k["launches_per_step"] == 0]
    cpu = None
    if args.cpu_baseline != "off":
        del model
        torch.cuda.empty_cache()
        cpu = cpu_baseline(torch, device, CONFIG1, args.cpu_seq_len, k_steps)

    line = {
        "metric": ("draft train tokens/sec (fwd+bwd) @Llama-3.1-70B EAGLE3 TTT5" if big else
                   "draft train tokens/sec (fwd+bwd) @Llama-3.1-8B EAGLE3 TTT7"),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": ("configs[3]: EAGLE3 draft, Llama-3.1-70B shape, one draft layer, " if big else
                                "configs[1]: EAGLE3 draft, Llama-3.1-8B shape, one draft layer, ")
                               +
                               f"batch 1, seq {t}, TTT {k_steps}, vocab 128256 -> draft 32000, "
                               f"{args.loss} loss, "
                               + ("fp32 master weights under torch.autocast(bf16), fp32 gradients "
                                  "(the reference Trainer's regime), " if autocast else
                                  "bf16 weights and activations (whole model cast), ")
                               + (f"sliding window {head_window} on every layer, " if head_window else "full attention, ")
                               + f"targets from {'verifier hidden states through the frozen verifier head' if args.targets == 'hidden' else 'full-vocab verifier logits gathered through d2t'}",
                   "seq_len": t, "ttt_steps": k_steps, "tokens_per_step": tokens,
                   "regime": args.regime, "final_loss": round(float(loss.detach()), 6),
                   "sliding_window": head_window, "decoder_gemm": _decoder_gemm_mode()},
        "reference_default_config": ref_default,
        "other_targets_entry": other_entry,
        "other_regime": {"regime": "bf16" if autocast else "autocast", "ms_per_step": round(other_ms, 3),
                         "value": round(tokens / (other_ms * 1e-3), 1), "unit": "tokens/s",
                         "final_loss": round(other_loss, 6)},
        "roofline": ({k: dominant[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
                     | {"kernel": dominant["kernel"]}) if dominant else None,
        "kernels": kernels,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
