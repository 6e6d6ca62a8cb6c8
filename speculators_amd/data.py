"""Batch layout producer: hidden-state files -> pinned staging -> one HIP launch that
writes the packed training row.

The reference builds its batch on the host (train/data.py:293-303 splits the layers of a
file, models/eagle3/data.py:8-44 shifts tokens against hidden states, ``CollateFn``
train/data.py:323-393 packs samples into ``[1, max_len, ...]`` with ``document_ids``)
and then copies six tensors to the device (train/trainer.py:452-457).  Here the raw
file tensors are read straight into pinned host buffers, uploaded once on a side
stream, and ``spx_pack_batch`` produces every tensor of the batch on the device: the
layer split, the shift, the bf16 cast, the truncation at ``max_len``, the zero padding,
``position_ids`` and ``document_ids``.  ``PackedBatchLoader`` stages batch i+1 on a
worker thread while the model runs on batch i.

Layouts (the preprocess function the reference pairs with each model,
scripts/train.py:641-646):

==========  =====  ==============================================================
layout      shift  batch keys
==========  =====  ==============================================================
``eagle3``  1      hidden_states (aux layers), verifier_last_hidden_states, ...
``dflash``  0      the same keys, no shift
``mtp``     0      hidden_states = the last layer; no verifier_last_hidden_states
==========  =====  ==============================================================

Every layout also returns ``input_ids``, ``loss_mask``, ``position_ids`` and
``document_ids``, all ``[1, max_len]``.
"""

from __future__ import annotations

import json
import queue
import struct
import threading
from dataclasses import dataclass
from pathlib import Path

import torch

from . import _lib

LAYOUTS = {
    # name: (shift, has aux output, key of the last-layer output)
    "eagle3": (1, True, "verifier_last_hidden_states"),
    "peagle": (1, True, "verifier_last_hidden_states"),
    "dflash": (0, True, "verifier_last_hidden_states"),
    "mtp": (0, False, "hidden_states"),
}

_ST_DTYPES = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16,
              "I64": torch.int64, "I32": torch.int32, "BOOL": torch.bool, "U8": torch.uint8}


# ------------------------------------------------------------------ hidden-state files
@dataclass
class _Entry:
    dtype: torch.dtype
    shape: tuple
    begin: int
    end: int


class HiddenStatesFile:
    """One ``hs_{idx}.safetensors`` file (hs_connectors/src/hs_connectors/transfer.py:136-155):
    ``hidden_states [seq, layers + 1, hidden]`` and ``token_ids [seq]``.  Only the header
    is parsed on opening; ``read_into`` reads each tensor's bytes directly into a caller
    buffer (pinned memory), without an intermediate tensor."""

    def __init__(self, path):
        self.path = Path(path)
        with open(self.path, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            if n > 100_000_000:
                raise ValueError(f"{self.path}: implausible safetensors header length {n}")
            header = json.loads(f.read(n))
        self._data_offset = 8 + n
        self.entries: dict[str, _Entry] = {}
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            if meta["dtype"] not in _ST_DTYPES:
                raise ValueError(f"{self.path}: unsupported dtype {meta['dtype']} for '{name}'")
            self.entries[name] = _Entry(_ST_DTYPES[meta["dtype"]], tuple(meta["shape"]),
                                        *meta["data_offsets"])
        for need in ("hidden_states", "token_ids"):
            if need not in self.entries:
                raise ValueError(f"{self.path}: no '{need}' tensor")
        hs = self.entries["hidden_states"]
        if len(hs.shape) != 3 or self.entries["token_ids"].shape != (hs.shape[0],):
            raise ValueError(f"{self.path}: expected hidden_states [seq, layers + 1, hidden] and "
                             f"token_ids [seq], got {hs.shape} and {self.entries['token_ids'].shape}")
        self.seq_len, self.layers_plus_one, self.hidden_size = hs.shape
        self.dtype = hs.dtype

    def read_into(self, name: str, dst: torch.Tensor) -> None:
        """Fill ``dst`` (contiguous CPU tensor of the entry's dtype and element count)."""
        e = self.entries[name]
        if dst.dtype != e.dtype or not dst.is_contiguous() or dst.device.type != "cpu":
            raise ValueError(f"destination for '{name}' must be a contiguous CPU {e.dtype} tensor")
        if dst.numel() * dst.element_size() != e.end - e.begin:
            raise ValueError(f"destination for '{name}' holds {dst.numel() * dst.element_size()} "
                             f"bytes, the file {e.end - e.begin}")
        if dst.numel() == 0:
            return
        view = dst.view(torch.uint8).reshape(-1).numpy()
        with open(self.path, "rb", buffering=0) as f:
            f.seek(self._data_offset + e.begin)
            got = f.readinto(memoryview(view))
            while got < view.nbytes:  # short reads on large files
                more = f.readinto(memoryview(view)[got:])
                if not more:
                    raise OSError(f"{self.path}: truncated tensor '{name}'")
                got += more

    def load(self) -> dict:
        """Both tensors as ordinary CPU tensors."""
        out = {}
        for name in ("hidden_states", "token_ids"):
            e = self.entries[name]
            out[name] = torch.empty(e.shape, dtype=e.dtype)
            self.read_into(name, out[name])
        return out


# ------------------------------------------------------------------ row plan
def plan_rows(lengths, max_len: int, shift: int):
    """(src_start, out_start), two lists of ``len(lengths) + 1`` ints: where document d
    starts among the staged source rows, and where it starts in the packed row.  A
    document contributes ``max(len - shift, 0)`` rows; the row is cut at ``max_len``
    (documents beyond it keep an empty range), as the length bookkeeping of
    train/data.py:369-381 does."""
    src, out = [0], [0]
    for n in lengths:
        n = int(n)
        src.append(src[-1] + n)
        out.append(min(out[-1] + max(n - shift, 0), max_len))
    return src, out


class _Slot:
    """Pinned staging + device staging for one batch in flight."""

    def __init__(self, rows: int, layers_plus_one: int, hidden: int, src_dtype, mask_dtype,
                 max_docs: int, device):
        self.hs = torch.empty(rows, layers_plus_one, hidden, dtype=src_dtype, pin_memory=True)
        self.ids = torch.empty(rows, dtype=torch.int64, pin_memory=True)
        self.mask = torch.empty(rows, dtype=mask_dtype, pin_memory=True)
        self.plan = torch.zeros(2, max_docs + 1, dtype=torch.int64, pin_memory=True)
        self.d_hs = torch.empty_like(self.hs, device=device)
        self.d_ids = torch.empty_like(self.ids, device=device)
        self.d_mask = torch.empty_like(self.mask, device=device)
        self.d_plan = torch.empty_like(self.plan, device=device)
        self.rows = 0
        self.n_docs = 1
        self.done = None  # event: the pack kernel of the last use has finished
        self.free = threading.Event()  # set once the last use has been handed to the device
        self.free.set()


class BatchPacker:
    """``packer(samples)`` -> the batch dict of device tensors.

    ``samples``: a list whose items are ``None`` (a failed sample: skipped, as the collate
    of the reference skips it) or dicts with ``"hidden_states"`` (a ``[seq, layers + 1,
    hidden]`` CPU tensor, or a :class:`HiddenStatesFile`), ``"token_ids"`` (int64 ``[seq]``; taken
    from the file when a file is given) and ``"loss_mask"`` (``[seq]``).  An empty list gives
    an all-padding batch.
    """

    def __init__(self, max_len: int, hidden_size: int, num_target_layers: int = 3,
                 layout: str = "eagle3", device="cuda", src_dtype=torch.bfloat16,
                 mask_dtype=torch.int64, max_source_rows: int | None = None,
                 max_docs: int = 4096, slots: int = 2):
        if layout not in LAYOUTS:
            raise ValueError(f"unknown layout '{layout}', expected one of {sorted(LAYOUTS)}")
        if src_dtype not in (torch.bfloat16, torch.float32):
            raise _lib.SpxError("hidden-state sources must be bf16 or fp32")
        _lib.load()  # no host fallback: fail here when the HIP library is missing
        self.max_len, self.hidden_size, self.layers = max_len, hidden_size, num_target_layers
        self.layout = layout
        self.shift, self.has_aux, self.last_key = LAYOUTS[layout]
        self.device = torch.device(device)
        self.src_dtype, self.mask_dtype = src_dtype, mask_dtype
        self.max_docs = max_docs
        # staged rows: what fits the packed row plus the one extra row per document the
        # shift consumes, unless the caller sizes it
        self.max_source_rows = max_source_rows or (max_len + max_docs)
        if slots < 1:
            raise ValueError("slots must be at least 1")
        self._slots = [None] * slots
        self._next = 0
        self._abort = False
        self.stream = torch.cuda.Stream(device=self.device)

    def _slot(self) -> _Slot:
        i = self._next
        self._next = (i + 1) % len(self._slots)
        if self._slots[i] is None:
            self._slots[i] = _Slot(self.max_source_rows, self.layers + 1, self.hidden_size,
                                   self.src_dtype, self.mask_dtype, self.max_docs, self.device)
        slot = self._slots[i]
        # staged but not yet packed: wait for pack() (another thread) to take it
        while not slot.free.wait(0.1):
            if self._abort:
                raise RuntimeError("batch staging abandoned")
        slot.free.clear()
        if slot.done is not None:
            slot.done.synchronize()  # its previous upload and pack have drained
        return slot

    def stage(self, samples) -> _Slot:
        """Host part: copy / read the samples into a pinned slot and write the row plan."""
        slot = self._slot()
        try:
            self._fill(slot, samples)
        except BaseException:
            slot.free.set()  # a rejected batch leaves the slot reusable
            raise
        return slot

    def _fill(self, slot: _Slot, samples) -> None:
        lengths, at = [], 0
        room = self.max_len  # packed rows still free
        for s in samples:
            if s is None:
                continue
            if len(lengths) >= self.max_docs:
                raise ValueError(f"more than max_docs={self.max_docs} samples in one batch")
            hs = s["hidden_states"]
            is_file = isinstance(hs, HiddenStatesFile)
            seq = hs.seq_len if is_file else hs.shape[0]
            shape = ((hs.layers_plus_one, hs.hidden_size) if is_file else tuple(hs.shape[1:]))
            if shape != (self.layers + 1, self.hidden_size):
                raise ValueError(f"sample hidden states are [seq, {shape[0]}, {shape[1]}], "
                                 f"expected [seq, {self.layers + 1}, {self.hidden_size}]")
            if hs.dtype != self.src_dtype:
                raise ValueError(f"sample hidden states are {hs.dtype}, the packer was built for "
                                 f"{self.src_dtype}")
            if s["loss_mask"].shape[0] != seq:
                raise ValueError("loss_mask and hidden_states differ in length")
            # rows past the cut are never read by the kernel: do not stage them
            keep = min(seq, room + self.shift) if room > 0 else 0
            if at + keep > self.max_source_rows:
                raise ValueError(f"batch needs more than max_source_rows={self.max_source_rows} "
                                 "staged rows")
            if keep:
                if is_file and keep == seq:
                    hs.read_into("hidden_states", slot.hs[at:at + seq])
                    hs.read_into("token_ids", slot.ids[at:at + seq])
                else:
                    loaded = hs.load() if is_file else {"hidden_states": hs, "token_ids": s["token_ids"]}
                    slot.hs[at:at + keep].copy_(loaded["hidden_states"][:keep])
                    slot.ids[at:at + keep].copy_(loaded["token_ids"][:keep])
                slot.mask[at:at + keep].copy_(s["loss_mask"][:keep])
            lengths.append(keep)
            at += keep
            room -= max(keep - self.shift, 0)
        if not lengths:
            lengths = [0]
        src, out = plan_rows(lengths, self.max_len, self.shift)
        slot.plan[0, :len(src)] = torch.tensor(src, dtype=torch.int64)
        slot.plan[1, :len(out)] = torch.tensor(out, dtype=torch.int64)
        slot.rows, slot.n_docs = at, len(lengths)

    def pack(self, slot: _Slot) -> dict:
        """Device part: one upload per staged tensor and one kernel, on the packer's side
        stream; the returned tensors are ordered after them on the current stream."""
        t, h, dev = self.max_len, self.hidden_size, self.device
        consumer = torch.cuda.current_stream(dev)
        with torch.cuda.stream(self.stream):
            n = slot.rows
            if n:
                slot.d_hs[:n].copy_(slot.hs[:n], non_blocking=True)
                slot.d_ids[:n].copy_(slot.ids[:n], non_blocking=True)
                slot.d_mask[:n].copy_(slot.mask[:n], non_blocking=True)
            slot.d_plan.copy_(slot.plan, non_blocking=True)
            aux = (torch.empty(1, t, self.layers * h, device=dev, dtype=torch.bfloat16)
                   if self.has_aux else None)
            last = torch.empty(1, t, h, device=dev, dtype=torch.bfloat16)
            ids = torch.empty(1, t, device=dev, dtype=torch.int64)
            mask = torch.empty(1, t, device=dev, dtype=self.mask_dtype)
            pos = torch.empty(1, t, device=dev, dtype=torch.int64)
            doc = torch.empty(1, t, device=dev, dtype=torch.int64)
            _lib.call("spx_pack_batch", _lib.ptr(slot.d_hs), _lib.dtype_code(slot.d_hs), n,
                      self.layers, h, _lib.ptr(slot.d_ids), _lib.ptr(slot.d_mask),
                      slot.d_mask.element_size(), None, _lib.ptr(slot.d_plan[0]),
                      _lib.ptr(slot.d_plan[1]), slot.n_docs, t, self.shift, _lib.ptr(aux),
                      _lib.ptr(last), _lib.ptr(ids), _lib.ptr(mask), _lib.ptr(pos), _lib.ptr(doc),
                      self.stream.cuda_stream)
            slot.done = torch.cuda.Event()
            slot.done.record(self.stream)
        slot.free.set()
        consumer.wait_event(slot.done)
        batch = {"input_ids": ids, "loss_mask": mask, "position_ids": pos, "document_ids": doc}
        if self.has_aux:
            batch["hidden_states"] = aux
        batch[self.last_key] = last
        for v in batch.values():
            v.record_stream(consumer)  # allocated on the side stream, consumed on this one
        return batch

    def __call__(self, samples) -> dict:
        return self.pack(self.stage(samples))


class PackedBatchLoader:
    """Iterates device batches over ``batches`` (an iterable of sample lists).  A worker
    thread stages the next batch into pinned memory (file reads included) while the caller
    computes on the current one; uploads and the pack kernel run on the packer's side
    stream, so the copy of batch i+1 overlaps the step on batch i."""

    def __init__(self, packer: BatchPacker, batches, prefetch: int | None = None):
        self.packer = packer
        self.batches = batches
        if len(packer._slots) < 2:
            raise ValueError("prefetching needs a packer with at least two slots")
        depth = prefetch if prefetch is not None else len(packer._slots) - 1
        self.depth = max(1, min(depth, len(packer._slots) - 1))

    def __iter__(self):
        q: queue.Queue = queue.Queue(maxsize=self.depth)
        stop = threading.Event()
        self.packer._abort = False

        def put(item) -> bool:
            while not stop.is_set():
                try:
                    q.put(item, timeout=0.1)
                    return True
                except queue.Full:
                    continue
            return False

        def work():
            try:
                for samples in self.batches:
                    if not put(("slot", self.packer.stage(samples))):
                        return
                put(("end", None))
            except BaseException as exc:  # noqa: BLE001 - handed to the consumer thread
                put(("error", exc))

        th = threading.Thread(target=work, daemon=True, name="spx-batch-stager")
        th.start()
        try:
            while True:
                kind, item = q.get()
                if kind == "end":
                    return
                if kind == "error":
                    raise item
                yield self.packer.pack(item)
        finally:
            stop.set()
            self.packer._abort = True
            th.join(timeout=5)
            self.packer._abort = False
            for slot in self.packer._slots:  # a slot staged but never packed is free again
                if slot is not None:
                    slot.free.set()
