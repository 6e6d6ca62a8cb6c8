"""Device batch producer (``spx_pack_batch`` through ``BatchPacker`` / ``PackedBatchLoader``)
against the CPU restatement of the reference's collate: bit-exact, every key."""

import pytest
import torch
from safetensors.torch import save_file

from oracle import data as OD

pytestmark = pytest.mark.gpu

_PRE = {"eagle3": OD.shift_eagle3, "dflash": None, "mtp": OD.shift_mtp}


def _raw(seq, layers, hidden, g, dtype, mask_dtype=torch.int64):
    return {"hidden_states": (torch.randn(seq, layers + 1, hidden, generator=g) * 3).to(dtype),
            "token_ids": torch.randint(0, 128000, (seq,), generator=g),
            "loss_mask": torch.randint(0, 2, (seq,), generator=g).to(mask_dtype)}


def _want(raws, max_len, hidden, layers, layout):
    samples = [None if r is None else OD.sample_from_file(r, r["loss_mask"]) for r in raws]
    return OD.collate(samples, max_len, hidden, layers, dtype=torch.bfloat16, preprocess=_PRE[layout])


def _check(got, want, empty=False):
    assert got.keys() == want.keys()
    for k, w in want.items():
        g = got[k].cpu()
        assert g.shape == w.shape, k
        if k == "loss_mask" and empty:
            assert not g.any()
            continue
        assert g.dtype == w.dtype, k
        if g.dtype == torch.bfloat16:
            assert torch.equal(g.view(torch.int16), w.view(torch.int16)), k
        else:
            assert torch.equal(g, w), k


@pytest.mark.parametrize("layout", ["eagle3", "dflash", "mtp"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("lens,max_len,hidden", [
    ([2, 6], 10, 8), ([5, 7], 11, 8), ([5, 1, 0, 7], 8, 16), ([1], 4, 8), ([9], 6, 8),
    ([3, 3, 3], 6, 8), ([], 5, 8), ([4, None, 3], 16, 8), ([37, 5, 90], 128, 64),
    ([6, 4], 9, 12),   # hidden not a multiple of 8: element-wise path
])
def test_pack_matches_collate(layout, dtype, lens, max_len, hidden):
    from speculators_amd.data import BatchPacker

    g = torch.Generator().manual_seed(sum(n or 0 for n in lens) + max_len)
    raws = [None if n is None else _raw(n, 3, hidden, g, dtype) for n in lens]
    packer = BatchPacker(max_len, hidden, 3, layout=layout, src_dtype=dtype)
    got = packer(raws)
    torch.cuda.synchronize()
    _check(got, _want(raws, max_len, hidden, 3, layout), empty=not lens)


@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.uint8, torch.int32, torch.int64])
def test_pack_mask_dtypes_and_slot_reuse(mask_dtype):
    from speculators_amd.data import BatchPacker

    g = torch.Generator().manual_seed(3)
    packer = BatchPacker(64, 32, 3, layout="eagle3", mask_dtype=mask_dtype, slots=2)
    for i in range(5):  # more batches than slots: every slot is staged again
        raws = [_raw(n, 3, 32, g, torch.bfloat16, mask_dtype) for n in (7 + i, 20, 3 * i + 1)]
        got = packer(raws)
        _check(got, _want(raws, 64, 32, 3, "eagle3"))


def test_pack_cast_special_values():
    """fp32 -> bf16 like the CPU cast of the collate: ties to even, NaN, infinities, denormals."""
    from speculators_amd.data import BatchPacker

    vals = torch.tensor([1.00390625, 1.01171875, -1.00390625, float("nan"), float("inf"), -float("inf"),
                         1e-40, 3.3895314e38, 0.0, -0.0, 65504.0, 1.0000001], dtype=torch.float32)
    hs = vals.repeat(4)[:32].reshape(1, 4, 8).repeat(3, 1, 1).contiguous()
    raw = {"hidden_states": hs, "token_ids": torch.arange(3), "loss_mask": torch.ones(3, dtype=torch.long)}
    got = BatchPacker(4, 8, 3, layout="dflash", src_dtype=torch.float32)([raw])
    want = _want([raw], 4, 8, 3, "dflash")
    for k in ("hidden_states", "verifier_last_hidden_states"):
        g, w = got[k].cpu(), want[k]
        nan = torch.isnan(w)
        assert nan.any() and torch.equal(torch.isnan(g), nan), k  # a NaN's payload is not defined
        assert torch.equal(g.view(torch.int16)[~nan], w.view(torch.int16)[~nan]), k


def test_pack_rejects_mismatched_samples():
    from speculators_amd._lib import SpxError
    from speculators_amd.data import BatchPacker

    g = torch.Generator().manual_seed(0)
    packer = BatchPacker(16, 8, 3)
    with pytest.raises(ValueError, match="expected"):
        packer([_raw(4, 2, 8, g, torch.bfloat16)])
    with pytest.raises(ValueError, match="built for"):
        packer([_raw(4, 3, 8, g, torch.float32)])
    bad = _raw(4, 3, 8, g, torch.bfloat16)
    bad["loss_mask"] = bad["loss_mask"][:3]
    with pytest.raises(ValueError, match="differ in length"):
        packer([bad])
    with pytest.raises(SpxError):
        BatchPacker(16, 8, 3, src_dtype=torch.float16)
    # the packer still works after the rejected batches
    raws = [_raw(5, 3, 8, g, torch.bfloat16)]
    _check(packer(raws), _want(raws, 16, 8, 3, "eagle3"))


@pytest.mark.parametrize("layout", ["eagle3", "mtp"])
def test_loader_over_hidden_state_files(tmp_path, layout):
    """hs_{idx}.safetensors files -> pinned staging on a worker thread -> device batches."""
    from speculators_amd.data import BatchPacker, HiddenStatesFile, PackedBatchLoader

    g = torch.Generator().manual_seed(11)
    hidden, layers, max_len = 64, 3, 96
    raws, idx = {}, 0
    batches = []
    for lens in ([30, 40, 20], [96], [50, 70], [10], [], [33, 33, 33]):
        batch = []
        for n in lens:
            r = _raw(n, layers, hidden, g, torch.bfloat16)
            save_file({"hidden_states": r["hidden_states"], "token_ids": r["token_ids"]},
                      tmp_path / f"hs_{idx}.safetensors")
            raws[idx] = r
            batch.append(idx)
            idx += 1
        batches.append(batch)

    def samples():
        for batch in batches:
            yield [{"hidden_states": HiddenStatesFile(tmp_path / f"hs_{i}.safetensors"),
                    "loss_mask": raws[i]["loss_mask"]} for i in batch]

    packer = BatchPacker(max_len, hidden, layers, layout=layout, slots=2)
    seen = 0
    for got, batch in zip(PackedBatchLoader(packer, samples()), batches, strict=True):
        # consume on the current stream, as a training step would
        probe = got["hidden_states"].float().sum()
        _check(got, _want([raws[i] for i in batch], max_len, hidden, layers, layout), empty=not batch)
        assert torch.isfinite(probe)
        seen += 1
    assert seen == len(batches)


def test_loader_hands_worker_errors_to_the_caller(tmp_path):
    from speculators_amd.data import BatchPacker, PackedBatchLoader

    g = torch.Generator().manual_seed(0)
    good = [_raw(5, 3, 8, g, torch.bfloat16)]
    packer = BatchPacker(16, 8, 3)
    it = iter(PackedBatchLoader(packer, [good, [_raw(5, 2, 8, g, torch.bfloat16)], good]))
    _check(next(it), _want(good, 16, 8, 3, "eagle3"))
    with pytest.raises(ValueError, match="expected"):
        next(it)
    # the packer is usable afterwards
    _check(packer(good), _want(good, 16, 8, 3, "eagle3"))


def test_packed_batch_feeds_the_draft_model():
    """The producer's keys are the keyword arguments of ``Eagle3DraftModel.forward``."""
    from speculators_amd.data import BatchPacker
    from speculators_amd.eagle3 import Eagle3Config, Eagle3DraftModel
    from speculators_amd.losses import resolve_loss_config

    g = torch.Generator().manual_seed(5)
    cfg = Eagle3Config(hidden_size=128, num_attention_heads=2, num_key_value_heads=1, head_dim=64,
                       intermediate_size=256, vocab_size=512, draft_vocab_size=512)
    torch.manual_seed(0)
    model = Eagle3DraftModel(cfg).cuda().to(torch.bfloat16)
    raws = [_raw(n, 3, 128, g, torch.bfloat16) for n in (40, 25)]
    for r in raws:
        r["token_ids"] %= 512
    batch = BatchPacker(64, 128, 3)(raws)
    _tokens, loss, metrics = model(**batch, ttt_steps=2, ttt_step_loss_decay=1.0,
                                   loss_config=resolve_loss_config("kl_div", "hip"))
    loss.backward()
    assert torch.isfinite(loss)
    want_total = float(_want(raws, 64, 128, 3, "eagle3")["loss_mask"].sum())
    assert float(metrics["full_acc_0_total"]) == want_total
