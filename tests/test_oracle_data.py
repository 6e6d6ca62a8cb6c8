"""Batch layout oracle against the reference's known answers, the row plan of the product
against the oracle (on the CPU, through an emulation of the kernel's index rule), and the
hidden-state file reader against the safetensors library."""

import pytest
import torch
from safetensors.torch import load_file, save_file

from oracle import data as OD
from speculators_amd import data as D


def _t(x, dtype=None):
    return torch.tensor(x, dtype=dtype)


# ---------------------------------------------------------------- known answers
def test_shift_known_answer():
    # tests/unit/train/test_data.py:16-51
    sample = {
        "input_ids": _t([0, 1, 2, 3, 4]),
        "hidden_states": _t([[0.0, 0.1, 0.2], [1.0, 1.1, 1.2], [2.0, 2.1, 2.2], [3.0, 3.1, 3.2],
                             [4.0, 4.1, 4.2]]),
        "verifier_last_hidden_states": _t([[10.0], [11.0], [12.0], [13.0], [14.0]]),
        "loss_mask": _t([0, 0, 1, 1, 1]),
        "lengths": _t([5]),
        "position_ids": _t([0, 1, 2, 3, 4]),
    }
    want = {
        "input_ids": _t([1, 2, 3, 4]),
        "hidden_states": _t([[0.0, 0.1, 0.2], [1.0, 1.1, 1.2], [2.0, 2.1, 2.2], [3.0, 3.1, 3.2]]),
        "verifier_last_hidden_states": _t([[11.0], [12.0], [13.0], [14.0]]),
        "loss_mask": _t([0, 1, 1, 1]),
        "lengths": _t([4]),
        "position_ids": _t([1, 2, 3, 4]),
    }
    got = OD.shift_eagle3(sample)
    assert got.keys() == want.keys()
    for k in want:
        assert torch.equal(got[k], want[k]), k


def _two_docs():
    return [
        {
            "input_ids": _t([0, 1]),
            "hidden_states": _t([[0.0, 0.1, 0.2], [1.0, 1.1, 1.2]]),
            "verifier_last_hidden_states": _t([[2.0], [3.0]]),
            "loss_mask": _t([0, 1]),
            "lengths": _t([2]),
            "position_ids": _t([0, 1]),
        },
        {
            "input_ids": _t([2, 3, 4, 5, 6, 7]),
            "hidden_states": _t([[4.0, 4.1, 4.2], [5.0, 5.1, 5.2], [6.0, 6.1, 6.2], [7.0, 7.1, 7.2],
                                 [8.0, 8.1, 8.2], [9.0, 9.1, 9.2]]),
            "verifier_last_hidden_states": _t([[10.0], [11.0], [12.0], [13.0], [14.0], [15.0]]),
            "loss_mask": _t([0, 0, 1, 0, 1, 1]),
            "lengths": _t([6]),
            "position_ids": _t([0, 1, 2, 3, 4, 5]),
        },
    ]


def test_collate_known_answer():
    # tests/unit/train/test_data.py:54-131 (the reference leaves the two padding rows
    # unchecked; they are zeros, document id -1)
    got = OD.collate(_two_docs(), 10, 1, 3, dtype=torch.float32)
    want = {
        "input_ids": _t([[0, 1, 2, 3, 4, 5, 6, 7, 0, 0]]),
        "hidden_states": _t([[[0.0, 0.1, 0.2], [1.0, 1.1, 1.2], [4.0, 4.1, 4.2], [5.0, 5.1, 5.2],
                              [6.0, 6.1, 6.2], [7.0, 7.1, 7.2], [8.0, 8.1, 8.2], [9.0, 9.1, 9.2],
                              [0, 0, 0], [0, 0, 0]]]),
        "verifier_last_hidden_states": _t([[[2.0], [3.0], [10.0], [11.0], [12.0], [13.0], [14.0],
                                            [15.0], [0], [0]]]),
        "loss_mask": _t([[0, 1, 0, 0, 1, 0, 1, 1, 0, 0]]),
        "document_ids": _t([[0, 0, 1, 1, 1, 1, 1, 1, -1, -1]]),
        "position_ids": _t([[0, 1, 0, 1, 2, 3, 4, 5, 0, 0]]),
    }
    assert got.keys() == want.keys()
    for k in want:
        assert got[k].dtype == want[k].dtype, k
        assert torch.equal(got[k], want[k]), k


def test_collate_casts_hidden_state_keys_only():
    # tests/unit/train/test_data.py:134-152
    got = OD.collate([{
        "input_ids": _t([0]), "hidden_states": torch.ones(1, 3),
        "verifier_last_hidden_states": torch.ones(1, 1), "loss_mask": _t([1]),
        "lengths": _t([1]), "position_ids": _t([0])}], 4, 1, dtype=torch.bfloat16)
    assert got["hidden_states"].dtype == torch.bfloat16
    assert got["verifier_last_hidden_states"].dtype == torch.bfloat16
    assert got["input_ids"].dtype == torch.long


def test_collate_truncation_known_answer():
    # tests/unit/train/test_data.py:155-200
    g = torch.Generator().manual_seed(0)
    docs = []
    for n in (5, 7):
        docs.append({"input_ids": torch.arange(n), "hidden_states": torch.randn(n, 24, generator=g),
                     "verifier_last_hidden_states": torch.randn(n, 8, generator=g),
                     "loss_mask": torch.ones(n, dtype=torch.long), "lengths": _t([n]),
                     "position_ids": torch.arange(n)})
    got = OD.collate(docs, 11, 8, 3, dtype=torch.float32)
    assert torch.equal(got["document_ids"], _t([[0] * 5 + [1] * 6]))
    assert "lengths" not in got
    for k in ("input_ids", "hidden_states", "verifier_last_hidden_states", "loss_mask", "position_ids"):
        assert got[k].shape[:2] == (1, 11)
    assert torch.equal(got["input_ids"][0], torch.cat([torch.arange(5), torch.arange(6)]))


def test_collate_empty_batch_is_all_padding():
    got = OD.collate([None, None], 6, 4, 3, dtype=torch.bfloat16, preprocess=OD.shift_eagle3)
    assert torch.equal(got["document_ids"], torch.full((1, 6), -1))
    assert got["hidden_states"].shape == (1, 6, 12) and not got["hidden_states"].any()
    assert got["loss_mask"].dtype == torch.bool


def test_kept_lengths():
    assert OD.kept_lengths([5, 7], 11) == [5, 6]
    assert OD.kept_lengths([5, 6, 3], 11) == [5, 6]  # reaching max_len exactly ends the row
    assert OD.kept_lengths([2, 0, 3], 11) == [2, 0, 3]
    assert OD.kept_lengths([0], 4) == [0]
    assert OD.kept_lengths([20, 3], 8) == [8]


# ---------------------------------------------------------------- row plan of the product
def _raw(seq, layers, hidden, g, dtype=torch.float32):
    return {"hidden_states": torch.randn(seq, layers + 1, hidden, generator=g).to(dtype),
            "token_ids": torch.randint(0, 1000, (seq,), generator=g),
            "loss_mask": torch.randint(0, 2, (seq,), generator=g)}


def _oracle_batch(raws, max_len, hidden, layers, layout, dtype=torch.bfloat16):
    pre = {"eagle3": OD.shift_eagle3, "dflash": None, "mtp": OD.shift_mtp}[layout]
    samples = [None if r is None else OD.sample_from_file(r, r["loss_mask"]) for r in raws]
    return OD.collate(samples, max_len, hidden, layers, dtype=dtype, preprocess=pre)


def _emulate_kernel(raws, max_len, layers, hidden, layout):
    """The index rule of the pack kernel, in Python, on the plan the product computes."""
    shift, has_aux, last_key = D.LAYOUTS[layout]
    live = [r for r in raws if r is not None]
    lengths = [r["token_ids"].shape[0] for r in live] or [0]
    src, out = D.plan_rows(lengths, max_len, shift)
    hs = (torch.cat([r["hidden_states"] for r in live]) if live
          else torch.zeros(0, layers + 1, hidden))
    ids = torch.cat([r["token_ids"] for r in live]) if live else torch.zeros(0, dtype=torch.long)
    mask = torch.cat([r["loss_mask"] for r in live]) if live else torch.zeros(0, dtype=torch.long)
    res = {"input_ids": torch.zeros(1, max_len, dtype=torch.long),
           "loss_mask": torch.zeros(1, max_len, dtype=mask.dtype),
           "position_ids": torch.zeros(1, max_len, dtype=torch.long),
           "document_ids": torch.full((1, max_len), -1, dtype=torch.long),
           last_key: torch.zeros(1, max_len, hidden, dtype=torch.bfloat16)}
    if has_aux:
        res["hidden_states"] = torch.zeros(1, max_len, layers * hidden, dtype=torch.bfloat16)
    n_docs = len(lengths)
    for r in range(out[n_docs]):
        d = max(i for i in range(n_docs) if out[i] <= r)
        o = r - out[d]
        s = src[d] + o
        if has_aux:
            res["hidden_states"][0, r] = hs[s, :layers].reshape(-1).to(torch.bfloat16)
        res[last_key][0, r] = hs[s + shift, layers].to(torch.bfloat16)
        res["input_ids"][0, r] = ids[s + shift]
        res["loss_mask"][0, r] = mask[s + shift]
        res["position_ids"][0, r] = o + shift
        res["document_ids"][0, r] = d
    return res


@pytest.mark.parametrize("layout", ["eagle3", "dflash", "mtp"])
@pytest.mark.parametrize("lens,max_len", [([2, 6], 10), ([5, 7], 11), ([5, 1, 0, 7], 8), ([1], 4),
                                          ([9], 6), ([3, 3, 3], 6), ([], 5), ([4, None, 3], 16)])
def test_row_plan_matches_oracle(layout, lens, max_len):
    g = torch.Generator().manual_seed(len(lens) * 100 + max_len)
    raws = [None if n is None else _raw(n, 3, 4, g) for n in lens]
    want = _oracle_batch(raws, max_len, 4, 3, layout)
    got = _emulate_kernel(raws, max_len, 3, 4, layout)
    assert got.keys() == want.keys()
    for k in want:
        if k == "loss_mask" and not lens:
            assert not got[k].any() and not want[k].any()  # the empty sample's mask is bool
            continue
        assert torch.equal(got[k], want[k]), k


# ---------------------------------------------------------------- file reader
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_hidden_states_file_reader(tmp_path, dtype):
    g = torch.Generator().manual_seed(1)
    hs = torch.randn(7, 4, 16, generator=g).to(dtype)
    ids = torch.randint(0, 50000, (7,), generator=g)
    path = tmp_path / "hs_3.safetensors"
    save_file({"token_ids": ids, "hidden_states": hs}, path)
    f = D.HiddenStatesFile(path)
    assert (f.seq_len, f.layers_plus_one, f.hidden_size, f.dtype) == (7, 4, 16, dtype)
    got, want = f.load(), load_file(path)
    assert torch.equal(got["hidden_states"], want["hidden_states"])
    assert torch.equal(got["token_ids"], want["token_ids"])
    # straight into a slice of a larger buffer
    big = torch.zeros(20, 4, 16, dtype=dtype)
    f.read_into("hidden_states", big[5:12])
    assert torch.equal(big[5:12], hs) and not big[:5].any() and not big[12:].any()
    with pytest.raises(ValueError, match="bytes"):
        f.read_into("hidden_states", big[5:11])
    with pytest.raises(ValueError, match="contiguous CPU"):
        f.read_into("token_ids", torch.zeros(7, dtype=torch.int32))


def test_hidden_states_file_rejects_other_files(tmp_path):
    save_file({"hidden_states": torch.zeros(3, 8)}, tmp_path / "a.safetensors")
    with pytest.raises(ValueError, match="token_ids"):
        D.HiddenStatesFile(tmp_path / "a.safetensors")
    save_file({"hidden_states": torch.zeros(3, 8), "token_ids": torch.zeros(3, dtype=torch.long)},
              tmp_path / "b.safetensors")
    with pytest.raises(ValueError, match="expected hidden_states"):
        D.HiddenStatesFile(tmp_path / "b.safetensors")


def test_packer_fails_without_a_device():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(Exception):  # noqa: B017 - no HIP device or library: never a host fallback
        D.BatchPacker(16, 8)(_raw(3, 3, 8, torch.Generator().manual_seed(0)))
    with pytest.raises(ValueError, match="unknown layout"):
        D.BatchPacker(16, 8, layout="nope")
