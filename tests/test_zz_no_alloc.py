"""The allocation-free attention forward (scratch in a static device array) against the
entry point that takes a caller-owned workspace: bit-identical outputs on two calls in a row,
the second with a smaller input, and a clear refusal above the scratch limit."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(name_static: bool, q, k, v, row_lo, t, step, hq, hkv, d):
    from speculators_amd import _lib

    dev = q.device
    out = torch.full((1, t, hq, d), float("nan"), device=dev, dtype=torch.bfloat16)
    lse = torch.full((hq, t), float("nan"), device=dev, dtype=torch.float32)
    common = (_lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1), _lib.ptr(v), v.stride(1),
              _lib.ptr(row_lo), t, step, hq, hkv, d, float(d ** -0.5), _lib.ptr(out), _lib.ptr(lse))
    if name_static:
        _lib.call("spx_ttt_attn_fwd_static", *common, _lib.stream_ptr(dev))
    else:
        n = _lib.load().spx_ttt_attn_workspace_bytes(t, hq, hkv, d, 0)
        ws = torch.empty(n, device=dev, dtype=torch.uint8)
        _lib.call("spx_ttt_attn_fwd", *common, _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
    torch.cuda.synchronize()
    return out, lse


def test_static_scratch_forward_equals_workspace_forward_twice_then_smaller():
    from speculators_amd import _lib
    from speculators_amd.attention import create_ttt_mask

    lib = _lib.load()
    assert lib.spx_ttt_attn_fwd_static_max_bytes() == 16 << 20
    g = torch.Generator().manual_seed(0)
    # the second call is smaller than the first (fewer rows, fewer heads, another head size):
    # whatever the first left in the array must not reach the second's result
    for t, hq, hkv, d, step, window in [(1000, 8, 2, 128, 2, None), (200, 4, 1, 64, 1, 16),
                                        (4096, 32, 8, 128, 0, None)]:
        print(f"case T={t} Hq={hq} Hkv={hkv} D={d} step={step}", flush=True)
        doc = torch.zeros(1, t, dtype=torch.long)
        doc[0, t - 7:] = -1
        mask = create_ttt_mask(doc.cuda(), t, window)
        q = torch.randn(1, hq, t, d, generator=g).bfloat16().cuda()
        k = torch.randn(1, hkv, (step + 1) * t, d, generator=g).bfloat16().cuda()
        v = torch.randn(1, hkv, (step + 1) * t, d, generator=g).bfloat16().cuda()
        ref, ref_lse = _run(False, q, k, v, mask.row_lo, t, step, hq, hkv, d)
        got, got_lse = _run(True, q, k, v, mask.row_lo, t, step, hq, hkv, d)
        assert torch.isfinite(ref.float()).all()
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
        assert torch.equal(got_lse, ref_lse)
        # a further call (the set-up of this device and head size is done) takes no memory from the
        # device and none from torch's pool: free bytes and allocated bytes stand still across it
        out = torch.empty(1, t, hq, d, device="cuda", dtype=torch.bfloat16)
        lse = torch.empty(hq, t, device="cuda", dtype=torch.float32)
        torch.cuda.synchronize()
        free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        _lib.call("spx_ttt_attn_fwd_static", _lib.ptr(q), q.stride(1), _lib.ptr(k), k.stride(1), _lib.ptr(v),
                  v.stride(1), _lib.ptr(mask.row_lo), t, step, hq, hkv, d, float(d ** -0.5), _lib.ptr(out),
                  _lib.ptr(lse), _lib.stream_ptr(q.device))
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_static_scratch_rejects_shapes_above_its_limit():
    from speculators_amd import _lib

    lib = _lib.load()
    # 8 kv heads x 128 x 16384 rows x 2 bytes = 32 MiB > 16 MiB: refused before anything is read
    rc = lib.spx_ttt_attn_fwd_static(None, 0, None, 0, None, 0, None, 16384, 0, 32, 8, 128, 0.1,
                                     None, None, None)
    assert rc == 1 and b"16 MiB" in lib.spx_last_error()
