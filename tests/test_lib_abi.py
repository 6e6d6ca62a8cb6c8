"""The C-ABI library loads on a machine without a GPU and exports every symbol
that include/spx.h declares (no compute calls here)."""

import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "spx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = _declared_symbols()
    assert "spx_fused_vocab_loss_fwd" in names and "spx_version" in names


def test_library_exports_every_declared_symbol():
    from speculators_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail("libspx_hip.so is not built; run __graft_entry__.build()")
    lib = _lib.load()
    assert lib.spx_version() >= 100
    for name in _declared_symbols():
        assert hasattr(lib, name), name
    # every bound signature is declared in the header and vice versa
    assert set(_lib.SIGNATURES) | {"spx_version", "spx_last_error"} == set(_declared_symbols())


def test_argument_errors_do_not_need_a_gpu():
    from speculators_amd import _lib

    lib = _lib.load()
    rc = lib.spx_fused_vocab_loss_fwd(99, None, 0, None, 0, 1, 8, 0, None, None, None, None, None,
                                      None, 0, None)
    assert rc == 1 and b"unknown loss op" in lib.spx_last_error()
    rc = lib.spx_fused_vocab_loss_fwd(0, None, 4, None, 4, 1, 8, 0, None, None, None, None, None,
                                      None, 0, None)
    assert rc == 1 and b"stride" in lib.spx_last_error()


def test_host_tensors_are_refused():
    import torch

    from speculators_amd import _lib, losses

    with pytest.raises(_lib.SpxError):
        losses.kl_div_loss(torch.randn(1, 2, 8), torch.randn(1, 2, 8))


def test_resolve_loss_config_mirrors_reference_errors():
    from speculators_amd import losses as L

    assert L.resolve_loss_config("kl_div")["kl_div"] == (L.kl_div_loss, 1.0)
    cfg = L.resolve_loss_config('{"ce": 0.1, "tv": 0.9}')
    assert cfg["ce"] == (L.ce_loss, 0.1) and cfg["tv"] == (L.tv_loss, 0.9)
    for name in ("kl_div", "rkl", "jsd", "ce", "tv", "nla", "lk_hybrid"):
        assert name in L.resolve_loss_config(name)
    with pytest.raises(ValueError, match="Unknown loss implementation"):
        L.resolve_loss_config("kl_div", "triton")
    with pytest.raises(ValueError, match="Unknown loss function"):
        L.resolve_loss_config("nope")
    with pytest.raises(ValueError, match="non-empty JSON dict"):
        L.resolve_loss_config("[]")
    with pytest.raises(ValueError, match="Unknown loss function 'zz'"):
        L.resolve_loss_config('{"zz": 1}')
    with pytest.raises(ValueError, match="must be a number"):
        L.resolve_loss_config('{"ce": "x"}')
