"""ctypes binding of ``libspx_hip.so``.

There is no CPU or PyTorch fallback: if the library is not built, or a call is
made with tensors that are not on a HIP device, the call raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SPX_LIB_PATH") or os.path.join(_HERE, "libspx_hip.so")

_P, _I64, _I, _F = c_void_p, c_int64, c_int, c_float

_I32 = c_int32

# name -> argument types (return type int unless listed in RESTYPES); mirrors include/spx.h
SIGNATURES: dict[str, list] = {
    "spx_vocab_gather": [_P, _I64, _P, _P, _I64, _I64, _I64, _I64, _I, _P],
    "spx_fused_vocab_loss_fwd": [_I, _P, _I64, _P, _I64, _I64, _I64, _I, _P, _P, _P, _P, _P, _P, _I,
                                 _P],
    "spx_fused_vocab_loss_bwd": [_I, _P, _I64, _P, _I64, _I64, _I64, _I, _P, _P, _P, _P, _P, _P, _P,
                                 _I64, _P],
    "spx_fused_vocab_loss_bwd_packed": [_I, _P, _I64, _P, _I64, _I64, _I64, _I, _P, _P, _P, _P, _P, _P, _P,
                                        _P, _I64, _P],
    "spx_ttt_step_reduce": [_P, _P, _P, _P, _I, _P, _I, _I64, _F, _P, _P, _P],
    "spx_block_reduce": [_P, _P, _P, _P, _I, _P, _I64, _I32, _P, _P, _P, _P, _P],
    "spx_ttt_row_lo": [_P, _I, _I64, _I64, _P, _P],
    "spx_ttt_attn_workspace_bytes": [_I64, _I32, _I32, _I32, _I32],
    "spx_ttt_attn_fwd": [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I32, _I32, _I32, _I32, _F, _P, _P,
                         _P, _I64, _P],
    "spx_ttt_attn_bwd": [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _I32,
                         _F, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _P],
}
SIGNATURES["spx_ttt_attn_bwd_accumulate"] = SIGNATURES["spx_ttt_attn_bwd"]
SIGNATURES["spx_vocab_loss_step_fwd"] = [_I, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I, _P, _P, _P,
                                         _P, _P, _P, _I, _P, _I, _P, _I, _P, _P]
SIGNATURES["spx_ttt_step_mean"] = [_P, _P, _I, _I64, _F, _P, _P, _P, _P]
SIGNATURES["spx_span_attn_fwd"] = [_P, _I64, _P, _I64, _P, _I64, _P, _P, _I64, _I32, _I32, _I32, _F, _P, _P,
                                   _P, _I64, _P]
SIGNATURES["spx_span_attn_bwd"] = [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _P, _P, _I64, _I32, _I32, _I32,
                                   _F, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _P]
SIGNATURES["spx_ttt_attn_fwd_static_max_bytes"] = []
SIGNATURES["spx_ttt_attn_fwd_static"] = [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I32, _I32, _I32, _I32, _F,
                                         _P, _P, _P]
SIGNATURES["spx_dflash_row_ranges"] = [_P, _I, _I64, _P, _I, _I64, _I32, _I64, _I32, _P, _P, _P, _P, _P, _P]
SIGNATURES["spx_dflash_attn_workspace_bytes"] = [_I64, _I64, _I32, _I32, _I32, _I32]
SIGNATURES["spx_dflash_attn_fwd"] = [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _P, _I64, _I64, _I32,
                                     _I32, _I32, _F, _P, _P, _P, _I64, _P]
SIGNATURES["spx_dflash_attn_bwd"] = [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _P, _P, _P, _P, _I64,
                                     _I64, _I32, _I32, _I32, _F, _P, _I64, _P, _I64, _P, _I64, _P,
                                     _I64, _P]
SIGNATURES["spx_rmsnorm_fwd"] = [_P, _I64, _P, _P, _I64, _P, _I64, _I64, _F, _P]
SIGNATURES["spx_rmsnorm_bwd_slots"] = [_I64, _I64]
SIGNATURES["spx_rmsnorm_bwd"] = [_P, _I64, _P, _P, _I64, _P, _P, _I64, _P, _P, _I64, _I64, _P]
SIGNATURES["spx_add_rmsnorm_fwd"] = [_P, _I64, _P, _I64, _P, _I64, _P, _P, _I64, _P, _I64, _I64, _F, _P]
SIGNATURES["spx_add_rmsnorm_bwd"] = [_P, _I64, _P, _P, _I64, _P, _I64, _P, _P, _I64, _P, _P, _I64, _I64, _P]
SIGNATURES["spx_rmsnorm_bwd_partial"] = [_P, _I64, _P, _P, _I64, _P, _I64, _P, _P, _I64, _P, _I32, _I64, _I64, _P]
SIGNATURES["spx_rmsnorm_dweight"] = [_P, _I64, _I64, _P, _P]
SIGNATURES["spx_rope_relayout"] = [_P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _I32, _I64, _P]
SIGNATURES["spx_swiglu_rows_fwd"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _P]
SIGNATURES["spx_swiglu_rows_bwd"] = [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _P]
SIGNATURES["spx_swiglu_fwd"] = [_P, _P, _P, _I64, _P]
SIGNATURES["spx_swiglu_bwd"] = [_P, _P, _P, _P, _P, _I64, _P]
SIGNATURES["spx_label_ce_fwd"] = [_P, _I64, _P, _I64, _I64, _I, _I64, _P, _P, _P, _P]
SIGNATURES["spx_label_ce_from_lse"] = [_P, _I64, _P, _I64, _I64, _I, _I64, _P, _P, _P]
SIGNATURES["spx_label_ce_bwd"] = [_P, _I64, _P, _P, _P, _I64, _I64, _I, _I64, _P, _I64, _P]
SIGNATURES["spx_label_ce_bwd_packed"] = [_P, _I64, _P, _P, _P, _I64, _I64, _I, _I64, _P, _P, _I64, _P]
SIGNATURES["spx_pack_batch"] = [_P, _I, _I64, _I64, _I64, _P, _P, _I, _P, _P, _P, _I64, _I64, _I,
                                _P, _P, _P, _P, _P, _P, _P]
SIGNATURES["spx_gemm_bf16_nt"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _P]
SIGNATURES["spx_pack_row_map"] = [_P, _P, _I64, _I64, _P, _P, _P]
SIGNATURES["spx_unpack_rows"] = [_P, _I64, _P, _I64, _I64, _I64, _P, _I64, _P]
SIGNATURES["spx_unpack_rows_scaled"] = [_P, _I64, _P, _P, _I64, _I64, _I64, _P, _I64, _P]
SIGNATURES["spx_vocab_loss_step_fwd_grad"] = [_I, _P, _I64, _P, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _I,
                                              _P, _I, _P, _I, _P, _P, _P, _I64, _P]
SIGNATURES["spx_gemm_bf16_nt_tail"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I32, _P, _I64, _P]
SIGNATURES["spx_gemm_tail_workspace_bytes"] = []
SIGNATURES["spx_gemm_bf16_nt_stats"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _P, _P, _P, _I64, _P]
SIGNATURES["spx_gemm_stats_workspace_bytes"] = [_I64, _I64]
SIGNATURES["spx_gemm_bf16_nt_rows"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _P, _P]
SIGNATURES["spx_gemm_bf16_nt_rows_split"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _P, _I32, _P, _I64, _P]
SIGNATURES["spx_gemm_bf16_tn"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I, _P]
SIGNATURES["spx_gemm_bf16_tn_f32"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I, _P]
SIGNATURES["spx_rope_relayout_partial"] = [_P, _I64, _I32, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _I32, _I32,
                                           _I64, _F, _P]
SIGNATURES["spx_sigmoid_gate_fwd"] = [_P, _I64, _P, _I64, _I32, _P, _I64, _I64, _I32, _I32, _P]
SIGNATURES["spx_sigmoid_gate_bwd"] = [_P, _I64, _P, _I64, _I32, _P, _I64, _P, _I64, _P, _I64, _I32, _I64, _I32,
                                      _I32, _P]
SIGNATURES["spx_gemm_grouped_workspace_bytes"] = [_I64, _I64]
SIGNATURES["spx_gemm_split_workspace_bytes"] = [_I64, _I64, _I32]
SIGNATURES["spx_gemm_bf16_nt_grouped"] = [_P, _I64, _P, _I64, _I64, _P, _I64, _I64, _I64, _I64, _P, _I64, _P,
                                          _I64, _P]
SIGNATURES["spx_gemm_bf16_tn_grouped"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I64, _P, _I64, _I, _I,
                                          _P]
SIGNATURES["spx_gemm_bf16_tn_grouped_multi"] = [_P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I64, _I64, _P, _I64,
                                                _I, _I, _P]
SIGNATURES["spx_transpose_bf16"] = [_P, _I64, _I64, _P, _I64, _I64, _I64, _I64, _I64, _P]
SIGNATURES["spx_moe_gather_rows"] = [_P, _I64, _I64, _P, _P, _P, _I64, _I64, _I64, _P]
SIGNATURES["spx_moe_combine_rows"] = [_P, _I64, _I64, _P, _P, _P, _I64, _I64, _I32, _I64, _P]
SIGNATURES["spx_moe_pair_dot"] = [_P, _I64, _P, _I64, _I64, _P, _P, _I64, _I32, _I64, _P]
RESTYPES = {"spx_gemm_grouped_workspace_bytes": c_int64, "spx_gemm_tail_workspace_bytes": c_int64, "spx_gemm_stats_workspace_bytes": c_int64, "spx_gemm_split_workspace_bytes": c_int64, "spx_ttt_attn_workspace_bytes": c_int64, "spx_ttt_attn_fwd_static_max_bytes": c_int64, "spx_dflash_attn_workspace_bytes": c_int64,
            "spx_rmsnorm_bwd_slots": c_int64}

_lib = None


class SpxError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SpxError(
            f"{LIB_PATH} is missing: build it with `make -C speculators_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path"
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.spx_version.restype = c_int
    lib.spx_version.argtypes = []
    lib.spx_last_error.restype = c_char_p
    lib.spx_last_error.argtypes = []
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = RESTYPES.get(name, c_int)
        fn.argtypes = argtypes
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise SpxError(f"{name} failed ({rc}): {lib.spx_last_error().decode()}")


def ptr(t: torch.Tensor | None):
    """Device pointer of a tensor (None -> NULL).  Refuses host tensors."""
    if t is None:
        return None
    if not t.is_cuda:
        raise SpxError("libspx_hip works on HIP device tensors only (got a CPU tensor)")
    return t.data_ptr()


def stream_ptr(device=None):
    return torch.cuda.current_stream(device).cuda_stream


DTYPE_CODE = {torch.bfloat16: 0, torch.float32: 1}
KIND_CODE = {
    torch.bool: 0, torch.uint8: 0, torch.int8: 0, torch.int32: 1, torch.int64: 2,
    torch.float32: 3, torch.bfloat16: 4,
}


def dtype_code(t: torch.Tensor) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise SpxError(f"unsupported dtype {t.dtype}: bf16 and f32 only") from None


def kind_code(t: torch.Tensor) -> int:
    try:
        return KIND_CODE[t.dtype]
    except KeyError:
        raise SpxError(f"unsupported mask dtype {t.dtype}") from None
