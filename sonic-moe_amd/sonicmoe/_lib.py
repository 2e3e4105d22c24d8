"""ctypes binding of libsonicmoe_hip.so (declared in include/sonicmoe_hip.h).

The library is the only compute path of the `sonicmoe` backend: if it is missing or fails to load, every operator
raises.  There is no eager / CPU fallback.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

_LIB: ctypes.CDLL | None = None

DT_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

_P, _I, _L, _Z = c_void_p, c_int, c_int64, c_size_t

_SIGNATURES = {
    "smoe_version": (c_int, []),
    "smoe_last_error": (c_char_p, []),
    "smoe_set_tuning": (c_int, [c_char_p, _I]),
    "smoe_count_cumsum": (c_int, [_P, _I, _L, _I, _P, _P, _P]),
    "smoe_topk_softmax_fwd": (c_int, [_P, _I, _L, _I, _I, _L, _P, _P, _I, _P]),
    "smoe_softmax_topk_bwd": (c_int, [_P, _I, _L, _P, _P, _P, _L, _I, _P]),
    "smoe_routing_metadata_workspace_bytes": (c_size_t, [_L, _I]),
    "smoe_routing_metadata": (c_int, [_P, _P, _L, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "smoe_routing_metadata_static_capacity": (c_size_t, []),
    "smoe_routing_metadata_static": (c_int, [_P, _P, _L, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P]),
    "smoe_gemm_workspace_bytes": (c_size_t, [_L, _I]),
    "smoe_fp8_gemm_workspace_bytes": (c_size_t, [_L, _I, _I]),
    "smoe_up_projection_forward": (
        c_int,
        [_P, _P, _L, _L, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _I, _P, _Z, _P],
    ),
    "smoe_down_projection_forward": (c_int, [_P, _P, _L, _L, _P, _P, _P, _P, _L, _I, _I, _I, _P, _Z, _P]),
    "smoe_down_projection_forward_combine": (c_int, [_P, _P, _L, _L, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _P, _Z, _P]),
    "smoe_gather_sum": (c_int, [_P, _P, _P, _P, _P, _L, _I, _I, _P]),
    "smoe_dz_partial_cols": (c_int, [_I]),
    "smoe_down_projection_backward": (
        c_int,
        [_P, _P, _P, _L, _L, _P, _P, _L, _L, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _I, _P, _Z,
         _P],
    ),
    "smoe_up_projection_backward": (
        c_int,
        [_P, _P, _L, _L, _P, _P, _L, _L, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _I, _P, _Z, _P],
    ),
    "smoe_router_weight_grad": (c_int, [_P, _P, _P, _L, _I, _I, _I, _P]),
    "smoe_router_fused_partials": (ctypes.c_int64, [_L, _I]),
    "smoe_router_forward_fused": (c_int, [_P, _P, _L, _I, _I, _I, _P, _P, _P, _P, _P]),
    "smoe_switch_loss_from_partials": (c_int, [_P, _L, _I, _P, _P, _P, _P]),
    "smoe_switch_loss_workspace_bytes": (c_size_t, [_L, _I]),
    "smoe_switch_loss_fwd": (c_int, [_P, _I, _L, _L, _I, _P, _P, _P, _P, _Z, _P]),
    "smoe_switch_loss_bwd": (c_int, [_P, _I, _L, _L, _I, _P, _P, _P, _P, _L, _P]),
    "smoe_tr_softmax": (c_int, [_P, _I, _L, _I, _L, _P, _P]),
    "smoe_tr_rank": (c_int, [_P, _P, _I, _P, _P, _L, _I, _I, _P]),
    "smoe_tr_select": (c_int, [_P, _I, _P, _P, _L, _I, _P]),
    "smoe_tr_row_counts": (c_int, [_P, _L, _I, _P, _P]),
    "smoe_tr_compact": (c_int, [_P, _P, _I, _P, _L, _I, _P, _P, _P, _P]),
    "smoe_mx_quantize": (c_int, [_P, _L, _L, _I, _P, _P, _P]),
    "smoe_mx_quantize_transposed": (c_int, [_P, _L, _L, _I, _I, _I, _P, _P, _P]),
    "smoe_mx_quantize_both": (c_int, [_P, _L, _L, _I, _I, _I, _P, _P, _P, _P, _P]),
    "smoe_down_projection_backward_fp8": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _I, _P, _Z, _P],
    ),
    "smoe_up_projection_forward_fp8": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _I, _P, _Z, _P],
    ),
    "smoe_down_projection_forward_fp8": (c_int, [_P, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _P, _Z, _P]),
    "smoe_score_grad_bias_term": (c_int, [_P, _P, _P, _P, _P, _P, _L, _I, _I, _P]),
}


def library_path() -> Path:
    env = os.environ.get("SONICMOE_HIP_LIB")
    return Path(env) if env else Path(__file__).resolve().parent / "lib" / "libsonicmoe_hip.so"


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = library_path()
        if not path.exists():
            raise RuntimeError(
                f"{path} not found: the HIP library is not built (run `python sonic-moe_amd/build.py`); "
                "the sonicmoe backend has no fallback path"
            )
        handle = ctypes.CDLL(str(path))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = handle
    return _LIB


def exported_symbols() -> list[str]:
    return list(_SIGNATURES)


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().smoe_last_error().decode(errors="replace")
        raise RuntimeError(f"{what} failed (status {rc}): {msg}")


def set_tuning(name: str, value: int) -> None:
    """Override a kernel-selection knob of the library (value < 0 restores the default)."""
    check(lib().smoe_set_tuning(name.encode(), int(value)), f"smoe_set_tuning({name}, {value})")


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def require_device(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("sonicmoe HIP operators need tensors on the GPU (got a CPU tensor)")


def current_stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream
