"""ctypes binding of libsonicmoe_hip.so and libsonicmoe_hip_f16.so (declared in include/sonicmoe_hip.h).

The two libraries are builds of the same sources with the same entry points: the first takes bfloat16 for the 16-bit
tensors of the GEMM-side operators, the second float16.  They are the only compute path of the `sonicmoe` backend: if
the one an operator needs is missing or fails to load, the operator raises.  There is no eager / CPU fallback.
"""

from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

_LIBS: dict[torch.dtype, ctypes.CDLL] = {}
_TLS = threading.local()           # .last = the library of this thread's latest lib() call: check() asks it for the
                                   # error text (the libraries keep their last error per thread as well)
_TUNING: dict[str, int] = {}       # overrides made so far, for a library that is loaded later

DT_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

_P, _I, _L, _Z = c_void_p, c_int, c_int64, c_size_t

_SIGNATURES = {
    "smoe_version": (c_int, []),
    "smoe_last_error": (c_char_p, []),
    "smoe_set_tuning": (c_int, [c_char_p, _I]),
    "smoe_count_cumsum": (c_int, [_P, _I, _L, _I, _P, _P, _P]),
    "smoe_topk_softmax_fwd": (c_int, [_P, _I, _L, _I, _I, _L, _P, _P, _I, _P]),
    "smoe_softmax_topk_bwd": (c_int, [_P, _I, _L, _P, _P, _P, _P, _L, _I, _P]),
    "smoe_topk_bwd": (c_int, [_P, _I, _L, _P, _P, _L, _I, _P]),
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


_LIB_FILES = {torch.bfloat16: ("libsonicmoe_hip.so", "SONICMOE_HIP_LIB"),
              torch.float16: ("libsonicmoe_hip_f16.so", "SONICMOE_HIP_LIB_F16")}


def library_path(dtype: torch.dtype = torch.bfloat16) -> Path:
    name, var = _LIB_FILES[dtype]
    env = os.environ.get(var)
    return Path(env) if env else Path(__file__).resolve().parent / "lib" / name


def lib(dtype: torch.dtype = torch.bfloat16) -> ctypes.CDLL:
    """The library whose 16-bit element type is `dtype` (operators without such tensors use the default)."""
    handle = _LIBS.get(dtype)
    if handle is None:
        if dtype not in _LIB_FILES:
            raise NotImplementedError(f"no build of the HIP library for {dtype} tensors (bfloat16 and float16 exist)")
        path = library_path(dtype)
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
        for name, value in _TUNING.items():
            handle.smoe_set_tuning(name.encode(), value)
        _LIBS[dtype] = handle
    _TLS.last = handle
    return handle


def exported_symbols() -> list[str]:
    return list(_SIGNATURES)


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = (getattr(_TLS, "last", None) or lib()).smoe_last_error().decode(errors="replace")
        raise RuntimeError(f"{what} failed (status {rc}): {msg}")


def set_tuning(name: str, value: int) -> None:
    """Override a kernel-selection knob (value < 0 restores the default) in every build of the library, those loaded
    later included."""
    for handle in list(_LIBS.values()) or [lib()]:
        rc = handle.smoe_set_tuning(name.encode(), int(value))
        if rc != 0:
            raise RuntimeError(f"smoe_set_tuning({name}, {value}) failed (status {rc}): "
                               f"{handle.smoe_last_error().decode(errors='replace')}")
    _TUNING[name] = int(value)


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def require_device(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("sonicmoe HIP operators need tensors on the GPU (got a CPU tensor)")


def current_stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream
