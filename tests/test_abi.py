"""The C-ABI library loads and exports every entry point that include/sonicmoe_hip.h declares; argument checks
that happen before any GPU work report the documented status codes.  No compute is launched here."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "sonicmoe_hip.h"


def declared_functions() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(smoe_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from sonicmoe import _lib

    if not _lib.library_path().exists():
        import __graft_entry__

        __graft_entry__.build()
    return _lib.lib()


def test_header_and_binding_agree(lib):
    from sonicmoe import _lib

    names = declared_functions()
    assert len(names) >= 14
    assert sorted(_lib.exported_symbols()) == names
    for n in names:
        assert getattr(lib, n) is not None


def test_version_and_error_text(lib):
    assert lib.smoe_version() >= 200
    assert isinstance(lib.smoe_last_error(), bytes)


def test_argument_checks_return_status_codes(lib):
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # E out of range -> SMOE_ERR_UNSUPPORTED (2), before anything is launched
    assert lib.smoe_count_cumsum(p, 0, 4, 0, p, p, None) == 2
    assert b"E=0" in lib.smoe_last_error()
    # null output -> SMOE_ERR_INVALID (1)
    assert lib.smoe_count_cumsum(p, 0, 4, 8, None, None, None) == 1
    # K > E
    assert lib.smoe_topk_softmax_fwd(p, 0, 4, 8, 9, 8, p, p, 1, None) == 2
    # H not a multiple of 64
    assert lib.smoe_up_projection_forward(p, p, 0, 0, None, p, p, p, None, p, 4, 8, 96, 64, 2, 0, p, 1 << 20,
                                          None) == 2
    assert b"multiple of 64" in lib.smoe_last_error()
    # workspace too small
    assert lib.smoe_down_projection_forward(p, p, 0, 0, None, p, p, None, 1 << 20, 64, 64, 2, p, 8, None) == 4
    # activation code outside the enum -> SMOE_ERR_INVALID
    assert lib.smoe_up_projection_forward(p, p, 0, 0, None, p, p, p, None, p, 4, 8, 64, 64, 2, 7, p, 1 << 20,
                                          None) == 1
    assert b"activation" in lib.smoe_last_error()
    # a backward call with every output null has nothing to do
    assert lib.smoe_up_projection_backward(p, p, 0, 0, p, None, 0, 0, None, None, p, None, p, 4, 8, 64, 64, 2, 0, p,
                                           1 << 20, None) == 1
    # switch loss: E outside [1, 4096] -> unsupported; workspace too small -> SMOE_ERR_WORKSPACE
    assert lib.smoe_switch_loss_fwd(p, 0, 8192, 16, 8192, p, p, p, p, 1 << 20, None) == 2
    assert b"E=8192" in lib.smoe_last_error()
    assert lib.smoe_switch_loss_fwd(p, 0, 128, 1024, 128, p, p, p, p, 16, None) == 4
    assert lib.smoe_switch_loss_bwd(p, 0, 64, 16, 128, p, p, p, p, 128, None) == 1  # row stride below E
    assert lib.smoe_switch_loss_workspace_bytes(32768, 128) == 256 * 128 * 4
    # workspace size queries are pure host functions
    assert lib.smoe_gemm_workspace_bytes(262144, 128) > 0
    # the fp8 operators with a gathered token operand: tile map + (K / 128) * TK scale words in grouped order
    assert lib.smoe_fp8_gemm_workspace_bytes(262144, 128, 4096) >= lib.smoe_gemm_workspace_bytes(262144, 128) + 32 * 262144 * 4
    assert lib.smoe_fp8_gemm_workspace_bytes(262144, 128, 64) == 0
    assert lib.smoe_routing_metadata_workspace_bytes(262144, 128) == 2 * 128 * 256 * 4
    assert lib.smoe_dz_partial_cols(1024) >= 4


def test_misaligned_operands_are_rejected(lib):
    buf = ctypes.create_string_buffer(256)
    base = ctypes.addressof(buf)
    base += (-base) % 16
    p, q = ctypes.c_void_p(base), ctypes.c_void_p(base + 2)
    # a weight pointer that is not 16-byte aligned, then a row stride that is not a multiple of 8 elements
    assert lib.smoe_up_projection_forward(p, q, 64, 64, None, p, p, p, None, p, 4, 8, 64, 64, 2, 0, p, 1 << 20,
                                          None) == 2
    assert b"16-byte aligned" in lib.smoe_last_error()
    assert lib.smoe_down_projection_forward(p, p, 64 * 64, 68, None, p, p, None, 8, 64, 64, 2, p, 1 << 20, None) == 2
    assert b"multiples of 8" in lib.smoe_last_error()


def test_tuning_knobs(lib):
    assert lib.smoe_set_tuning(b"no_such_knob", 1) == 1
    assert b"unknown knob" in lib.smoe_last_error()
    assert lib.smoe_set_tuning(b"varlen_k_tile_order", 7) == 1
    assert lib.smoe_set_tuning(b"gemm_stream", 0) == 0
    assert lib.smoe_set_tuning(b"gemm_stream", -1) == 0  # back to the default


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from sonicmoe import _lib

    import torch

    monkeypatch.setenv("SONICMOE_HIP_LIB", str(tmp_path / "nope.so"))
    monkeypatch.setenv("SONICMOE_HIP_LIB_F16", str(tmp_path / "nope_f16.so"))
    monkeypatch.setattr(_lib, "_LIBS", {})
    with pytest.raises(RuntimeError, match="not found"):
        _lib.lib()
    with pytest.raises(RuntimeError, match="not found"):
        _lib.lib(torch.float16)
    with pytest.raises(NotImplementedError, match="no build"):
        _lib.lib(torch.float32)


def test_the_fp16_build_exports_the_same_entry_points(lib):
    """libsonicmoe_hip_f16.so is the same sources with fp16 as the 16-bit element type: same symbols, same argument
    checks; the fused router (bf16 bit tricks) refuses."""
    import torch

    from sonicmoe import _lib

    lib16 = _lib.lib(torch.float16)
    assert lib16 is not lib and lib16._name.endswith("libsonicmoe_hip_f16.so")
    for n in declared_functions():
        assert getattr(lib16, n) is not None
    assert lib16.smoe_version() == lib.smoe_version()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib16.smoe_up_projection_forward(p, p, 0, 0, None, p, p, p, None, p, 4, 8, 96, 64, 2, 0, p, 1 << 20,
                                            None) == 2
    assert b"multiple of 64" in lib16.smoe_last_error()
    assert lib16.smoe_router_forward_fused(p, p, 16, 512, 16, 2, p, p, p, None, None) == 2
    assert b"bf16 only" in lib16.smoe_last_error()
    # a knob set through the binding reaches both builds
    _lib.set_tuning("gemm_stream", 0)
    _lib.set_tuning("gemm_stream", -1)


def test_element_type_of_an_operator_call():
    """Host logic that picks the library build: one 16-bit element type per operator call, bf16 or fp16."""
    import torch

    from sonicmoe.functional.forward import _elem_dtype

    b, h, f = (torch.empty(2, dtype=d) for d in (torch.bfloat16, torch.float16, torch.float32))
    assert _elem_dtype(("x", b), ("bias", None), ("y", b)) == torch.bfloat16
    assert _elem_dtype(("x", h), ("y", h)) == torch.float16
    assert _elem_dtype(("bias", None)) == torch.bfloat16   # nothing to go by: the default build
    with pytest.raises(NotImplementedError, match="one element type"):
        _elem_dtype(("x", b), ("w", h))
    with pytest.raises(NotImplementedError, match="bfloat16 or float16"):
        _elem_dtype(("x", f))
