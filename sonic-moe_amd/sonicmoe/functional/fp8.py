"""fp8 path: block-scaled e4m3 operands for the two forward grouped GEMMs and the two activation-gradient GEMMs.

The reference has no fp8 path; this module has the shape of its `enable_quack_gemm` switch
(sonicmoe/functional/utils.py:9-25): inside `with enable_fp8_forward():` the expert forward quantises x, W1, y1 and W2
(one power-of-two scale per 32 contraction elements) and runs the fp8 MFMA kernels; z is still stored in bf16.
A layer called inside `with enable_fp8_backward():` computes dz (from quantised dout and W2^T) and dx (from the dz the
dz kernel quantises in its epilogue and W1^T) in fp8 as well; the two weight-gradient GEMMs, which contract over the
tokens, stay in bf16 and read the bf16 dz / y1s.
"""

from __future__ import annotations

import weakref
from contextlib import contextmanager

import torch

from .. import _lib
from ..enums import ACTIVATION_CODE, LIBRARY_NAME, ActivationType
from .forward import _elem_dtype, _gemm_workspace

_FP8_FORWARD = False


@contextmanager
def enable_fp8_forward(enable: bool = True):
    global _FP8_FORWARD
    previous, _FP8_FORWARD = _FP8_FORWARD, enable
    try:
        yield
    finally:
        _FP8_FORWARD = previous


def is_using_fp8_forward() -> bool:
    return _FP8_FORWARD


_FP8_BACKWARD = False


@contextmanager
def enable_fp8_backward(enable: bool = True):
    """Layers whose FORWARD runs inside this block compute their activation gradients (dz, dx) with fp8 operands."""
    global _FP8_BACKWARD
    previous, _FP8_BACKWARD = _FP8_BACKWARD, enable
    try:
        yield
    finally:
        _FP8_BACKWARD = previous


def is_using_fp8_backward() -> bool:
    return _FP8_BACKWARD


@torch.library.custom_op(f"{LIBRARY_NAME}::_mx_quantize", mutates_args={"q", "scales"})
def _mx_quantize(src: torch.Tensor, q: torch.Tensor, scales: torch.Tensor) -> None:
    """src (R, C) bf16 -> q (R, C) uint8 e4m3 codes, scales (C/128, R) int32 (four exponent bytes per word)."""
    _lib.require_device(src, q, scales)
    dt = _elem_dtype(("src", src))
    R, C = src.shape
    assert src.stride(1) == 1 and q.is_contiguous() and scales.is_contiguous()
    assert q.dtype == torch.uint8 and q.shape == (R, C) and scales.dtype == torch.int32 and scales.shape == (C // 128, R)
    rc = _lib.lib(dt).smoe_mx_quantize(
        _lib.ptr(src), src.stride(0), R, C, _lib.ptr(q), _lib.ptr(scales), _lib.current_stream_handle()
    )
    _lib.check(rc, "_mx_quantize")


def mx_quantize(t: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantise the rows of a 2-D bf16 tensor; see `_mx_quantize` for the layouts."""
    R, C = t.shape
    if C % 128:
        raise NotImplementedError(f"mx_quantize: {C} columns are not a multiple of 128")
    q = torch.empty(R, C, dtype=torch.uint8, device=t.device)
    scales = torch.empty(C // 128, R, dtype=torch.int32, device=t.device)
    _mx_quantize(t, q, scales)
    return q, scales


# Quantised copies of expert weights, reused while the tensor that owns the storage is alive and has not been written
# to (same object, same version counter): inference and repeated forwards quantise a weight once, a training step
# re-quantises after the optimizer.  An entry holds only a weak reference to that tensor and is dropped with it, so a
# new parameter that lands at a freed parameter's address never meets the old one's entry.  Weights that have to be
# copied into (E, out, in) order first are never cached: the copy is a fresh tensor every call.  Writes that bypass
# the version counter (`param.data.copy_()`, raw pointers) are not seen; use cache_quantized_weights(False) there.
_WEIGHT_CACHE: dict[tuple, tuple] = {}
_WEIGHT_CACHE_MAX = 8
_CACHE_WEIGHTS = True


@contextmanager
def cache_quantized_weights(enable: bool = True):
    global _CACHE_WEIGHTS
    previous, _CACHE_WEIGHTS = _CACHE_WEIGHTS, enable
    try:
        yield
    finally:
        _CACHE_WEIGHTS = previous


def quantize_expert_weight(w_view: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """w_view is the (out, in, E) permuted view of an (E, out, in) parameter; quantised along `in`."""
    w = w_view.permute(2, 0, 1)
    aliases_caller = w.is_contiguous()
    if not aliases_caller:
        w = w.contiguous()
    E, N, K = w.shape
    if not aliases_caller or not _CACHE_WEIGHTS or torch.compiler.is_compiling():
        return mx_quantize(w.detach().reshape(E * N, K))
    owner = w_view._base if w_view._base is not None else w_view  # the tensor whose version counter sees every write
    key = (id(owner), w.data_ptr(), tuple(w.shape), w.device.index)
    hit = _WEIGHT_CACHE.get(key)
    if hit is not None and hit[0]() is owner and hit[1] == owner._version:
        return hit[2], hit[3]
    q, scales = mx_quantize(w.detach().reshape(E * N, K))
    if len(_WEIGHT_CACHE) >= _WEIGHT_CACHE_MAX:
        _WEIGHT_CACHE.pop(next(iter(_WEIGHT_CACHE)))
    _WEIGHT_CACHE[key] = (weakref.ref(owner, lambda _ref, k=key: _WEIGHT_CACHE.pop(k, None)), owner._version, q, scales)
    return q, scales


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_up_projection_forward_fp8", mutates_args={"z", "y1", "y1q", "y1q_scales"}
)
def _up_projection_forward_fp8(
    xq: torch.Tensor,
    x_scales: torch.Tensor,
    w1q: torch.Tensor,
    w1_scales: torch.Tensor,
    z: torch.Tensor | None,
    y1: torch.Tensor | None,
    b1: torch.Tensor | None,
    expert_frequency_offset: torch.Tensor,
    x_gather_idx: torch.Tensor,
    E: int,
    stream_id: int,
    activation_type: str,
    is_glu_activation: bool,
    y1q: torch.Tensor | None = None,
    y1q_scales: torch.Tensor | None = None,
) -> None:
    """z = gather(xq) w1q^T (+ b1) with the block scales applied, y1 = act(z); xq (T, H), w1q (E*N1, H).  y1 comes back
    in bf16 (`y1`) and / or quantised in the epilogue (`y1q` (TK, I) uint8 with `y1q_scales` (I/128, TK) int32)."""
    _lib.require_device(xq, x_scales, w1q, w1_scales, y1, y1q, y1q_scales, b1, expert_frequency_offset, x_gather_idx)
    dt = _elem_dtype(("z", z), ("y1", y1), ("b1", b1))
    T, H = xq.shape
    TK, I = (y1 if y1 is not None else y1q).shape
    assert y1q is None or (y1q.dtype == torch.uint8 and y1q.is_contiguous() and y1q_scales.shape == (I // 128, TK))
    N1 = 2 * I if is_glu_activation else I
    assert w1q.shape == (E * N1, H) and x_scales.shape == (H // 128, T) and w1_scales.shape == (H // 128, E * N1)
    assert z is None or (z.shape == (TK, N1) and z.is_contiguous())
    ws = _gemm_workspace(TK, E, xq.device, stream_id, fp8_gathered_k=H)
    rc = _lib.lib(dt).smoe_up_projection_forward_fp8(
        _lib.ptr(xq),
        _lib.ptr(x_scales),
        _lib.ptr(w1q),
        _lib.ptr(w1_scales),
        _lib.ptr(b1),
        _lib.ptr(z),
        _lib.ptr(y1),
        _lib.ptr(y1q),
        _lib.ptr(y1q_scales),
        _lib.ptr(expert_frequency_offset),
        _lib.ptr(x_gather_idx),
        T,
        TK,
        H,
        I,
        E,
        ACTIVATION_CODE[ActivationType(activation_type)],
        _lib.ptr(ws),
        ws.numel(),
        stream_id,
    )
    _lib.check(rc, "_up_projection_forward_fp8")


@torch.library.custom_op(f"{LIBRARY_NAME}::_down_projection_forward_fp8", mutates_args={"y2"})
def _down_projection_forward_fp8(
    y1q: torch.Tensor,
    y1_scales: torch.Tensor,
    w2q: torch.Tensor,
    w2_scales: torch.Tensor,
    y2: torch.Tensor,
    b2: torch.Tensor | None,
    expert_frequency_offset: torch.Tensor,
    E: int,
    stream_id: int,
) -> None:
    """y2 = y1q w2q^T (+ b2) with the block scales applied; y1q (TK, I), w2q (E*H, I)."""
    _lib.require_device(y1q, y1_scales, w2q, w2_scales, y2, b2, expert_frequency_offset)
    dt = _elem_dtype(("y2", y2), ("b2", b2))
    TK, I = y1q.shape
    H = y2.size(1)
    assert w2q.shape == (E * H, I) and y1_scales.shape == (I // 128, TK) and w2_scales.shape == (I // 128, E * H)
    ws = _gemm_workspace(TK, E, y1q.device, stream_id)
    rc = _lib.lib(dt).smoe_down_projection_forward_fp8(
        _lib.ptr(y1q),
        _lib.ptr(y1_scales),
        _lib.ptr(w2q),
        _lib.ptr(w2_scales),
        _lib.ptr(b2),
        _lib.ptr(y2),
        _lib.ptr(expert_frequency_offset),
        TK,
        H,
        I,
        E,
        _lib.ptr(ws),
        ws.numel(),
        stream_id,
    )
    _lib.check(rc, "_down_projection_forward_fp8")


@torch.library.custom_op(f"{LIBRARY_NAME}::_mx_quantize_transposed", mutates_args={"q", "scales"})
def _mx_quantize_transposed(src: torch.Tensor, q: torch.Tensor, scales: torch.Tensor) -> None:
    """src (E, R, C) bf16 (last dimension contiguous) -> q (E, C, R) uint8, the transposed matrices quantised along R,
    scales (R/128, E*C) int32."""
    _lib.require_device(src, q, scales)
    dt = _elem_dtype(("src", src))
    E, R, C = src.shape
    assert src.stride(2) == 1 and q.is_contiguous() and scales.is_contiguous()
    assert q.dtype == torch.uint8 and q.shape == (E, C, R)
    assert scales.dtype == torch.int32 and scales.shape == (R // 128, E * C)
    rc = _lib.lib(dt).smoe_mx_quantize_transposed(
        _lib.ptr(src), src.stride(0), src.stride(1), E, R, C, _lib.ptr(q), _lib.ptr(scales),
        _lib.current_stream_handle()
    )
    _lib.check(rc, "_mx_quantize_transposed")


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_mx_quantize_both", mutates_args={"q_rows", "scales_rows", "q_t", "scales_t"}
)
def _mx_quantize_both(src: torch.Tensor, q_rows: torch.Tensor, scales_rows: torch.Tensor, q_t: torch.Tensor,
                      scales_t: torch.Tensor) -> None:
    """src (E, R, C) bf16 -> both quantised copies from one pass over src: q_rows (E*R, C) / scales_rows (C/128, E*R) as
    `_mx_quantize` of the (E*R, C) matrix, q_t (E, C, R) / scales_t (R/128, E*C) as `_mx_quantize_transposed`."""
    _lib.require_device(src, q_rows, scales_rows, q_t, scales_t)
    dt = _elem_dtype(("src", src))
    E, R, C = src.shape
    assert src.stride(2) == 1 and all(t.is_contiguous() for t in (q_rows, scales_rows, q_t, scales_t))
    assert q_rows.dtype == torch.uint8 and q_rows.shape == (E * R, C) and q_t.dtype == torch.uint8 and q_t.shape == (E, C, R)
    assert scales_rows.dtype == torch.int32 and scales_rows.shape == (C // 128, E * R)
    assert scales_t.dtype == torch.int32 and scales_t.shape == (R // 128, E * C)
    rc = _lib.lib(dt).smoe_mx_quantize_both(
        _lib.ptr(src), src.stride(0), src.stride(1), E, R, C, _lib.ptr(q_rows), _lib.ptr(scales_rows), _lib.ptr(q_t),
        _lib.ptr(scales_t), _lib.current_stream_handle()
    )
    _lib.check(rc, "_mx_quantize_both")


# Transposed quantised weights a forward pass made together with the row-quantised ones (one read of the weight for
# both), waiting for the backward pass of the same step: key -> (weak owner, version, codes, scales).  An entry is used
# once, and only while the weight is unchanged.
_TRANSPOSED_STASH: dict = {}
_TRANSPOSED_STASH_MAX = 16


def _weight_key(w_view: torch.Tensor, w: torch.Tensor):
    owner = w_view._base if w_view._base is not None else w_view  # the tensor whose version counter sees every write
    return owner, (id(owner), w.data_ptr(), tuple(w.shape), w.device.index)


def quantize_expert_weight_both(w_view: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """`quantize_expert_weight` for a step whose backward pass will ask for `quantize_expert_weight_transposed` of the
    same weight: one kernel reads the weight once and writes both copies; the transposed one is kept for that call."""
    w = w_view.permute(2, 0, 1)
    E, N, K = w.shape
    if not w.is_contiguous() or N % 128 or K % 128 or torch.compiler.is_compiling():
        return quantize_expert_weight(w_view)
    owner, key = _weight_key(w_view, w)
    if _CACHE_WEIGHTS:
        hit = _WEIGHT_CACHE.get(key)
        if hit is not None and hit[0]() is owner and hit[1] == owner._version:
            return hit[2], hit[3]  # unchanged since an earlier forward pass: only the transposed copy is missing
    q = torch.empty(E * N, K, dtype=torch.uint8, device=w.device)
    scales = torch.empty(K // 128, E * N, dtype=torch.int32, device=w.device)
    qt = torch.empty(E, K, N, dtype=torch.uint8, device=w.device)
    scales_t = torch.empty(N // 128, E * K, dtype=torch.int32, device=w.device)
    _mx_quantize_both(w.detach(), q, scales, qt, scales_t)
    if _CACHE_WEIGHTS:
        if len(_WEIGHT_CACHE) >= _WEIGHT_CACHE_MAX:
            _WEIGHT_CACHE.pop(next(iter(_WEIGHT_CACHE)))
        _WEIGHT_CACHE[key] = (weakref.ref(owner, lambda _ref, k=key: _WEIGHT_CACHE.pop(k, None)), owner._version, q, scales)
    if len(_TRANSPOSED_STASH) >= _TRANSPOSED_STASH_MAX:
        _TRANSPOSED_STASH.pop(next(iter(_TRANSPOSED_STASH)))
    _TRANSPOSED_STASH[key] = (weakref.ref(owner, lambda _ref, k=key: _TRANSPOSED_STASH.pop(k, None)), owner._version,
                              qt.view(E * K, N), scales_t)
    return q, scales


def quantize_expert_weight_transposed(w_view: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """w_view is the (out, in, E) permuted view of an (E, out, in) parameter; returns the (E * in, out) codes of the
    transposed matrices, quantised along `out`, and their scale table: the weight operand of the activation-gradient
    GEMMs, which contract over `out`.  Taken from the forward pass of the same step when that made it
    (`quantize_expert_weight_both`); otherwise quantised here.  Not cached beyond that: a training step writes the
    weights between two backward passes."""
    w = w_view.permute(2, 0, 1)
    if w.stride(2) != 1:
        w = w.contiguous()
    elif not torch.compiler.is_compiling():
        owner, key = _weight_key(w_view, w)
        hit = _TRANSPOSED_STASH.pop(key, None)
        if hit is not None and hit[0]() is owner and hit[1] == owner._version:
            return hit[2], hit[3]
    E, N, K = w.shape
    if N % 128 or K % 64:
        raise NotImplementedError(f"quantize_expert_weight_transposed: ({N}, {K}) matrices need out % 128 == 0 and "
                                  f"in % 64 == 0")
    q = torch.empty(E, K, N, dtype=torch.uint8, device=w.device)
    scales = torch.empty(N // 128, E * K, dtype=torch.int32, device=w.device)
    _mx_quantize_transposed(w.detach(), q, scales)
    return q.view(E * K, N), scales


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_down_projection_backward_fp8", mutates_args={"dz", "dzq", "dzq_scales", "y1s", "ds"}
)
def _down_projection_backward_fp8(
    doutq: torch.Tensor,
    dout_scales: torch.Tensor,
    w2tq: torch.Tensor,
    w2t_scales: torch.Tensor,
    z: torch.Tensor,
    dz: torch.Tensor,
    dzq: torch.Tensor,
    dzq_scales: torch.Tensor,
    y1s: torch.Tensor,
    ds: torch.Tensor,
    topk_scores: torch.Tensor,
    expert_frequency_offset: torch.Tensor,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    E: int,
    stream_id: int,
    activation_type: str,
    is_glu_activation: bool,
) -> None:
    """The activation-gradient half of `_down_projection_backward` with fp8 operands: dy1 = gather(doutq) w2tq^T with
    the block scales applied, then dz (bf16, and once more quantised: dzq (TK, N1) uint8 with dzq_scales (N1/128, TK)),
    y1s = s * act(z) and ds exactly as the bf16 operator forms them.  doutq (T, H), w2tq (E*I, H)."""
    _lib.require_device(doutq, dout_scales, w2tq, w2t_scales, z, dz, dzq, dzq_scales, y1s, ds, topk_scores,
                        expert_frequency_offset, x_gather_idx, s_scatter_idx)
    dt = _elem_dtype(("z", z), ("dz", dz), ("y1s", y1s))
    T, H = doutq.shape
    TK, N1 = z.shape
    I = N1 // 2 if is_glu_activation else N1
    assert w2tq.shape == (E * I, H) and dout_scales.shape == (H // 128, T) and w2t_scales.shape == (H // 128, E * I)
    assert z.is_contiguous() and dz.is_contiguous() and dz.shape == z.shape and y1s.shape == (TK, I) and y1s.is_contiguous()
    assert dzq.dtype == torch.uint8 and dzq.shape == (TK, N1) and dzq.is_contiguous()
    assert dzq_scales.dtype == torch.int32 and dzq_scales.shape == (N1 // 128, TK) and dzq_scales.is_contiguous()
    assert ds.dtype == torch.float32 and ds.numel() == TK and topk_scores.dtype == torch.float32
    ncols = _lib.lib(dt).smoe_dz_partial_cols(I)
    ds_partial = torch.empty(max(TK, 1), ncols, dtype=torch.float32, device=z.device)
    ws = _gemm_workspace(TK, E, z.device, stream_id, fp8_gathered_k=H)
    rc = _lib.lib(dt).smoe_down_projection_backward_fp8(
        _lib.ptr(doutq),
        _lib.ptr(dout_scales),
        _lib.ptr(w2tq),
        _lib.ptr(w2t_scales),
        _lib.ptr(z),
        _lib.ptr(dz),
        _lib.ptr(dzq),
        _lib.ptr(dzq_scales),
        _lib.ptr(y1s),
        _lib.ptr(ds),
        _lib.ptr(ds_partial),
        _lib.ptr(topk_scores),
        _lib.ptr(expert_frequency_offset),
        _lib.ptr(x_gather_idx),
        _lib.ptr(s_scatter_idx),
        T,
        TK,
        H,
        I,
        E,
        ACTIVATION_CODE[ActivationType(activation_type)],
        _lib.ptr(ws),
        ws.numel(),
        stream_id,
    )
    _lib.check(rc, "_down_projection_backward_fp8")


@torch.library.custom_op(f"{LIBRARY_NAME}::_score_grad_bias_term", mutates_args={"ds"})
def _score_grad_bias_term(
    dout: torch.Tensor,
    b2: torch.Tensor,
    ds: torch.Tensor,
    expert_frequency_offset: torch.Tensor,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    stream_id: int,
) -> None:
    """ds[s_scatter_idx[m]] += <dout[x_gather_idx[m]], b2[expert of m]>: the part of the score gradient that the
    down-projection bias causes (the reference folds it into db2_and_ds_kernel, sonicmoe/functional/backward.py:36-107).
    `_down_projection_backward` adds it itself; `_down_projection_backward_fp8` does not know b2."""
    _lib.require_device(dout, b2, ds, expert_frequency_offset, x_gather_idx, s_scatter_idx)
    dt = _elem_dtype(("dout", dout), ("b2", b2))
    T, H = dout.shape
    E = expert_frequency_offset.numel() - 1
    TK = x_gather_idx.numel()
    assert dout.is_contiguous() and b2.shape == (E, H) and b2.is_contiguous()
    assert ds.dtype == torch.float32 and ds.numel() == TK and ds.is_contiguous() and s_scatter_idx.numel() == TK
    rc = _lib.lib(dt).smoe_score_grad_bias_term(
        _lib.ptr(dout), _lib.ptr(b2), _lib.ptr(expert_frequency_offset), _lib.ptr(x_gather_idx), _lib.ptr(s_scatter_idx),
        _lib.ptr(ds), TK, H, E, stream_id,
    )
    _lib.check(rc, "_score_grad_bias_term")
