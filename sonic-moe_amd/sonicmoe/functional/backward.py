"""Backward operators `sonicmoe::*` (names, arguments and mutation contracts of sonicmoe/functional/backward.py)."""

from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ..enums import ACTIVATION_CODE, LIBRARY_NAME, ActivationType
from ..utils import expert_major_strides
from .forward import _check_schedule_order, _elem_dtype, _gather_sum, _gemm_workspace


@torch.library.custom_op(f"{LIBRARY_NAME}::_up_projection_backward", mutates_args={"dw1", "dx_expanded", "db1"})
def _up_projection_backward(
    x: torch.Tensor,
    w1: torch.Tensor,
    dx_expanded: torch.Tensor | None,
    dw1: torch.Tensor | None,
    dz: torch.Tensor,
    db1: torch.Tensor | None,
    expert_frequency_offset: torch.Tensor,
    expert_schedule_order: torch.Tensor | None,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    is_glu_activation: bool,
    stream_id: int,
) -> None:
    """dw1[e] = sum_m dz[m]^T x[t_m], db1[e] = sum_m dz[m] (zeros for empty experts), dx_expanded = dz W1[e]; any
    output may be None to skip it."""
    _lib.require_device(x, w1, dx_expanded, dw1, db1, dz, expert_frequency_offset, expert_schedule_order, x_gather_idx)
    _check_schedule_order(expert_schedule_order, w1.size(2))
    dt = _elem_dtype(("x", x), ("w1", w1), ("dx_expanded", dx_expanded), ("dw1", dw1), ("db1", db1), ("dz", dz))
    N1, H, E = w1.shape
    I = N1 // 2 if is_glu_activation else N1
    T, TK = x.size(0), dz.size(0)
    assert x.is_contiguous() and dz.is_contiguous() and (dx_expanded is None or dx_expanded.is_contiguous())
    assert dz.size(1) == N1 and (db1 is None or (db1.shape == (E, N1) and db1.is_contiguous()))
    w_se, w_sr = expert_major_strides(w1, "w1")
    d_se, d_sr = expert_major_strides(dw1, "dw1") if dw1 is not None else (0, 0)
    ws = _gemm_workspace(TK, E, x.device, stream_id)
    rc = _lib.lib(dt).smoe_up_projection_backward(
        _lib.ptr(x),
        _lib.ptr(w1),
        w_se,
        w_sr,
        _lib.ptr(dz),
        _lib.ptr(dw1),
        d_se,
        d_sr,
        _lib.ptr(db1),
        _lib.ptr(dx_expanded),
        _lib.ptr(expert_frequency_offset),
        _lib.ptr(expert_schedule_order),
        _lib.ptr(x_gather_idx),
        T,
        TK,
        H,
        I,
        E,
        # only the column count of dz depends on the activation here: any gated / any plain code will do
        ACTIVATION_CODE[ActivationType.SWIGLU if is_glu_activation else ActivationType.SILU],
        _lib.ptr(ws),
        ws.numel(),
        stream_id,
    )
    _lib.check(rc, "_up_projection_backward")


@torch.library.custom_op(f"{LIBRARY_NAME}::_down_projection_backward", mutates_args={"dw2", "dz", "ds", "db2"})
def _down_projection_backward(
    dout: torch.Tensor,
    z: torch.Tensor,
    w2: torch.Tensor,
    dw2: torch.Tensor | None,
    dz: torch.Tensor,
    ds: torch.Tensor,
    b2: torch.Tensor | None,
    db2: torch.Tensor | None,
    topk_scores: torch.Tensor,
    expert_frequency_offset: torch.Tensor,
    expert_schedule_order: torch.Tensor | None,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    stream_id: int,
    is_glu_activation: bool,
    activation_type: str,
) -> None:
    """dz, ds (flat routing-slot order), dw2 and db2 of the down projection + weighted combine; y1 is recomputed from z
    and the dout rows are re-gathered, nothing of size (TK, H) is kept from the forward."""
    _lib.require_device(dout, z, w2, dw2, dz, ds, b2, db2, topk_scores, expert_frequency_offset, expert_schedule_order,
                        x_gather_idx, s_scatter_idx)
    _check_schedule_order(expert_schedule_order, w2.size(2))
    dt = _elem_dtype(("dout", dout), ("z", z), ("w2", w2), ("dw2", dw2), ("dz", dz), ("b2", b2), ("db2", db2))
    H, I, E = w2.shape
    assert (b2 is None) == (db2 is None), "b2 and db2 have to be given together"
    assert b2 is None or (b2.shape == (E, H) and b2.is_contiguous() and db2.shape == (E, H) and db2.is_contiguous())
    assert z.size(1) == (2 * I if is_glu_activation else I)
    T, TK = dout.size(0), x_gather_idx.size(0)
    dout = dout.contiguous()
    assert z.is_contiguous() and dz.is_contiguous() and ds.is_contiguous() and ds.dtype == torch.float32
    assert topk_scores.dtype == torch.float32 and topk_scores.is_contiguous()
    w_se, w_sr = expert_major_strides(w2, "w2")
    d_se, d_sr = expert_major_strides(dw2, "dw2") if dw2 is not None else (0, 0)
    y1s = torch.empty(TK, I, dtype=z.dtype, device=z.device)
    ncols = _lib.lib(dt).smoe_dz_partial_cols(I)
    ds_partial = torch.empty(max(TK, 1), ncols, dtype=torch.float32, device=z.device)
    ws = _gemm_workspace(TK, E, z.device, stream_id)
    rc = _lib.lib(dt).smoe_down_projection_backward(
        _lib.ptr(dout),
        _lib.ptr(z),
        _lib.ptr(w2),
        w_se,
        w_sr,
        _lib.ptr(b2),
        _lib.ptr(dw2),
        d_se,
        d_sr,
        _lib.ptr(db2),
        _lib.ptr(dz),
        _lib.ptr(y1s),
        _lib.ptr(ds),
        _lib.ptr(ds_partial),
        _lib.ptr(topk_scores),
        _lib.ptr(expert_frequency_offset),
        _lib.ptr(expert_schedule_order),
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
    _lib.check(rc, "_down_projection_backward")


@torch.library.custom_op(f"{LIBRARY_NAME}::_down_projection_weight_grad", mutates_args={"dw2", "db2"})
def _down_projection_weight_grad(
    dout: torch.Tensor,
    y1s: torch.Tensor,
    dw2: torch.Tensor | None,
    db2: torch.Tensor | None,
    topk_scores: torch.Tensor,
    expert_frequency_offset: torch.Tensor,
    expert_schedule_order: torch.Tensor | None,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    stream_id: int,
) -> None:
    """The weight-gradient half of `_down_projection_backward` alone: dw2[e] = sum_m dout[t_m]^T y1s[m] and
    db2[e] = sum_m s dout[t_m], from the y1s = s * act(z) an earlier call (the fp8 activation-gradient operator) left."""
    _lib.require_device(dout, y1s, dw2, db2, topk_scores, expert_frequency_offset, expert_schedule_order, x_gather_idx,
                        s_scatter_idx)
    dt = _elem_dtype(("dout", dout), ("y1s", y1s), ("dw2", dw2), ("db2", db2))
    T, H = dout.shape
    TK, I = y1s.shape
    E = expert_frequency_offset.numel() - 1
    _check_schedule_order(expert_schedule_order, E)
    dout = dout.contiguous()
    assert y1s.is_contiguous() and topk_scores.dtype == torch.float32 and topk_scores.is_contiguous()
    assert dw2 is None or dw2.shape == (H, I, E)
    assert db2 is None or (db2.shape == (E, H) and db2.is_contiguous())
    d_se, d_sr = expert_major_strides(dw2, "dw2") if dw2 is not None else (0, 0)
    ws = _gemm_workspace(TK, E, dout.device, stream_id)
    rc = _lib.lib(dt).smoe_down_projection_backward(
        _lib.ptr(dout), None, None, 0, 0, None, _lib.ptr(dw2), d_se, d_sr, _lib.ptr(db2), None, _lib.ptr(y1s), None,
        None, _lib.ptr(topk_scores), _lib.ptr(expert_frequency_offset), _lib.ptr(expert_schedule_order),
        _lib.ptr(x_gather_idx), _lib.ptr(s_scatter_idx), T, TK, H, I, E, 0, _lib.ptr(ws), ws.numel(), stream_id,
    )
    _lib.check(rc, "_down_projection_weight_grad")


@torch.library.custom_op(f"{LIBRARY_NAME}::_token_broadcast_backward", mutates_args={"dx_reduced"})
def _token_broadcast_backward(
    dx_reduced: torch.Tensor,
    dx_expanded: torch.Tensor,
    s_reverse_scatter_idx: torch.Tensor,
    num_activated_expert_per_token_offset: torch.Tensor,
    varlen_K_max: int,
    H: int,
    is_varlen_K: bool,
) -> None:
    """dx_reduced[t] = sum over the token's routing slots j of dx_expanded[s_reverse_scatter_idx[j]]."""
    _gather_sum(
        dx_expanded,
        dx_reduced,
        None,
        s_reverse_scatter_idx,
        num_activated_expert_per_token_offset,
        varlen_K_max,
        H,
        is_varlen_K,
        "_token_broadcast_backward",
    )


@torch.library.custom_op(f"{LIBRARY_NAME}::_softmax_topk_bwd", mutates_args={"dlogits_full"})
def _softmax_topk_bwd(
    dlogits_full: torch.Tensor,
    dlogits: Optional[torch.Tensor],
    dtopk_score: torch.Tensor,
    topk_router_score: torch.Tensor,
    topk_router_indices: torch.Tensor,
    K: int,
) -> None:
    """dlogits_full[t, idx[t,k]] = s_k (ds_k - sum_j ds_j s_j) (+ dlogits[t, idx[t,k]] when `dlogits` is given, as in
    the reference: a gradient that reached the selected logits some other way); the caller zero-fills dlogits_full."""
    _lib.require_device(dlogits_full, dlogits, dtopk_score, topk_router_score, topk_router_indices)
    if dlogits_full.dtype not in _lib.DT_CODE:
        raise NotImplementedError(f"_softmax_topk_bwd: unsupported dtype {dlogits_full.dtype}")
    if dlogits is not None and (dlogits.dtype != dlogits_full.dtype or dlogits.shape != dlogits_full.shape
                                or dlogits.stride() != dlogits_full.stride()):
        raise ValueError("_softmax_topk_bwd: dlogits must have the dtype, shape and strides of dlogits_full")
    dtopk_score = dtopk_score.contiguous().float()
    assert topk_router_score.is_contiguous() and topk_router_indices.is_contiguous() and dlogits_full.stride(1) == 1
    rc = _lib.lib().smoe_softmax_topk_bwd(
        _lib.ptr(dlogits_full),
        _lib.DT_CODE[dlogits_full.dtype],
        dlogits_full.stride(0),
        _lib.ptr(dlogits),
        _lib.ptr(dtopk_score),
        _lib.ptr(topk_router_score),
        _lib.ptr(topk_router_indices),
        dtopk_score.size(0),
        K,
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "_softmax_topk_bwd")


@torch.library.custom_op(f"{LIBRARY_NAME}::_topk_bwd", mutates_args={"dlogits_full"})
def _topk_bwd(dlogits_full: torch.Tensor, dtopk_values: torch.Tensor, topk_indices: torch.Tensor, K: int) -> None:
    """dlogits_full[t, idx[t,k]] = dtopk_values[t,k]: backward of `_topk_fwd` without the softmax fusion; the caller
    zero-fills dlogits_full (sonicmoe/functional/backward.py:589-610 of the reference, which has no caller for it)."""
    _lib.require_device(dlogits_full, dtopk_values, topk_indices)
    if dlogits_full.dtype not in _lib.DT_CODE:
        raise NotImplementedError(f"_topk_bwd: unsupported dtype {dlogits_full.dtype}")
    dtopk_values = dtopk_values.contiguous().float()
    assert topk_indices.is_contiguous() and topk_indices.dtype == torch.int32 and dlogits_full.stride(1) == 1
    assert dtopk_values.shape == topk_indices.shape and dtopk_values.size(1) == K
    rc = _lib.lib().smoe_topk_bwd(
        _lib.ptr(dlogits_full), _lib.DT_CODE[dlogits_full.dtype], dlogits_full.stride(0), _lib.ptr(dtopk_values),
        _lib.ptr(topk_indices), dtopk_values.size(0), K, _lib.current_stream_handle(),
    )
    _lib.check(rc, "_topk_bwd")


@torch.library.custom_op(f"{LIBRARY_NAME}::_router_weight_grad", mutates_args={"partial"})
def _router_weight_grad(dlogits: torch.Tensor, x: torch.Tensor, partial: torch.Tensor) -> None:
    """partial[c] (E, H) = dlogits[rows of chunk c]^T x[rows of chunk c]; the chunks are partial.size(0) equal token
    ranges.  Their sum is the weight gradient of router_logits = F.linear(x, router_w)."""
    _lib.require_device(dlogits, x, partial)
    dt = _elem_dtype(("dlogits", dlogits), ("x", x), ("partial", partial))
    T, E = dlogits.shape
    H = x.size(1)
    assert dlogits.is_contiguous() and x.is_contiguous() and partial.is_contiguous()
    assert x.size(0) == T and partial.shape[1:] == (E, H)
    rc = _lib.lib(dt).smoe_router_weight_grad(
        _lib.ptr(dlogits), _lib.ptr(x), _lib.ptr(partial), T, E, H, partial.size(0), _lib.current_stream_handle()
    )
    _lib.check(rc, "_router_weight_grad")


def router_weight_grad_chunks(T: int, E: int, H: int) -> int:
    """Token chunks that give the split GEMM at least one 256 x 256 output tile per compute unit, each chunk at least
    256 tokens long."""
    tiles = -(-E // 256) * -(-H // 256)
    return max(1, min(64, -(-256 // tiles), T // 256))


@torch.library.custom_op(f"{LIBRARY_NAME}::_switch_loss_bwd", mutates_args={"dlogits"})
def _switch_loss_bwd(router_logits: torch.Tensor, expert_frequency: torch.Tensor, acc: torch.Tensor,
                     grad_aux: torch.Tensor, dlogits: torch.Tensor) -> None:
    """dlogits (T, E) = grad_aux * d aux / d router_logits for the switch loss; acc as left by _switch_loss_fwd.  The
    reference differentiates its six torch ops with autograd (sonicmoe/moe.py:261-274)."""
    _lib.require_device(router_logits, expert_frequency, acc, grad_aux, dlogits)
    if router_logits.dtype not in _lib.DT_CODE or dlogits.dtype != router_logits.dtype:
        raise NotImplementedError(f"_switch_loss_bwd: unsupported dtypes {router_logits.dtype}, {dlogits.dtype}")
    T, E = router_logits.shape
    assert router_logits.stride(1) == 1 and dlogits.stride(1) == 1 and dlogits.shape == router_logits.shape
    assert grad_aux.numel() == 1 and grad_aux.dtype == torch.float32 and acc.dtype == torch.float32
    rc = _lib.lib().smoe_switch_loss_bwd(
        _lib.ptr(router_logits), _lib.DT_CODE[router_logits.dtype], router_logits.stride(0), T, E,
        _lib.ptr(expert_frequency), _lib.ptr(acc), _lib.ptr(grad_aux), _lib.ptr(dlogits), dlogits.stride(0),
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "_switch_loss_bwd")
