"""Autograd layer of the MoE hot path (public entry points of sonicmoe/functional/__init__.py).

    moe_TC_softmax_topk_layer      router GEMM -> top-K softmax -> routing metadata -> experts -> combine
    moe_general_routing_inputs     same expert path for caller-supplied (score, token, expert) triples

What is kept for the backward pass is x, z (the pre-activation) and the routing metadata; the gathered inputs, y1, y2
and dx_expanded are transient.  y1 is rebuilt from z inside the dz kernel and the token rows are gathered again
inside the weight-gradient kernels.
"""

from __future__ import annotations

import os
from contextlib import contextmanager

import torch
import torch.nn.functional as F

from .. import _lib
from ..count_cumsum import count_cumsum
from ..enums import LIBRARY_NAME, ActivationType, is_glu
from .backward import (
    _down_projection_backward,
    _down_projection_weight_grad,
    _router_weight_grad,
    _softmax_topk_bwd,
    _switch_loss_bwd,
    _token_broadcast_backward,
    _up_projection_backward,
    router_weight_grad_chunks,
)
from .forward import (
    _down_projection_forward,
    _down_projection_forward_combine,
    _router_forward,
    _router_forward_fused,
    _softmax_topk_fwd,
    _switch_loss_from_partials,
    _switch_loss_fwd,
    _up_projection_forward,
    router_fused_partials,
    router_fused_supported,
)
from .fp8 import (
    _down_projection_backward_fp8,
    _down_projection_forward_fp8,
    _score_grad_bias_term,
    _up_projection_forward_fp8,
    enable_fp8_backward,
    enable_fp8_forward,
    is_using_fp8_backward,
    is_using_fp8_forward,
    mx_quantize,
    quantize_expert_weight,
    quantize_expert_weight_both,
    quantize_expert_weight_transposed,
)
from .utils import enable_quack_gemm, is_using_quack_gemm


# ---------------------------------------------------------------------------------------------------------------
# routing metadata (one stable counting sort on the device instead of argsort + bincount + index arithmetic)
# ---------------------------------------------------------------------------------------------------------------


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_routing_metadata",
    mutates_args={"freq", "off", "x_gather_idx", "s_scatter_idx", "s_reverse_scatter_idx", "tok_off"},
)
def _routing_metadata(
    expert_idx: torch.Tensor,
    token_idx: torch.Tensor | None,
    T: int,
    K: int,
    freq: torch.Tensor,
    off: torch.Tensor,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    s_reverse_scatter_idx: torch.Tensor,
    tok_off: torch.Tensor,
) -> None:
    _lib.require_device(expert_idx, token_idx, freq, off, x_gather_idx, s_scatter_idx, s_reverse_scatter_idx, tok_off)
    assert expert_idx.dtype == torch.int32 and expert_idx.is_contiguous()
    assert token_idx is None or (token_idx.dtype == torch.int32 and token_idx.is_contiguous())
    TK, E = expert_idx.numel(), freq.numel()
    L = _lib.lib()
    ws_bytes = L.smoe_routing_metadata_workspace_bytes(TK, E)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=expert_idx.device)
    rc = L.smoe_routing_metadata(
        _lib.ptr(expert_idx),
        _lib.ptr(token_idx),
        TK,
        T,
        E,
        K,
        _lib.ptr(freq),
        _lib.ptr(off),
        _lib.ptr(x_gather_idx),
        _lib.ptr(s_scatter_idx),
        _lib.ptr(s_reverse_scatter_idx),
        _lib.ptr(tok_off),
        _lib.ptr(ws),
        ws.numel(),
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "_routing_metadata")


@torch.no_grad()
def _build_metadata(expert_idx: torch.Tensor, token_idx: torch.Tensor | None, T: int, E: int, K: int):
    dev = expert_idx.device
    TK = expert_idx.numel()
    i32 = dict(dtype=torch.int32, device=dev)
    freq = torch.empty(E, **i32)
    off = torch.empty(E + 1, **i32)
    gidx = torch.empty(TK, **i32)
    sidx = torch.empty(TK, **i32)
    ridx = torch.empty(TK, **i32)
    tok_off = torch.empty(T + 1, **i32)
    expert_idx = expert_idx.contiguous().to(torch.int32)
    if token_idx is not None:
        token_idx = token_idx.contiguous().to(torch.int32)
    _routing_metadata(expert_idx, token_idx, T, K, freq, off, gidx, sidx, ridx, tok_off)
    return freq, off, gidx, sidx, ridx, tok_off


def TC_topk_router_metadata(topk_router_indices: torch.Tensor, expert_frequency_offset: torch.Tensor, K: int):
    """Token-choice top-K metadata (interface of sonicmoe/functional/__init__.py:19-46).  `expert_frequency_offset` is
    the (E,) inclusive cumsum the reference passes in; only its length is used, the offsets are recomputed together
    with the sort.  Returns (expert_frequency_offset (E+1,), x_gather_idx, s_scatter_idx, s_reverse_scatter_idx,
    num_activated_expert_per_token_offset); the order inside an expert is ascending flat slot (stable)."""
    T = topk_router_indices.size(0)
    E = expert_frequency_offset.numel()
    _, off, gidx, sidx, ridx, tok_off = _build_metadata(topk_router_indices.reshape(-1), None, T, E, K)
    return off, gidx, sidx, ridx, tok_off


def general_routing_router_metadata(
    router_scores_selected: torch.Tensor, sorted_selected_T: torch.Tensor, selected_E: torch.Tensor, T: int, E: int
):
    """Metadata for arbitrary (token, expert) pairs with tokens sorted ascending (interface of
    sonicmoe/functional/__init__.py:49-82).  Returns (expert_frequency, expert_frequency_offset, x_gather_idx,
    s_scatter_idx, s_reverse_scatter_idx, num_activated_expert_per_token_offset)."""
    freq, off, gidx, sidx, ridx, tok_off = _build_metadata(selected_E, sorted_selected_T, T, E, 1)
    return freq, off, gidx, sidx, ridx, tok_off


# ---------------------------------------------------------------------------------------------------------------
# autograd functions
# ---------------------------------------------------------------------------------------------------------------


class _RouterLinearFunction(torch.autograd.Function):
    """router_logits = F.linear(x, router_w) (sonicmoe/functional/__init__.py:438 of the reference) with the weight
    gradient as a token-split GEMM (_router_wgrad)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, router_w: torch.Tensor):
        ctx.save_for_backward(x, router_w)
        return F.linear(x, router_w)

    @staticmethod
    def backward(ctx, dlogits: torch.Tensor):
        x, router_w = ctx.saved_tensors
        dx = dlogits @ router_w if ctx.needs_input_grad[0] else None
        dw = _router_wgrad(dlogits, x, router_w) if ctx.needs_input_grad[1] else None
        return dx, dw


class TC_Softmax_Topk_Router_Function(torch.autograd.Function):
    """(scores fp32 (T, K), indices int32 (T, K)) = softmax(top-K(logits)); backward scatters into a zero (T, E)."""

    @staticmethod
    def forward(ctx, router_logits: torch.Tensor, E: int, K: int):
        T = router_logits.size(0)
        scores = torch.empty(T, K, dtype=torch.float32, device=router_logits.device)
        indices = torch.empty(T, K, dtype=torch.int32, device=router_logits.device)
        _softmax_topk_fwd(router_logits, scores, indices, E, K)
        ctx.save_for_backward(scores, indices)
        ctx.E, ctx.K, ctx.logits_dtype = E, K, router_logits.dtype
        ctx.mark_non_differentiable(indices)
        return scores, indices

    @staticmethod
    def backward(ctx, dscores: torch.Tensor, _unused):
        scores, indices = ctx.saved_tensors
        dlogits = torch.zeros(scores.size(0), ctx.E, dtype=ctx.logits_dtype, device=scores.device)
        _softmax_topk_bwd(dlogits, None, dscores, scores, indices, ctx.K)
        return dlogits, None, None


_FUSED_ROUTER = os.environ.get("SMOE_FUSED_ROUTER", "0") == "1"


@contextmanager
def fused_router(enable: bool = True):
    """Inside the block `moe_TC_softmax_topk_layer` computes logits, top-K scores / indices and the softmax column sums
    of the load-balancing loss in ONE kernel over x (`_router_forward_fused`) instead of F.linear followed by the
    top-K kernel (and a third pass for the loss).  Off by default: the kernel's logits differ from the library GEMM's in
    the last bf16 bit, so tokens whose K-th and (K+1)-th logits nearly tie may be routed differently than after
    F.linear; everything downstream is computed from the logits the kernel stores.  Shapes it does not take
    (`router_fused_supported`) use the unfused chain."""
    global _FUSED_ROUTER
    previous, _FUSED_ROUTER = _FUSED_ROUTER, enable
    try:
        yield
    finally:
        _FUSED_ROUTER = previous


_FUSED_COMBINE = os.environ.get("SMOE_FUSED_COMBINE", "0") == "1"


@contextmanager
def fused_combine(enable: bool = True):
    """Inside the block the bf16 forward pass runs the down projection and the score-weighted combine as ONE kernel
    (`_down_projection_forward_combine`): every output tile is scaled by its rows' routing scores and added onto the
    tokens' output rows with packed-bf16 atomics, `y2` (TK, H) is never stored.  Off by default: on MI355X the atomic
    traffic costs more than the stores of `y2` plus the separate gather-sum, the result carries bf16 accumulation error
    (K roundings instead of one) and is not bit-reproducible from run to run.  The backward pass is unchanged (it never
    reads `y2`)."""
    global _FUSED_COMBINE
    previous, _FUSED_COMBINE = _FUSED_COMBINE, enable
    try:
        yield
    finally:
        _FUSED_COMBINE = previous


_SCHEDULE_POLICY = "expert_index"


@contextmanager
def expert_schedule(policy: str = "largest_first"):
    """Order in which the grouped GEMMs of the layers called inside take up the experts' tiles: "expert_index" (default;
    what the reference runs, whose layers pass expert_schedule_order=None, sonicmoe/functional/__init__.py:161, :248)
    or "largest_first" (longest processing time first: the experts sorted by token count, descending).  Results do not
    depend on it."""
    global _SCHEDULE_POLICY
    if policy not in ("expert_index", "largest_first"):
        raise ValueError(f"unknown expert schedule policy {policy!r}")
    previous, _SCHEDULE_POLICY = _SCHEDULE_POLICY, policy
    try:
        yield
    finally:
        _SCHEDULE_POLICY = previous


def largest_first_schedule_order(expert_frequency_offset: torch.Tensor) -> torch.Tensor:
    """An expert_schedule_order for the grouped-GEMM operators: the experts by descending token count (ties by expert
    index), int32 (E,)."""
    counts = expert_frequency_offset[1:] - expert_frequency_offset[:-1]
    return torch.argsort(counts, descending=True, stable=True).to(torch.int32)


def _fp8_backward_requested(b1, b2, w1=None, w2=None) -> bool:
    """The fp8-backward switch as it stands while the forward pass runs (the backward pass may run outside the block).
    What the fp8 backward cannot do is refused here, in forward, not in the middle of a backward pass: weight shapes
    whose transposed quantised copies do not split into 128-element blocks.  (The fp8 kernels take the experts in index
    order: an expert_schedule policy only reorders the bf16 weight-gradient GEMMs of such a step.)"""
    if not is_using_fp8_backward():
        return False
    if w1 is not None and (w1.size(0) % 128 != 0 or w1.size(1) % 128 != 0):
        # the activation gradients contract over the up-projection's output columns (dx) and over H (dz): both are
        # quantised in blocks along those indices
        raise NotImplementedError(
            f"enable_fp8_backward: up-projection width {w1.size(0)} and hidden size {w1.size(1)} must be multiples of 128")
    return True


def _schedule_order(off):
    return largest_first_schedule_order(off) if _SCHEDULE_POLICY == "largest_first" else None


def _experts_forward(x, w1, b1, w2, b2, scores_flat, off, gidx, ridx, tok_off, K_or_maxK, is_varlen_K, activation_type,
                     stream_id, inference, order=None, sidx=None):
    """o = combine(down(act(up(gather(x))))); returns (o, z) with z = None in inference mode."""
    T, H = x.shape
    N1, _, E = w1.shape
    glu = is_glu(activation_type)
    I = N1 // 2 if glu else N1
    TK = gidx.numel()

    z = None if inference else torch.empty(TK, N1, dtype=x.dtype, device=x.device)
    y1 = None if is_using_fp8_forward() else torch.empty(TK, I, dtype=x.dtype, device=x.device)
    if _FUSED_COMBINE and sidx is not None and not is_using_fp8_forward():
        # down projection + combine in one kernel (atomic adds onto a zeroed output); y2 does not exist
        _up_projection_forward(x, w1, z, y1, b1, off, order, gidx, stream_id, activation_type.value, glu, inference)
        o = torch.zeros(T, H, dtype=x.dtype, device=x.device)
        _down_projection_forward_combine(w2, y1, o, b2, scores_flat, off, order, gidx, sidx, stream_id)
        return o, z
    y2 = torch.empty(TK, H, dtype=x.dtype, device=x.device)
    if is_using_fp8_forward():
        # a step whose backward pass runs on fp8 operands too reads each weight once for both quantised copies
        both = is_using_fp8_backward() and not inference
        quantize_weight = quantize_expert_weight_both if both else quantize_expert_weight
        xq, xs = mx_quantize(x)
        w1q, w1s = quantize_weight(w1)
        # y1 leaves the up-projection already quantised (from the fp32 accumulator); its bf16 form is not stored
        y1q = torch.empty(TK, I, dtype=torch.uint8, device=x.device)
        y1s = torch.empty(I // 128, TK, dtype=torch.int32, device=x.device)
        _up_projection_forward_fp8(
            xq, xs, w1q, w1s, z, None, b1, off, gidx, E, stream_id, activation_type.value, glu, y1q, y1s
        )
        del xq, xs, w1q, w1s
        w2q, w2s = quantize_weight(w2)
        _down_projection_forward_fp8(y1q, y1s, w2q, w2s, y2, b2, off, E, stream_id)
        del y1q, y1s, w2q, w2s
    else:
        _up_projection_forward(x, w1, z, y1, b1, off, order, gidx, stream_id, activation_type.value, glu, inference)
        _down_projection_forward(w2, y1, y2, b2, off, order, gidx, stream_id)
    del y1
    o = torch.empty(T, H, dtype=x.dtype, device=x.device)
    _router_forward(y2, o, scores_flat, ridx, tok_off, K_or_maxK, H, is_varlen_K)
    return o, z


def _experts_backward(dout, x, w1, w2, b2, z, scores_flat, off, gidx, sidx, ridx, tok_off, K_or_maxK, is_varlen_K,
                      activation_type, stream_id, has_b1, order=None, fp8=False):
    """Returns (dx, dw1, db1, dw2, db2, ds) of _experts_forward; `has_b1` says whether the forward pass had an
    up-projection bias (b1 itself is not needed for any gradient and is not kept)."""
    T, H = x.shape
    TK = gidx.numel()
    glu = is_glu(activation_type)
    dout = dout.contiguous()

    if fp8:
        return _experts_backward_fp8(dout, x, w1, w2, b2, z, scores_flat, off, gidx, sidx, ridx, tok_off, K_or_maxK,
                                     is_varlen_K, activation_type, stream_id, has_b1, order)

    dw2 = torch.empty_like(w2)  # keeps the (E, H, I)-contiguous layout of the parameter view
    db2 = None if b2 is None else torch.empty_like(b2)
    dz = torch.empty_like(z)
    ds = torch.empty(TK, dtype=torch.float32, device=x.device)
    _down_projection_backward(
        dout, z, w2, dw2, dz, ds, b2, db2, scores_flat, off, order, gidx, sidx, stream_id, glu, activation_type.value
    )
    dw1 = torch.empty_like(w1)
    db1 = torch.empty(w1.size(2), w1.size(0), dtype=x.dtype, device=x.device) if has_b1 else None
    dx_expanded = torch.empty(TK, H, dtype=x.dtype, device=x.device)
    _up_projection_backward(x, w1, dx_expanded, dw1, dz, db1, off, order, gidx, sidx, glu, stream_id)
    del dz
    dx = torch.empty(T, H, dtype=x.dtype, device=x.device)
    _token_broadcast_backward(dx, dx_expanded, ridx, tok_off, K_or_maxK, H, is_varlen_K)
    return dx, dw1, db1, dw2, db2, ds


def _experts_backward_fp8(dout, x, w1, w2, b2, z, scores_flat, off, gidx, sidx, ridx, tok_off, K_or_maxK, is_varlen_K,
                          activation_type, stream_id, has_b1, order):
    """_experts_backward with the two activation-gradient GEMMs on fp8 operands: dout and W2^T are quantised for dz,
    the dz kernel leaves dz in bf16 (for dW1 and db1) and quantised (for dx), W1^T is quantised for dx; dW2 and dW1
    are the bf16 weight-gradient GEMMs, and the bias gradients and the bias term of ds are the bf16 step's kernels."""
    T, H = x.shape
    TK = gidx.numel()
    N1, _, E = w1.shape
    glu = is_glu(activation_type)
    I = N1 // 2 if glu else N1
    doutq, dout_scales = mx_quantize(dout)
    w2tq, w2t_scales = quantize_expert_weight_transposed(w2)
    dz = torch.empty_like(z)
    dzq = torch.empty(TK, N1, dtype=torch.uint8, device=x.device)
    dzq_scales = torch.empty(N1 // 128, TK, dtype=torch.int32, device=x.device)
    y1s = torch.empty(TK, I, dtype=x.dtype, device=x.device)
    ds = torch.empty(TK, dtype=torch.float32, device=x.device)
    _down_projection_backward_fp8(doutq, dout_scales, w2tq, w2t_scales, z, dz, dzq, dzq_scales, y1s, ds, scores_flat,
                                  off, gidx, sidx, E, stream_id, activation_type.value, glu)
    del doutq, dout_scales, w2tq, w2t_scales
    if b2 is not None:  # y2 = y1 W2^T + b2 puts <dout, b2> into the score gradient
        _score_grad_bias_term(dout, b2, ds, off, gidx, sidx, stream_id)
    dw2 = torch.empty_like(w2)
    db2 = None if b2 is None else torch.empty_like(b2)
    _down_projection_weight_grad(dout, y1s, dw2, db2, scores_flat, off, order, gidx, sidx, stream_id)
    del y1s
    w1tq, w1t_scales = quantize_expert_weight_transposed(w1)
    dx_expanded = torch.empty(TK, H, dtype=x.dtype, device=x.device)
    _down_projection_forward_fp8(dzq, dzq_scales, w1tq, w1t_scales, dx_expanded, None, off, E, stream_id)
    del dzq, dzq_scales, w1tq, w1t_scales
    dw1 = torch.empty_like(w1)
    db1 = torch.empty(w1.size(2), w1.size(0), dtype=x.dtype, device=x.device) if has_b1 else None
    _up_projection_backward(x, w1, None, dw1, dz, db1, off, order, gidx, sidx, glu, stream_id)
    del dz
    dx = torch.empty(T, H, dtype=x.dtype, device=x.device)
    _token_broadcast_backward(dx, dx_expanded, ridx, tok_off, K_or_maxK, H, is_varlen_K)
    return dx, dw1, db1, dw2, db2, ds


class _ExpertsFunction(torch.autograd.Function):
    """o = combine(down(act(up(gather(x))))) over the routed (token, expert) pairs.

    Differentiable inputs: x (T, H), w1 (N1, H, E) view, b1 (E, N1) or None, w2 (H, I, E) view, b2 (E, H) or None,
    scores (flat, fp32); N1 = 2I for the gated activations, I otherwise.
    """

    @staticmethod
    def forward(
        ctx,
        x,
        w1,
        b1,
        w2,
        b2,
        scores_flat,
        off,
        gidx,
        sidx,
        ridx,
        tok_off,
        K_or_maxK: int,
        is_varlen_K: bool,
        activation_type: ActivationType,
        stream_id: int,
        inference: bool,
    ):
        x = x.contiguous()
        scores_flat = scores_flat.contiguous()
        order = _schedule_order(off)
        o, z = _experts_forward(x, w1, b1, w2, b2, scores_flat, off, gidx, ridx, tok_off, K_or_maxK, is_varlen_K,
                                activation_type, stream_id, inference, order, sidx)
        ctx.order = order
        ctx.fp8_backward = _fp8_backward_requested(b1, b2, w1, w2)
        if not inference:
            ctx.save_for_backward(x, w1, w2, b2, z, scores_flat, off, gidx, sidx, ridx, tok_off)
        ctx.cfg = (K_or_maxK, is_varlen_K, activation_type, stream_id, inference, b1 is not None)
        return o

    @staticmethod
    def backward(ctx, dout):
        K_or_maxK, is_varlen_K, activation_type, stream_id, inference, has_b1 = ctx.cfg
        if inference:
            raise RuntimeError("backward through an inference-mode MoE forward: z was not stored")
        x, w1, w2, b2, z, scores_flat, off, gidx, sidx, ridx, tok_off = ctx.saved_tensors
        dx, dw1, db1, dw2, db2, ds = _experts_backward(
            dout, x, w1, w2, b2, z, scores_flat, off, gidx, sidx, ridx, tok_off, K_or_maxK, is_varlen_K, activation_type,
            stream_id, has_b1, ctx.order, ctx.fp8_backward,
        )
        return dx, dw1, db1, dw2, db2, ds, None, None, None, None, None, None, None, None, None, None


def _router_wgrad(dlogits: torch.Tensor, x: torch.Tensor, like: torch.Tensor) -> torch.Tensor:
    """dWr = dlogits^T x: a token-split GEMM where the kernel supports the shape (it has only E output rows and T
    contraction elements, which a library GEMM without a split runs on an eighth of the chip), torch otherwise."""
    T, E = dlogits.shape
    H = x.size(1)
    fast = (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and dlogits.dtype == x.dtype and E % 8 == 0
            and H % 8 == 0)
    if fast and T >= 256 and os.environ.get("SMOE_ROUTER_WGRAD", "1") != "0":
        partial = torch.empty(router_weight_grad_chunks(T, E, H), E, H, dtype=x.dtype, device=x.device)
        _router_weight_grad(dlogits.contiguous(), x.contiguous(), partial)
        return partial.sum(0, dtype=torch.float32).to(like.dtype) if partial.size(0) > 1 else partial[0]
    return dlogits.t() @ x


class _TCLayerFunction(torch.autograd.Function):
    """The whole token-choice layer as one autograd node: router GEMM -> top-K softmax -> metadata -> experts.

    One node instead of three lets the backward pass form dx = dx_experts + dlogits Wr inside the router GEMM
    (`addmm_` on the experts' dx) instead of leaving the sum of the two paths to autograd's elementwise add, and
    adds a gradient arriving at router_logits from outside (an auxiliary loss) before the router GEMMs."""

    @staticmethod
    def forward(ctx, x, router_w, w1, b1, w2, b2, K: int, activation_type: ActivationType, stream_id: int,
                inference: bool):
        T, E = x.size(0), router_w.size(0)
        x = x.contiguous()
        scores = torch.empty(T, K, dtype=torch.float32, device=x.device)
        indices = torch.empty(T, K, dtype=torch.int32, device=x.device)
        if _FUSED_ROUTER and router_fused_supported(x, router_w):
            router_logits = torch.empty(T, E, dtype=x.dtype, device=x.device)
            colsum = torch.empty(router_fused_partials(T, E), E, dtype=torch.float32, device=x.device)
            _router_forward_fused(x, router_w.contiguous(), router_logits, scores, indices, colsum)
            # picked up by switch_loss() when it is handed this very tensor (MoE.forward does that).  Under torch.compile
            # a tensor attribute does not survive tracing: the loss then takes its own pass over the logits.
            if not torch.compiler.is_compiling():
                router_logits._smoe_softmax_colsum_partials = (colsum, router_logits._version)
        else:
            router_logits = F.linear(x, router_w)
            _softmax_topk_fwd(router_logits, scores, indices, E, K)
        freq, off, gidx, sidx, ridx, tok_off = _build_metadata(indices.view(-1), None, T, E, K)
        scores_flat = scores.view(-1)
        order = _schedule_order(off)
        o, z = _experts_forward(x, w1, b1, w2, b2, scores_flat, off, gidx, ridx, tok_off, K, False, activation_type,
                                stream_id, inference, order, sidx)
        ctx.order = order
        ctx.fp8_backward = _fp8_backward_requested(b1, b2, w1, w2)
        if not inference:
            ctx.save_for_backward(x, router_w, w1, w2, b2, z, scores, indices, off, gidx, sidx, ridx, tok_off)
        ctx.cfg = (K, activation_type, stream_id, inference, router_logits.dtype, b1 is not None)
        ctx.mark_non_differentiable(freq)
        return o, router_logits, freq

    @staticmethod
    def backward(ctx, dout, dlogits_outside, _dfreq):
        K, activation_type, stream_id, inference, logits_dtype, has_b1 = ctx.cfg
        if inference:
            raise RuntimeError("backward through an inference-mode MoE forward: z was not stored")
        x, router_w, w1, w2, b2, z, scores, indices, off, gidx, sidx, ridx, tok_off = ctx.saved_tensors
        T, E = x.size(0), router_w.size(0)
        dx, dw1, db1, dw2, db2, ds = _experts_backward(
            dout, x, w1, w2, b2, z, scores.view(-1), off, gidx, sidx, ridx, tok_off, K, False, activation_type, stream_id,
            has_b1, ctx.order, ctx.fp8_backward,
        )
        dlogits = torch.zeros(T, E, dtype=logits_dtype, device=x.device)
        _softmax_topk_bwd(dlogits, None, ds.view(T, K), scores, indices, K)
        if dlogits_outside is not None:
            dlogits = dlogits + dlogits_outside
        dwr = _router_wgrad(dlogits, x, router_w) if ctx.needs_input_grad[1] else None
        if ctx.needs_input_grad[0]:
            dx.addmm_(dlogits, router_w)  # dx_experts + dlogits Wr in the GEMM's epilogue
        else:
            dx = None
        return dx, dwr, dw1, db1, dw2, db2, None, None, None, None


class _SwitchLossFunction(torch.autograd.Function):
    """aux = E * <norm_1(sum_t softmax(logits)), norm_1(freq)> (fp32 scalar); the gradient reaches the logits only."""

    @staticmethod
    def forward(ctx, router_logits: torch.Tensor, expert_frequency: torch.Tensor):
        E = router_logits.size(-1)
        logits = router_logits.reshape(-1, E)
        if logits.stride(1) != 1:
            logits = logits.contiguous()
        freq = expert_frequency.to(torch.int32).contiguous()
        acc = torch.empty(E, dtype=torch.float32, device=logits.device)
        aux = torch.empty(1, dtype=torch.float32, device=logits.device)
        partials, version = getattr(router_logits, "_smoe_softmax_colsum_partials", (None, None))
        if partials is not None and version == router_logits._version and router_logits.dim() == 2:
            _switch_loss_from_partials(partials, freq, acc, aux)  # the fused router already summed the softmax columns
        else:
            _switch_loss_fwd(logits, freq, acc, aux)
        ctx.save_for_backward(logits, freq, acc)
        ctx.logits_shape = router_logits.shape
        return aux.view(())

    @staticmethod
    def backward(ctx, grad_aux: torch.Tensor):
        logits, freq, acc = ctx.saved_tensors
        dlogits = torch.empty_like(logits, memory_format=torch.contiguous_format)
        _switch_loss_bwd(logits, freq, acc, grad_aux.reshape(1).float().contiguous(), dlogits)
        return dlogits.view(ctx.logits_shape), None


def switch_loss(router_logits: torch.Tensor, expert_frequency: torch.Tensor) -> torch.Tensor:
    """Load-balancing loss of the reference's MoE._compute_switch_loss (sonicmoe/moe.py:261-274) from the router
    logits (..., E) and the per-expert token counts (E): the softmax, its column sums, both normalisations and the dot
    product in two launches forward and one backward, without a (T, E) fp32 tensor."""
    if router_logits.numel() == 0:  # no tokens: both normalisations clamp and the loss is 0, as in the reference
        acc = F.softmax(router_logits.reshape(-1, router_logits.size(-1)), dim=-1, dtype=torch.float32).sum(0)
        f = F.normalize(expert_frequency.float(), p=1, dim=0)
        return router_logits.size(-1) * (F.normalize(acc, p=1, dim=0) * f).sum()
    return _SwitchLossFunction.apply(router_logits, expert_frequency)


def _check_bias(b1, b2):
    assert (b1 is None) == (b2 is None), "b1 and b2 has to be None or not None at the same time!"
    if b1 is not None:
        return b1.contiguous(), b2.contiguous()
    return None, None


def _as_activation(activation_type) -> ActivationType:
    return ActivationType(activation_type) if isinstance(activation_type, str) else activation_type


# ---------------------------------------------------------------------------------------------------------------
# layer entry points
# ---------------------------------------------------------------------------------------------------------------


def moe_TC_softmax_topk_layer(
    x: torch.Tensor,
    router_w: torch.Tensor,
    w1: torch.Tensor,
    b1: torch.Tensor | None,
    w2: torch.Tensor,
    b2: torch.Tensor | None,
    K: int,
    stream_id: int,
    activation_type: ActivationType | str = ActivationType.SWIGLU,
    is_inference_mode_enabled: bool = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Token-choice top-K MoE layer (interface of sonicmoe/functional/__init__.py:423-490).

    x (T, H); router_w (E, H); w1 (2I, H, E) and w2 (H, I, E) are permuted views of the (E, out, in) parameters.
    Returns (o (T, H), router_logits (T, E), expert_frequency (E,) int32).
    """
    b1, b2 = _check_bias(b1, b2)
    activation_type = _as_activation(activation_type)
    if os.environ.get("SMOE_FUSED_TC_LAYER", "1") == "0":  # the layer as three autograd nodes, as the reference builds it
        T, E = x.size(0), router_w.size(0)
        router_logits = _RouterLinearFunction.apply(x, router_w)
        topk_scores, topk_indices = TC_Softmax_Topk_Router_Function.apply(router_logits, E, K)
        freq, off, gidx, sidx, ridx, tok_off = _build_metadata(topk_indices.view(-1), None, T, E, K)
        o = _ExpertsFunction.apply(
            x, w1, b1, w2, b2, topk_scores.view(-1), off, gidx, sidx, ridx, tok_off, K, False, activation_type,
            stream_id, is_inference_mode_enabled,
        )
        return o, router_logits, freq
    return _TCLayerFunction.apply(
        x, router_w, w1, b1, w2, b2, K, activation_type, stream_id, is_inference_mode_enabled
    )


def moe_general_routing_inputs(
    x: torch.Tensor,
    router_scores: torch.Tensor,
    token_indices: torch.Tensor,
    expert_indices: torch.Tensor,
    w1: torch.Tensor,
    b1: torch.Tensor | None,
    w2: torch.Tensor,
    b2: torch.Tensor | None,
    E: int,
    stream_id: int,
    activation_type: ActivationType,
    is_inference_mode_enabled: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """MoE layer for arbitrary routing (interface of sonicmoe/functional/__init__.py:497-562): pair j sends token
    token_indices[j] (SORTED ascending) to expert expert_indices[j] with weight router_scores[j].
    Returns (o (T, H), expert_frequency (E,) int32); d(router_scores) comes back in the pairs' order."""
    b1, b2 = _check_bias(b1, b2)
    activation_type = _as_activation(activation_type)
    T = x.size(0)
    E = w2.size(-1)
    freq, off, gidx, sidx, ridx, tok_off = _build_metadata(expert_indices, token_indices, T, E, 1)
    o = _ExpertsFunction.apply(
        x, w1, b1, w2, b2, router_scores.float(), off, gidx, sidx, ridx, tok_off, E, True, activation_type, stream_id,
        is_inference_mode_enabled,
    )
    return o, freq


__all__ = [
    "TC_Softmax_Topk_Router_Function",
    "TC_topk_router_metadata",
    "general_routing_router_metadata",
    "count_cumsum",
    "enable_quack_gemm",
    "is_using_quack_gemm",
    "enable_fp8_forward",
    "is_using_fp8_forward",
    "enable_fp8_backward",
    "is_using_fp8_backward",
    "expert_schedule",
    "fused_combine",
    "fused_router",
    "largest_first_schedule_order",
    "moe_TC_softmax_topk_layer",
    "moe_general_routing_inputs",
    "switch_loss",
]
