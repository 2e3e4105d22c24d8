"""Forward operators `sonicmoe::*` (names, arguments and mutation contracts of sonicmoe/functional/forward.py).

Every operator is an out-variant: the caller allocates the outputs, the operator fills them through the C ABI of
libsonicmoe_hip.so on the given stream and returns None.
"""

from __future__ import annotations

import torch

from .. import _lib
from ..enums import ACTIVATION_CODE, LIBRARY_NAME, ActivationType
from ..utils import expert_major_strides


def _gemm_workspace(TK: int, E: int, device, stream_id: int, fp8_gathered_k: int = 0) -> torch.Tensor:
    """Tile-map scratch of one grouped-GEMM launch (`fp8_gathered_k`: contraction size of an fp8 operator with a gathered
    token operand, whose workspace also holds the gathered rows' scale words).  It comes from PyTorch's caching allocator, which orders its reuse
    on the CURRENT stream, and the routing / combine kernels around the GEMM run on the current stream as well: a
    GEMM launched on any other stream would race with both, so that is refused."""
    current = _lib.current_stream_handle()
    if stream_id != current:
        raise RuntimeError(
            f"grouped GEMM asked to run on stream {stream_id:#x} while PyTorch's current stream is {current:#x}: pass "
            "torch.cuda.current_stream().cuda_stream (a MoE module keeps the stream it was constructed under in "
            "`.stream_id`; set it again when calling the module under another stream)"
        )
    if fp8_gathered_k:
        n = _lib.lib().smoe_fp8_gemm_workspace_bytes(TK, E, fp8_gathered_k)
    else:
        n = _lib.lib().smoe_gemm_workspace_bytes(TK, E)
    return torch.empty(max(n, 16), dtype=torch.uint8, device=device)


def _check_bf16(*named):
    for name, t in named:
        if t is not None and t.dtype != torch.bfloat16:
            raise NotImplementedError(f"{name}: this operator takes bfloat16 tensors, got {t.dtype}")


def _elem_dtype(*named) -> torch.dtype:
    """The 16-bit element type of an operator call (it selects the library build, `_lib.lib(dtype)`): every tensor
    given has the same one, bfloat16 or float16 -- the types the reference's grouped GEMMs take
    (sonicmoe/functional/grouped_gemm.py:3033-3044)."""
    dt = None
    for name, t in named:
        if t is None:
            continue
        if t.dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"{name}: the HIP grouped GEMMs take bfloat16 or float16 tensors, got {t.dtype}")
        if dt is None:
            dt = t.dtype
        elif t.dtype != dt:
            raise NotImplementedError(f"{name} is {t.dtype} next to {dt} tensors: one operator call, one element type")
    return dt or torch.bfloat16


def _check_schedule_order(order: torch.Tensor | None, E: int) -> None:
    """expert_schedule_order: None or E int32 holding a permutation of the experts (position i of the tile schedule works
    on expert order[i]); the values are not inspected -- that would cost a host round trip."""
    if order is not None and (order.dtype != torch.int32 or order.shape != (E,) or not order.is_contiguous()):
        raise ValueError(f"expert_schedule_order must be a contiguous int32 tensor of {E} experts, got "
                         f"{order.dtype} {tuple(order.shape)}")


@torch.library.custom_op(f"{LIBRARY_NAME}::_topk_fwd", mutates_args={"values", "indices"})
def _topk_fwd(
    x: torch.Tensor, k: int, values: torch.Tensor, indices: torch.Tensor, require_softmax_fusion: bool = True
) -> None:
    """Row-wise top-k of x (M, N) -> values (M, k) fp32 (softmax over the winners if requested), indices (M, k) int32."""
    _lib.require_device(x, values, indices)
    if x.dtype not in _lib.DT_CODE:
        raise NotImplementedError(f"_topk_fwd: unsupported logits dtype {x.dtype}")
    assert values.dtype == torch.float32 and indices.dtype == torch.int32
    assert values.is_contiguous() and indices.is_contiguous() and x.stride(1) == 1
    M, N = x.shape
    rc = _lib.lib().smoe_topk_softmax_fwd(
        _lib.ptr(x),
        _lib.DT_CODE[x.dtype],
        M,
        N,
        k,
        x.stride(0),
        _lib.ptr(values),
        _lib.ptr(indices),
        1 if require_softmax_fusion else 0,
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "_topk_fwd")


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_softmax_topk_fwd", mutates_args={"topk_router_score", "topk_router_indices"}
)
def _softmax_topk_fwd(
    router_logits: torch.Tensor, topk_router_score: torch.Tensor, topk_router_indices: torch.Tensor, E: int, K: int
) -> None:
    _topk_fwd(router_logits, K, topk_router_score, topk_router_indices, True)


@torch.library.custom_op(f"{LIBRARY_NAME}::_up_projection_forward", mutates_args={"z", "y1"})
def _up_projection_forward(
    x: torch.Tensor,
    w1: torch.Tensor,
    z: torch.Tensor | None,
    y1: torch.Tensor,
    b1: torch.Tensor | None,
    expert_frequency_offset: torch.Tensor,
    expert_schedule_order: torch.Tensor | None,
    x_gather_idx: torch.Tensor,
    stream_id: int,
    activation_type: str,
    is_glu_activation: bool,
    is_inference_mode_enabled: bool = False,
) -> None:
    """z = gather(x) W1^T (+ b1), y1 = act(z); w1 is the (N1, H, E) view of the (E, N1, H) parameter, N1 = 2I for the
    gated activations and I otherwise; b1 is (E, N1)."""
    _lib.require_device(x, w1, y1, b1, expert_frequency_offset, expert_schedule_order, x_gather_idx)
    _check_schedule_order(expert_schedule_order, w1.size(2))
    dt = _elem_dtype(("x", x), ("w1", w1), ("z", z), ("y1", y1), ("b1", b1))
    N1, H, E = w1.shape
    I = N1 // 2 if is_glu_activation else N1
    T, TK = x.size(0), y1.size(0)
    assert x.is_contiguous() and y1.is_contiguous() and (z is None or z.is_contiguous())
    assert b1 is None or (b1.shape == (E, N1) and b1.is_contiguous())
    s_e, s_row = expert_major_strides(w1, "w1")
    ws = _gemm_workspace(TK, E, x.device, stream_id)
    rc = _lib.lib(dt).smoe_up_projection_forward(
        _lib.ptr(x),
        _lib.ptr(w1),
        s_e,
        s_row,
        _lib.ptr(b1),
        None if is_inference_mode_enabled else _lib.ptr(z),
        _lib.ptr(y1),
        _lib.ptr(expert_frequency_offset),
        _lib.ptr(expert_schedule_order),
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
    _lib.check(rc, "_up_projection_forward")


@torch.library.custom_op(f"{LIBRARY_NAME}::_down_projection_forward", mutates_args={"y2"})
def _down_projection_forward(
    w2: torch.Tensor,
    y1: torch.Tensor,
    y2: torch.Tensor,
    b2: torch.Tensor | None,
    expert_frequency_offset: torch.Tensor,
    expert_schedule_order: torch.Tensor | None,
    x_gather_idx: torch.Tensor,
    stream_id: int,
) -> None:
    """y2 = y1 W2^T (+ b2) per expert; w2 is the (H, I, E) view of the (E, H, I) parameter, b2 is (E, H)."""
    _lib.require_device(w2, y1, y2, b2, expert_frequency_offset, expert_schedule_order)
    _check_schedule_order(expert_schedule_order, w2.size(2))
    dt = _elem_dtype(("w2", w2), ("y1", y1), ("y2", y2), ("b2", b2))
    H, I, E = w2.shape
    TK = y1.size(0)
    assert y1.is_contiguous() and y2.is_contiguous()
    assert b2 is None or (b2.shape == (E, H) and b2.is_contiguous())
    s_e, s_row = expert_major_strides(w2, "w2")
    ws = _gemm_workspace(TK, E, y1.device, stream_id)
    rc = _lib.lib(dt).smoe_down_projection_forward(
        _lib.ptr(y1),
        _lib.ptr(w2),
        s_e,
        s_row,
        _lib.ptr(b2),
        _lib.ptr(y2),
        _lib.ptr(expert_frequency_offset),
        _lib.ptr(expert_schedule_order),
        TK,
        H,
        I,
        E,
        _lib.ptr(ws),
        ws.numel(),
        stream_id,
    )
    _lib.check(rc, "_down_projection_forward")


@torch.library.custom_op(f"{LIBRARY_NAME}::_down_projection_forward_combine", mutates_args={"o"})
def _down_projection_forward_combine(
    w2: torch.Tensor,
    y1: torch.Tensor,
    o: torch.Tensor,
    b2: torch.Tensor | None,
    topk_scores: torch.Tensor,
    expert_frequency_offset: torch.Tensor,
    expert_schedule_order: torch.Tensor | None,
    x_gather_idx: torch.Tensor,
    s_scatter_idx: torch.Tensor,
    stream_id: int,
) -> None:
    """o[x_gather_idx[m]] += topk_scores[s_scatter_idx[m]] * (y1[m] W2[e]^T (+ b2[e])): the down projection and the
    score-weighted combine (`_down_projection_forward` + `_router_forward`, sonicmoe/functional/forward.py:132-236) as
    ONE kernel that never stores y2.  `o` (T, H) must be zero on entry.  The additions are packed-bf16 atomics: within
    bf16 accumulation error of the two-kernel path, not bit-reproducible from run to run, and slower on MI355X; an
    option (`sonicmoe.functional.fused_combine()`), not the default."""
    _lib.require_device(w2, y1, o, b2, topk_scores, expert_frequency_offset, expert_schedule_order, x_gather_idx,
                        s_scatter_idx)
    _check_schedule_order(expert_schedule_order, w2.size(2))
    dt = _elem_dtype(("w2", w2), ("y1", y1), ("o", o), ("b2", b2))
    H, I, E = w2.shape
    T, TK = o.size(0), y1.size(0)
    assert y1.is_contiguous() and o.is_contiguous() and o.size(1) == H
    assert topk_scores.dtype == torch.float32 and topk_scores.is_contiguous()
    assert x_gather_idx.dtype == torch.int32 and s_scatter_idx.dtype == torch.int32
    assert x_gather_idx.numel() == TK and s_scatter_idx.numel() == TK
    assert b2 is None or (b2.shape == (E, H) and b2.is_contiguous())
    s_e, s_row = expert_major_strides(w2, "w2")
    ws = _gemm_workspace(TK, E, y1.device, stream_id)
    rc = _lib.lib(dt).smoe_down_projection_forward_combine(
        _lib.ptr(y1),
        _lib.ptr(w2),
        s_e,
        s_row,
        _lib.ptr(b2),
        _lib.ptr(o),
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
        _lib.ptr(ws),
        ws.numel(),
        stream_id,
    )
    _lib.check(rc, "_down_projection_forward_combine")


def _gather_sum(src, out, weights, ridx, tok_off, K, H, is_varlen_K, what):
    _lib.require_device(src, out, weights, ridx, tok_off)
    dt = _elem_dtype((what + ".src", src), (what + ".out", out))
    assert src.is_contiguous() and out.is_contiguous() and ridx.dtype == torch.int32
    if weights is not None:
        assert weights.dtype == torch.float32 and weights.is_contiguous()
    if src.size(0) == 0:  # no routed row at all: every token's sum is empty
        out.zero_()
        return
    rc = _lib.lib(dt).smoe_gather_sum(
        _lib.ptr(src),
        _lib.ptr(out),
        _lib.ptr(weights),
        _lib.ptr(ridx),
        _lib.ptr(tok_off) if is_varlen_K else None,
        out.size(0),
        K,
        H,
        _lib.current_stream_handle(),
    )
    _lib.check(rc, what)


@torch.library.custom_op(f"{LIBRARY_NAME}::_router_forward", mutates_args={"o"})
def _router_forward(
    y2: torch.Tensor,
    o: torch.Tensor,
    topk_scores: torch.Tensor,
    s_reverse_scatter_idx: torch.Tensor,
    num_activated_expert_per_token_offset: torch.Tensor,
    varlen_K_max: int,
    H: int,
    is_varlen_K: bool,
) -> None:
    """o[t] = sum over the token's routing slots j of topk_scores[j] * y2[s_reverse_scatter_idx[j]]."""
    _gather_sum(
        y2,
        o,
        topk_scores,
        s_reverse_scatter_idx,
        num_activated_expert_per_token_offset,
        varlen_K_max,
        H,
        is_varlen_K,
        "_router_forward",
    )


@torch.library.custom_op(f"{LIBRARY_NAME}::_switch_loss_fwd", mutates_args={"acc", "aux"})
def _switch_loss_fwd(router_logits: torch.Tensor, expert_frequency: torch.Tensor, acc: torch.Tensor,
                     aux: torch.Tensor) -> None:
    """acc (E) fp32 = column sums of softmax(router_logits) in fp32; aux (1) fp32 = E * <acc / |acc|_1, freq / |freq|_1>:
    the switch loss of the reference's MoE._compute_switch_loss (sonicmoe/moe.py:261-274) in one pass over the
    logits."""
    _lib.require_device(router_logits, expert_frequency, acc, aux)
    if router_logits.dtype not in _lib.DT_CODE:
        raise NotImplementedError(f"_switch_loss_fwd: unsupported dtype {router_logits.dtype}")
    T, E = router_logits.shape
    assert router_logits.stride(1) == 1 and expert_frequency.dtype == torch.int32 and expert_frequency.is_contiguous()
    assert expert_frequency.numel() == E and acc.numel() == E and acc.dtype == torch.float32 and acc.is_contiguous()
    assert aux.numel() == 1 and aux.dtype == torch.float32
    ws_bytes = _lib.lib().smoe_switch_loss_workspace_bytes(T, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=router_logits.device)
    rc = _lib.lib().smoe_switch_loss_fwd(
        _lib.ptr(router_logits), _lib.DT_CODE[router_logits.dtype], router_logits.stride(0), T, E,
        _lib.ptr(expert_frequency), _lib.ptr(acc), _lib.ptr(aux), _lib.ptr(ws), ws_bytes,
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "_switch_loss_fwd")


def router_fused_supported(x: torch.Tensor, router_w: torch.Tensor) -> bool:
    """Shapes and dtypes `_router_forward_fused` takes: bf16, E a multiple of 16 up to 256, H a multiple of 256."""
    E, H = router_w.shape
    return (x.is_cuda and x.dtype == torch.bfloat16 and router_w.dtype == torch.bfloat16 and E % 16 == 0
            and 16 <= E <= 256 and H % 256 == 0 and x.size(0) > 0)


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_router_forward_fused", mutates_args={"router_logits", "topk_scores", "topk_indices", "colsum_partial"}
)
def _router_forward_fused(x: torch.Tensor, router_w: torch.Tensor, router_logits: torch.Tensor,
                          topk_scores: torch.Tensor, topk_indices: torch.Tensor,
                          colsum_partial: torch.Tensor | None) -> None:
    """router_logits = x router_w^T, the top-K of every row with softmax scores, and (if colsum_partial is given) the
    per-workgroup column sums of softmax(router_logits), in one kernel: the reference's F.linear followed by
    sonicmoe::_softmax_topk_fwd (sonicmoe/functional/__init__.py:438-439) and the softmax column sums of
    MoE._compute_switch_loss (sonicmoe/moe.py:261-264).  colsum_partial: (router_fused_partials(T, E), E) fp32."""
    _lib.require_device(x, router_w, router_logits, topk_scores, topk_indices, colsum_partial)
    _check_bf16(("x", x), ("router_w", router_w), ("router_logits", router_logits))
    T, H = x.shape
    E = router_w.size(0)
    K = topk_scores.size(1)
    assert x.is_contiguous() and router_w.is_contiguous() and router_logits.is_contiguous()
    assert router_w.shape == (E, H) and router_logits.shape == (T, E)
    assert topk_scores.shape == (T, K) and topk_scores.dtype == torch.float32 and topk_scores.is_contiguous()
    assert topk_indices.shape == (T, K) and topk_indices.dtype == torch.int32 and topk_indices.is_contiguous()
    if colsum_partial is not None:
        assert colsum_partial.dtype == torch.float32 and colsum_partial.is_contiguous()
        assert colsum_partial.shape == (_lib.lib().smoe_router_fused_partials(T, E), E)
    rc = _lib.lib().smoe_router_forward_fused(
        _lib.ptr(x), _lib.ptr(router_w), T, H, E, K, _lib.ptr(router_logits), _lib.ptr(topk_scores),
        _lib.ptr(topk_indices), _lib.ptr(colsum_partial), _lib.current_stream_handle(),
    )
    _lib.check(rc, "_router_forward_fused")


def router_fused_partials(T: int, E: int) -> int:
    return int(_lib.lib().smoe_router_fused_partials(T, E))


@torch.library.custom_op(f"{LIBRARY_NAME}::_switch_loss_from_partials", mutates_args={"acc", "aux"})
def _switch_loss_from_partials(colsum_partial: torch.Tensor, expert_frequency: torch.Tensor, acc: torch.Tensor,
                               aux: torch.Tensor) -> None:
    """acc, aux of `_switch_loss_fwd` from the column-sum partials `_router_forward_fused` wrote."""
    _lib.require_device(colsum_partial, expert_frequency, acc, aux)
    n, E = colsum_partial.shape
    assert colsum_partial.dtype == torch.float32 and colsum_partial.is_contiguous()
    assert expert_frequency.dtype == torch.int32 and expert_frequency.is_contiguous() and expert_frequency.numel() == E
    assert acc.numel() == E and acc.dtype == torch.float32 and acc.is_contiguous() and aux.numel() == 1
    rc = _lib.lib().smoe_switch_loss_from_partials(
        _lib.ptr(colsum_partial), n, E, _lib.ptr(expert_frequency), _lib.ptr(acc), _lib.ptr(aux),
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "_switch_loss_from_partials")
