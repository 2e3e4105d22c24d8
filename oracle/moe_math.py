"""Floating-point side of the hot path, restated with plain torch on the CPU.  TEST INFRASTRUCTURE ONLY.

Two layers are restated:

* `moe_torch_backend`  - the reference's own torch backend (sonicmoe/moe.py:276-363), the parity target
  named by the reference's tests (tests/moe_test.py:87-118).  Differentiable through torch.autograd.
* the operator-level functions (`up_projection_forward` ... `softmax_topk_bwd`) - what each
  `sonicmoe::*` operator computes, with the hand-derived backward formulas of the fused epilogues
  (sonicmoe/functional/grouped_gemm.py:1154-1168, :1311-1333, :2536-2561; functional/backward.py).

All functions take weights in the PARAMETER layout: w1 (E, 2I, H), w2 (E, H, I); gate rows of w1 are the
even rows, up rows the odd rows (moe.py:24-27).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def swiglu(z: torch.Tensor) -> torch.Tensor:
    """moe.py:24-27: up = odd columns, gate = even columns."""
    return z[..., 1::2] * F.silu(z[..., ::2])


# moe.py:24-60 (activation definitions of the torch backend) and enums.py:18-30 (names, which ones are gated).
# The torch backend evaluates GELU in its exact (erf) form.
GLU_ACTIVATIONS = ("swiglu", "geglu", "reglu")
_POINTWISE = {
    "swiglu": F.silu,
    "geglu": F.gelu,
    "reglu": F.relu,
    "relu_sq": lambda t: F.relu(t) ** 2,
    "relu": F.relu,
    "gelu": F.gelu,
    "silu": F.silu,
}


def is_glu(activation: str) -> bool:
    return activation in GLU_ACTIVATIONS


def activation_forward(z: torch.Tensor, activation: str = "swiglu") -> torch.Tensor:
    """y1 = f(z_even) * z_odd for the gated activations, f(z) otherwise (moe.py:24-60)."""
    f = _POINTWISE[activation]
    if is_glu(activation):
        return f(z[..., ::2]) * z[..., 1::2]
    return f(z)


def _pointwise_with_derivative(t: torch.Tensor, activation: str):
    """(f(t), f'(t)) written out by hand (the forms the fused epilogues evaluate: grouped_gemm.py:1154-1271, with the
    exact GELU of the torch backend in place of the tanh approximation)."""
    if activation in ("swiglu", "silu"):
        sig = torch.sigmoid(t)
        return t * sig, t * sig * (1 - sig) + sig
    if activation in ("geglu", "gelu"):
        cdf = 0.5 * (1 + torch.erf(t * 0.7071067811865476))
        pdf = torch.exp(-0.5 * t * t) * 0.3989422804014327
        return t * cdf, cdf + t * pdf
    if activation in ("reglu", "relu"):
        return t.clamp_min(0), (t > 0).to(t.dtype)
    if activation == "relu_sq":
        r = t.clamp_min(0)
        return r * r, 2 * r
    raise ValueError(activation)


def activation_backward(z: torch.Tensor, dy1: torch.Tensor, activation: str = "swiglu"):
    """(dz, y1) for upstream gradient dy1 of y1 = activation_forward(z)."""
    if is_glu(activation):
        g, u = z[..., ::2], z[..., 1::2]
        f, fp = _pointwise_with_derivative(g, activation)
        dz = torch.empty_like(z)
        dz[..., ::2] = dy1 * u * fp
        dz[..., 1::2] = dy1 * f
        return dz, f * u
    f, fp = _pointwise_with_derivative(z, activation)
    return dy1 * fp, f


def switch_aux_loss(logits: torch.Tensor, expert_frequency: torch.Tensor) -> torch.Tensor:
    """moe.py:261-274 with probs = softmax(logits, fp32) (moe.py:253)."""
    logits = logits.reshape(-1, logits.size(-1))
    probs = F.softmax(logits, dim=-1, dtype=torch.float32)
    E = logits.size(1)
    acc = probs.sum(0)
    f = expert_frequency.float()
    return E * (F.normalize(acc, p=1, dim=0) * F.normalize(f, p=1, dim=0)).sum()


def moe_torch_backend(
    x: torch.Tensor,
    router_w: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    K: int,
    b1: torch.Tensor | None = None,
    b2: torch.Tensor | None = None,
    selected_experts: torch.Tensor | None = None,
    math_dtype: torch.dtype = torch.float32,
    gate_dtype: torch.dtype | None = None,
    activation: str = "swiglu",
):
    """Restatement of MoE.forward(kernel_backend_moe=torch) (moe.py:232-245, :276-363).

    The reference test runs it under autocast(float32) (tests/moe_test.py:87), i.e. the linears are evaluated
    in `math_dtype` on the (bf16-rounded) parameters and activations, while the gates are rounded to the
    activation dtype (moe.py:286-287; `gate_dtype`, default x.dtype).

    `selected_experts` (T, K) overrides torch.topk's choice so that downstream tensors can be compared
    when logits hold ties (torch.topk's tie order is unspecified).
    Returns (out (T, H) math_dtype, router_logits (T, E), expert_frequency (E,) int32).
    """
    T, H = x.shape
    E = router_w.size(0)
    gate_dtype = x.dtype if gate_dtype is None else gate_dtype
    xm = x.to(math_dtype)
    logits = F.linear(xm, router_w.to(math_dtype))  # moe.py:278
    if selected_experts is None:
        top_v, sel = logits.topk(K, dim=-1)  # moe.py:365-371
    else:
        sel = selected_experts.long()
        top_v = logits.gather(1, sel)
    gates = F.softmax(top_v.float(), dim=-1).to(gate_dtype)  # moe.py:286-287
    flat = sel.flatten()
    _, sorted_scattered = flat.sort(stable=True)  # moe.py:301
    freq = flat.bincount(minlength=E).to(torch.int32)  # moe.py:303-309
    fan_in = sorted_scattered // K  # moe.py:342
    batch_gates = gates.flatten()[sorted_scattered]  # moe.py:345-346
    xs = xm[fan_in].split(freq.tolist(), dim=0)  # moe.py:348, :141
    # unbind (not w[e]) so that autograd stacks the per-expert weight gradients instead of adding E full-size tensors
    w1m, w2m = w1.to(math_dtype).unbind(0), w2.to(math_dtype).unbind(0)
    outs = []
    for e in range(E):  # moe.py:145-148, :354-355
        h = F.linear(xs[e], w1m[e], None if b1 is None else b1[e].to(math_dtype))
        h = activation_forward(h, activation)
        outs.append(F.linear(h, w2m[e], None if b2 is None else b2[e].to(math_dtype)))
    y = torch.cat(outs, dim=0) * batch_gates.to(math_dtype).unsqueeze(-1)  # moe.py:357
    out = torch.zeros(T, H, dtype=math_dtype, device=x.device).index_add(0, fan_in, y)  # moe.py:358-359
    return out, logits, freq


def general_routing_reference(
    x, scores, token_idx, expert_idx, w1, w2, E, b1=None, b2=None, math_dtype=torch.float32, activation="swiglu"
):
    """benchmarks/moe-token-rounding.py:21-50: per-expert masked loop, fp32 accumulate."""
    T, H = x.shape
    xm = x.to(math_dtype)
    out = torch.zeros(T, H, dtype=math_dtype, device=x.device)
    for e in range(E):
        pos = expert_idx == e
        t_idx = token_idx[pos].long()
        if t_idx.numel() == 0:
            continue
        h = F.linear(xm[t_idx], w1[e].to(math_dtype), None if b1 is None else b1[e].to(math_dtype))
        h = activation_forward(h, activation)
        y = F.linear(h, w2[e].to(math_dtype), None if b2 is None else b2[e].to(math_dtype))
        out.index_add_(0, t_idx, y * scores[pos].to(math_dtype)[:, None])
    return out


# ----------------------------------------------------------------------------------------------------------
# operator level (what each sonicmoe::* op computes); m = grouped row, t = x_gather_idx[m], f = s_scatter_idx[m]
# ----------------------------------------------------------------------------------------------------------


def _rnd(t: torch.Tensor, round_dtype):
    return t if round_dtype is None else t.to(round_dtype).to(t.dtype)


def up_projection_forward(x, w1, off, gidx, b1=None, math_dtype=torch.float32, round_dtype=None, activation="swiglu"):
    """z[m] = x[t] W1[e]^T (+b1[e]);  y1[m] = act(z[m]), both taken from the un-rounded accumulator
    (functional/forward.py:53-129; grouped_gemm.py:1287-1288, :2463-2469)."""
    E = w1.size(0)
    off = off.tolist()
    xg = x.to(math_dtype)[gidx.long()]
    zs = []
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        zs.append(F.linear(xg[a:b], w1[e].to(math_dtype), None if b1 is None else b1[e].to(math_dtype)))
    z = torch.cat(zs, dim=0)
    y1 = activation_forward(z, activation)
    return _rnd(z, round_dtype), _rnd(y1, round_dtype)


def down_projection_forward(y1, w2, off, b2=None, math_dtype=torch.float32, round_dtype=None):
    """y2[m] = y1[m] W2[e]^T (+b2[e]) (functional/forward.py:132-178)."""
    E = w2.size(0)
    off = off.tolist()
    ys = []
    y1 = y1.to(math_dtype)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        ys.append(F.linear(y1[a:b], w2[e].to(math_dtype), None if b2 is None else b2[e].to(math_dtype)))
    return _rnd(torch.cat(ys, dim=0), round_dtype)


def router_forward(y2, scores_flat, ridx, tok_off, math_dtype=torch.float32, round_dtype=None):
    """o[t] = sum_{j in [tok_off[t], tok_off[t+1])} scores_flat[j] * y2[ridx[j]]
    (functional/reduction_over_k_gather.py:441-517; forward.py:181-202)."""
    T = tok_off.numel() - 1
    H = y2.size(1)
    TK = ridx.numel()
    counts = (tok_off[1:] - tok_off[:-1]).long()
    tok_of_slot = torch.repeat_interleave(torch.arange(T, device=y2.device), counts, output_size=TK)
    rows = y2.to(math_dtype)[ridx.long()]
    if scores_flat is not None:
        rows = rows * scores_flat.to(math_dtype)[:, None]
    o = torch.zeros(T, H, dtype=math_dtype, device=y2.device).index_add(0, tok_of_slot, rows)
    return _rnd(o, round_dtype)


def down_projection_backward(
    dout, z, w2, scores_flat, off, gidx, sidx, math_dtype=torch.float32, round_dtype=None, b2=None, activation="swiglu"
):
    """Backward of (down projection + weighted combine), with y1 recomputed from the STORED z
    (functional/backward.py:31-107, :286-461; grouped_gemm.py:1154-1271, :1311-1333, :2536-2561).

      dy1[m]   = dout[t] W2[e]                               (not scaled by s)
      ds[f]    = sum_i dy1[m,i] y1[m,i] (+ <dout[t], b2[e]>) (written in flat-slot order)
      dz[m]    = s * d(act)/dz applied to dy1                (SwiGLU: dz_2i = s dy1 u (silu(g)(1-sig) + sig), dz_2i+1 = s dy1 silu(g))
      y1s[m]   = s y1[m] ;  dW2[e] = sum_m dout[t]^T (x) y1s[m] ;  db2[e] = sum_m s dout[t]
    Returns (dz, y1s (TK, I), ds (TK,) fp32-like, dw2 (E, H, I)) and, when b2 is given, db2 (E, H) as a fifth value.
    """
    E, H, I = w2.shape
    TK = gidx.numel()
    zf = z.to(math_dtype)
    dg = dout.to(math_dtype)[gidx.long()]
    s = scores_flat.to(math_dtype)[sidx.long()]
    dev = z.device
    off = off.tolist()
    dy1 = torch.empty(TK, I, dtype=math_dtype, device=dev)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        dy1[a:b] = dg[a:b] @ w2[e].to(math_dtype)
    dz, y1 = activation_backward(zf, s[:, None] * dy1, activation)
    row_ds = (dy1 * y1).sum(dim=1)
    db2 = None
    if b2 is not None:
        db2 = torch.zeros(E, H, dtype=math_dtype, device=dev)
        for e in range(E):
            a, b = int(off[e]), int(off[e + 1])
            row_ds[a:b] += dg[a:b] @ b2[e].to(math_dtype)
            db2[e] = (s[a:b, None] * dg[a:b]).sum(dim=0)
    ds = torch.zeros(TK, dtype=math_dtype, device=dev)
    ds[sidx.long()] = row_ds
    y1s = _rnd(s[:, None] * y1, round_dtype)
    dw2 = torch.zeros(E, H, I, dtype=math_dtype, device=dev)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        if b > a:
            dw2[e] = dg[a:b].t() @ y1s[a:b]
    if b2 is None:
        return _rnd(dz, round_dtype), y1s, ds, _rnd(dw2, round_dtype)
    return _rnd(dz, round_dtype), y1s, ds, _rnd(dw2, round_dtype), _rnd(db2, round_dtype)


def up_projection_backward(x, w1, dz, off, gidx, math_dtype=torch.float32, round_dtype=None, with_db1=False):
    """dW1[e] = sum_m dz[m]^T (x) x[t];  dx_expanded[m] = dz[m] W1[e];  db1[e] = sum_m dz[m]
    (functional/backward.py:109-168, :195-283).  Returns (dw1, dx_expanded) and db1 (E, N1) as a third value on request."""
    E, N1, H = w1.shape
    TK = gidx.numel()
    xg = x.to(math_dtype)[gidx.long()]
    dzf = dz.to(math_dtype)
    dev = dz.device
    off = off.tolist()
    dw1 = torch.zeros(E, N1, H, dtype=math_dtype, device=dev)
    db1 = torch.zeros(E, N1, dtype=math_dtype, device=dev)
    dxe = torch.empty(TK, H, dtype=math_dtype, device=dev)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        if b > a:
            dw1[e] = dzf[a:b].t() @ xg[a:b]
            db1[e] = dzf[a:b].sum(dim=0)
        dxe[a:b] = dzf[a:b] @ w1[e].to(math_dtype)
    if with_db1:
        return _rnd(dw1, round_dtype), _rnd(dxe, round_dtype), _rnd(db1, round_dtype)
    return _rnd(dw1, round_dtype), _rnd(dxe, round_dtype)


def token_broadcast_backward(dx_expanded, ridx, tok_off, math_dtype=torch.float32, round_dtype=None):
    """dx[t] = sum_j dx_expanded[ridx[j]] over the token's slots (functional/backward.py:464-484)."""
    return router_forward(dx_expanded, None, ridx, tok_off, math_dtype, round_dtype)


def softmax_topk_bwd(dscore, score, idx, E):
    """functional/backward.py:487-525."""
    g, s = dscore.float(), score.float()
    dot = (g * s).sum(dim=1, keepdim=True)
    out = torch.zeros(score.size(0), E, dtype=torch.float32, device=score.device)
    out.scatter_(1, idx.long(), s * (g - dot))
    return out


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    """||a-b|| / ||b|| in float64."""
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))
