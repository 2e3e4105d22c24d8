"""Pins the floating-point side of the oracle: the hand-derived operator-level backward formulas against
torch.autograd through the restated forward (fp64), special cases that reduce to library routines, closed forms."""

import numpy as np
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_math as M
from oracle import routing as R

D = torch.float64


def _problem(T=40, H=16, I=8, E=4, K=2, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=D)
    w1 = torch.randn(E, 2 * I, H, generator=g, dtype=D) * 0.3
    w2 = torch.randn(E, H, I, generator=g, dtype=D) * 0.3
    wr = torch.randn(E, H, generator=g, dtype=D) * 0.3
    idx = np.stack([np.random.default_rng(seed + t).choice(E, size=K, replace=False) for t in range(T)]).astype(np.int32)
    meta = {k: torch.from_numpy(v) for k, v in R.tc_topk_router_metadata(idx, E).items()}
    scores = torch.rand(T, K, generator=g, dtype=D) + 0.1
    dout = torch.randn(T, H, generator=g, dtype=D)
    return x, w1, w2, wr, idx, meta, scores, dout


def test_operator_chain_equals_torch_backend():
    """up -> down -> combine (operator level) == the restated torch backend driven with the same routing."""
    T, K = 40, 2
    x, w1, w2, wr, idx, meta, _, _ = _problem()
    out_ref, logits, freq = M.moe_torch_backend(x, wr, w1, w2, K, selected_experts=torch.from_numpy(idx), math_dtype=D,
                                                gate_dtype=D)
    gates = F.softmax(logits.gather(1, torch.from_numpy(idx).long()), dim=-1)
    off, gidx, ridx, tok_off = (meta[k] for k in ("expert_frequency_offset", "x_gather_idx", "s_reverse_scatter_idx",
                                                  "num_activated_expert_per_token_offset"))
    z, y1 = M.up_projection_forward(x, w1, off, gidx, math_dtype=D)
    y2 = M.down_projection_forward(y1, w2, off, math_dtype=D)
    o = M.router_forward(y2, gates.reshape(-1), ridx, tok_off, math_dtype=D)
    # the torch backend evaluates the gate softmax in fp32 (moe.py:286), everything else here is fp64
    torch.testing.assert_close(o, out_ref, rtol=1e-5, atol=1e-7)
    np.testing.assert_array_equal(freq.numpy(), meta["expert_frequency"].numpy())


def test_explicit_backward_matches_autograd():
    """dz, ds, dW2, dW1, dx_expanded, dx from the hand-written formulas == autograd of the operator chain (fp64)."""
    x, w1, w2, wr, idx, meta, scores, dout = _problem(seed=3)
    off, gidx, sidx, ridx, tok_off = (meta[k] for k in ("expert_frequency_offset", "x_gather_idx", "s_scatter_idx",
                                                        "s_reverse_scatter_idx", "num_activated_expert_per_token_offset"))
    xr, w1r, w2r, sr = (t.clone().requires_grad_() for t in (x, w1, w2, scores))
    z, y1 = M.up_projection_forward(xr, w1r, off, gidx, math_dtype=D)
    y2 = M.down_projection_forward(y1, w2r, off, math_dtype=D)
    o = M.router_forward(y2, sr.reshape(-1), ridx, tok_off, math_dtype=D)
    gx, gw1, gw2, gs, gz = torch.autograd.grad(o, [xr, w1r, w2r, sr, z], grad_outputs=dout)

    dz, y1s, ds, dw2 = M.down_projection_backward(dout, z.detach(), w2, scores.reshape(-1), off, gidx, sidx, math_dtype=D)
    dw1, dxe = M.up_projection_backward(x, w1, dz, off, gidx, math_dtype=D)
    dx = M.token_broadcast_backward(dxe, ridx, tok_off, math_dtype=D)
    kw = dict(rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(dz, gz, **kw)
    torch.testing.assert_close(ds.view_as(gs), gs, **kw)
    torch.testing.assert_close(dw2, gw2, **kw)
    torch.testing.assert_close(dw1, gw1, **kw)
    torch.testing.assert_close(dx, gx, **kw)
    torch.testing.assert_close(y1s, scores.reshape(-1)[sidx.long()][:, None] * M.swiglu(z.detach()), **kw)


ALL_ACTIVATIONS = ["swiglu", "geglu", "reglu", "relu_sq", "relu", "gelu", "silu"]


@pytest.mark.parametrize("activation", ALL_ACTIVATIONS)
def test_activation_forms(activation):
    """activation_forward reduces to the library routines the reference's torch backend calls (moe.py:24-60); the
    hand-written derivative equals autograd's, and the gated forms split gate = even / up = odd columns."""
    g = torch.Generator().manual_seed(1)
    z = torch.randn(7, 12, generator=g, dtype=D)
    z[0, 0] = 0.25  # keep clear of the kink of relu at 0
    lib = {"swiglu": F.silu, "geglu": F.gelu, "reglu": F.relu, "relu_sq": lambda t: F.relu(t).square(),
           "relu": F.relu, "gelu": F.gelu, "silu": F.silu}[activation]
    y = M.activation_forward(z, activation)
    if M.is_glu(activation):
        assert y.shape == (7, 6)
        torch.testing.assert_close(y, lib(z[:, 0::2]) * z[:, 1::2], rtol=1e-12, atol=1e-12)
    else:
        assert y.shape == z.shape
        torch.testing.assert_close(y, lib(z), rtol=1e-12, atol=1e-12)
    zr = z.clone().requires_grad_()
    dy = torch.randn(y.shape, generator=g, dtype=D)
    (gz,) = torch.autograd.grad(M.activation_forward(zr, activation), zr, grad_outputs=dy)
    dz, y_again = M.activation_backward(z, dy, activation)
    torch.testing.assert_close(dz, gz, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(y_again, y, rtol=1e-12, atol=1e-12)


def test_gelu_is_the_erf_form():
    """Known answers: gelu(t) = t * Phi(t) with the normal distribution function (tables: Phi(1) = 0.8413447460685429,
    Phi(2) = 0.9772498680518208, Phi(-0.5) = 0.3085375387259869).  The tanh approximation the reference's fused kernels
    use (grouped_gemm.py:432-433) gives 0.841192 at t = 1: the two forms differ from the fourth digit on."""
    t = torch.tensor([[1.0, 2.0, -0.5, 0.0]], dtype=D)
    want = torch.tensor([[0.8413447460685429, 2 * 0.9772498680518208, -0.5 * 0.3085375387259869, 0.0]], dtype=D)
    torch.testing.assert_close(M.activation_forward(t, "gelu"), want, rtol=1e-12, atol=1e-14)
    tanh_form = 0.5 * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (1.0 + 0.044715)))
    assert abs(float(M.activation_forward(t, "gelu")[0, 0]) - tanh_form) > 1e-4


@pytest.mark.parametrize("activation", ALL_ACTIVATIONS)
def test_explicit_backward_with_bias_and_activation(activation):
    """dz, ds, dW2, db2, dW1, db1, dx with expert biases, for every activation == autograd of the operator chain."""
    glu = M.is_glu(activation)
    x, w1, w2, wr, idx, meta, scores, dout = _problem(seed=4)
    if not glu:
        w1 = w1[:, : w1.size(1) // 2].contiguous()  # (E, I, H)
    E, N1, H = w1.shape
    g = torch.Generator().manual_seed(8)
    b1 = torch.randn(E, N1, generator=g, dtype=D) * 0.2
    b2 = torch.randn(E, H, generator=g, dtype=D) * 0.2
    off, gidx, sidx, ridx, tok_off = (meta[k] for k in ("expert_frequency_offset", "x_gather_idx", "s_scatter_idx",
                                                        "s_reverse_scatter_idx", "num_activated_expert_per_token_offset"))
    xr, w1r, w2r, sr, b1r, b2r = (t.clone().requires_grad_() for t in (x, w1, w2, scores, b1, b2))
    z, y1 = M.up_projection_forward(xr, w1r, off, gidx, b1=b1r, math_dtype=D, activation=activation)
    y2 = M.down_projection_forward(y1, w2r, off, b2=b2r, math_dtype=D)
    o = M.router_forward(y2, sr.reshape(-1), ridx, tok_off, math_dtype=D)
    gx, gw1, gw2, gs, gz, gb1, gb2 = torch.autograd.grad(o, [xr, w1r, w2r, sr, z, b1r, b2r], grad_outputs=dout)

    dz, y1s, ds, dw2, db2 = M.down_projection_backward(dout, z.detach(), w2, scores.reshape(-1), off, gidx, sidx,
                                                       math_dtype=D, b2=b2, activation=activation)
    dw1, dxe, db1 = M.up_projection_backward(x, w1, dz, off, gidx, math_dtype=D, with_db1=True)
    dx = M.token_broadcast_backward(dxe, ridx, tok_off, math_dtype=D)
    kw = dict(rtol=1e-9, atol=1e-11)
    for name, a, b in [("dz", dz, gz), ("ds", ds.view_as(gs), gs), ("dw2", dw2, gw2), ("db2", db2, gb2),
                       ("dw1", dw1, gw1), ("db1", db1, gb1), ("dx", dx, gx)]:
        torch.testing.assert_close(a, b, msg=lambda m, n=name: f"{n}: {m}", **kw)

    # the layer-level restatement with the same biases and activation is the same function
    out_ref, logits, _ = M.moe_torch_backend(x, wr, w1, w2, idx.shape[1], b1=b1, b2=b2,
                                             selected_experts=torch.from_numpy(idx), math_dtype=D, gate_dtype=D,
                                             activation=activation)
    gates = F.softmax(logits.gather(1, torch.from_numpy(idx).long()), dim=-1).reshape(-1)
    z2, y1b = M.up_projection_forward(x, w1, off, gidx, b1=b1, math_dtype=D, activation=activation)
    o2 = M.router_forward(M.down_projection_forward(y1b, w2, off, b2=b2, math_dtype=D), gates, ridx, tok_off, math_dtype=D)
    torch.testing.assert_close(o2, out_ref, rtol=1e-5, atol=1e-7)


def test_single_expert_is_a_dense_swiglu_mlp():
    g = torch.Generator().manual_seed(5)
    T, H, I = 30, 12, 6
    x = torch.randn(T, H, generator=g, dtype=D)
    w1 = torch.randn(1, 2 * I, H, generator=g, dtype=D)
    w2 = torch.randn(1, H, I, generator=g, dtype=D)
    wr = torch.randn(1, H, generator=g, dtype=D)
    out, _, freq = M.moe_torch_backend(x, wr, w1, w2, 1, math_dtype=D, gate_dtype=D)
    h = x @ w1[0].t()
    ref = (F.silu(h[:, 0::2]) * h[:, 1::2]) @ w2[0].t()  # gate = even columns, up = odd columns; gate weight == 1
    torch.testing.assert_close(out, ref, rtol=1e-12, atol=1e-12)
    assert int(freq[0]) == T


def test_top1_scores_are_one_and_router_gets_no_gradient():
    x, w1, w2, wr, _, _, _, dout = _problem(K=1, seed=9)
    wrr = wr.clone().requires_grad_()
    out, logits, _ = M.moe_torch_backend(x, wrr, w1, w2, 1, math_dtype=D, gate_dtype=D)
    (g,) = torch.autograd.grad(out, wrr, grad_outputs=dout)
    assert float(g.abs().max()) < 1e-12  # softmax over one value is constant
    s, i = R.topk_softmax(logits.detach().float().numpy(), 1)
    assert (s == 1.0).all()
    dl = M.softmax_topk_bwd(torch.randn(x.size(0), 1), torch.from_numpy(s), torch.from_numpy(i), wr.size(0))
    assert float(dl.abs().max()) == 0.0


def test_torch_backend_equals_masked_expert_loop():
    """The sorted/grouped evaluation and the reference benchmark's per-expert masked loop are the same function."""
    x, w1, w2, wr, idx, meta, _, _ = _problem(seed=11)
    T, K = idx.shape
    out, logits, _ = M.moe_torch_backend(x, wr, w1, w2, K, selected_experts=torch.from_numpy(idx), math_dtype=D,
                                         gate_dtype=D)
    gates = F.softmax(logits.gather(1, torch.from_numpy(idx).long()), dim=-1).reshape(-1)
    tok = torch.arange(T).repeat_interleave(K)
    ref = M.general_routing_reference(x, gates, tok, torch.from_numpy(idx).reshape(-1), w1, w2, w1.size(0), math_dtype=D)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-7)


def test_aux_loss_closed_forms():
    E = 8
    # uniform probabilities and uniform load -> E * sum((1/E)*(1/E)) = 1
    assert abs(float(M.switch_aux_loss(torch.zeros(64, E), torch.full((E,), 16))) - 1.0) < 1e-6
    # everything on one expert with a (numerically) one-hot router -> E * 1 * 1 = E
    logits = torch.full((64, E), -40.0)
    logits[:, 3] = 40.0
    f = torch.zeros(E)
    f[3] = 64
    assert abs(float(M.switch_aux_loss(logits, f)) - E) < 1e-4


def test_module_torch_backend_on_cpu_matches_oracle():
    """The CPU-runnable configuration (T=1024, H=512, I=256, E=8, K=2): the module's torch backend in fp32, forward and
    backward."""
    from sonicmoe import KernelBackendMoE, MoE
    from sonicmoe.enums import ActivationType

    torch.manual_seed(0)
    T, H, I, E, K = 1024, 512, 256, 8, 2
    moe = MoE(E, K, H, I, ActivationType.SWIGLU, False, 0.02)
    x = torch.randn(T, H, requires_grad=True)
    g = torch.randn(T, H)
    out, aux = moe(x, kernel_backend_moe=KernelBackendMoE.torch)
    params = [moe.router.weight, moe.c_fc.weight, moe.c_proj.weight]
    grads = torch.autograd.grad((out * g).sum(), [x] + params)
    xr = x.detach().clone().requires_grad_()
    pr = [p.detach().clone().requires_grad_() for p in params]
    out_ref, logits, freq = M.moe_torch_backend(xr, pr[0], pr[1], pr[2], K)
    grads_ref = torch.autograd.grad((out_ref * g).sum(), [xr] + pr)
    torch.testing.assert_close(out, out_ref, rtol=1e-5, atol=1e-6)
    for a, b in zip(grads, grads_ref):
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-5)  # fp32 summation order differs
    assert abs(float(aux) - float(M.switch_aux_loss(logits, freq))) < 1e-5


def test_sonicmoe_backend_refuses_cpu_tensors():
    from sonicmoe import KernelBackendMoE, MoE
    from sonicmoe.enums import ActivationType

    moe = MoE(8, 2, 512, 256, ActivationType.SWIGLU, False, 0.02)
    with pytest.raises(RuntimeError, match="GPU"):
        moe(torch.randn(16, 512), kernel_backend_moe=KernelBackendMoE.sonicmoe)
