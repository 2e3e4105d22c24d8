"""GPU parity of expert biases and of the seven activation functions, operator level and module level.

Operator level: every sonicmoe::* grouped-GEMM operator with b1 / b2 given, for each activation, against the oracle's
operator restatement on the same bf16 inputs.  Module level: MoE(add_bias=True) forward + backward (the add_bias axis of the reference's
tests/moe_test.py:40, :72-75) against the oracle's restatement of the torch backend.
Tolerance: relative L2 <= 1e-2 (bf16); ds is fp32 and is held to 2e-3.
"""

import pytest
import torch

from helpers import make_tc_routing, rel_l2
from oracle import moe_math as M

pytestmark = pytest.mark.gpu
TOL = 1e-2
ACTIVATIONS = ["swiglu", "geglu", "reglu", "relu_sq", "relu", "gelu", "silu"]


def _problem(dev, T, H, I, E, K, activation, seed, skew=0.0, empty=()):
    glu = M.is_glu(activation)
    N1 = 2 * I if glu else I
    g = torch.Generator().manual_seed(seed)
    # std chosen so that z = O(1): the activations are then exercised on both sides of their bends
    w1 = (torch.randn(E, N1, H, generator=g) / H**0.5).to(torch.bfloat16).to(dev)
    w2 = (torch.randn(E, H, I, generator=g) / I**0.5).to(torch.bfloat16).to(dev)
    b1 = (0.5 * torch.randn(E, N1, generator=g)).to(torch.bfloat16).to(dev)
    b2 = (0.5 * torch.randn(E, H, generator=g)).to(torch.bfloat16).to(dev)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    dout = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    idx, scores, meta, md = make_tc_routing(T, E, K, dev, seed=seed + 1, skew=skew, empty=empty)
    return glu, N1, w1, w2, b1, b2, x, dout, torch.from_numpy(scores).to(dev).view(-1), md


@pytest.mark.parametrize("activation", ACTIVATIONS)
@pytest.mark.parametrize("with_bias", [False, True])
def test_operators_bias_activation(dev, activation, with_bias):
    from sonicmoe.functional import backward as bwd
    from sonicmoe.functional import forward as fwd

    T, H, I, E, K = 1500, 320, 192, 8, 2  # ragged tiles in every dimension, one empty expert
    glu, N1, w1, w2, b1, b2, x, dout, s_flat, md = _problem(dev, T, H, I, E, K, activation, 7, skew=0.7, empty=(5,))
    if not with_bias:
        b1 = b2 = None
    TK = T * K
    off, gidx, sidx, ridx, tok_off = (md[k] for k in ("expert_frequency_offset", "x_gather_idx", "s_scatter_idx",
                                                      "s_reverse_scatter_idx",
                                                      "num_activated_expert_per_token_offset"))
    stream = torch.cuda.current_stream().cuda_stream
    bf = dict(dtype=torch.bfloat16, device=dev)

    z = torch.empty(TK, N1, **bf)
    y1 = torch.empty(TK, I, **bf)
    fwd._up_projection_forward(x, w1.permute(1, 2, 0), z, y1, b1, off, None, gidx, stream, activation, glu, False)
    z_ref, y1_ref = M.up_projection_forward(x, w1, off, gidx, b1=b1, activation=activation)
    assert rel_l2(z, z_ref) < TOL
    assert rel_l2(y1, y1_ref) < TOL
    y1b = torch.empty_like(y1)
    fwd._up_projection_forward(x, w1.permute(1, 2, 0), None, y1b, b1, off, None, gidx, stream, activation, glu, True)
    assert torch.equal(y1b, y1)

    y2 = torch.empty(TK, H, **bf)
    fwd._down_projection_forward(w2.permute(1, 2, 0), y1, y2, b2, off, None, gidx, stream)
    assert rel_l2(y2, M.down_projection_forward(y1, w2, off, b2=b2)) < TOL

    dw2 = torch.full((E, H, I), 3.0, **bf).permute(1, 2, 0)
    db2 = torch.full((E, H), 3.0, **bf) if with_bias else None
    dz = torch.empty(TK, N1, **bf)
    ds = torch.empty(TK, dtype=torch.float32, device=dev)
    bwd._down_projection_backward(dout, z, w2.permute(1, 2, 0), dw2, dz, ds, b2, db2, s_flat, off, None, gidx, sidx,
                                  stream, glu, activation)
    ref = M.down_projection_backward(dout, z, w2, s_flat, off, gidx, sidx, round_dtype=torch.bfloat16, b2=b2,
                                     activation=activation)
    assert rel_l2(dz, ref[0]) < TOL
    assert rel_l2(ds, ref[2]) < 2e-3
    assert rel_l2(dw2.permute(2, 0, 1), ref[3]) < TOL
    assert bool((dw2[..., 5] == 0).all())
    if with_bias:
        assert rel_l2(db2, ref[4]) < TOL
        assert bool((db2[5] == 0).all())

    dw1 = torch.full((E, N1, H), 3.0, **bf).permute(1, 2, 0)
    db1 = torch.full((E, N1), 3.0, **bf) if with_bias else None
    dxe = torch.empty(TK, H, **bf)
    bwd._up_projection_backward(x, w1.permute(1, 2, 0), dxe, dw1, dz, db1, off, None, gidx, sidx, glu, stream)
    dw1_ref, dxe_ref, db1_ref = M.up_projection_backward(x, w1, dz, off, gidx, with_db1=True)
    assert rel_l2(dxe, dxe_ref) < TOL
    assert rel_l2(dw1.permute(2, 0, 1), dw1_ref) < TOL
    if with_bias:
        assert rel_l2(db1, db1_ref) < TOL
        assert bool((db1[5] == 0).all())


@pytest.mark.parametrize("activation", ["swiglu", "geglu", "gelu", "relu_sq"])
@pytest.mark.parametrize("shape", [(2048, 768, 256, 16, 4), (1024, 1536, 512, 64, 4)])
def test_module_with_bias(dev, activation, shape):
    """MoE(add_bias=True): forward and all gradients of the sonicmoe backend against the oracle's torch backend."""
    from sonicmoe import MoE
    from sonicmoe.enums import ActivationType

    T, H, I, E, K = shape
    torch.manual_seed(42)
    moe = MoE(E, K, H, I, ActivationType(activation), True, 0.02).to(device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        moe.c_fc.bias.normal_(0, 0.01)
        moe.c_proj.bias.normal_(0, 0.01)
    x = (0.02 * torch.randn(T, H, device=dev)).to(torch.bfloat16).requires_grad_()
    dy = (0.02 * torch.randn(T, H, device=dev)).to(torch.bfloat16)
    params = [moe.router.weight, moe.c_fc.weight, moe.c_fc.bias, moe.c_proj.weight, moe.c_proj.bias]
    names = ["dx", "d_router", "dw1", "db1", "dw2", "db2"]

    out, _ = moe(x)
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=dy)

    # oracle, fp32 math on the same bf16 parameters, driven with the kernel's routing choice (bf16 logits hold ties)
    from sonicmoe.functional import forward as fwd

    with torch.no_grad():
        logits = torch.nn.functional.linear(x, moe.router.weight)
        sc = torch.empty(T, K, dtype=torch.float32, device=dev)
        sel = torch.empty(T, K, dtype=torch.int32, device=dev)
        fwd._topk_fwd(logits, K, sc, sel, True)
    xr = x.detach().float().requires_grad_()
    pr = [p.detach().float().requires_grad_() for p in params]
    out_ref, _, _ = M.moe_torch_backend(xr, pr[0], pr[1], pr[3], K, b1=pr[2], b2=pr[4], selected_experts=sel,
                                        gate_dtype=torch.float32, activation=activation)
    grads_ref = torch.autograd.grad(out_ref, [xr] + pr, grad_outputs=dy.float())
    assert rel_l2(out, out_ref) < TOL
    for n, a, b in zip(names, grads, grads_ref):
        assert rel_l2(a, b) < TOL, (n, rel_l2(a, b))
