"""GPU parity of the float16 build of the library (libsonicmoe_hip_f16.so: the same kernels with fp16 as the 16-bit
element type, which the reference's grouped GEMMs accept next to bf16, sonicmoe/functional/grouped_gemm.py:3033-3044).

Same oracle, same inputs rounded to fp16.  fp16 keeps three more mantissa bits than bf16, so the bound is tighter than
the bf16 tests' 1e-2: relative L2 <= 1.5e-3 per operator (measured ~3e-4, the output rounding); a kernel that rounded
through bf16 on its way would sit at 2e-3 .. 4e-3 and fail it.
"""

from pathlib import Path

import pytest
import torch

from helpers import make_tc_routing, make_weights, rel_l2
from oracle import moe_math as M
from oracle import routing as R

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
F16 = torch.float16
TOL = 1.5e-3

SHAPES = [
    # T, H, I, E, K, skew, empty experts, biases
    (1024, 512, 256, 8, 2, 0.0, (), False),          # C1 shape
    (1500, 768, 192, 16, 4, 1.2, (3, 15), True),     # skewed, empty experts, N tails, biases
    (4096, 1024, 512, 32, 8, 0.8, (0,), False),      # the hand-scheduled loops, several tiles per workgroup
    (300, 64, 64, 4, 1, 0.0, (), True),              # contraction of one stage: the one-tile kernels
    (1536, 2048, 1024, 12, 2, 1.5, (2, 7), False),   # weight gradients as tile streams
]


@pytest.mark.parametrize("gemm_asm", [1, 0])
@pytest.mark.parametrize("T,H,I,E,K,skew,empty,bias", SHAPES)
def test_fp16_operator_chain(dev, tuning, gemm_asm, T, H, I, E, K, skew, empty, bias):
    """Every GEMM-side operator of a training step on fp16 tensors, each against the oracle on the operator's own
    inputs, with the hand-scheduled loops and with the compiler-scheduled kernels."""
    from sonicmoe.functional import backward as bwd
    from sonicmoe.functional import forward as fwd

    tuning("gemm_asm", gemm_asm)
    _, w1, w2 = make_weights(E, H, I, dev, dtype=F16, seed=T)
    idx, scores, meta, md = make_tc_routing(T, E, K, dev, seed=T + 1, skew=skew, empty=empty)
    g = torch.Generator().manual_seed(T + 2)
    x = torch.randn(T, H, generator=g).to(F16).to(dev)
    dout = torch.randn(T, H, generator=g).to(F16).to(dev)
    b1 = (torch.randn(E, 2 * I, generator=g) * 0.1).to(F16).to(dev) if bias else None
    b2 = (torch.randn(E, H, generator=g) * 0.1).to(F16).to(dev) if bias else None
    TK = T * K
    off, gidx, sidx, ridx, tok_off = (md[k] for k in (
        "expert_frequency_offset", "x_gather_idx", "s_scatter_idx", "s_reverse_scatter_idx",
        "num_activated_expert_per_token_offset"))
    s_flat = torch.from_numpy(scores).to(dev).view(-1)
    stream = torch.cuda.current_stream().cuda_stream
    w1v, w2v = w1.permute(1, 2, 0), w2.permute(1, 2, 0)
    h = dict(dtype=F16, device=dev)

    z, y1 = torch.empty(TK, 2 * I, **h), torch.empty(TK, I, **h)
    fwd._up_projection_forward(x, w1v, z, y1, b1, off, None, gidx, stream, "swiglu", True, False)
    z_ref, y1_ref = M.up_projection_forward(x, w1, off, gidx, b1=b1)
    assert rel_l2(z, z_ref) < TOL and rel_l2(y1, y1_ref) < TOL

    y2 = torch.empty(TK, H, **h)
    fwd._down_projection_forward(w2v, y1, y2, b2, off, None, gidx, stream)
    assert rel_l2(y2, M.down_projection_forward(y1, w2, off, b2=b2)) < TOL

    o = torch.empty(T, H, **h)
    fwd._router_forward(y2, o, s_flat, ridx, tok_off, K, H, False)
    o_ref = M.router_forward(y2, s_flat, ridx, tok_off)
    assert rel_l2(o, o_ref) < TOL

    # the same two steps as one kernel: atomic adds round to fp16 once per contribution
    o_fused = torch.zeros(T, H, **h)
    fwd._down_projection_forward_combine(w2v, y1, o_fused, b2, s_flat, off, None, gidx, sidx, stream)
    assert rel_l2(o_fused, o_ref) < 4 * TOL

    dz, ds = torch.empty_like(z), torch.empty(TK, dtype=torch.float32, device=dev)
    dw2 = torch.empty(E, H, I, **h).permute(1, 2, 0)
    db2 = torch.empty(E, H, **h) if bias else None
    bwd._down_projection_backward(dout, z, w2v, dw2, dz, ds, b2, db2, s_flat, off, None, gidx, sidx, stream, True,
                                  "swiglu")
    ref = M.down_projection_backward(dout, z, w2, s_flat, off, gidx, sidx, b2=b2)
    dz_ref, ds_ref, dw2_ref = ref[0], ref[2], ref[3]
    assert rel_l2(dz, dz_ref) < TOL
    assert rel_l2(dw2.permute(2, 0, 1), dw2_ref) < TOL
    assert rel_l2(ds, ds_ref) < TOL
    if bias:
        assert rel_l2(db2, ref[4]) < TOL

    dw1 = torch.empty(E, 2 * I, H, **h).permute(1, 2, 0)
    db1 = torch.empty(E, 2 * I, **h) if bias else None
    dxe = torch.empty(TK, H, **h)
    bwd._up_projection_backward(x, w1v, dxe, dw1, dz, db1, off, None, gidx, sidx, True, stream)
    ref = M.up_projection_backward(x, w1, dz, off, gidx)
    assert rel_l2(dw1.permute(2, 0, 1), ref[0]) < TOL
    assert rel_l2(dxe, ref[1]) < TOL
    if bias:
        db1_ref = torch.stack([dz[off[e]:off[e + 1]].float().sum(0) for e in range(E)])
        assert rel_l2(db1, db1_ref) < TOL
    dx = torch.empty(T, H, **h)
    bwd._token_broadcast_backward(dx, dxe, ridx, tok_off, K, H, False)
    assert rel_l2(dx, M.router_forward(dxe, None, ridx, tok_off)) < TOL


def test_operator_rejects_mixed_element_types(dev):
    from sonicmoe.functional import forward as fwd

    T, H, I, E, K = 256, 64, 64, 2, 1
    _, w1, _ = make_weights(E, H, I, dev, dtype=F16, seed=1)
    _, _, _, md = make_tc_routing(T, E, K, dev, seed=2)
    x = torch.randn(T, H, device=dev).to(torch.bfloat16)
    z, y1 = torch.empty(T, 2 * I, dtype=F16, device=dev), torch.empty(T, I, dtype=F16, device=dev)
    with pytest.raises(NotImplementedError, match="one element type"):
        fwd._up_projection_forward(x, w1.permute(1, 2, 0), z, y1, None, md["expert_frequency_offset"], None,
                                   md["x_gather_idx"], torch.cuda.current_stream().cuda_stream, "swiglu", True, False)
    with pytest.raises(NotImplementedError, match="bfloat16 or float16"):
        fwd._up_projection_forward(x.float(), w1.permute(1, 2, 0).float(), z.float(), y1.float(), None,
                                   md["expert_frequency_offset"], None, md["x_gather_idx"],
                                   torch.cuda.current_stream().cuda_stream, "swiglu", True, False)


@pytest.mark.parametrize("T,H,I,E,K,add_bias", [
    (1024, 512, 256, 8, 2, False),     # C1 shape
    (2048, 768, 256, 128, 8, True),    # a reference test shape (tests/moe_test.py:26-37) at T=2048, with biases
    (8192, 4096, 1024, 128, 8, False), # reference test shape at full T
])
def test_fp16_moe_forward_backward(dev, T, H, I, E, K, add_bias):
    """The module in fp16, forward and every gradient, against the oracle in fp32 on the same fp16-rounded values
    (driven with the HIP path's expert choice).  Through the whole layer the errors of several fp16 roundings add up:
    bound 3e-3 (the bf16 layer test allows 1e-2)."""
    from sonicmoe import KernelBackendMoE, MoE
    from sonicmoe.enums import ActivationType

    torch.manual_seed(42)
    moe = MoE(E, K, H, I, ActivationType.SWIGLU, add_bias, 0.02).to(device=dev, dtype=F16)
    with torch.no_grad():
        moe.router.weight.normal_(0, 0.02)
        if add_bias:
            moe.c_fc.bias.normal_(0, 0.1)
            moe.c_proj.bias.normal_(0, 0.1)
    x = torch.randn(T, H, device=dev).to(F16).requires_grad_()
    dy = torch.randn(T, H, device=dev).to(F16)
    out, aux = moe(x, kernel_backend_moe=KernelBackendMoE.sonicmoe)
    assert out.dtype == F16
    params = [moe.router.weight, moe.c_fc.weight, moe.c_proj.weight]
    if add_bias:
        params += [moe.c_fc.bias, moe.c_proj.bias]
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=dy)

    with torch.no_grad():
        logits = torch.nn.functional.linear(x, moe.router.weight)
    _, i_ref = R.topk_softmax(logits.float().cpu().numpy(), K)
    sel = torch.from_numpy(i_ref).to(dev)
    xr = x.detach().clone().requires_grad_()
    pr = [p.detach().clone().requires_grad_() for p in params]
    kw = dict(b1=pr[3], b2=pr[4]) if add_bias else {}
    out_ref, _, freq_ref = M.moe_torch_backend(xr, pr[0], pr[1], pr[2], K, selected_experts=sel, **kw)
    grads_ref = torch.autograd.grad(out_ref, [xr] + pr, grad_outputs=dy.float())
    assert rel_l2(out, out_ref) < 3e-3
    for n, g, gr in zip(["dx", "d_router_w", "d_w1", "d_w2", "d_b1", "d_b2"], grads, grads_ref):
        assert g.shape == gr.shape and g.dtype == F16
        assert rel_l2(g, gr) < 3e-3, n
    aux_ref = M.switch_aux_loss(logits, freq_ref)
    assert abs(float(aux) - float(aux_ref)) < 1e-3 * abs(float(aux_ref))


def test_fp16_layer_with_fp8_gemms(dev):
    """The block-scaled e4m3 path on fp16 tensors (quantisers read fp16, the fp8 GEMMs write fp16): against the fp16
    path of the same module, with the bounds of the bf16 test of the same name in test_fp8_gpu.py."""
    from sonicmoe import MoE, enable_fp8_backward, enable_fp8_forward
    from sonicmoe.enums import ActivationType

    T, H, I, E, K = 2048, 1024, 512, 16, 4
    torch.manual_seed(3)
    moe = MoE(E, K, H, I, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=F16)
    x = torch.randn(T, H, device=dev).to(F16).requires_grad_()
    dy = torch.randn(T, H, device=dev).to(F16)
    params = [moe.router.weight, moe.c_fc.weight, moe.c_proj.weight]
    out, _ = moe(x)
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=dy)
    with enable_fp8_forward(), enable_fp8_backward():
        out8, _ = moe(x)
        grads8 = torch.autograd.grad(out8, [x] + params, grad_outputs=dy)
    assert out8.dtype == F16
    errs = [rel_l2(out8, out)] + [rel_l2(a, b) for a, b in zip(grads8, grads)]
    print("fp16 tensors, fp8 GEMMs: out, dx, dWr, dW1, dW2 rel-L2 vs the fp16 path:", errs)
    assert all(1e-2 < e < 9e-2 for e in errs), errs


def test_libraries_do_not_interpose_each_other(dev):
    """The two builds define the same symbols.  A host program that has loaded the bf16 library with RTLD_GLOBAL must
    still get fp16 arithmetic from the fp16 library (each is linked to bind its own definitions): a child process does
    exactly that and runs one fp16 up-projection against torch."""
    import subprocess
    import sys
    import textwrap

    code = textwrap.dedent("""
        import ctypes, sys, torch
        sys.path[:0] = [%r, %r]
        from sonicmoe import _lib
        ctypes.CDLL(str(_lib.library_path(torch.bfloat16)), mode=ctypes.RTLD_GLOBAL)
        from sonicmoe.functional import forward
        dev = torch.device("cuda:0")
        T, H, I, E = 512, 256, 128, 2
        g = torch.Generator().manual_seed(1)
        x = torch.randn(T, H, generator=g).half().to(dev)
        w1 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).half().to(dev)
        off = torch.tensor([0, 200, T], dtype=torch.int32, device=dev)
        gidx = torch.randperm(T, generator=g).to(torch.int32).to(dev)
        z = torch.empty(T, 2 * I, dtype=torch.float16, device=dev)
        y1 = torch.empty(T, I, dtype=torch.float16, device=dev)
        forward._up_projection_forward(x, w1.permute(1, 2, 0), z, y1, None, off, None, gidx,
                                       torch.cuda.current_stream().cuda_stream, "swiglu", True, False)
        xg = x[gidx.long()].float()
        ref = torch.cat([xg[:200] @ w1[0].float().t(), xg[200:] @ w1[1].float().t()])
        err = float((z.float() - ref).norm() / ref.norm())
        print("rel-L2", err)
        assert err < 1.5e-3, err
    """) % (str(ROOT / "sonic-moe_amd"), str(ROOT))
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr
