"""GPU parity of the whole layer (module API, forward + all gradients) against the restated torch backend.

The oracle is evaluated in fp32 on the same bf16-rounded inputs and parameters (what the reference's own test does
under autocast(float32), tests/moe_test.py:87-118) and is driven with the HIP path's expert choice, because
torch.topk's order among tied logits is unspecified.  Bar: relative L2 <= 1e-2 for the output and every gradient.
"""

import pytest
import torch

from helpers import rel_l2
from oracle import moe_math as M
from oracle import routing as R

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _build(dev, T, H, I, E, K, seed=42, x_scale=1.0):
    from sonicmoe import MoE
    from sonicmoe.enums import ActivationType

    torch.manual_seed(seed)
    moe = MoE(E, K, H, I, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        moe.router.weight.normal_(0, 0.02)
    x = (x_scale * torch.randn(T, H, device=dev)).to(torch.bfloat16).requires_grad_()
    dy = (x_scale * torch.randn(T, H, device=dev)).to(torch.bfloat16)
    return moe, x, dy


@pytest.mark.parametrize(
    "T,H,I,E,K",
    [
        (1024, 512, 256, 8, 2),     # C1 shape
        (2048, 768, 256, 128, 8),   # reference test shapes (tests/moe_test.py:26-37) at T=2048
        (2048, 1536, 512, 64, 4),
        (2048, 4096, 1024, 32, 2),
        (1024, 4096, 256, 256, 16),
        (8192, 4096, 1024, 128, 8), # reference test shape at full T
    ],
)
def test_moe_forward_backward(dev, T, H, I, E, K):
    from sonicmoe import KernelBackendMoE

    moe, x, dy = _build(dev, T, H, I, E, K)
    out, aux = moe(x, kernel_backend_moe=KernelBackendMoE.sonicmoe)
    params = [moe.router.weight, moe.c_fc.weight, moe.c_proj.weight]
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=dy)

    # routing: bit-exact against the oracle on the very logits the layer saw
    with torch.no_grad():
        logits = torch.nn.functional.linear(x, moe.router.weight)
    s_ref, i_ref = R.topk_softmax(logits.float().cpu().numpy(), K)
    sel = torch.from_numpy(i_ref).to(dev)

    xr = x.detach().clone().requires_grad_()
    pr = [p.detach().clone().requires_grad_() for p in params]
    out_ref, logits_ref, freq_ref = M.moe_torch_backend(xr, pr[0], pr[1], pr[2], K, selected_experts=sel)
    grads_ref = torch.autograd.grad(out_ref, [xr] + pr, grad_outputs=dy.float())

    assert rel_l2(out, out_ref) < TOL
    names = ["dx", "d_router_w", "d_w1", "d_w2"]
    for n, g, gr in zip(names, grads, grads_ref):
        assert g.shape == gr.shape
        assert rel_l2(g, gr) < TOL, n
    aux_ref = M.switch_aux_loss(logits, freq_ref)
    assert abs(float(aux) - float(aux_ref)) < 1e-3 * abs(float(aux_ref))


def test_fused_layer_node_matches_three_nodes(dev, monkeypatch):
    """The token-choice layer as one autograd node (dx formed inside the router GEMM, the outside gradient of the
    logits added before the router GEMMs) against the same layer as three nodes whose dx contributions autograd adds;
    the loss also reads router_logits directly, as an auxiliary loss does."""
    from sonicmoe.functional import moe_TC_softmax_topk_layer
    from helpers import make_weights

    T, H, I, E, K = 2048, 768, 256, 32, 4
    wr, w1, w2 = make_weights(E, H, I, dev, seed=7)
    g = torch.Generator().manual_seed(8)
    x0 = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    dl = (torch.randn(T, E, generator=g) * 0.01).to(torch.bfloat16).to(dev)

    def run(fused):
        monkeypatch.setenv("SMOE_FUSED_TC_LAYER", "1" if fused else "0")
        x = x0.clone().requires_grad_()
        ps = [p.detach().clone().requires_grad_() for p in (wr, w1, w2)]
        o, logits, freq = moe_TC_softmax_topk_layer(x, ps[0], ps[1].permute(1, 2, 0), None, ps[2].permute(1, 2, 0), None,
                                                    K, 0)
        loss = (o.float() * dy.float()).sum() + (logits.float() * dl.float()).sum()
        return o, logits, freq, torch.autograd.grad(loss, [x] + ps)

    o1, l1, f1, g1 = run(True)
    o0, l0, f0, g0 = run(False)
    assert torch.equal(o1, o0) and torch.equal(l1, l0) and torch.equal(f1, f0)
    for name, a, b in zip(["dx", "d_router_w", "d_w1", "d_w2"], g1, g0):
        assert rel_l2(a, b) < 5e-3, name  # dx and d_router_w: one rounding less in the fused node
    assert torch.equal(g1[2], g0[2]) and torch.equal(g1[3], g0[3])


def test_layer_with_fused_combine(dev):
    """`with fused_combine():` - the down projection adds its score-weighted rows onto the output itself (atomics, no
    y2): the output stays within the layer's tolerance of the two-kernel path, every gradient is bit-identical (the
    backward pass never reads y2 or o), and the general-routing entry takes the same path."""
    from sonicmoe.functional import fused_combine, moe_TC_softmax_topk_layer, moe_general_routing_inputs
    from helpers import make_weights

    T, H, I, E, K = 2048, 768, 256, 32, 4
    wr, w1, w2 = make_weights(E, H, I, dev, seed=17)
    g = torch.Generator().manual_seed(18)
    x0 = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)

    def run(fused):
        x = x0.clone().requires_grad_()
        ps = [p.detach().clone().requires_grad_() for p in (wr, w1, w2)]
        with fused_combine(fused):
            o, logits, freq = moe_TC_softmax_topk_layer(x, ps[0], ps[1].permute(1, 2, 0), None, ps[2].permute(1, 2, 0),
                                                        None, K, 0)
        return o, torch.autograd.grad((o.float() * dy.float()).sum(), [x] + ps)

    o1, g1 = run(True)
    o0, g0 = run(False)
    assert rel_l2(o1, o0) < 1e-2
    for a, b in zip(g1, g0):
        assert torch.equal(a, b)

    # general routing: explicit (token, expert, score) triples
    scores = torch.softmax(torch.randn(T, K, generator=g), dim=-1).to(dev)
    experts = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32).to(dev)
    tokens = torch.arange(T, dtype=torch.int32, device=dev).repeat_interleave(K)

    def run_general(fused):
        with fused_combine(fused), torch.no_grad():
            out, _ = moe_general_routing_inputs(x0, scores.view(-1), tokens, experts.view(-1), w1.permute(1, 2, 0), None,
                                                w2.permute(1, 2, 0), None, E, 0, "swiglu")
        return out

    assert rel_l2(run_general(True), run_general(False)) < 1e-2


def test_module_aux_loss_value_and_gradient(dev):
    """MoE.forward's auxiliary loss on the HIP path (fused switch-loss kernels) against the oracle's formula on the
    same router logits and expert counts, differentiated by autograd: the value, and the gradients a loss of
    10 * aux sends to the router weight and the input."""
    from sonicmoe import KernelBackendMoE

    moe, x, dy = _build(dev, 2048, 512, 256, 32, 4, seed=5, x_scale=1.0)
    out, aux = moe(x, kernel_backend_moe=KernelBackendMoE.sonicmoe)
    grads = torch.autograd.grad(10.0 * aux, [x, moe.router.weight])
    assert aux.dtype == torch.float32

    xr = x.detach().clone().requires_grad_()
    wr = moe.router.weight.detach().clone().requires_grad_()
    logits = torch.nn.functional.linear(xr, wr)
    s_ref, i_ref = R.topk_softmax(logits.detach().float().cpu().numpy(), 4)
    freq = torch.bincount(torch.from_numpy(i_ref).flatten().long(), minlength=32).to(dev)
    aux_ref = M.switch_aux_loss(logits, freq)
    grads_ref = torch.autograd.grad(10.0 * aux_ref, [xr, wr])
    assert abs(float(aux.detach()) - float(aux_ref.detach())) < 1e-5 * abs(float(aux_ref.detach()))
    for n, g, gr in zip(["dx", "d_router_w"], grads, grads_ref):
        assert g.shape == gr.shape and rel_l2(g, gr) < TOL, n


def test_inference_mode_matches_training_forward(dev):
    from sonicmoe import KernelBackendMoE

    moe, x, _ = _build(dev, 1024, 512, 256, 8, 2)
    out_train, _ = moe(x, kernel_backend_moe=KernelBackendMoE.sonicmoe)
    with torch.no_grad():
        out_inf, _ = moe(x, kernel_backend_moe=KernelBackendMoE.sonicmoe, is_inference_mode=True)
    assert torch.equal(out_train, out_inf)


def test_torch_backend_of_module_matches_oracle(dev):
    """The module's own torch backend (the CPU-runnable configuration) against the oracle restatement, fp32 on GPU."""
    from sonicmoe import KernelBackendMoE, MoE
    from sonicmoe.enums import ActivationType

    torch.manual_seed(0)
    moe = MoE(8, 2, 512, 256, ActivationType.SWIGLU, False, 0.02).to(dev)
    x = torch.randn(1024, 512, device=dev)
    out, _ = moe(x, kernel_backend_moe=KernelBackendMoE.torch)
    out_ref, _, _ = M.moe_torch_backend(x, moe.router.weight, moe.c_fc.weight, moe.c_proj.weight, 2)
    assert rel_l2(out, out_ref) < 1e-5


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, TOL), (torch.float16, 3e-3)], ids=["bf16", "fp16"])
def test_general_routing_layer(dev, dtype, tol):
    """moe_general_routing_inputs against the per-expert masked loop of the reference's benchmark, on bf16 tensors and
    on fp16 ones (the second build of the library)."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import moe_general_routing_inputs
    from helpers import make_weights

    T, H, I, E = 1024, 512, 256, 16
    _, w1, w2 = make_weights(E, H, I, dev, dtype=dtype, seed=3)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(T, H, generator=g).to(dtype).to(dev).requires_grad_()
    # ragged: token t gets (t % 5) experts, so some tokens get none
    tok, exp = [], []
    for t in range(T):
        k = t % 5
        if k:
            tok += [t] * k
            exp += torch.randperm(E, generator=g)[:k].tolist()
    tok = torch.tensor(tok, dtype=torch.int32, device=dev)
    exp = torch.tensor(exp, dtype=torch.int32, device=dev)
    scores = torch.rand(tok.numel(), generator=g).to(dev).requires_grad_()
    w1p, w2p = w1.requires_grad_(), w2.requires_grad_()
    o, freq = moe_general_routing_inputs(x, scores, tok, exp, w1p.permute(1, 2, 0), None, w2p.permute(1, 2, 0), None, E,
                                         torch.cuda.current_stream().cuda_stream, ActivationType.SWIGLU, False)
    dy = torch.randn(T, H, generator=g).to(dtype).to(dev)
    grads = torch.autograd.grad(o, [x, scores, w1p, w2p], grad_outputs=dy)

    xr, sr = x.detach().clone().requires_grad_(), scores.detach().clone().requires_grad_()
    w1r, w2r = w1.detach().clone().requires_grad_(), w2.detach().clone().requires_grad_()
    o_ref = M.general_routing_reference(xr, sr, tok, exp, w1r, w2r, E)
    grads_ref = torch.autograd.grad(o_ref, [xr, sr, w1r, w2r], grad_outputs=dy.float())
    assert torch.equal(freq.cpu(), torch.bincount(exp.long().cpu(), minlength=E).int())
    assert o.dtype == dtype and rel_l2(o, o_ref) < tol
    for n, a, b in zip(["dx", "dscores", "dw1", "dw2"], grads, grads_ref):
        assert rel_l2(a, b) < tol, n
    # tokens without any expert get exactly zero
    assert bool((o[::5] == 0).all())


def test_torch_compile_fullgraph(dev):
    """The operators are registered custom ops with declared mutations, so the module compiles with fullgraph=True
    (the reference tests the same: tests/moe_test.py:80-81); results must match eager."""
    from sonicmoe import KernelBackendMoE

    moe, x, dy = _build(dev, 1024, 512, 256, 8, 2)
    params = [moe.router.weight, moe.c_fc.weight, moe.c_proj.weight]
    out, _ = moe(x, kernel_backend_moe=KernelBackendMoE.sonicmoe)
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=dy)
    compiled = torch.compile(moe, fullgraph=True)
    out_c, _ = compiled(x)
    grads_c = torch.autograd.grad(out_c, [x] + params, grad_outputs=dy)
    assert torch.equal(out, out_c)
    for a, b in zip(grads, grads_c):
        assert rel_l2(a, b) < 5e-3  # dx: the compiled graph fuses the two dx contributions before the bf16 rounding


def test_module_on_another_stream(dev):
    """The grouped GEMMs take an explicit stream while the routing / combine kernels and the allocator follow PyTorch's
    current stream: a mismatch is refused instead of racing; with `.stream_id` set to the current stream the module
    gives the same result as on the default stream."""
    moe, x, dy = _build(dev, 1024, 512, 256, 8, 2)
    with torch.no_grad():
        ref, _ = moe(x)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with pytest.raises(RuntimeError, match="current stream"):
            with torch.no_grad():
                moe(x)
        constructed_under, moe.stream_id = moe.stream_id, side.cuda_stream
        with torch.no_grad():
            out, _ = moe(x)
        moe.stream_id = constructed_under
    side.synchronize()
    assert torch.equal(out, ref)


def test_empty_batch(dev):
    """Zero tokens: every operator accepts empty tensors; the weight gradients are zeros."""
    from sonicmoe import MoE
    from sonicmoe.enums import ActivationType

    torch.manual_seed(0)
    moe = MoE(8, 2, 256, 128, ActivationType.SWIGLU, True, 0.02).to(device=dev, dtype=torch.bfloat16)
    x = torch.zeros(0, 256, dtype=torch.bfloat16, device=dev, requires_grad=True)
    out, aux = moe(x)
    assert out.shape == (0, 256)
    params = [moe.c_fc.weight, moe.c_fc.bias, moe.c_proj.weight, moe.c_proj.bias]
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=torch.zeros_like(out))
    assert grads[0].shape == (0, 256)
    for g in grads[1:]:
        assert bool((g == 0).all())


def test_general_routing_without_pairs(dev):
    """General routing entry with no (token, expert) pair at all: the output is zero."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import moe_general_routing_inputs
    from helpers import make_weights

    T, H, I, E = 64, 256, 128, 4
    _, w1, w2 = make_weights(E, H, I, dev, seed=1)
    x = torch.randn(T, H, device=dev).to(torch.bfloat16)
    empty_i = torch.zeros(0, dtype=torch.int32, device=dev)
    o, freq = moe_general_routing_inputs(x, torch.zeros(0, device=dev), empty_i, empty_i, w1.permute(1, 2, 0), None,
                                         w2.permute(1, 2, 0), None, E, torch.cuda.current_stream().cuda_stream,
                                         ActivationType.SWIGLU, False)
    assert o.shape == (T, H) and bool((o == 0).all()) and bool((freq == 0).all())
