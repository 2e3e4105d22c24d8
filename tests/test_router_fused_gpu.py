"""The router in one pass over x (`_router_forward_fused`): logits against the fp32 product, top-K scores and indices
bit-exact against the stand-alone top-K kernel (and the oracle) applied to the logits the kernel stored, the softmax
column sums against the oracle's switch loss, and the layer with `fused_router()` against the oracle routed by the
layer's own logits."""

import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import moe_math as M
from oracle import routing as R

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,H,E,K", [(1000, 256, 16, 2), (4096, 1024, 128, 8), (777, 512, 64, 4), (2048, 2048, 256, 8),
                                     (64, 256, 48, 3), (5, 256, 128, 8)])
def test_router_forward_fused(dev, T, H, E, K):
    from sonicmoe.functional import forward as fwd

    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    wr = (torch.randn(E, H, generator=g) / H**0.5).to(torch.bfloat16).to(dev)
    if E >= 64:
        wr[7] = wr[3]  # two experts with identical logits: the lower column has to win every tie
    logits = torch.full((T, E), 9.0, dtype=torch.bfloat16, device=dev)
    scores = torch.full((T, K), 9.0, dtype=torch.float32, device=dev)
    idx = torch.full((T, K), -1, dtype=torch.int32, device=dev)
    part = torch.full((fwd.router_fused_partials(T, E), E), 9.0, dtype=torch.float32, device=dev)
    assert fwd.router_fused_supported(x, wr)
    fwd._router_forward_fused(x, wr, logits, scores, idx, part)

    assert rel_l2(logits, x.float() @ wr.float().t()) < 5e-3
    # top-K of the logits as stored: the stand-alone kernel and the oracle
    s2 = torch.empty_like(scores)
    i2 = torch.empty_like(idx)
    fwd._softmax_topk_fwd(logits, s2, i2, E, K)
    assert torch.equal(idx, i2) and torch.equal(scores, s2)
    s_ref, i_ref = R.topk_softmax(logits.float().cpu().numpy(), K)
    assert np.array_equal(idx.cpu().numpy(), i_ref)
    np.testing.assert_allclose(scores.cpu().numpy(), s_ref, rtol=2e-6, atol=1e-7)
    # column sums of the row softmax, and the loss from them
    acc_ref = torch.softmax(logits.float(), dim=-1).sum(0)
    assert rel_l2(part.sum(0), acc_ref) < 1e-5
    freq = torch.bincount(idx.view(-1).long(), minlength=E).to(torch.int32)
    acc = torch.empty(E, dtype=torch.float32, device=dev)
    aux = torch.empty(1, dtype=torch.float32, device=dev)
    fwd._switch_loss_from_partials(part, freq, acc, aux)
    aux_ref = M.switch_aux_loss(logits.float().cpu(), freq.cpu())
    assert abs(float(aux) - float(aux_ref)) < 1e-5 * max(1.0, abs(float(aux_ref)))
    # without the column sums: same logits, scores, indices
    l3, s3, i3 = torch.empty_like(logits), torch.empty_like(scores), torch.empty_like(idx)
    fwd._router_forward_fused(x, wr, l3, s3, i3, None)
    assert torch.equal(l3, logits) and torch.equal(s3, scores) and torch.equal(i3, idx)


def test_unsupported_router_shapes(dev):
    from sonicmoe.functional import forward as fwd

    x = torch.zeros(8, 256, dtype=torch.bfloat16, device=dev)
    assert not fwd.router_fused_supported(x, torch.zeros(24, 256, dtype=torch.bfloat16, device=dev))     # E % 16
    assert not fwd.router_fused_supported(x[:, :192].contiguous(), torch.zeros(32, 192, dtype=torch.bfloat16, device=dev))
    assert not fwd.router_fused_supported(x.float(), torch.zeros(32, 256, device=dev))
    with pytest.raises(RuntimeError, match="multiple of 16"):
        fwd._router_forward_fused(x, torch.zeros(24, 256, dtype=torch.bfloat16, device=dev),
                                  torch.empty(8, 24, dtype=torch.bfloat16, device=dev),
                                  torch.empty(8, 2, dtype=torch.float32, device=dev),
                                  torch.empty(8, 2, dtype=torch.int32, device=dev), None)


def test_layer_with_fused_router(dev):
    """MoE forward + backward with the fused router against the oracle, routed by the logits the layer returns."""
    from sonicmoe import MoE
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import fused_router

    T, H, I, E, K = 2048, 1024, 256, 32, 4
    torch.manual_seed(11)
    moe = MoE(E, K, H, I, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=torch.bfloat16)
    x = torch.randn(T, H, device=dev).to(torch.bfloat16).requires_grad_()
    dy = torch.randn(T, H, device=dev).to(torch.bfloat16)
    params = [moe.router.weight, moe.c_fc.weight, moe.c_proj.weight]
    out0, aux0 = moe(x)
    with fused_router():
        out, aux = moe(x)
        grads = torch.autograd.grad(out + 0.0 * aux, [x] + params, grad_outputs=dy)
        out_b, aux_b = moe(x)
    assert torch.equal(out, out_b) and torch.equal(aux, aux_b)
    # against the unfused path of the same module: same routing except for near-ties, so close, not identical
    assert rel_l2(out, out0) < 2e-2 and abs(float(aux) - float(aux0)) < 1e-3 * abs(float(aux0))
    grads0 = torch.autograd.grad(out0, [x] + params, grad_outputs=dy)
    for a, b in zip(grads, grads0):
        assert rel_l2(a, b) < 3e-2
    # the auxiliary loss through the fused column sums, with its gradient
    with fused_router():
        out2, aux2 = moe(x)
        g_aux = torch.autograd.grad(aux2, [moe.router.weight])[0]
    out3, aux3 = moe(x)
    g_aux0 = torch.autograd.grad(aux3, [moe.router.weight])[0]
    assert rel_l2(g_aux, g_aux0) < 2e-2


@pytest.mark.gpu
def test_fused_router_hands_its_column_sums_to_the_loss(dev, monkeypatch):
    """Inside `with fused_router(): moe(x)` the auxiliary loss is formed from the column sums the router kernel wrote
    (one pass over x), not from a second pass over the logits; outside it the stand-alone pass runs."""
    import sonicmoe.functional as SF
    from sonicmoe import MoE
    from sonicmoe.enums import ActivationType

    calls = {"partials": 0, "full": 0}
    real_p, real_f = SF._switch_loss_from_partials, SF._switch_loss_fwd
    monkeypatch.setattr(SF, "_switch_loss_from_partials", lambda *a: (calls.__setitem__("partials", calls["partials"] + 1), real_p(*a))[1])
    monkeypatch.setattr(SF, "_switch_loss_fwd", lambda *a: (calls.__setitem__("full", calls["full"] + 1), real_f(*a))[1])
    torch.manual_seed(3)
    moe = MoE(32, 4, 1024, 256, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=torch.bfloat16)
    x = torch.randn(1024, 1024, device=dev).to(torch.bfloat16)
    with SF.fused_router():
        _, aux = moe(x)
    assert calls == {"partials": 1, "full": 0}
    _, aux0 = moe(x)
    assert calls == {"partials": 1, "full": 1}
    assert abs(float(aux) - float(aux0)) < 1e-3 * abs(float(aux0))
