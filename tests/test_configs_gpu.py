"""GPU parity at the remaining benchmark configurations: Zipf-skewed load with empty experts (config 3, reduced T so
that the fp32 oracle finishes in seconds), token-rounding routing through moe_general_routing_inputs (config 4), and
size-independent properties at the full size of config 2."""

import pytest
import torch

from helpers import make_weights, rel_l2
from oracle import moe_math as M
from oracle import routing as R

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _zipf_bias(E, dev):
    e = torch.arange(E, device=dev, dtype=torch.float32)
    return 2.0 * torch.log(1.0 / (e + 1.0))


def test_zipf_skewed_load_with_empty_experts(dev):
    """Config 3 semantics: logits + 2*log(1/(e+1)); the tail experts receive no token, the head ones thousands."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import TC_Softmax_Topk_Router_Function, _build_metadata, _ExpertsFunction

    T, H, I, E, K = 4096, 1024, 384, 128, 8
    wr, w1, w2 = make_weights(E, H, I, dev, seed=21)
    g = torch.Generator().manual_seed(22)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev).requires_grad_()
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    w1.requires_grad_(); w2.requires_grad_(); wr.requires_grad_()
    logits = torch.nn.functional.linear(x, wr) + _zipf_bias(E, dev).to(torch.bfloat16)
    s, i = TC_Softmax_Topk_Router_Function.apply(logits, E, K)
    freq, off, gidx, sidx, ridx, tok_off = _build_metadata(i.view(-1), None, T, E, K)
    assert int((freq == 0).sum()) > 0, "the skew should leave some experts empty"
    assert int(freq.max()) > 4 * T * K // E
    o = _ExpertsFunction.apply(x, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, s.view(-1), off, gidx, sidx, ridx,
                               tok_off, K, False, ActivationType.SWIGLU, torch.cuda.current_stream().cuda_stream, False)
    grads = torch.autograd.grad(o, [x, wr, w1, w2], grad_outputs=dy)

    # routing bit-exact against the oracle on the same logits
    s_ref, i_ref = R.topk_softmax(logits.detach().float().cpu().numpy(), K)
    assert torch.equal(i.cpu(), torch.from_numpy(i_ref))
    meta = R.tc_topk_router_metadata(i_ref, E)
    for name, t in zip(["expert_frequency", "expert_frequency_offset", "x_gather_idx", "s_scatter_idx",
                        "s_reverse_scatter_idx"], [freq, off, gidx, sidx, ridx]):
        assert torch.equal(t.cpu(), torch.from_numpy(meta[name])), name

    # float parity: the same function in fp32 torch (logit bias added by hand, so restate the few lines here)
    xr, wrr, w1r, w2r = (t.detach().clone().float().requires_grad_() for t in (x, wr, w1, w2))
    lin = torch.nn.functional.linear(xr, wrr)
    # value: the bf16-rounded biased logits the layer saw; gradient: that of the linear map
    lg = (lin.detach().to(torch.bfloat16) + _zipf_bias(E, dev).to(torch.bfloat16)).float() + (lin - lin.detach())
    gates = torch.softmax(lg.gather(1, i.long()), dim=-1)
    tok = torch.arange(T, device=dev).repeat_interleave(K)
    o_ref = M.general_routing_reference(xr, gates.reshape(-1), tok, i.reshape(-1), w1r, w2r, E)
    grads_ref = torch.autograd.grad(o_ref, [xr, wrr, w1r, w2r], grad_outputs=dy.float())
    assert rel_l2(o, o_ref) < TOL
    for n, a, b in zip(["dx", "d_router", "dw1", "dw2"], grads, grads_ref):
        assert rel_l2(a, b) < TOL, (n, rel_l2(a, b))
    empty = (freq == 0).nonzero().flatten().tolist()
    assert bool((grads[2][empty] == 0).all()) and bool((grads[3][empty] == 0).all())


@pytest.mark.parametrize("routing", ["nr", "up", "down"])
def test_token_rounding_general_routing(dev, routing):
    """Config 4 semantics at T=4096: expert counts rounded to multiples of the 128-token tile, general-routing entry."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import moe_general_routing_inputs
    from sonicmoe.routing import token_choice_rounding

    T, H, I, E, K, tile = 4096, 1024, 256, 64, 4, 128
    wr, w1, w2 = make_weights(E, H, I, dev, seed=31)
    g = torch.Generator().manual_seed(32)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev).requires_grad_()
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    with torch.no_grad():
        logits = torch.nn.functional.linear(x, wr)
        scores, tok, exp = token_choice_rounding(logits, K, tile, routing)
    scores = scores.float().requires_grad_()
    w1.requires_grad_(); w2.requires_grad_()
    o, freq = moe_general_routing_inputs(x, scores, tok, exp, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, E,
                                         torch.cuda.current_stream().cuda_stream, ActivationType.SWIGLU, False)
    assert bool((freq % tile == 0).all()) and int(freq.sum()) == tok.numel()
    grads = torch.autograd.grad(o, [x, scores, w1, w2], grad_outputs=dy)
    xr, sr, w1r, w2r = (t.detach().clone().float().requires_grad_() for t in (x, scores, w1, w2))
    o_ref = M.general_routing_reference(xr, sr, tok, exp, w1r, w2r, E)
    grads_ref = torch.autograd.grad(o_ref, [xr, sr, w1r, w2r], grad_outputs=dy.float())
    assert rel_l2(o, o_ref) < TOL
    for n, a, b in zip(["dx", "dscores", "dw1", "dw2"], grads, grads_ref):
        assert rel_l2(a, b) < TOL, n


def test_full_size_properties(dev):
    """Config 2 at full size (T=32768,H=4096,I=1024,E=128,K=8): properties that need no second implementation.
    (1) the routing metadata is a stable sort of the router's choice; (2) two runs are bit-identical; (3) the layer is
    linear in the upstream gradient: grads(2*dout) == 2*grads(dout) exactly in bf16 (power-of-two scaling);
    (4) 64 sampled tokens agree with a dense fp32 evaluation of just those tokens."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import _build_metadata, fused_combine, moe_TC_softmax_topk_layer

    T, H, I, E, K = 32768, 4096, 1024, 128, 8
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16).requires_grad_()
    wr = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w1 = (0.02 * torch.randn(E, 2 * I, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    dout = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    st = torch.cuda.current_stream().cuda_stream

    def run(dy):
        # the default forward: the opt-in combine by atomic adds is not reproducible bit for bit, whatever the environment
        with fused_combine(False):
            o, logits, freq = moe_TC_softmax_topk_layer(x, wr, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, K,
                                                        st, ActivationType.SWIGLU, False)
        return o, logits, freq, torch.autograd.grad(o, [x, wr, w1, w2], grad_outputs=dy)

    o1, logits, freq, g1 = run(dout)
    o2, _, _, g2 = run(dout)
    assert torch.equal(o1, o2) and all(torch.equal(a, b) for a, b in zip(g1, g2)), "not deterministic"
    _, _, _, g3 = run(dout * 2)
    for a, b in zip(g1[2:], g3[2:]):  # weight gradients: exactly linear (scores' path does not enter them twice)
        assert torch.equal(a * 2, b)

    # metadata invariants on the real routing
    with torch.no_grad():
        from sonicmoe.functional import forward

        scores = torch.empty(T, K, dtype=torch.float32, device=dev)
        idx = torch.empty(T, K, dtype=torch.int32, device=dev)
        forward._topk_fwd(logits, K, scores, idx, True)
        f, off, gidx, sidx, ridx, tok_off = _build_metadata(idx.view(-1), None, T, E, K)
    flat = idx.view(-1).long()
    assert torch.equal(f, freq) and int(f.sum()) == T * K and int(off[-1]) == T * K
    assert torch.equal(sidx.long(), torch.sort(flat, stable=True).indices)
    assert torch.equal(ridx[sidx.long()].long(), torch.arange(T * K, device=dev))
    assert torch.equal(gidx, sidx // K)
    assert bool((idx[:, :-1] != idx[:, 1:]).all()) and bool((scores[:, :-1] >= scores[:, 1:]).all())

    # sampled tokens against a dense fp32 evaluation
    sample = torch.randperm(T, generator=torch.Generator().manual_seed(1))[:64].to(dev)
    xs = x.detach()[sample].float()
    ref = torch.zeros(64, H, device=dev)
    for j in range(K):
        e = idx[sample, j].long()
        h = torch.einsum("th,tnh->tn", xs, w1.detach()[e].float())
        y = torch.nn.functional.silu(h[:, 0::2]) * h[:, 1::2]
        ref += scores[sample, j, None] * torch.einsum("ti,thi->th", y, w2.detach()[e].float())
    assert rel_l2(o1.detach()[sample], ref) < TOL

    # gradient VALUES at full size: the weight gradients of two experts against a dense fp32 evaluation of just those
    # experts, and dx of a few tokens against autograd through a dense fp32 restatement of their K expert MLPs
    with torch.no_grad():
        for e in (0, E - 1):
            a, b = int(off[e]), int(off[e + 1])
            tok = gidx[a:b].long()
            sc = scores.view(-1)[sidx[a:b].long()]
            dw1_ref, dw2_ref = _dense_expert_weight_grads(x, dout, w1, w2, e, tok, sc)
            assert rel_l2(g1[2][e], dw1_ref) < TOL, e
            assert rel_l2(g1[3][e], dw2_ref) < TOL, e
    few = sample[:8]
    xs = x.detach()[few].float().requires_grad_()
    lg = xs @ wr.detach().float().t()
    out = torch.zeros(8, H, device=dev)
    sc_few = torch.softmax(torch.gather(lg, 1, idx[few].long()), dim=-1)   # softmax over the K winners
    for j in range(K):
        e = idx[few, j].long()
        h = torch.einsum("th,tnh->tn", xs, w1.detach()[e].float())
        y = torch.nn.functional.silu(h[:, 0::2]) * h[:, 1::2]
        out = out + sc_few[:, j, None] * torch.einsum("ti,thi->th", y, w2.detach()[e].float())
    (dx_ref,) = torch.autograd.grad(out, xs, grad_outputs=dout[few].float())
    assert rel_l2(g1[0][few], dx_ref) < 2e-2   # incl. the path through the router scores (bf16 logits in the product)


def test_tensors_beyond_2_31_elements(dev):
    """T=65536, K=8, H=4096: the grouped (TK, H) tensors hold 2^31 elements, so any 32-bit element index would wrap.
    The LAST expert's rows sit at the highest addresses: its weight gradients and the outputs of the last tokens are
    compared with a dense fp32 evaluation of that expert alone."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import _build_metadata, forward, moe_TC_softmax_topk_layer

    T, H, I, E, K = 65536, 4096, 512, 64, 8
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16).requires_grad_()
    wr = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    w1 = (0.02 * torch.randn(E, 2 * I, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    dout = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    st = torch.cuda.current_stream().cuda_stream
    o, logits, freq = moe_TC_softmax_topk_layer(x, wr, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, K, st,
                                                ActivationType.SWIGLU, False)
    dx, dw1, dw2 = torch.autograd.grad(o, [x, w1, w2], grad_outputs=dout)
    assert T * K * H >= 2**31

    with torch.no_grad():
        scores = torch.empty(T, K, dtype=torch.float32, device=dev)
        idx = torch.empty(T, K, dtype=torch.int32, device=dev)
        forward._topk_fwd(logits, K, scores, idx, True)
        _, off, gidx, sidx, _, _ = _build_metadata(idx.view(-1), None, T, E, K)
        e = E - 1
        a, b = int(off[e]), int(off[e + 1])
        assert b == T * K and b - a > 1000
        tok = gidx[a:b].long()
        s = scores.view(-1)[sidx[a:b].long()]
        xe, de = x.detach()[tok].float(), dout[tok].float()
        z = xe @ w1.detach()[e].float().t()
        gate, up = z[:, 0::2], z[:, 1::2]
        sig = torch.sigmoid(gate)
        y1 = gate * sig * up
        dy1 = de @ w2.detach()[e].float()
        dz = torch.empty_like(z)
        dz[:, 0::2] = s[:, None] * dy1 * up * (gate * sig * (1 - sig) + sig)
        dz[:, 1::2] = s[:, None] * dy1 * gate * sig
        dw2_ref = de.t() @ (s[:, None] * y1)
        dw1_ref = dz.t() @ xe
    assert rel_l2(dw2[e], dw2_ref) < TOL
    assert rel_l2(dw1[e], dw1_ref) < TOL

    # forward of the last 32 tokens, densely
    with torch.no_grad():
        sample = torch.arange(T - 32, T, device=dev)
        xs = x.detach()[sample].float()
        ref = torch.zeros(32, H, device=dev)
        for j in range(K):
            ee = idx[sample, j].long()
            h = torch.einsum("th,tnh->tn", xs, w1.detach()[ee].float())
            y = torch.nn.functional.silu(h[:, 0::2]) * h[:, 1::2]
            ref += scores[sample, j, None] * torch.einsum("ti,thi->th", y, w2.detach()[ee].float())
    assert rel_l2(o.detach()[sample], ref) < TOL
    assert bool(torch.isfinite(dx.float()).all())


def _dense_tokens(x, w1, w2, pairs_tok, pairs_exp, pairs_score, sample):
    """fp32 forward of the sampled tokens only: sum over a token's routed pairs of score * W2[e] swiglu(W1[e] x)."""
    ref = torch.zeros(sample.numel(), x.size(1), device=x.device)
    for n, t in enumerate(sample.tolist()):
        sel = (pairs_tok == t).nonzero().flatten()
        for j in sel.tolist():
            e = int(pairs_exp[j])
            h = w1.detach()[e].float() @ x.detach()[t].float()
            y = torch.nn.functional.silu(h[0::2]) * h[1::2]
            ref[n] += float(pairs_score[j]) * (w2.detach()[e].float() @ y)
    return ref


def _dense_expert_weight_grads(x, dout, w1, w2, e, tok, s):
    """fp32 weight gradients of ONE expert from its routed tokens `tok` with scores `s` (the formulas of the layer)."""
    xe, de = x.detach()[tok].float(), dout[tok].float()
    z = xe @ w1.detach()[e].float().t()
    gate, up = z[:, 0::2], z[:, 1::2]
    sig = torch.sigmoid(gate)
    y1 = gate * sig * up
    dy1 = de @ w2.detach()[e].float()
    dz = torch.empty_like(z)
    dz[:, 0::2] = s[:, None] * dy1 * up * (gate * sig * (1 - sig) + sig)
    dz[:, 1::2] = s[:, None] * dy1 * gate * sig
    return dz.t() @ xe, de.t() @ (s[:, None] * y1)


def test_config3_full_size_properties(dev):
    """Config 3 at full size (T=32768,H=4096,I=1536,E=128,K=8, Zipf logit bias 2*log(1/(e+1))): the head experts hold
    tens of thousands of rows, the tail ones none; I=1536 gives the weight-gradient kernels 6 column tiles.  Checked
    without a second full implementation: routing metadata = stable sort of the router's choice, two runs bit-identical,
    zero weight gradients for experts without tokens, sampled tokens against a dense fp32 forward, and the weight
    gradients of one mid-sized and the largest expert against a dense fp32 evaluation of just those experts."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import TC_Softmax_Topk_Router_Function, _build_metadata, _ExpertsFunction

    T, H, I, E, K = 32768, 4096, 1536, 128, 8
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16).requires_grad_()
    wr = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    w1 = (0.02 * torch.randn(E, 2 * I, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    dout = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    st = torch.cuda.current_stream().cuda_stream
    bias = _zipf_bias(E, dev).to(torch.bfloat16)

    def run():
        logits = torch.nn.functional.linear(x.detach(), wr) + bias
        s, i = TC_Softmax_Topk_Router_Function.apply(logits, E, K)
        freq, off, gidx, sidx, ridx, tok_off = _build_metadata(i.view(-1), None, T, E, K)
        o = _ExpertsFunction.apply(x, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, s.view(-1), off, gidx, sidx,
                                   ridx, tok_off, K, False, ActivationType.SWIGLU, st, False)
        return o, torch.autograd.grad(o, [x, w1, w2], grad_outputs=dout), (s, i, freq, off, gidx, sidx, ridx)

    o1, g1, (s, i, freq, off, gidx, sidx, ridx) = run()
    o2, g2, _ = run()
    assert torch.equal(o1, o2) and all(torch.equal(a, b) for a, b in zip(g1, g2)), "not deterministic"
    flat = i.view(-1).long()
    assert int(freq.sum()) == T * K and int(off[-1]) == T * K
    assert torch.equal(sidx.long(), torch.sort(flat, stable=True).indices)
    assert torch.equal(ridx[sidx.long()].long(), torch.arange(T * K, device=dev))
    assert torch.equal(gidx, sidx // K)
    empty = (freq == 0).nonzero().flatten()
    assert empty.numel() > 0 and int(freq.max()) > 20000, "the Zipf bias should empty the tail and overload the head"
    dx, dw1, dw2 = g1
    assert bool((dw1[empty] == 0).all()) and bool((dw2[empty] == 0).all())
    assert bool(torch.isfinite(dx.float()).all())

    with torch.no_grad():
        sample = torch.randperm(T, generator=torch.Generator().manual_seed(1))[:32].to(dev)
        tok_of_pair = torch.arange(T, device=dev).repeat_interleave(K)
        ref = _dense_tokens(x, w1, w2, tok_of_pair, i.view(-1), s.view(-1), sample)
        assert rel_l2(o1.detach()[sample], ref) < TOL
        # one mid-sized expert (its last token tile is ragged) and the largest one
        counts = freq.tolist()
        mid = min((e for e in range(E) if 300 <= counts[e] <= 6000), key=lambda e: counts[e], default=None)
        for e in [e for e in (mid, int(freq.argmax())) if e is not None]:
            a, b = int(off[e]), int(off[e + 1])
            tok = gidx[a:b].long()
            sc = s.view(-1)[sidx[a:b].long()]
            dw1_ref, dw2_ref = _dense_expert_weight_grads(x, dout, w1, w2, e, tok, sc)
            assert rel_l2(dw1[e], dw1_ref) < TOL, e
            assert rel_l2(dw2[e], dw2_ref) < TOL, e


def test_config4_full_size_properties(dev):
    """Config 4 at full size (T=16384,H=4096,I=1024,E=256,K=8, token rounding "nr" to tiles of 128, general-routing
    entry): every expert's count is a multiple of 128, the pairs are sorted by token, two runs are bit-identical,
    sampled tokens match a dense fp32 forward over their pairs and one expert's weight gradients a dense evaluation."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import _build_metadata, moe_general_routing_inputs
    from sonicmoe.routing import token_choice_rounding

    T, H, I, E, K, tile = 16384, 4096, 1024, 256, 8, 128
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16).requires_grad_()
    wr = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    w1 = (0.02 * torch.randn(E, 2 * I, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    dout = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    st = torch.cuda.current_stream().cuda_stream
    with torch.no_grad():
        scores, tok, exp = token_choice_rounding(torch.nn.functional.linear(x, wr), K, tile, "nr")
    scores = scores.float().requires_grad_()
    assert bool((tok[1:] >= tok[:-1]).all())

    def run():
        o, freq = moe_general_routing_inputs(x, scores, tok, exp, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, E,
                                             st, ActivationType.SWIGLU, False)
        return o, freq, torch.autograd.grad(o, [x, scores, w1, w2], grad_outputs=dout)

    o1, freq, g1 = run()
    o2, _, g2 = run()
    assert torch.equal(o1, o2) and all(torch.equal(a, b) for a, b in zip(g1, g2)), "not deterministic"
    assert bool((freq % tile == 0).all()) and int(freq.sum()) == tok.numel()
    assert abs(tok.numel() - T * K) <= E * tile // 2
    with torch.no_grad():
        sample = torch.randperm(T, generator=torch.Generator().manual_seed(2))[:32].to(dev)
        ref = _dense_tokens(x, w1, w2, tok, exp, scores.detach(), sample)
        assert rel_l2(o1.detach()[sample], ref) < TOL
        _, off, gidx, sidx, _, _ = _build_metadata(exp, tok, T, E, 1)
        e = int((freq > 0).nonzero().flatten()[7])
        a, b = int(off[e]), int(off[e + 1])
        dw1_ref, dw2_ref = _dense_expert_weight_grads(x, dout, w1, w2, e, gidx[a:b].long(),
                                                      scores.detach()[sidx[a:b].long()])
        assert rel_l2(g1[2][e], dw1_ref) < TOL
        assert rel_l2(g1[3][e], dw2_ref) < TOL


def test_config5_full_size_fp8(dev):
    """Config 5 (config 2's shape with fp8 operands) at full size, forward and backward: deterministic; the routing is
    the bf16 path's (the router is not quantised); output and gradients against the bf16 path of the same layer, with
    the bounds measured at the small shapes (tests/test_fp8_gpu.py): one quantised GEMM stays inside the 5e-2 stated
    for fp8, chains of two or three land at 5e-2 .. 7e-2 -- recorded, not claimed as within tolerance; 64 sampled
    tokens against a dense fp32 evaluation.  The scales are one power of two per 32 elements (what the fp8 matrix
    instruction applies itself), not the amax/448 per 128 elements of the config's wording:
    tests/test_fp8_recipe_numerics.py pins the difference of the two on the CPU.  Weight gradients are bf16 GEMMs."""
    from sonicmoe import enable_fp8_backward, enable_fp8_forward
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import moe_TC_softmax_topk_layer

    T, H, I, E, K = 32768, 4096, 1024, 128, 8
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16).requires_grad_()
    wr = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w1 = (0.02 * torch.randn(E, 2 * I, H, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I, generator=g, device=dev)).to(torch.bfloat16).requires_grad_()
    dout = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    st = torch.cuda.current_stream().cuda_stream

    def run():
        o, logits, freq = moe_TC_softmax_topk_layer(x, wr, w1.permute(1, 2, 0), None, w2.permute(1, 2, 0), None, K, st,
                                                    ActivationType.SWIGLU, False)
        return o, logits, freq, torch.autograd.grad(o, [x, wr, w1, w2], grad_outputs=dout)

    o_ref, logits_ref, freq_ref, g_ref = run()
    with enable_fp8_forward(), enable_fp8_backward():
        o8, logits8, freq8, g8 = run()
        o8b, _, _, g8b = run()
    assert torch.equal(o8, o8b) and all(torch.equal(a, b) for a, b in zip(g8, g8b)), "not deterministic"
    assert torch.equal(logits8, logits_ref) and torch.equal(freq8, freq_ref)
    errs = dict(out=rel_l2(o8, o_ref), **{n: rel_l2(a, b) for n, a, b in zip(("dx", "dwr", "dw1", "dw2"), g8, g_ref)})
    print("config 5 full size, fp8 against bf16:", {k: round(v, 4) for k, v in errs.items()})
    assert all(1e-3 < v < 9e-2 for v in errs.values()), errs
    del g_ref, g8, g8b, o8b

    # sampled tokens of the fp8 output against a dense fp32 evaluation (same bound as the fp8 layer test: 8e-2)
    with torch.no_grad():
        from sonicmoe.functional import forward

        scores = torch.empty(T, K, dtype=torch.float32, device=dev)
        idx = torch.empty(T, K, dtype=torch.int32, device=dev)
        forward._topk_fwd(logits8, K, scores, idx, True)
    sample = torch.randperm(T, generator=torch.Generator().manual_seed(1))[:64].to(dev)
    xs = x.detach()[sample].float()
    ref = torch.zeros(64, H, device=dev)
    for j in range(K):
        e = idx[sample, j].long()
        h = torch.einsum("th,tnh->tn", xs, w1.detach()[e].float())
        y = torch.nn.functional.silu(h[:, 0::2]) * h[:, 1::2]
        ref += scores[sample, j, None] * torch.einsum("ti,thi->th", y, w2.detach()[e].float())
    err = rel_l2(o8.detach()[sample], ref)
    assert 1e-2 < err < 8e-2, err
