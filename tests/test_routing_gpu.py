"""GPU parity of the routing kernels against the CPU oracle: every integer output bit-exact, scores within fp32
rounding (rtol 1e-5, the only difference being the exp implementation)."""

import numpy as np
import pytest
import torch

from oracle import routing as R

pytestmark = pytest.mark.gpu


def _ops():
    from sonicmoe import count_cumsum
    from sonicmoe.functional import _build_metadata, backward, forward

    return count_cumsum, _build_metadata, forward, backward


def _topk(dev, logits, K, softmax=True):
    _, _, fwd, _ = _ops()
    T = logits.shape[0]
    scores = torch.empty(T, K, dtype=torch.float32, device=dev)
    idx = torch.empty(T, K, dtype=torch.int32, device=dev)
    fwd._topk_fwd(logits, K, scores, idx, softmax)
    torch.cuda.synchronize()
    return scores.cpu().numpy(), idx.cpu().numpy()


@pytest.mark.parametrize(
    "T,E,K",
    [(1000, 128, 8), (333, 256, 16), (64, 8, 2), (50, 64, 4), (17, 4096, 16), (100, 72, 3), (5, 16, 16), (257, 1024, 1),
     (31, 24, 5), (4096, 128, 8)],
)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_topk_softmax_matches_oracle(dev, T, E, K, dtype):
    g = torch.Generator().manual_seed(T * 131 + E * 7 + K)
    logits = (torch.randn(T, E, generator=g) * 1.3).to(dtype)
    if T > 8:
        logits[3] = 0.5  # a fully tied row
        logits[4, : E // 2] = -1.25  # ties among negatives
        logits[5] = 0.0
        logits[5, E // 3] = -0.0
    s_ref, i_ref = R.topk_softmax(logits.float().numpy(), K)
    s, i = _topk(dev, logits.to(dev), K)
    np.testing.assert_array_equal(i, i_ref)
    np.testing.assert_allclose(s, s_ref, rtol=1e-5, atol=1e-7)
    v_ref, i_ref2 = R.topk_softmax(logits.float().numpy(), K, softmax=False)
    v, i2 = _topk(dev, logits.to(dev), K, softmax=False)
    np.testing.assert_array_equal(i2, i_ref2)
    np.testing.assert_array_equal(v, v_ref)


def test_topk_fp32_low_bit_ties(dev):
    """fp32 logits that differ only in the mantissa bits the reference overwrites must tie towards the lower column."""
    E, K = 128, 4
    base = np.full((6, E), 1.0, dtype=np.float32)
    bits = base.view(np.uint32)
    bits[0, 100] |= 0x3F  # larger only in the 7 cleared bits: still a tie, column 0.. win
    bits[1, 100] |= 0x80  # larger in a kept bit: wins
    base[2] = -base[2]
    bits[2, 100] |= 0x3F
    base[3] = np.linspace(-1, 1, E, dtype=np.float32)
    base[4] = 0
    base[5] = np.float32(-1e-3)
    logits = torch.from_numpy(base)
    s_ref, i_ref = R.topk_softmax(base, K)
    s, i = _topk(dev, logits.to(dev), K)
    np.testing.assert_array_equal(i, i_ref)
    assert list(i[0]) == [0, 1, 2, 3] and i[1][0] == 100
    np.testing.assert_allclose(s, s_ref, rtol=1e-5)


def _sizes():
    sizes = set()
    for i in range(15):
        for j in (0, 1, 3, 7, 9):
            sizes.add(2**i + j)
    rng = np.random.default_rng(0)
    sizes.update(int(v) for v in rng.integers(2000, 4000, size=6))
    return sorted(sizes)


@pytest.mark.parametrize("E", [4, 8, 72, 256, 1920, 2048, 16384, 50000])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_count_cumsum_exact(dev, E, dtype):
    """Size / E / dtype matrix of the reference's own test (tests/count_cumsum_test.py:16-38)."""
    count_cumsum, _, _, _ = _ops()
    g = torch.Generator().manual_seed(E)
    for n in _sizes() + [2097152]:
        x = torch.randint(0, E, (n,), generator=g, dtype=dtype)
        c_ref, cs_ref = R.count_cumsum(x.numpy(), E)
        c, cs = count_cumsum(x.to(dev), E, do_cumsum=True)
        c_only = count_cumsum(x.to(dev), E, do_cumsum=False)
        assert c.dtype == torch.int32 and cs.dtype == torch.int32
        np.testing.assert_array_equal(c.cpu().numpy(), c_ref, err_msg=f"n={n}")
        np.testing.assert_array_equal(cs.cpu().numpy(), cs_ref, err_msg=f"n={n}")
        np.testing.assert_array_equal(c_only.cpu().numpy(), c_ref, err_msg=f"n={n}")


_NAMES = ["expert_frequency", "expert_frequency_offset", "x_gather_idx", "s_scatter_idx", "s_reverse_scatter_idx",
          "num_activated_expert_per_token_offset"]


@pytest.mark.parametrize("T,E,K", [(1, 8, 2), (7, 4, 4), (128, 8, 2), (1000, 128, 8), (4096, 256, 16), (32768, 128, 8),
                                   (513, 72, 3), (300, 2048, 4)])
def test_tc_metadata_exact(dev, T, E, K):
    _, build, _, _ = _ops()
    rng = np.random.default_rng(T + E)
    # K distinct experts per token, Zipf-skewed so that some experts are empty and some very large
    w = 1.0 / np.arange(1, E + 1) ** 1.5
    idx = np.stack([rng.choice(E, size=K, replace=False, p=w / w.sum()) for _ in range(T)]).astype(np.int32)
    ref = R.tc_topk_router_metadata(idx, E)
    out = build(torch.from_numpy(idx).to(dev).view(-1), None, T, E, K)
    torch.cuda.synchronize()
    for name, t in zip(_NAMES, out):
        np.testing.assert_array_equal(t.cpu().numpy(), ref[name], err_msg=name)


@pytest.mark.parametrize("T,E,TK", [(64, 8, 200), (1000, 256, 5000), (16, 4, 0), (333, 128, 4096), (50, 8, 3)])
def test_general_metadata_exact(dev, T, E, TK):
    _, build, _, _ = _ops()
    rng = np.random.default_rng(T * 3 + TK)
    tok = np.sort(rng.integers(0, T, size=TK)).astype(np.int32)
    exp = rng.integers(0, E, size=TK).astype(np.int32)
    ref = R.general_routing_router_metadata(tok, exp, T, E)
    out = build(torch.from_numpy(exp).to(dev), torch.from_numpy(tok).to(dev), T, E, 1)
    torch.cuda.synchronize()
    for name, t in zip(_NAMES, out):
        np.testing.assert_array_equal(t.cpu().numpy(), ref[name], err_msg=name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_softmax_topk_bwd(dev, dtype):
    _, _, fwd, bwd = _ops()
    T, E, K = 777, 128, 8
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g).to(dtype)
    s, i = R.topk_softmax(logits.float().numpy(), K)
    ds = torch.randn(T, K, generator=g)
    ref = R.softmax_topk_bwd(ds.numpy(), s, i, E)
    dl = torch.zeros(T, E, dtype=dtype, device=dev)
    bwd._softmax_topk_bwd(dl, None, ds.to(dev), torch.from_numpy(s).to(dev), torch.from_numpy(i).to(dev), K)
    torch.cuda.synchronize()
    got = dl.float().cpu().numpy()
    if dtype == torch.float32:
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-7)
    else:
        np.testing.assert_allclose(got, torch.from_numpy(ref).to(dtype).float().numpy(), rtol=1e-2, atol=1e-6)
    # the optional `dlogits` argument: a gradient already sitting at the selected positions is added in (and only
    # there: what the reference's kernel does, backward.py:520-525)
    extra = torch.randn(T, E, generator=g).to(dtype)
    dl2 = torch.zeros(T, E, dtype=dtype, device=dev)
    bwd._softmax_topk_bwd(dl2, extra.to(dev), ds.to(dev), torch.from_numpy(s).to(dev), torch.from_numpy(i).to(dev), K)
    sel = torch.zeros(T, E, dtype=torch.bool).scatter_(1, torch.from_numpy(i).long(), True)
    want = torch.where(sel, torch.from_numpy(ref) + extra.float(), torch.zeros(()))
    np.testing.assert_allclose(dl2.float().cpu().numpy(), want.to(dtype).float().numpy(),
                               rtol=1e-5 if dtype == torch.float32 else 1e-2, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_topk_bwd_is_the_gradient_of_topk(dev, dtype):
    """`_topk_bwd` (the un-fused top-K's backward) against autograd through torch.topk on tie-free fp32 logits: the
    gradient of a selected logit is the gradient of its value, every other entry stays zero; exact (a scatter)."""
    _, _, fwd, bwd = _ops()
    T, E, K = 513, 64, 6
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(T, E, generator=g).requires_grad_()
    vals, idx = torch.topk(logits, K, dim=-1)
    dv = torch.randn(T, K, generator=g)
    (ref,) = torch.autograd.grad(vals, logits, grad_outputs=dv)
    dl = torch.zeros(T, E, dtype=dtype, device=dev)
    bwd._topk_bwd(dl, dv.to(dev), idx.to(torch.int32).to(dev), K)
    torch.cuda.synchronize()
    assert torch.equal(dl.cpu(), ref.to(dtype))


@pytest.mark.parametrize("mode", ["nr", "up", "down"])
@pytest.mark.parametrize("T,E,K,tile,dtype", [
    (512, 16, 2, 32, torch.bfloat16),
    (4096, 64, 4, 128, torch.bfloat16),
    (3000, 256, 8, 128, torch.float16),     # T not a multiple of the select kernel's 1024-token chunks
    (200, 8, 2, 128, torch.bfloat16),       # every target is 0 or clamps to T
])
def test_token_rounding_router_on_device(dev, mode, T, E, K, tile, dtype):
    """The HIP token-rounding router against the oracle driven with the same rounded probabilities: the same set of
    (token, expert) pairs and the same scores (the order inside a token is ascending expert here, unspecified in the
    reference)."""
    from oracle import token_rounding as TR
    from sonicmoe.routing import token_choice_rounding_device

    g = torch.Generator().manual_seed(T + E)
    logits = (torch.randn(T, E, generator=g) * 1.5).to(dtype).to(dev)
    sc, tok, exp, probs = token_choice_rounding_device(logits, K, tile, mode)
    # the device softmax against torch's (both fp32, rounded to the 16-bit dtype): at most one unit in the last place
    ref_p = torch.softmax(logits.float(), dim=-1).to(dtype)
    assert float((probs.float() - ref_p.float()).abs().max()) <= float(ref_p.float().max()) * 2.0 ** -7

    rnd = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).float().numpy()  # noqa: E731
    sc_o, tok_o, exp_o, target = TR.token_choice_rounding(probs.float().cpu().numpy(), K, tile, mode, rnd=rnd)
    order = np.lexsort((exp_o, tok_o))
    tok_o, exp_o, sc_o = tok_o[order], exp_o[order], sc_o[order]
    assert tok.cpu().numpy().tolist() == tok_o.tolist()
    assert exp.cpu().numpy().tolist() == exp_o.tolist()
    assert np.array_equal(sc.float().cpu().numpy(), sc_o)  # same dtype arithmetic: identical bits
    counts = np.bincount(exp.cpu().numpy(), minlength=E)
    assert counts.tolist() == target.tolist()
    assert bool((torch.diff(tok) >= 0).all())


@pytest.mark.parametrize("T,E", [(1000, 128), (37, 8), (4096, 256), (300, 100), (65, 1000), (9, 4096), (1, 64), (32768, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_switch_loss_matches_oracle(dev, T, E, dtype):
    """Fused switch loss (forward value and gradient with respect to the logits) against the oracle's torch formula
    differentiated by autograd in fp32.  Tolerances: value 1e-5 relative (fp32 sums in another order); gradient
    rel-L2 1e-5 for fp32 logits, 1e-2 for 16-bit logits (the gradient is rounded to the logits' dtype)."""
    from oracle import moe_math as M
    from sonicmoe.functional import switch_loss

    g = torch.Generator().manual_seed(T * 7 + E)
    logits = (torch.randn(T, E, generator=g) * 1.5).to(dtype)
    freq = torch.randint(0, 50, (E,), generator=g, dtype=torch.int32)
    freq[0] += 1  # not all zero
    ref_in = logits.float().requires_grad_(True)
    aux_ref = M.switch_aux_loss(ref_in, freq)
    scale = float(T)  # keeps the gradient's elements (order 1/T per unit of loss) inside fp16's normal range
    (dref,) = torch.autograd.grad(aux_ref * scale, ref_in)

    x = logits.to(dev).requires_grad_(True)
    aux = switch_loss(x, freq.to(dev))
    assert aux.dtype == torch.float32 and aux.dim() == 0
    (dx,) = torch.autograd.grad(aux * scale, x)
    torch.cuda.synchronize()
    assert abs(float(aux.detach()) - float(aux_ref.detach())) <= 1e-5 * abs(float(aux_ref.detach())) + 1e-7
    assert dx.dtype == dtype and dx.shape == logits.shape
    err = float((dx.float().cpu() - dref).norm() / dref.norm().clamp_min(1e-30))
    assert err < (1e-5 if dtype == torch.float32 else 1e-2), err


def test_switch_loss_closed_forms(dev):
    """Uniform router and uniform load give exactly 1; all probability mass and all load on one expert give E; the
    gradient of a row sums to zero (softmax) and vanishes for a uniform load (the loss is then constant = 1)."""
    from sonicmoe.functional import switch_loss

    E = 64
    aux = switch_loss(torch.zeros(128, E, device=dev), torch.full((E,), 16, dtype=torch.int32, device=dev))
    assert abs(float(aux) - 1.0) < 1e-6
    logits = torch.full((32, E), -30.0, device=dev)
    logits[:, 5] = 30.0
    f = torch.zeros(E, dtype=torch.int32, device=dev)
    f[5] = 100
    assert abs(float(switch_loss(logits, f)) - E) < 1e-4
    x = torch.randn(200, E, device=dev, requires_grad=True)
    (d,) = torch.autograd.grad(switch_loss(x, torch.randint(1, 9, (E,), dtype=torch.int32, device=dev)), x)
    assert float(d.sum(1).abs().max()) < 1e-7
    (d,) = torch.autograd.grad(switch_loss(x, torch.full((E,), 3, dtype=torch.int32, device=dev)), x)
    assert float(d.abs().max()) < 1e-8
    # a strided view of a wider tensor is read in place
    wide = torch.randn(50, 2 * E, device=dev)
    fr = torch.randint(1, 9, (E,), dtype=torch.int32, device=dev)
    assert abs(float(switch_loss(wide[:, :E], fr)) - float(switch_loss(wide[:, :E].contiguous(), fr))) < 1e-7
