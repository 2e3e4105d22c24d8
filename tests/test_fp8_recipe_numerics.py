"""CPU simulation of an fp8 recipe for the layer at its headline shape (OCP e4m3, one fp32 scale amax/448 per 128 contiguous
elements of the contraction, fp32 accumulation, both operands of every GEMM quantised).

The reference has no fp8 path to compare with (parity unpinned); this test records what
the recipe itself can deliver against the fp32 evaluation: the first GEMM stays inside the 5e-2 bar, but the error of
SwiGLU(z) and of everything downstream of a second quantised GEMM lands between 5e-2 and 8e-2.  e4m3 keeps 3 mantissa
bits, i.e. ~2.6 % rms relative rounding error per element, ~3.7 % per product; block scaling cannot change that."""

import torch


def _qdq(t: torch.Tensor, dim: int = -1, blk: int = 128) -> torch.Tensor:
    t = t.transpose(dim, -1)
    sh = t.shape
    tb = t.reshape(*sh[:-1], sh[-1] // blk, blk)
    s = tb.abs().amax(-1, keepdim=True).clamp_min(1e-12) / 448.0
    out = (tb / s).to(torch.float8_e4m3fn).float() * s
    return out.reshape(sh).transpose(dim, -1)


def _rel(a, b):
    return float((a - b).norm() / b.norm())


def test_e4m3_block_scaled_recipe_error_levels():
    torch.manual_seed(0)
    T, H, I = 1024, 1024, 256
    x, dout = torch.randn(T, H), torch.randn(T, H)
    w1, w2 = torch.randn(2 * I, H) * 0.02, torch.randn(H, I) * 0.02

    def forward(Q):
        z = Q(x) @ Q(w1).t()
        y1 = torch.nn.functional.silu(z[:, 0::2]) * z[:, 1::2]
        return z, y1, Q(y1) @ Q(w2).t()

    ident = lambda t, dim=-1: t  # noqa: E731
    z0, y0, o0 = forward(ident)
    z1, y1, o1 = forward(_qdq)
    ez, ey, eo = _rel(z1, z0), _rel(y1, y0), _rel(o1, o0)
    assert 0.02 < ez < 0.05, ez  # one quantised GEMM: ~3.6 %
    assert 0.04 < ey < 0.08, ey  # gate * up multiplies two such errors: ~5 %
    assert 0.05 < eo < 0.09, eo  # second quantised GEMM on top: ~6 %  (outside the 5e-2 bar of config 5)
    # activation gradient through W2 quantised along its contraction dimension (H)
    d0 = dout @ w2
    d1 = _qdq(dout) @ _qdq(w2, dim=0)
    assert 0.02 < _rel(d1, d0) < 0.05


def test_power_of_two_scales_per_32_against_fp32_scales_per_128():
    """Config 5 of the benchmark list words its recipe as "per-128-element block scales (amax/448)"; the kernels use the
    format the fp8 matrix instruction multiplies natively instead: one power-of-two scale per 32 elements.  Same
    problem, both recipes, against the fp32 evaluation.  An fp32 scale amax/448 puts each block's largest element
    exactly on the top code, so the elements that carry most of the norm round a little better than under a
    power-of-two scale, which leaves the data's own mantissas in place; the smaller block does not make up for that.
    Measured: the built format is 3 .. 10 % less accurate in relative L2 at every stage, in the same regime (one
    quantised GEMM ~3.5e-2).  The bounds below pin that difference."""
    from oracle import fp8 as Q

    torch.manual_seed(1)
    T, H, I = 512, 1024, 256
    x, dout = torch.randn(T, H), torch.randn(T, H)
    x[:, ::7] *= 30.0  # outlier channels
    w1, w2 = torch.randn(2 * I, H) * 0.02, torch.randn(H, I) * 0.02

    def mx(t, dim=-1):
        t2 = t.transpose(dim, -1).contiguous()
        return Q.fake_quant(t2).transpose(dim, -1)

    def run(Qf):
        z = Qf(x) @ Qf(w1).t()
        y1 = torch.nn.functional.silu(z[:, 0::2]) * z[:, 1::2]
        out = Qf(y1) @ Qf(w2).t()
        dy1 = Qf(dout) @ Qf(w2, dim=0)
        return z, y1, out, dy1

    ref = run(lambda t, dim=-1: t)
    per128 = [_rel(a, b) for a, b in zip(run(_qdq), ref)]
    per32 = [_rel(a, b) for a, b in zip(run(mx), ref)]
    for name, e32, e128 in zip(("z", "y1", "out", "dy1"), per32, per128):
        assert 0.95 * e128 < e32 < 1.15 * e128, (name, e32, e128)
    assert per32[0] < 5e-2 and per128[0] < 5e-2 and per32[3] < 5e-2 and per128[3] < 5e-2  # one quantised GEMM
