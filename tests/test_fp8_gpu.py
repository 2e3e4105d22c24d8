"""GPU tests of the fp8 forward path (block-scaled e4m3): quantiser bit-exact against the oracle, the two fp8 grouped
GEMMs against the oracle evaluated on the same de-quantised operands (tight) and against the unquantised fp32 oracle
within the fp8 tolerance 5e-2, and the layer with `enable_fp8_forward()`.

Parity against the reference is unpinned for this path (the reference has no fp8 code).  Per operator the format stays
inside 5e-2; through the whole layer (two quantised GEMMs and a gated activation in series) the relative L2 against
the bf16 oracle is about 6e-2, which the last test records with its measured bound."""

import numpy as np
import pytest
import torch

from helpers import make_tc_routing, rel_l2
from oracle import fp8 as Q
from oracle import moe_math as M

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("R,C", [(1, 128), (77, 256), (1000, 1024), (4096, 4096)])
def test_quantiser_bit_exact(dev, R, C):
    from sonicmoe.functional.fp8 import mx_quantize

    g = torch.Generator().manual_seed(R + C)
    x = torch.randn(R, C, generator=g) * torch.logspace(-5, 3, R)[:, None]
    x[0, :32] = 0.0
    if R > 5:
        x[5, 0] = 448.0 * 8
        x[4, 32:64] = torch.linspace(-1.75, 1.75, 32)
    x = x.to(torch.bfloat16)
    q, s = mx_quantize(x.to(dev))
    q_ref, ex_ref = Q.mx_quantize(x)
    s_ref = Q.pack_scales(ex_ref)
    assert torch.equal(s.cpu(), s_ref)
    got, ref = q.cpu(), q_ref
    zero = ((got & 0x7F) == 0) & ((ref & 0x7F) == 0)  # the sign of a zero carries no value
    assert bool(((got == ref) | zero).all())


def _problem(dev, T, H, I, E, K, seed, activation="swiglu", skew=0.0, empty=()):
    glu = M.is_glu(activation)
    N1 = 2 * I if glu else I
    g = torch.Generator().manual_seed(seed)
    w1 = (torch.randn(E, N1, H, generator=g) / H**0.5).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, generator=g) / I**0.5).to(torch.bfloat16)
    b1 = (0.3 * torch.randn(E, N1, generator=g)).to(torch.bfloat16)
    b2 = (0.3 * torch.randn(E, H, generator=g)).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    _, scores, meta, md = make_tc_routing(T, E, K, dev, seed=seed + 1, skew=skew, empty=empty)
    return glu, N1, w1, w2, b1, b2, x, md, meta


@pytest.mark.parametrize("T,H,I,E,K,activation,with_bias,skew,empty", [
    (512, 256, 128, 8, 2, "swiglu", False, 0.0, ()),
    (1500, 384, 256, 8, 2, "swiglu", True, 0.8, (5,)),     # ragged tiles, an empty expert, biases
    (2048, 1024, 512, 16, 4, "geglu", False, 0.5, ()),
    (1024, 512, 384, 4, 2, "gelu", True, 0.0, ()),         # not gated: z has I columns
])
def test_fp8_forward_operators(dev, T, H, I, E, K, activation, with_bias, skew, empty):
    from sonicmoe.functional import fp8

    glu, N1, w1, w2, b1, b2, x, md, meta = _problem(dev, T, H, I, E, K, T + H, activation, skew, empty)
    if not with_bias:
        b1 = b2 = None
    TK = T * K
    off, gidx = md["expert_frequency_offset"], md["x_gather_idx"]
    stream = torch.cuda.current_stream().cuda_stream
    bf = dict(dtype=torch.bfloat16, device=dev)
    dv = lambda t: None if t is None else t.to(dev)  # noqa: E731

    xq, xs = fp8.mx_quantize(x.to(dev))
    w1q, w1s = fp8.quantize_expert_weight(w1.to(dev).permute(1, 2, 0))
    z = torch.empty(TK, N1, **bf)
    y1 = torch.empty(TK, I, **bf)
    y1q_f = torch.empty(TK, I, dtype=torch.uint8, device=dev)
    y1s_f = torch.zeros(I // 128, TK, dtype=torch.int32, device=dev)
    fp8._up_projection_forward_fp8(xq, xs, w1q, w1s, z, y1, dv(b1), off, gidx, E, stream, activation, glu, y1q_f, y1s_f)
    z_fq, y1_fq = Q.up_projection_forward_fp8(x, w1, off, gidx, b1=b1, activation=activation)
    assert rel_l2(z, z_fq) < 5e-3      # same operands, fp32 accumulation: what is left is the bf16 rounding of z
    assert rel_l2(y1, y1_fq) < 5e-3
    z_ref, y1_ref = M.up_projection_forward(x, w1, off.cpu(), gidx.cpu(), b1=b1, activation=activation)
    assert rel_l2(z, z_ref) < 5e-2     # one quantised GEMM against the unquantised one: the fp8 tolerance

    # y1 quantised inside the epilogue (from the fp32 values): de-quantised it is y1 up to the e4m3 rounding, every
    # block's scale is the smallest power of two that avoids saturation, and without the bf16 output the bytes are the same
    words = y1s_f.cpu().numpy().view(np.uint32).T                        # (TK, I/128)
    ex = np.stack([(words >> (8 * b)) & 0xFF for b in range(4)], axis=-1).reshape(TK, I // 32).astype(np.uint8)
    y1_deq = Q.mx_dequantize(y1q_f.cpu(), torch.from_numpy(ex))
    assert rel_l2(y1_deq, y1_fq) < 4e-2
    blocks = y1_fq.reshape(TK, I // 32, 32).abs().amax(-1).numpy()
    scale = 2.0 ** (ex.astype(np.float64) - 127)
    live = blocks > 1e-6
    ratio = blocks[live] / scale[live]
    assert bool((ratio < 448 * 1.02).all()) and bool((ratio > 224 * 0.98).all())
    y1q_only = torch.empty_like(y1q_f)
    y1s_only = torch.zeros_like(y1s_f)
    fp8._up_projection_forward_fp8(xq, xs, w1q, w1s, None, None, dv(b1), off, gidx, E, stream, activation, glu,
                                   y1q_only, y1s_only)
    assert torch.equal(y1q_only, y1q_f) and torch.equal(y1s_only, y1s_f)

    y1q, y1s = fp8.mx_quantize(y1)
    w2q, w2s = fp8.quantize_expert_weight(w2.to(dev).permute(1, 2, 0))
    y2 = torch.empty(TK, H, **bf)
    fp8._down_projection_forward_fp8(y1q, y1s, w2q, w2s, y2, dv(b2), off, E, stream)
    y2_fq = Q.down_projection_forward_fp8(y1.float().cpu(), w2, off, b2=b2)
    assert rel_l2(y2, y2_fq) < 5e-3
    y2_ref = M.down_projection_forward(y1.float().cpu(), w2, off.cpu(), b2=b2)
    assert rel_l2(y2, y2_ref) < 5e-2


def test_layer_with_fp8_forward(dev):
    """MoE forward in fp8, backward in bf16: output and gradients against the bf16 path of the same module."""
    from sonicmoe import MoE, enable_fp8_forward
    from sonicmoe.enums import ActivationType

    T, H, I, E, K = 2048, 1024, 512, 16, 4
    torch.manual_seed(3)
    moe = MoE(E, K, H, I, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=torch.bfloat16)
    x = torch.randn(T, H, device=dev).to(torch.bfloat16).requires_grad_()
    dy = torch.randn(T, H, device=dev).to(torch.bfloat16)
    params = [moe.c_fc.weight, moe.c_proj.weight]
    out, _ = moe(x)
    grads = torch.autograd.grad(out, [x] + params, grad_outputs=dy)
    with enable_fp8_forward():
        out8, _ = moe(x)
        grads8 = torch.autograd.grad(out8, [x] + params, grad_outputs=dy)
        with torch.no_grad():
            out8_inf, _ = moe(x, is_inference_mode=True)
    assert torch.equal(out8, out8_inf)
    err = rel_l2(out8, out)
    assert 1e-2 < err < 8e-2, err   # measured ~6e-2: two quantised GEMMs in series exceed the per-operator 5e-2
    for a, b in zip(grads8, grads):
        assert rel_l2(a, b) < 8e-2  # bf16 backward from the fp8-forward z


def test_quantised_weight_cache_follows_parameter_updates(dev):
    """The cached quantised weights are dropped when the parameter is written to (optimizer step)."""
    from sonicmoe import MoE, enable_fp8_forward
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional.fp8 import cache_quantized_weights

    torch.manual_seed(5)
    moe = MoE(8, 2, 256, 128, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=torch.bfloat16)
    x = torch.randn(512, 256, device=dev).to(torch.bfloat16)
    with torch.no_grad(), enable_fp8_forward():
        a, _ = moe(x)
        b, _ = moe(x)                      # second call: cache hit
        moe.c_proj.weight.mul_(2.0)        # in-place update bumps the version counter
        c, _ = moe(x)
        with cache_quantized_weights(False):
            d, _ = moe(x)
    assert torch.equal(a, b)
    assert torch.equal(c, d)
    assert rel_l2(c, 2.0 * a.float()) < 1e-2


def test_quantised_weight_cache_is_not_fooled_by_address_reuse(dev):
    """A module is freed and another of the same shape is built: its parameters may land at the freed addresses with
    the same version counter, and must not meet the first module's quantised weights."""
    import gc

    from sonicmoe import MoE, enable_fp8_forward
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional.fp8 import cache_quantized_weights

    x = torch.randn(512, 256, device=dev).to(torch.bfloat16)
    outs = []
    for seed in (11, 12):
        torch.manual_seed(seed)
        moe = MoE(8, 2, 256, 128, ActivationType.SWIGLU, False, 0.02).to(device=dev, dtype=torch.bfloat16)
        with torch.no_grad(), enable_fp8_forward():
            cached, _ = moe(x)
            with cache_quantized_weights(False):
                fresh, _ = moe(x)
        assert torch.equal(cached, fresh), seed
        outs.append(cached)
        del moe
        gc.collect()
    assert not torch.equal(outs[0], outs[1])


def test_weights_in_another_physical_layout_are_requantised_every_call(dev):
    """Expert weights stored physically as (out, in, E) have to be copied into (E, out, in) order before quantising:
    the copy is a new tensor every call and must never be served from the cache after an in-place update."""
    from sonicmoe.functional import fp8

    E, N, K = 4, 128, 256
    g = torch.Generator().manual_seed(21)
    w_phys = torch.randn(N, K, E, generator=g).to(torch.bfloat16).to(dev)   # the (out, in, E) "view" IS the storage
    q0, s0 = fp8.quantize_expert_weight(w_phys)
    w_phys.mul_(3.0)
    q1, s1 = fp8.quantize_expert_weight(w_phys)
    q_ref, s_ref = fp8.mx_quantize(w_phys.permute(2, 0, 1).contiguous().reshape(E * N, K))
    assert torch.equal(q1, q_ref) and torch.equal(s1, s_ref)
    assert not (torch.equal(q0, q1) and torch.equal(s0, s1))
