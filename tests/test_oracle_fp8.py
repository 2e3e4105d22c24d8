"""Pins the fp8 side of the oracle (format only: the reference has no fp8 path, parity against it is unpinned).

Every check is against something the oracle does not compute itself: torch's own float8_e4m3fn decoding and casting,
and the inequalities that define a block scale."""

import numpy as np
import torch

from oracle import fp8 as Q


def test_decode_table_matches_torch_float8():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    got = Q.e4m3_table()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(got[ok].astype(np.float32), ref[ok])
    assert np.nanmax(got) == Q.E4M3_MAX


def test_quantised_elements_match_torch_cast_and_scales_are_tight():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 256, generator=g) * torch.logspace(-6, 4, 64)[:, None]
    x[3, 32:64] = 0.0                      # an all-zero block
    x[5, 0] = 448.0 * 2.0**3               # amax exactly at the top of a binade of scales
    x[6, :32] = torch.linspace(-1.75, 1.75, 32)  # includes exact ties between neighbouring codes
    x = x.to(torch.bfloat16).float()       # the kernels quantise bf16 inputs
    codes, ex = Q.mx_quantize(x)
    scale = torch.from_numpy(2.0 ** (ex.numpy().astype(np.float64) - 127)).float()
    blocks = x.reshape(64, 8, 32)
    amax = blocks.abs().amax(-1)
    nz = amax > 0
    ratio = (amax / scale)[nz]
    assert bool((ratio <= 448.0).all()) and bool((ratio > 224.0).all())  # smallest power of two that avoids saturation
    assert bool((ex[~nz] == 0).all())
    # elements: torch's own cast of the scaled values (round to nearest even)
    ref = (blocks / scale[:, :, None]).to(torch.float8_e4m3fn).view(torch.uint8).reshape(64, 256)
    same = codes == ref
    zero = (codes & 0x7F) == 0  # +0 and -0 are the same value
    assert bool((same | (zero & ((ref & 0x7F) == 0))).all())
    # round trip error bound: half a unit in the last place of a 3-bit mantissa, relative to the block's amax
    back = Q.mx_dequantize(codes, ex).reshape(64, 8, 32)
    assert bool(((back - blocks).abs() <= amax[:, :, None] / 16 + 1e-30).all())


def test_scale_table_layout():
    ex = torch.arange(2 * 8, dtype=torch.uint8).reshape(2, 8) + 100  # 2 rows, 8 blocks = 2 groups of 128 elements
    words = Q.pack_scales(ex)
    assert words.shape == (2, 2) and words.dtype == torch.int32      # (groups, rows)
    w = words.numpy().view(np.uint32)
    for r in range(2):
        for grp in range(2):
            for b in range(4):
                assert (int(w[grp, r]) >> (8 * b)) & 0xFF == int(ex[r, 4 * grp + b])


def test_one_quantised_gemm_stays_inside_the_fp8_tolerance():
    """The per-operator error of the format: a GEMM of two fake-quantised operands against the unquantised one."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(256, 512, generator=g)
    w = torch.randn(128, 512, generator=g) * 0.02
    ref = x @ w.t()
    got = Q.fake_quant(x) @ Q.fake_quant(w).t()
    rel = float((got - ref).norm() / ref.norm())
    assert 0.02 < rel < 0.05, rel
