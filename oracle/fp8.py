"""CPU restatement of the fp8 path (block-scaled OCP e4m3).  TEST INFRASTRUCTURE ONLY.

PARITY UNPINNED against the reference: the reference (sonicmoe/functional/*.py) computes in bf16 only and holds no fp8
code, test or number.  What is pinned here is the format, not a reference behaviour:

  e4m3_table        pinned: every one of the 256 codes against torch.float8_e4m3fn's own decoding
  mx_quantize       pinned: elements against torch's float -> float8_e4m3fn cast of x / scale (round to nearest even);
                    scales against their defining inequalities (power of two, amax / scale in (224, 448])
  *_forward_fp8,    the operator restatements of oracle.moe_math evaluated on the de-quantised operands: the product
  *_backward_fp8    kernels must match THESE tightly (same operands, fp32 accumulation), and the unquantised oracle
                    within the fp8 tolerance

Format: along the contraction dimension every 32 consecutive elements share one power-of-two scale 2^(byte - 127);
elements are e4m3 (1 sign, 4 exponent bits with bias 7, 3 mantissa bits, no infinities, 0x7f / 0xff = NaN, max 448).
"""

from __future__ import annotations

import numpy as np
import torch

from . import moe_math as M

BLOCK = 32
E4M3_MAX = 448.0


def e4m3_table() -> np.ndarray:
    """Value of each of the 256 e4m3 codes (NaN for 0x7f and 0xff)."""
    out = np.empty(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        ex, man = (code >> 3) & 15, code & 7
        if ex == 15 and man == 7:
            out[code] = np.nan
        elif ex == 0:
            out[code] = sign * man * 2.0**-9
        else:
            out[code] = sign * (1 + man / 8.0) * 2.0 ** (ex - 7)
    return out


def _round_to_e4m3(v: np.ndarray) -> np.ndarray:
    """Nearest e4m3 code of each |v| <= 448 (ties to the even mantissa), by search over the 127 non-negative codes."""
    table = e4m3_table()[:127]  # codes 0x00..0x7e, ascending
    a = np.abs(v).astype(np.float64)
    hi = np.searchsorted(table, a, side="left").clip(1, 126)
    lo = hi - 1
    dlo, dhi = a - table[lo], table[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo)
    code = np.where(a == 0, 0, code)
    return (code | np.where(np.signbit(v), 0x80, 0)).astype(np.uint8)


def mx_scale_exponent(amax: np.ndarray) -> np.ndarray:
    """Biased exponent byte of the smallest power of two s with amax / s <= 448; 0 for an all-zero block."""
    amax = amax.astype(np.float64)
    with np.errstate(divide="ignore"):
        k = np.ceil(np.log2(amax / E4M3_MAX))
    k = np.where(amax > 0, k, -127)
    # log2 can be off by one ulp at exact powers: fix up with the defining inequality
    k = np.where((amax > 0) & (amax / 2.0**k > E4M3_MAX), k + 1, k)
    k = np.where((amax > 0) & (amax / 2.0 ** (k - 1) <= E4M3_MAX), k - 1, k)
    return np.clip(k + 127, 0, 254).astype(np.uint8)


def mx_quantize(x: torch.Tensor):
    """x (R, C), C % 32 == 0 -> (codes uint8 (R, C), exponent bytes uint8 (R, C/32))."""
    a = x.detach().float().cpu().numpy().astype(np.float64)
    R, C = a.shape
    blocks = a.reshape(R, C // BLOCK, BLOCK)
    ex = mx_scale_exponent(np.abs(blocks).max(axis=2))
    scaled = blocks / (2.0 ** (ex.astype(np.float64) - 127))[:, :, None]
    return torch.from_numpy(_round_to_e4m3(scaled).reshape(R, C)), torch.from_numpy(ex)


def mx_dequantize(codes: torch.Tensor, ex: torch.Tensor) -> torch.Tensor:
    R, C = codes.shape
    vals = e4m3_table()[codes.cpu().numpy()].reshape(R, C // BLOCK, BLOCK)
    vals = vals * (2.0 ** (ex.cpu().numpy().astype(np.float64) - 127))[:, :, None]
    return torch.from_numpy(vals.reshape(R, C)).float()


def pack_scales(ex: torch.Tensor) -> torch.Tensor:
    """(R, C/32) exponent bytes -> the kernels' table (C/128, R) of 32-bit words, byte b = block 4g + b of row r."""
    R, nb = ex.shape
    e = ex.cpu().numpy().astype(np.uint32).reshape(R, nb // 4, 4)
    words = e[:, :, 0] | (e[:, :, 1] << 8) | (e[:, :, 2] << 16) | (e[:, :, 3] << 24)
    return torch.from_numpy(np.ascontiguousarray(words.T).view(np.int32).copy())


def fake_quant(x: torch.Tensor) -> torch.Tensor:
    """Quantise then de-quantise the rows of a 2-D tensor (or of every matrix of a 3-D one)."""
    shape = x.shape
    q, ex = mx_quantize(x.reshape(-1, shape[-1]))
    return mx_dequantize(q, ex).reshape(shape)


def up_projection_forward_fp8(x, w1, off, gidx, b1=None, activation="swiglu"):
    """moe_math.up_projection_forward on the de-quantised x and W1 (contraction along H)."""
    return M.up_projection_forward(fake_quant(x), fake_quant(w1), off.cpu(), gidx.cpu(),
                                   b1=None if b1 is None else b1.cpu(), activation=activation)


def down_projection_forward_fp8(y1, w2, off, b2=None):
    """moe_math.down_projection_forward on the de-quantised y1 and W2 (contraction along I)."""
    return M.down_projection_forward(fake_quant(y1), fake_quant(w2), off.cpu(), b2=None if b2 is None else b2.cpu())


def fake_quant_transposed(w: torch.Tensor) -> torch.Tensor:
    """(E, R, C): every matrix quantised along R (32 consecutive r of a column share a scale), de-quantised, same shape."""
    return fake_quant(w.transpose(1, 2).contiguous()).transpose(1, 2).contiguous()


def down_projection_backward_fp8(dout, z, w2, scores_flat, off, gidx, sidx, activation="swiglu"):
    """The activation-gradient half of moe_math.down_projection_backward with dy1 formed from the de-quantised dout
    (blocks along H) and W2 (blocks along H, i.e. along the rows of each (H, I) matrix).  Returns (dz, y1s, ds)."""
    dz, y1s, ds, _ = M.down_projection_backward(fake_quant(dout), z, fake_quant_transposed(w2), scores_flat, off.cpu(),
                                                gidx.cpu(), sidx.cpu(), activation=activation)
    return dz, y1s, ds


def dx_fp8(dz, w1, off):
    """dx_expanded[m] = dz[m] W1[e] on the de-quantised dz (blocks along its N1 columns) and W1 (blocks along N1, the
    rows of each (N1, H) matrix)."""
    dzq, w1q = fake_quant(dz), fake_quant_transposed(w1)
    out = torch.empty(dz.size(0), w1.size(2))
    o = off.tolist()
    for e in range(w1.size(0)):
        out[o[e]:o[e + 1]] = dzq[o[e]:o[e + 1]] @ w1q[e].float()
    return out
