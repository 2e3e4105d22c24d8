"""Integer / index side of the hot path, restated with numpy.  TEST INFRASTRUCTURE ONLY.

Every function cites the reference lines it follows (paths relative to the reference tree).
All outputs that the reference defines as integers are produced bit-exactly.
"""

from __future__ import annotations

import numpy as np


def _next_pow2(n: int) -> int:
    p = 1
    while p < n:
        p *= 2
    return p


def topk_softmax(logits_f32: np.ndarray, K: int, softmax: bool = True) -> tuple[np.ndarray, np.ndarray]:
    """Fused top-K + softmax router (sonicmoe/functional/topk_softmax.py:118-174).

    `logits_f32` is the (T, E) logit matrix already widened to float32 (bf16/fp16 logits widen exactly).
    The reference overwrites the low log2(next_pow2(E)) mantissa bits of every fp32 logit with an encoded
    column index (inverted for values >= 0) so that the bitonic top-k orders ties towards the LOWER column
    (:127-142), then clears those bits again before the softmax (:151-161).  For bf16/fp16 logits the low
    16/13 bits are zero, so this is lossless; for fp32 logits values that differ only in those bits tie and
    the softmax sees the truncated value.  Both are reproduced here.

    Returns (scores float32 (T, K), indices int32 (T, K)), ordered by descending value, ties by ascending
    column.  With softmax=False the (bit-cleared) top-K values are returned instead of scores.
    """
    x = np.ascontiguousarray(logits_f32, dtype=np.float32)
    T, E = x.shape
    assert 1 <= K <= E
    mask = np.uint32(_next_pow2(E) - 1)
    bits = x.view(np.uint32)
    col = np.arange(E, dtype=np.uint32)[None, :]
    enc = np.where(x >= 0, ~col, col) & mask
    packed = ((bits & ~mask) | enc).view(np.float32)
    # all packed values of a row are distinct (the column is embedded), so a plain descending sort is the
    # bitonic network's result; NaNs are outside the contract
    order = np.argsort(-packed.astype(np.float64), axis=1, kind="stable")[:, :K]
    top_packed = np.take_along_axis(packed, order, axis=1).view(np.uint32)
    vals = (top_packed & ~mask).view(np.float32)
    e_idx = top_packed & mask
    idx = (np.where(vals >= 0, ~e_idx, e_idx) & mask).astype(np.int32)
    if not softmax:
        return vals, idx
    m = vals.max(axis=1, keepdims=True)
    ex = np.exp((vals - m).astype(np.float32)).astype(np.float32)
    s = np.zeros((T, 1), dtype=np.float32)
    for k in range(K):  # sequential fp32 sum, as in :167-171
        s = (s + ex[:, k : k + 1]).astype(np.float32)
    return (ex / s).astype(np.float32), idx


def count_cumsum(x: np.ndarray, E: int) -> tuple[np.ndarray, np.ndarray]:
    """Expert histogram and INCLUSIVE prefix sum, both int32 (sonicmoe/count_cumsum/kernel.cu:92-145,
    sonicmoe/count_cumsum/__init__.py:16-29)."""
    x = np.asarray(x).reshape(-1)
    count = np.bincount(x.astype(np.int64), minlength=E).astype(np.int32)
    return count, np.cumsum(count, dtype=np.int64).astype(np.int32)


def tc_topk_router_metadata(topk_indices: np.ndarray, E: int):
    """Routing metadata for token-choice top-K (sonicmoe/functional/__init__.py:19-46).

    The reference uses torch.argsort, whose order inside one expert is unspecified; the canonical answer
    (and the one the HIP path produces) is the STABLE sort, i.e. ascending flat slot inside every expert.

    Returns dict with expert_frequency (E,), expert_frequency_offset (E+1,), x_gather_idx, s_scatter_idx,
    s_reverse_scatter_idx (TK,), num_activated_expert_per_token_offset (T+1,) - all int32.
    """
    T, K = topk_indices.shape
    flat = np.asarray(topk_indices).reshape(-1)
    freq, cums = count_cumsum(flat, E)
    s_scatter = np.argsort(flat, kind="stable").astype(np.int32)  # :22
    off = np.concatenate([np.zeros(1, np.int32), cums])  # :23-28
    s_rev = np.empty_like(s_scatter)
    s_rev[s_scatter] = np.arange(T * K, dtype=np.int32)  # :30-33
    tok_off = np.arange(0, T * K + 1, K, dtype=np.int32)  # :35-37
    x_gather = (s_scatter // K).astype(np.int32)  # :38
    return dict(
        expert_frequency=freq,
        expert_frequency_offset=off,
        x_gather_idx=x_gather,
        s_scatter_idx=s_scatter,
        s_reverse_scatter_idx=s_rev,
        num_activated_expert_per_token_offset=tok_off,
    )


def general_routing_router_metadata(sorted_token_idx: np.ndarray, expert_idx: np.ndarray, T: int, E: int):
    """Routing metadata for caller-supplied (token, expert) pairs, tokens sorted ascending
    (sonicmoe/functional/__init__.py:49-82)."""
    tok = np.asarray(sorted_token_idx).reshape(-1)
    exp = np.asarray(expert_idx).reshape(-1)
    TK = tok.shape[0]
    assert exp.shape[0] == TK
    freq, cums = count_cumsum(exp, E)  # :55
    off = np.concatenate([np.zeros(1, np.int32), cums])  # :56
    s_scatter = np.argsort(exp, kind="stable").astype(np.int32)  # :58
    s_rev = np.empty_like(s_scatter)
    s_rev[s_scatter] = np.arange(TK, dtype=np.int32)  # :59-62
    x_gather = tok[s_scatter].astype(np.int32)  # :64
    _, tcum = count_cumsum(tok, T)  # :66-69
    tok_off = np.concatenate([np.zeros(1, np.int32), tcum])  # :71-73
    return dict(
        expert_frequency=freq,
        expert_frequency_offset=off,
        x_gather_idx=x_gather,
        s_scatter_idx=s_scatter,
        s_reverse_scatter_idx=s_rev,
        num_activated_expert_per_token_offset=tok_off,
    )


def softmax_topk_bwd(dscore: np.ndarray, score: np.ndarray, idx: np.ndarray, E: int) -> np.ndarray:
    """dlogits[t, idx[t,k]] = s_k (ds_k - sum_j ds_j s_j), zero elsewhere
    (sonicmoe/functional/backward.py:487-525; caller zero-fills, functional/__init__.py:107)."""
    T, K = score.shape
    g = dscore.astype(np.float32)
    s = score.astype(np.float32)
    dot = (g * s).sum(axis=1, keepdims=True, dtype=np.float32)
    add = s * (g - dot)
    out = np.zeros((T, E), dtype=np.float32)
    np.put_along_axis(out, idx.astype(np.int64), add, axis=1)
    return out


def round_half_even_multiple(freq: np.ndarray, tile: int, mode: str) -> np.ndarray:
    """Per-expert count rounded to a multiple of `tile` (benchmarks/moe-token-rounding.py:155-156, :169-179).
    'nr' uses torch.round = round-half-to-even on freq/tile (float32 division in the reference)."""
    f = freq.astype(np.float32) / np.float32(tile)
    if mode == "up":
        return (np.ceil(f) * tile).astype(np.int32)
    if mode == "down":
        return (freq // tile * tile).astype(np.int32)
    if mode == "nr":
        return np.rint(f).astype(np.int32) * np.int32(tile)
    raise NotImplementedError(mode)
