"""Token-rounding router restated with explicit per-expert loops (numpy).  TEST INFRASTRUCTURE ONLY.

Follows benchmarks/moe-token-rounding.py:139-191 of the reference step by step; the dense (T, E) argsort of the
reference becomes a per-expert sort here.  Ties in the ranking value are outside the contract (the reference's argsort
is not stable); callers use tie-free inputs.
"""

from __future__ import annotations

import numpy as np

from .routing import round_half_even_multiple


def token_choice_rounding(probs: np.ndarray, K: int, tile: int, mode: str, rnd=None):
    """`probs` (T, E) float32: softmax probabilities already rounded to the activation dtype (:149).
    `rnd` rounds a float32 array to the activation dtype (the reference's tensors are in that dtype, so the sum of the
    picks, their quotients and `scores - 1` are each rounded to it: :158, :163); None = float32 tensors.
    Returns (scores (TK',), token_idx (TK',) int32 ascending, expert_idx (TK',) int32, rounded counts (E,))."""
    T, E = probs.shape
    rnd = (lambda a: a) if rnd is None else rnd
    p = probs.astype(np.float32).copy()
    top_i = np.argsort(-p, axis=1, kind="stable")[:, :K]  # :152
    top_v = np.take_along_axis(p, top_i, axis=1)
    freq = np.bincount(top_i.reshape(-1), minlength=E).astype(np.int32)  # :154
    top_v = rnd(top_v / rnd(top_v.sum(axis=1, keepdims=True, dtype=np.float32)))  # :158
    np.put_along_axis(p, top_i, top_v, axis=1)  # :160
    rank = rnd(p - np.float32(1.0))  # :162-163
    np.put_along_axis(rank, top_i, top_v, axis=1)  # :164
    target = np.minimum(round_half_even_multiple(freq, tile, mode), T)  # :169-179
    order = np.stack([np.argsort(-rank[:, e], kind="stable") for e in range(E)], axis=1)  # :167, (T, E)
    toks, exps = [], []
    for r in range(T):  # boolean-mask selection enumerates (rank position, expert) row-major: :181-184
        for e in range(E):
            if r < target[e]:
                toks.append(order[r, e])
                exps.append(e)
    tok = np.asarray(toks, dtype=np.int32)
    exp = np.asarray(exps, dtype=np.int32)
    by_token = np.argsort(tok, kind="stable")  # :187-189 (the reference's argsort is unstable: the order of one
    # token's pairs is unspecified there; stable = ascending rank position, then expert)
    tok, exp = tok[by_token], exp[by_token]
    return p[tok, exp], tok, exp, target
