"""Shared builders for the parity tests: seeded synthetic inputs and routing, on a given device."""

from __future__ import annotations

import numpy as np
import torch

from oracle import routing as R


def make_weights(E, H, I, device, dtype=torch.bfloat16, seed=0, std=0.02):
    g = torch.Generator().manual_seed(seed)
    w1 = (torch.randn(E, 2 * I, H, generator=g) * std).to(dtype).to(device)
    w2 = (torch.randn(E, H, I, generator=g) * std).to(dtype).to(device)
    wr = (torch.randn(E, H, generator=g) * std).to(dtype).to(device)
    return wr, w1, w2


def make_tc_routing(T, E, K, device, seed=0, skew=0.0, empty=()):
    """Random token-choice routing: K distinct experts per token, optional Zipf skew, experts in `empty` never
    chosen.  Returns numpy metadata dict (oracle) and the same tensors on `device`."""
    rng = np.random.default_rng(seed)
    w = 1.0 / np.arange(1, E + 1) ** skew
    for e in empty:
        w[e] = 0.0
    w = w / w.sum()
    idx = np.stack([rng.choice(E, size=K, replace=False, p=w) for _ in range(T)]).astype(np.int32)
    meta = R.tc_topk_router_metadata(idx, E)
    scores = rng.random((T, K), dtype=np.float32) + 0.05
    scores = (scores / scores.sum(1, keepdims=True)).astype(np.float32)
    dev = {k: torch.from_numpy(v).to(device) for k, v in meta.items()}
    return idx, scores, meta, dev


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))
