"""Host-side routers that produce inputs for `moe_general_routing_inputs`.

`token_choice_rounding` is the token-rounding router of the reference's benchmark
(benchmarks/moe-token-rounding.py:139-191): token-choice top-K first, then every expert's token count is rounded to a
multiple of the GEMM token tile by dropping its lowest-ranked picks or adding its best non-picked tokens.  Plain torch
on whatever device the logits live on; it runs outside the timed region in the reference as well.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def token_choice_rounding(
    router_logits: torch.Tensor, K: int, tile: int = 128, routing: str = "nr"
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (router_scores (TK',), token_indices (TK',) int32 ascending, expert_indices (TK',) int32).

    routing: 'nr' rounds each expert's count to the nearest multiple of `tile` (half to even), 'up' / 'down' round
    up / down.  Scores are the softmax probabilities, with the K token-choice picks renormalised to sum to 1."""
    T, E = router_logits.shape
    dev, dtype = router_logits.device, router_logits.dtype
    probs = F.softmax(router_logits, dim=-1, dtype=torch.float32).to(dtype)
    top_v, top_i = probs.topk(K, dim=-1)
    freq = torch.bincount(top_i.reshape(-1), minlength=E).to(torch.int32)
    top_v = top_v / top_v.sum(dim=-1, keepdim=True)
    probs = probs.scatter(-1, top_i, top_v)
    # ranking value: token-choice picks keep their (renormalised) score, everything else is pushed below them by -1
    rank_val = (probs - 1).scatter(1, top_i, top_v)
    order = rank_val.argsort(dim=0, descending=True).int()  # (T, E): per expert, tokens best first
    if routing == "down":
        target = freq // tile * tile
    elif routing == "up":
        target = (torch.ceil(freq / tile) * tile).to(torch.int32)
    elif routing == "nr":
        target = torch.round(freq / tile).to(torch.int32) * tile
    else:
        raise NotImplementedError(routing)
    target = target.clamp(max=T)
    keep = torch.arange(T, device=dev, dtype=torch.int32)[:, None] < target[None, :]
    tok = order[keep]
    exp = torch.arange(E, device=dev, dtype=torch.int32)[None, :].expand(T, -1)[keep]
    by_token = tok.argsort(stable=True)
    tok, exp = tok[by_token], exp[by_token]
    return probs[tok.long(), exp.long()].contiguous(), tok.contiguous(), exp.contiguous()
