"""Host-side routers that produce inputs for `moe_general_routing_inputs`.

`token_choice_rounding` is the token-rounding router of the reference's benchmark
(benchmarks/moe-token-rounding.py:139-191): token-choice top-K first, then every expert's token count is rounded to a
multiple of the GEMM token tile by dropping its lowest-ranked picks or adding its best non-picked tokens.  For 16-bit
logits on the GPU the whole router runs in HIP kernels (a radix select per expert instead of the reference's dense
(T, E) argsort); otherwise it is plain torch on whatever device the logits live on, as in the reference.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from . import _lib
from .count_cumsum import count_cumsum


def token_choice_rounding(
    router_logits: torch.Tensor, K: int, tile: int = 128, routing: str = "nr"
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (router_scores (TK',), token_indices (TK',) int32 ascending, expert_indices (TK',) int32).

    routing: 'nr' rounds each expert's count to the nearest multiple of `tile` (half to even), 'up' / 'down' round
    up / down.  Scores are the softmax probabilities, with the K token-choice picks renormalised to sum to 1."""
    T, E = router_logits.shape
    dev, dtype = router_logits.device, router_logits.dtype
    if router_logits.is_cuda and dtype in (torch.bfloat16, torch.float16) and E <= 4096 and K <= min(E, 64) and T > 0:
        return token_choice_rounding_device(router_logits, K, tile, routing)[:3]
    probs = F.softmax(router_logits, dim=-1, dtype=torch.float32).to(dtype)
    top_v, top_i = probs.topk(K, dim=-1)
    freq = torch.bincount(top_i.reshape(-1), minlength=E).to(torch.int32)
    top_v = top_v / top_v.sum(dim=-1, keepdim=True)
    probs = probs.scatter(-1, top_i, top_v)
    # ranking value: token-choice picks keep their (renormalised) score, everything else is pushed below them by -1
    rank_val = (probs - 1).scatter(1, top_i, top_v)
    order = rank_val.argsort(dim=0, descending=True).int()  # (T, E): per expert, tokens best first
    target = _rounded_counts(freq, tile, routing, T)
    keep = torch.arange(T, device=dev, dtype=torch.int32)[:, None] < target[None, :]
    tok = order[keep]
    exp = torch.arange(E, device=dev, dtype=torch.int32)[None, :].expand(T, -1)[keep]
    by_token = tok.argsort(stable=True)
    tok, exp = tok[by_token], exp[by_token]
    return probs[tok.long(), exp.long()].contiguous(), tok.contiguous(), exp.contiguous()


def _rounded_counts(freq: torch.Tensor, tile: int, routing: str, T: int) -> torch.Tensor:
    if routing == "down":
        target = freq // tile * tile
    elif routing == "up":
        target = (torch.ceil(freq / tile) * tile).to(torch.int32)
    elif routing == "nr":
        target = torch.round(freq / tile).to(torch.int32) * tile
    else:
        raise NotImplementedError(routing)
    return target.clamp(max=T).to(torch.int32)


def token_choice_rounding_device(router_logits: torch.Tensor, K: int, tile: int = 128, routing: str = "nr"):
    """The router above in HIP kernels.  Returns (scores, token_indices, expert_indices, probs) where probs (T, E) is
    the rounded softmax the selection was made from; inside a token the pairs are in ascending expert order (the
    reference leaves that order unspecified)."""
    _lib.require_device(router_logits)
    T, E = router_logits.shape
    dev, dtype = router_logits.device, router_logits.dtype
    code = _lib.DT_CODE[dtype]
    lib, st = _lib.lib(), _lib.current_stream_handle()
    logits = router_logits if router_logits.stride(1) == 1 else router_logits.contiguous()
    probs = torch.empty(T, E, dtype=dtype, device=dev)
    _lib.check(lib.smoe_tr_softmax(_lib.ptr(logits), code, T, E, logits.stride(0), _lib.ptr(probs), st), "tr_softmax")
    softmax_probs = probs.clone()
    top_v = torch.empty(T, K, dtype=torch.float32, device=dev)
    top_i = torch.empty(T, K, dtype=torch.int32, device=dev)
    _lib.check(lib.smoe_topk_softmax_fwd(_lib.ptr(probs), code, T, E, K, E, _lib.ptr(top_v), _lib.ptr(top_i), 0, st),
               "topk")
    freq = count_cumsum(top_i.view(-1), E, do_cumsum=False)
    rank = torch.empty_like(probs)
    _lib.check(lib.smoe_tr_rank(_lib.ptr(probs), _lib.ptr(rank), code, _lib.ptr(top_v), _lib.ptr(top_i), T, E, K, st),
               "tr_rank")
    target = _rounded_counts(freq, tile, routing, T)
    keep = torch.empty(T, E, dtype=torch.uint8, device=dev)
    _lib.check(lib.smoe_tr_select(_lib.ptr(rank), code, _lib.ptr(target), _lib.ptr(keep), T, E, st), "tr_select")
    counts = torch.empty(T, dtype=torch.int32, device=dev)
    _lib.check(lib.smoe_tr_row_counts(_lib.ptr(keep), T, E, _lib.ptr(counts), st), "tr_row_counts")
    tok_off = torch.zeros(T + 1, dtype=torch.int32, device=dev)
    tok_off[1:] = counts.cumsum(0)
    n = int(tok_off[-1])  # the one host synchronisation: the number of routed pairs sizes the outputs
    scores = torch.empty(n, dtype=dtype, device=dev)
    tok = torch.empty(n, dtype=torch.int32, device=dev)
    exp = torch.empty(n, dtype=torch.int32, device=dev)
    _lib.check(lib.smoe_tr_compact(_lib.ptr(keep), _lib.ptr(probs), code, _lib.ptr(tok_off), T, E, _lib.ptr(scores),
                                   _lib.ptr(tok), _lib.ptr(exp), st), "tr_compact")
    return scores, tok, exp, softmax_probs
