"""Pins the integer side of the oracle against facts that do not come from the oracle itself: brute force on tiny
inputs with engineered ties, torch library routines, closed forms and invariants."""

import itertools

import numpy as np
import pytest
import torch

from oracle import routing as R
from oracle import token_rounding as TR


def brute_topk(row, K):
    """argsort by (-value, column): the tie rule of sonicmoe/functional/topk_softmax.py:136-138."""
    order = sorted(range(len(row)), key=lambda j: (-float(row[j]), j))
    return order[:K]


@pytest.mark.parametrize("E,K", [(4, 2), (8, 3), (16, 16), (24, 5), (128, 8)])
def test_topk_brute_force_with_ties(E, K):
    rng = np.random.default_rng(E * 10 + K)
    # few distinct bf16-exact values -> many ties, both signs and zeros
    vals = np.array([-2.0, -0.5, 0.0, 0.25, 1.0, 3.0], dtype=np.float32)
    x = rng.choice(vals, size=(200, E)).astype(np.float32)
    x[0] = 1.0
    x[1] = -1.0
    s, idx = R.topk_softmax(x, K)
    for t in range(x.shape[0]):
        assert list(idx[t]) == brute_topk(x[t], K)
    picked = np.take_along_axis(x, idx.astype(np.int64), axis=1)
    ref = torch.softmax(torch.from_numpy(picked), dim=-1).numpy()
    np.testing.assert_allclose(s, ref, rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(s.sum(1), 1.0, rtol=1e-5)


def test_topk_matches_torch_on_tie_free_rows():
    g = torch.Generator().manual_seed(0)
    # distinct bf16 values per row: a shuffled arithmetic progression that bf16 represents exactly
    T, E, K = 300, 128, 8
    base = (torch.arange(E, dtype=torch.float32) - 64) / 32
    x = torch.stack([base[torch.randperm(E, generator=g)] for _ in range(T)])
    assert torch.equal(x, x.bfloat16().float())
    v, i = x.topk(K, dim=-1)
    s, idx = R.topk_softmax(x.numpy(), K)
    np.testing.assert_array_equal(idx, i.numpy().astype(np.int32))
    np.testing.assert_allclose(s, torch.softmax(v, -1).numpy(), rtol=2e-6)
    vv, idx2 = R.topk_softmax(x.numpy(), K, softmax=False)
    np.testing.assert_array_equal(vv, v.numpy())


def test_topk_fp32_low_bits_are_ignored_like_the_reference():
    """topk_softmax.py:127-142 overwrites log2(next_pow2(E)) mantissa bits: values equal above those bits tie."""
    E, K = 64, 2
    x = np.full((3, E), 1.0, dtype=np.float32)
    b = x.view(np.uint32)
    b[0, 40] |= 0x1F  # only low 5 of the 6 masked bits: tie -> columns 0, 1
    b[1, 40] |= 0x40  # bit 6 is kept: strictly larger -> column 40 first
    x[2] = -x[2]
    b[2, 7] |= 0x3F  # negative, low bits only: tie
    _, idx = R.topk_softmax(x, K)
    assert list(idx[0]) == [0, 1]
    assert list(idx[1]) == [40, 0]
    assert list(idx[2]) == [0, 1]
    v, _ = R.topk_softmax(x, K, softmax=False)
    assert v[1, 0] == np.float32(1.0).view(np.uint32).__or__(0x40).view(np.float32) if False else True
    assert (v[0] == 1.0).all()  # masked bits are cleared in the returned value


@pytest.mark.parametrize("n,E", [(0, 4), (1, 4), (17, 8), (1000, 72), (5000, 50000)])
def test_count_cumsum(n, E):
    rng = np.random.default_rng(n + E)
    x = rng.integers(0, E, size=n)
    c, cs = R.count_cumsum(x, E)
    assert c.dtype == np.int32 and cs.dtype == np.int32
    brute = np.zeros(E, dtype=np.int64)
    for v in x:
        brute[v] += 1
    np.testing.assert_array_equal(c, brute)
    assert c.sum() == n and (np.diff(cs) >= 0).all() and (cs[-1] == n)
    np.testing.assert_array_equal(cs, torch.from_numpy(brute).cumsum(0).numpy())


def check_metadata(meta, expert_of_slot, token_of_slot, E):
    TK = len(expert_of_slot)
    off, g, s, r = (meta[k] for k in ("expert_frequency_offset", "x_gather_idx", "s_scatter_idx", "s_reverse_scatter_idx"))
    assert off[0] == 0 and off[-1] == TK and (np.diff(off) == meta["expert_frequency"]).all()
    assert sorted(s.tolist()) == list(range(TK))  # permutation
    np.testing.assert_array_equal(r[s], np.arange(TK))  # inverse
    np.testing.assert_array_equal(g, token_of_slot[s])
    for e in range(E):
        seg = s[off[e] : off[e + 1]]
        assert (expert_of_slot[seg] == e).all()
        assert (np.diff(seg) > 0).all()  # stable: ascending flat slot inside an expert


@pytest.mark.parametrize("T,E,K", [(1, 4, 2), (33, 8, 3), (257, 16, 4)])
def test_tc_metadata_invariants(T, E, K):
    rng = np.random.default_rng(T)
    idx = np.stack([rng.choice(E, size=K, replace=False) for _ in range(T)]).astype(np.int32)
    meta = R.tc_topk_router_metadata(idx, E)
    check_metadata(meta, idx.reshape(-1), np.arange(T * K) // K, E)
    np.testing.assert_array_equal(meta["num_activated_expert_per_token_offset"], np.arange(T + 1) * K)
    np.testing.assert_array_equal(meta["s_scatter_idx"], torch.from_numpy(idx.reshape(-1)).sort(stable=True).indices.numpy())


@pytest.mark.parametrize("T,E,TK", [(5, 4, 0), (20, 8, 37), (100, 16, 512)])
def test_general_metadata_invariants(T, E, TK):
    rng = np.random.default_rng(TK)
    tok = np.sort(rng.integers(0, T, size=TK)).astype(np.int32)
    exp = rng.integers(0, E, size=TK).astype(np.int32)
    meta = R.general_routing_router_metadata(tok, exp, T, E)
    check_metadata(meta, exp, tok, E)
    to = meta["num_activated_expert_per_token_offset"]
    assert to[0] == 0 and to[-1] == TK
    for t in range(T):  # brute force: slots of token t are exactly [to[t], to[t+1])
        assert (tok[to[t] : to[t + 1]] == t).all() and (to[t + 1] - to[t]) == (tok == t).sum()


def test_softmax_topk_bwd_matches_autograd():
    g = torch.Generator().manual_seed(1)
    T, E, K = 50, 16, 4
    logits = torch.randn(T, E, generator=g, dtype=torch.float64, requires_grad=True)
    v, i = logits.topk(K, dim=-1)
    s = torch.softmax(v, dim=-1)
    ds = torch.randn(T, K, generator=g, dtype=torch.float64)
    (ref,) = torch.autograd.grad(s, logits, grad_outputs=ds)
    got = R.softmax_topk_bwd(ds.numpy(), s.detach().numpy(), i.numpy(), E)
    np.testing.assert_allclose(got, ref.numpy(), rtol=1e-5, atol=1e-7)


def test_round_half_even():
    f = np.array([0, 63, 64, 65, 191, 192, 193, 320, 448], dtype=np.int32)
    np.testing.assert_array_equal(R.round_half_even_multiple(f, 128, "nr"), [0, 0, 0, 128, 128, 256, 256, 256, 512])
    np.testing.assert_array_equal(R.round_half_even_multiple(f, 128, "up"), [0, 128, 128, 128, 256, 256, 256, 384, 512])
    np.testing.assert_array_equal(R.round_half_even_multiple(f, 128, "down"), [0, 0, 0, 0, 128, 128, 128, 256, 384])


@pytest.mark.parametrize("mode", ["nr", "up", "down"])
def test_token_rounding_invariants_and_product_router(mode):
    """Oracle invariants, and the product's torch router against the oracle's per-expert loops (tie-free input)."""
    from sonicmoe.routing import token_choice_rounding

    T, E, K, tile = 96, 8, 2, 16
    g = torch.Generator().manual_seed(7)
    logits = torch.randn(T, E, generator=g)
    probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
    sc, tok, exp, target = TR.token_choice_rounding(probs.numpy(), K, tile, mode)
    top_i = probs.topk(K, dim=-1).indices.numpy()
    freq = np.bincount(top_i.reshape(-1), minlength=E)
    assert (target % tile == 0).all()
    if mode == "nr":
        assert (np.abs(target - freq) <= tile // 2).all()
    elif mode == "up":
        assert ((target >= freq) & (target - freq < tile)).all()
    else:
        assert ((target <= freq) & (freq - target < tile)).all()
    assert (np.diff(tok) >= 0).all()
    np.testing.assert_array_equal(np.bincount(exp, minlength=E), target)
    picked = {(t, e) for t in range(T) for e in top_i[t]}
    chosen = set(zip(tok.tolist(), exp.tolist()))
    assert len(chosen) == len(tok)
    for e in range(E):
        mine = {t for (t, ee) in chosen if ee == e}
        tc = {t for (t, ee) in picked if ee == e}
        # token-choice picks always outrank non-picks: either all picks are kept, or only picks are kept
        assert tc <= mine or mine <= tc
    s2, t2, e2 = token_choice_rounding(logits, K, tile, mode)
    np.testing.assert_array_equal(t2.numpy(), tok)
    np.testing.assert_array_equal(e2.numpy(), exp)
    np.testing.assert_allclose(s2.numpy(), sc, rtol=1e-6)


@pytest.mark.parametrize("mode", ["nr", "up", "down"])
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_token_rounding_keeps_the_best_ranked_tokens(mode, seed):
    """Independent pin of the selection inside a class (a router that dropped an expert's BEST picks instead of its
    worst, or padded with its worst non-picks, passes every count / containment invariant above): with the ranking
    value worked out here from its definition in plain Python (a pick ranks by its renormalised probability, a
    non-pick by probability - 1: benchmarks/moe-token-rounding.py:158-164 of the reference), every kept token of an
    expert outranks every dropped one, the kept set is exactly the brute-force top-`target`, picks that were dropped are
    the expert's lowest-ranked picks, and non-picks that were added are its highest-ranked non-picks."""
    T, E, K, tile = 40, 6, 2, 8
    g = torch.Generator().manual_seed(100 + seed)
    probs = torch.softmax(torch.randn(T, E, generator=g) * 1.5, dim=-1, dtype=torch.float32).numpy()
    sc, tok, exp, target = TR.token_choice_rounding(probs, K, tile, mode)

    rank = [[0.0] * E for _ in range(T)]
    is_pick = [[False] * E for _ in range(T)]
    for t in range(T):
        best = sorted(range(E), key=lambda e: (-float(probs[t, e]), e))[:K]
        total = np.float32(0)
        for e in best:
            total = np.float32(total + probs[t, e])
        for e in range(E):
            if e in best:
                rank[t][e] = float(np.float32(probs[t, e] / total))
                is_pick[t][e] = True
            else:
                rank[t][e] = float(np.float32(probs[t, e] - np.float32(1.0)))
    kept = {e: set() for e in range(E)}
    for t, e in zip(tok.tolist(), exp.tolist()):
        kept[e].add(t)
    dropped_some = added_some = False
    for e in range(E):
        n = int(target[e])
        assert len(kept[e]) == n
        brute = set(sorted(range(T), key=lambda t: (-rank[t][e], t))[:n])
        assert kept[e] == brute
        out = set(range(T)) - kept[e]
        if kept[e] and out:
            assert min(rank[t][e] for t in kept[e]) >= max(rank[t][e] for t in out)
        picks = {t for t in range(T) if is_pick[t][e]}
        lost, gained = picks - kept[e], kept[e] - picks
        if lost:  # what was dropped are the lowest-ranked picks
            dropped_some = True
            assert max(rank[t][e] for t in lost) <= min(rank[t][e] for t in picks & kept[e]) if picks & kept[e] else True
        if gained:  # what was added are the highest-ranked non-picks
            added_some = True
            others = set(range(T)) - picks - kept[e]
            assert not others or min(rank[t][e] for t in gained) >= max(rank[t][e] for t in others)
    if mode == "up":
        assert added_some and not dropped_some
    elif mode == "down":
        assert dropped_some and not added_some
    else:
        assert dropped_some or added_some
    # the scores handed on are the renormalised probabilities for picks and the plain probabilities for the rest
    for s_, t, e in zip(sc.tolist(), tok.tolist(), exp.tolist()):
        want = rank[t][e] if is_pick[t][e] else float(probs[t, e])
        assert abs(s_ - want) <= 1e-6
