"""The hand-scheduled tile loop, checked on the host before it ever runs on a GPU: the committed header is what the
generator emits, and a replay of the generated text on a symbolic machine (tests/tile_loop_sim.py) finds every load
inside its buffer, every LDS access inside its ring and ordered by waits and barriers, and every matrix instruction
multiplying the operand elements its accumulator stands for."""

from __future__ import annotations

import numpy as np
import pytest

import tile_loop_sim as sim
from tile_loop_sim import G


def test_header_matches_generator():
    assert G.OUT.read_text() == G.header(), "run python sonic-moe_amd/csrc/gen_tile_loop.py"


def _problem(qmn, S, N, tiles, gather, seed=0, ntok=700, p_pad=0):
    rng = np.random.default_rng(seed)
    K = S * G.BK
    TK = max(t[2] for t in tiles)
    if gather:
        gidx = rng.integers(0, ntok, size=TK).astype(np.int64)
        p_rows = ntok
    else:
        gidx, p_rows = None, TK
    nexp = max(t[0] for t in tiles) + 1
    if qmn:
        q_stride_row, q_stride_e = N + 8, (N + 8) * K  # (E, K, N) with padded rows
    else:
        q_stride_row, q_stride_e = K, N * K + 64 * 8
    assert nexp * q_stride_e * 2 < 2**47
    return sim.Problem(qmn=qmn, S=S, N=N, p_stride=K + p_pad, p_rows=p_rows, q_stride_e=q_stride_e,
                       q_stride_row=q_stride_row, gidx=gidx, tiles=tiles)


# (expert, row0, row_end, n0): full tiles, a ragged last token tile, a one-row tile, the same panel twice
TILES = [(0, 0, 600, 0), (0, 256, 600, 256), (0, 512, 600, 0), (3, 600, 601, 256), (5, 601, 1113, 0), (5, 857, 1113, 0)]


@pytest.mark.parametrize("qmn", [False, True])
@pytest.mark.parametrize("S", [3, 4, 5, 7])
@pytest.mark.parametrize("gather", [False, True])
def test_replay_multi_tile(qmn, S, gather):
    prob = _problem(qmn, S, 512, TILES, gather)
    out = sim.simulate(prob)
    assert out["mfma"] == len(TILES) * G.NW * 64 * 2 * S
    assert out["barriers"] == len(TILES) * (S + 1)


@pytest.mark.parametrize("qmn", [False, True])
def test_replay_single_tile_and_ragged_columns(qmn):
    # one tile only (the streams run on into a repeat of it); N = 320: the second feature tile has 64 valid columns
    sim.simulate(_problem(qmn, 3, 320, [(1, 10, 200, 256)], True, seed=1))
    sim.simulate(_problem(qmn, 6, 320, [(0, 0, 256, 0), (0, 0, 256, 256)], False, seed=2, p_pad=8))


@pytest.mark.parametrize("qmn", [False, True])
def test_replay_rereads_the_last_row_next_to_the_32_bit_limit(qmn):
    # Rows behind an expert's end are normally not fetched (offset = the tensor's end, dropped by the range check).
    # With a token tensor that ends within one stage offset of 4 GiB that offset could wrap around into the tensor, so
    # the kernel re-reads the expert's last row instead: both conventions have to replay clean.
    small = _problem(qmn, 4, 512, TILES, True)
    assert sim.drop_rows(small)
    big = _problem(qmn, 4, 512, TILES, True, ntok=(0xffffffff - 64) // (4 * G.BK * 2))
    assert not sim.drop_rows(big) and sim.p_extent(big) <= 0xffffffff
    sim.simulate(big)


def test_replay_nonzero_lds_base():
    sim.simulate(_problem(False, 4, 256, TILES[:3], True), lds_base=0)


def test_replay_catches_a_missing_wait():
    # the checker must not be vacuous: drop the wait in front of the barrier of the steady-state stage
    lines = G.emit_tile(False)
    idx = [i for i, ln in enumerate(lines) if ln.startswith("s_waitcnt vmcnt(8)")]
    assert idx
    broken = [ln for i, ln in enumerate(lines) if i not in idx]
    orig = sim.asm_lines
    sim.asm_lines = lambda qmn: broken
    try:
        with pytest.raises(sim.SimError):
            sim.simulate(_problem(False, 5, 256, TILES[:2], True))
    finally:
        sim.asm_lines = orig


def test_replay_catches_a_wrong_slot():
    # token operand refilled into the slot that is being read: must be flagged
    lines = [ln.replace(f"s_xor_b32 s{G.S_T0}, s{G.S_T0}, {G.P_STAGE}", f"s_xor_b32 s{G.S_T0}, s{G.S_T0}, 0") for ln in G.emit_tile(False)]
    orig = sim.asm_lines
    sim.asm_lines = lambda qmn: lines
    try:
        with pytest.raises(sim.SimError):
            sim.simulate(_problem(False, 4, 256, TILES[:2], False))
    finally:
        sim.asm_lines = orig


# ---- weight-gradient loop ------------------------------------------------------------------------------------------------
def _problem_mm(gp, experts, NA, NB, seed=0, before=37, after=90, ntok=500, tiles_of=None):
    """experts: row counts; the workgroup walks through one tile of every expert (a0, b0 vary), in order"""
    rng = np.random.default_rng(seed)
    total = before + sum(experts) + after
    gidx = rng.integers(0, ntok, size=total).astype(np.int64)
    tiles, row = [], before
    for i, n in enumerate(experts):
        a0 = (i * 256) % (-(-NA // 256) * 256)
        b0 = ((i + 1) * 256) % (-(-NB // 256) * 256)
        tiles.append((row, row + n, a0, b0))
        row += n
    return sim.ProblemMM(gp=gp, NA=NA, NB=NB, r_stride=NA + (8 if seed & 1 else 0), s_stride=NB, gather_rows=ntok,
                         gidx_flat=gidx, tiles=tiles)


@pytest.mark.parametrize("gp", [False, True])
@pytest.mark.parametrize("rows", [0, 1, 63, 64, 130, 192, 257, 448])
def test_replay_weight_gradient_loop(gp, rows):
    # one expert of 0 .. 7 stages with a ragged last stage, in the middle of the grouped rows
    out = sim.simulate_mm(_problem_mm(gp, [rows], 512, 768, seed=rows))
    assert out["mfma"] == G.NW * 64 * 2 * max(3, -(-rows // 64))


@pytest.mark.parametrize("gp", [False, True])
def test_replay_weight_gradient_stream(gp):
    # a stream of tiles of different experts: long, empty, one row, ragged, exactly three stages, long
    sim.simulate_mm(_problem_mm(gp, [300, 0, 1, 130, 192, 450, 64], 512, 768, seed=11))
    sim.simulate_mm(_problem_mm(gp, [192, 192, 0, 0, 200], 768, 512, seed=12, before=0))


@pytest.mark.parametrize("gp", [False, True])
def test_replay_weight_gradient_edges(gp):
    # the last expert ends exactly at the end of the grouped rows (index loads run past the array: range-checked);
    # ragged output tiles in both directions (NA = 320, NB = 448: the last tiles have 64 resp. 192 valid columns)
    sim.simulate_mm(_problem_mm(gp, [100, 70], 320, 448, seed=5, after=0))
    sim.simulate_mm(_problem_mm(gp, [300], 320, 448, seed=6, before=0, after=0))


def test_replay_weight_gradient_catches_missing_fix():
    # without the replacement of indices past the expert's end the next expert's rows would be multiplied in
    orig = G.mm_ragged_fix
    G.mm_ragged_fix = lambda em: [f"s_sub_i32 s{G.MS_RLEFT}, s{G.MS_RLEFT}, {G.BK}"]
    try:
        with pytest.raises(sim.SimError):
            sim.simulate_mm(_problem_mm(False, [100, 100], 512, 512, seed=7))
    finally:
        G.mm_ragged_fix = orig
