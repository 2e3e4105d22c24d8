"""Generator of the hand-scheduled main loop of the grouped GEMMs (gfx950, one wavefront per SIMD).

    python sonic-moe_amd/csrc/gen_tile_loop.py            # rewrites csrc/tile_loop_gen.h

The loop is ONE inline-assembly statement per output tile: every matrix instruction, LDS fragment read, direct-to-LDS
load, wait and barrier of a 256 x 256 tile's contraction is placed here, in program order, for a workgroup of four
wavefronts (2 x 2 wave tiles of 128 tokens x 128 features, 256 accumulator registers in a[0:255]).  The C++ kernel
around it (varlen_m_asm_kernel in gemm_varlen_m.hip) owns everything that happens once per tile: which tile, the
per-lane source offsets, the epilogue.

Pipeline (stage = 64 of the contraction = two k-slices of 32; token operand P: ring of 2 LDS slots, weight operand Q:
ring of 3):

    entry    barrier (the epilogue of the previous tile parked rows in the two vacated slots); request the next stage of
             either stream into those slots; read k-slice 0 of stage 0 into fragment set A
    stage s  k-slice 0: 64 MFMAs on set A; between them the reads of k-slice 1 into set B, then the LDS addresses of
                        stage s+1
             wait until this wave's loads of stage s+1 have landed (vmcnt) and its reads have returned (lgkmcnt);
             barrier: stage s+1 is complete in LDS and nobody reads the slots of stage s any more
             k-slice 1: 64 MFMAs on set B; between them the reads of (s+1, k-slice 0) into set A and the loads
                        P(s+2), Q(s+3) into the slots stage s has just vacated
    last     k-slice 1 has nothing to read or request: the next tile's first stages were requested earlier (the streams
             run across tile boundaries), its slots are left to the epilogue

A stream that has requested the tile's last stage moves on to the next tile's offsets (pvn / qvn / next expert base).

Everything about register numbers and LDS geometry the C++ side needs is emitted into the header as constants and as
the operand list of the statement, so the two cannot drift apart; tests/test_tile_loop_gen.py replays the address
arithmetic of this file on the host and checks the committed header against the generator.
"""

from __future__ import annotations

import sys
from pathlib import Path

# ---- geometry (must match Cfg<256, 256, 2, 2, QMN, 64> in gemm_varlen_m.hip) ------------------------------------------
BM = BN = 256
BK = 64
NW = 4
TM = TN = 128
FR = 16  # v_mfma_f32_16x16x32_bf16
KSTEP = 32
FM = TM // FR
FN = TN // FR
P_STAGE = BM * BK * 2
Q_STAGE = BN * BK * 2
P_SLOTS, Q_SLOTS = 2, 3
P_INSTR = P_STAGE // 1024 // NW
Q_INSTR = Q_STAGE // 1024 // NW
KROW = BK * 2  # bytes per row of a K-major stage
ROWB = BN * 2  # bytes per contraction row of an MN-major stage

# ---- register map -----------------------------------------------------------------------------------------------------
# accumulators: fragment (fn, fm) = a[4 * (fn * FM + fm) .. + 3]
def acc_reg(fn: int, fm: int) -> int:
    return 4 * (fn * FM + fm)


V_SET = (0, 64)  # fragment sets A, B: 8 weight fragments of 4 registers, then 8 token fragments
V_PV, V_QV, V_PVN, V_QVN = 128, 136, 144, 152  # per-lane source offsets of the two streams: current tile, next tile
V_POFF = 160  # p_off[2]: fragment read offsets inside a slot, k-slice 0 / 1
V_QOFF = 162  # K-major: q_off[2]; MN-major: q_off[16] (fragment fn, half h -> 2 * fn + h)
V_PRA = 178  # read addresses of the stage being read (offset + slot), same shapes
V_QRA = 180
V_LAST = 195

S_PRSRC, S_QRSRC, S_QNB = 40, 44, 48
S_PSOFF, S_QSOFF, S_PEND, S_QEND, S_QSTEP, S_NMID = 50, 51, 52, 53, 54, 55
S_PFILL, S_QFILL, S_LDSP, S_LDSQ, S_WLDS = 56, 57, 58, 59, 60
S_PCUR, S_QCUR, S_PFW, S_QFW, S_CNT, S_T0, S_QFWN = 61, 62, 63, 64, 65, 66, 67
S_LAST = 67


def qfrag(setno: int, q: int) -> int:
    return V_SET[setno] + 4 * q


def pfrag(setno: int, p: int) -> int:
    return V_SET[setno] + 32 + 4 * p


class Emitter:
    def __init__(self) -> None:
        self.lines: list[str] = []
        self.nlabel = 0

    def __call__(self, s: str) -> None:
        self.lines.append(s)

    def label(self, stem: str) -> str:
        self.nlabel += 1
        return f"L{stem}{self.nlabel}_%="


def fragment_order(idx: int) -> tuple[int, int]:
    """The idx-th matrix instruction of a k-slice works on fragment (fn, fm).  Two weight fragments at a time, zigzag over
    the token fragments, every other pair backwards: consecutive instructions always share one operand fragment.
    Measured against weight-fragment-major order: 1.3 % of the kernels (2 x 2 blocks 0.9 %, a Hilbert curve 1.2 %, 4 x 4
    blocks slower); the instruction reads its operands from the register file either way, so this is power, not issue."""
    pair, w = idx // (2 * FM), idx % (2 * FM)
    fm = w // 2
    fn = 2 * pair + ((w % 2) ^ (fm & 1))
    if pair & 1:
        fm = FM - 1 - fm
    return fn, fm


def mfma(setno: int, idx: int, fresh: bool) -> str:
    fn, fm = fragment_order(idx)
    a = acc_reg(fn, fm)
    q, p = qfrag(setno, fn), pfrag(setno, fm)
    c = "0" if fresh else f"a[{a}:{a + 3}]"
    return f"v_mfma_f32_16x16x32_bf16 a[{a}:{a + 3}], v[{q}:{q + 3}], v[{p}:{p + 3}], {c}"


def fragment_reads(setno: int, ks: int, qmn: bool) -> list[str]:
    """LDS reads of k-slice ks of the stage the read addresses point at, into fragment set setno."""
    out = []
    for q in range(FN):
        r = qfrag(setno, q)
        if not qmn:
            out.append(f"ds_read_b128 v[{r}:{r + 3}], v{V_QRA + ks} offset:{q * FR * KROW}")
        else:
            off = ks * KSTEP * ROWB
            out.append(f"ds_read_b64_tr_b16 v[{r}:{r + 1}], v{V_QRA + 2 * q} offset:{off}")
            out.append(f"ds_read_b64_tr_b16 v[{r + 2}:{r + 3}], v{V_QRA + 2 * q + 1} offset:{off}")
    for p in range(FM):
        r = pfrag(setno, p)
        out.append(f"ds_read_b128 v[{r}:{r + 3}], v{V_PRA + ks} offset:{p * FR * KROW}")
    return out


def n_qoff(qmn: bool) -> int:
    return 2 * FN if qmn else 2


def read_addresses(qmn: bool) -> list[str]:
    """read address = offset inside a slot + LDS address of the slot the stream of stages is on (s_pcur / s_qcur)"""
    out = [f"v_add_u32 v{V_PRA + k}, s{S_PCUR}, v{V_POFF + k}" for k in range(2)]
    out += [f"v_add_u32 v{V_QRA + k}, s{S_QCUR}, v{V_QOFF + k}" for k in range(n_qoff(qmn))]
    return out


def next_slots(qfw: int = S_QFW) -> list[str]:
    """the slots of the current stage become the ones to refill; move on to the slots of the next stage.  qfw: where
    this wave's weight fill address goes (loads into the previous weight slot may still be due: they use S_QFW)"""
    return [
        f"s_add_u32 s{S_PFW}, s{S_PCUR}, s{S_WLDS}",
        f"s_add_u32 s{qfw}, s{S_QCUR}, s{S_WLDS}",
        f"s_mov_b32 s{S_PFILL}, s{S_PCUR}",
        f"s_mov_b32 s{S_QFILL}, s{S_QCUR}",
        # P: two slots, toggle
        f"s_sub_u32 s{S_T0}, s{S_PCUR}, s{S_LDSP}",
        f"s_xor_b32 s{S_T0}, s{S_T0}, {P_STAGE}",
        f"s_add_u32 s{S_PCUR}, s{S_T0}, s{S_LDSP}",
        # Q: three slots, rotate
        f"s_add_u32 s{S_QCUR}, s{S_QCUR}, {Q_STAGE}",
        f"s_sub_u32 s{S_T0}, s{S_QCUR}, s{S_LDSQ}",
        f"s_cmp_ge_u32 s{S_T0}, {Q_SLOTS * Q_STAGE}",
        f"s_cselect_b32 s{S_T0}, {Q_SLOTS * Q_STAGE}, 0",
        f"s_sub_u32 s{S_QCUR}, s{S_QCUR}, s{S_T0}",
    ]


def load_pair(which: str, i: int) -> tuple[str, str]:
    """(set M0, direct-to-LDS load) of this wave's i-th load of a stage of stream `which`"""
    if which == "p":
        return (f"s_add_u32 m0, s{S_PFW}, {i * 1024}",
                f"buffer_load_dwordx4 v{V_PV + i}, s[{S_PRSRC}:{S_PRSRC + 3}], s{S_PSOFF} offen lds")
    return (f"s_add_u32 m0, s{S_QFW}, {i * 1024}",
            f"buffer_load_dwordx4 v{V_QV + i}, s[{S_QRSRC}:{S_QRSRC + 3}], s{S_QSOFF} offen lds")


def advance_stream(em: Emitter, which: str) -> list[str]:
    """a stage of the stream has been requested: move along the contraction; behind the tile's last stage switch to
    the next tile's offsets"""
    lab = em.label("adv")
    if which == "p":
        out = [f"s_add_u32 s{S_PSOFF}, s{S_PSOFF}, {KROW}", f"s_cmp_lg_u32 s{S_PSOFF}, s{S_PEND}",
               f"s_cbranch_scc1 {lab}"]
        out += [f"v_mov_b32 v{V_PV + i}, v{V_PVN + i}" for i in range(P_INSTR)]
        out += [f"s_mov_b32 s{S_PSOFF}, 0", f"{lab}:"]
    else:
        out = [f"s_add_u32 s{S_QSOFF}, s{S_QSOFF}, s{S_QSTEP}", f"s_cmp_lg_u32 s{S_QSOFF}, s{S_QEND}",
               f"s_cbranch_scc1 {lab}"]
        out += [f"v_mov_b32 v{V_QV + i}, v{V_QVN + i}" for i in range(Q_INSTR)]
        out += [f"s_mov_b32 s{S_QRSRC}, s{S_QNB}", f"s_mov_b32 s{S_QRSRC + 1}, s{S_QNB + 1}",
                f"s_mov_b32 s{S_QSOFF}, 0", f"{lab}:"]
    return out


# Placement of the non-matrix instructions of a stage (index = the matrix instruction, 0..63 of a k-slice, they follow).
# Loads issued in bursts are slower than loads issued evenly (measured: the same 16 loads of a stage bunched into the
# first 30 matrix instructions of k-slice 1 cost 5 % of the kernel against loads 4 apart), so they are spread as far as
# the ring allows: the token operand's over the first half of k-slice 1 (its ring has a slot less, so its loads have the
# least time to land), the weight operand's over the rest of k-slice 1 and, Q_TAIL of them, over k-slice 0 of the NEXT
# stage (the slot they fill was vacated at the same barrier; in program order they still follow the token loads, so the
# counted wait is unchanged).
SCHED = dict(
    read_step_kk=2,  # K-major weights: one fragment read per this many matrix instructions
    read_step_km=1,  # MN-major weights (two transpose reads per weight fragment)
    p_first=2,
    p_step=6,
    q_first=50,
    q_step=6,
    q_tail=8,        # weight-operand loads of a stage issued during the next stage's k-slice 0 ...
    q_tail_first=2,  # ... from this matrix instruction on,
    q_tail_step=7,   # ... this far apart
)


def schedule(qmn: bool) -> dict:
    nreads = FM + (2 * FN if qmn else FN)
    rstep = SCHED["read_step_km"] if qmn else SCHED["read_step_kk"]
    k0_reads = [r * rstep for r in range(nreads)]  # reads of k-slice 1
    k1_reads = [r * rstep for r in range(nreads)]
    nt = SCHED["q_tail"]
    p_at = [SCHED["p_first"] + SCHED["p_step"] * i for i in range(P_INSTR)]
    q_at = [SCHED["q_first"] + SCHED["q_step"] * i for i in range(Q_INSTR - nt)]
    q_tail_at = [SCHED["q_tail_first"] + SCHED["q_tail_step"] * i for i in range(nt)]
    # the slot bookkeeping and the read addresses of the next stage follow the last read (the tail loads keep their own
    # copy of the fill address)
    k0_addr = max(k0_reads) + 2
    assert p_at[0] >= 1 and (not q_at or (q_at[0] > p_at[-1] + 1 and q_at[-1] + 2 < 64))
    assert not q_tail_at or q_tail_at[0] >= 1
    assert k0_addr + 4 + n_qoff(qmn) + 2 < 64 and (not q_tail_at or q_tail_at[-1] + 1 < 63)
    return dict(k0_reads=k0_reads, k0_addr=k0_addr, k1_reads=k1_reads, p_at=p_at, q_at=q_at, q_tail_at=q_tail_at)


def emit_kslice(em: Emitter, setno: int, fresh: bool, extras: dict[int, list[str]]) -> None:
    for line in extras.get(-1, []):
        em(line)
    for idx in range(FN * FM):
        em(mfma(setno, idx, fresh))
        for line in extras.get(idx, []):
            em(line)


def add_extra(extras: dict[int, list[str]], at: int, lines: list[str]) -> None:
    extras.setdefault(at, []).extend(lines)


def emit_stage(em: Emitter, qmn: bool, kind: str) -> None:
    """kind: 'first' (accumulators start from zero, stores of the previous epilogue may be outstanding; the entry has
    requested whole stages, so no loads are left over), 'mid', 'last' (requests nothing new)"""
    sch = schedule(qmn)
    nt = len(sch["q_tail_at"])
    # ---- k-slice 0 on set A (its reads were issued during the previous k-slice 1, or at the entry)
    ex: dict[int, list[str]] = {-1: ["s_waitcnt lgkmcnt(0)"]}
    for at, line in zip(sch["k0_reads"], fragment_reads(1, 1, qmn)):
        add_extra(ex, at, [line])
    if kind != "first" and nt:
        # the rest of the weight stage whose first loads went out during the previous k-slice 1
        for j, at in enumerate(sch["q_tail_at"]):
            m0, ld = load_pair("q", Q_INSTR - nt + j)
            add_extra(ex, at - 1, [m0])
            add_extra(ex, at, [ld])
        add_extra(ex, sch["q_tail_at"][-1] + 1, advance_stream(em, "q"))
    if kind != "last":
        # all reads that use the old slots have been issued: derive the next stage's
        slots = next_slots(S_QFWN)
        at = sch["k0_addr"]
        for j in range(0, len(slots), 4):
            add_extra(ex, at, slots[j:j + 4])
            at += 1
        for line in read_addresses(qmn):
            add_extra(ex, at, [line])
            at += 1
    if kind != "last":
        add_extra(ex, FN * FM - 1, [f"s_mov_b32 s{S_QFW}, s{S_QFWN}"])
    emit_kslice(em, 0, kind == "first", ex)
    # stage s+1 has landed (only the weight stage after it may still be on its way); the reads of set B have returned
    em(f"s_waitcnt vmcnt({0 if kind == 'first' else Q_INSTR}) lgkmcnt(0)")
    em("s_barrier")
    # ---- k-slice 1 on set B
    ex = {}
    if kind != "last":
        for at, line in zip(sch["k1_reads"], fragment_reads(0, 0, qmn)):
            add_extra(ex, at, [line])
        for i, at in enumerate(sch["p_at"]):
            m0, ld = load_pair("p", i)
            add_extra(ex, at - 1, [m0])
            add_extra(ex, at, [ld])
        add_extra(ex, sch["p_at"][-1] + 1, advance_stream(em, "p"))
        for i, at in enumerate(sch["q_at"]):
            m0, ld = load_pair("q", i)
            add_extra(ex, at - 1, [m0])
            add_extra(ex, at, [ld])
        if nt == 0:
            add_extra(ex, sch["q_at"][-1] + 1, advance_stream(em, "q"))
    emit_kslice(em, 1, False, ex)


def emit_tile(qmn: bool) -> list[str]:
    em = Emitter()
    # ---- entry: refill the two slots the previous tile's last stage left (the epilogue parked rows there)
    em("s_barrier")
    em(f"s_add_u32 s{S_PFW}, s{S_PFILL}, s{S_WLDS}")
    em(f"s_add_u32 s{S_QFW}, s{S_QFILL}, s{S_WLDS}")
    for which, n in (("p", P_INSTR), ("q", Q_INSTR)):
        for i in range(n):
            m0, ld = load_pair(which, i)
            em(m0)
            em("s_nop 0")
            em(ld)
        for line in advance_stream(em, which):
            em(line)
    # stage 0 sits in the other token slot and in the weight slot after the vacated one
    em(f"s_mov_b32 s{S_PCUR}, s{S_PFILL}")
    em(f"s_mov_b32 s{S_QCUR}, s{S_QFILL}")
    for line in next_slots()[4:]:
        em(line)
    for line in read_addresses(qmn):
        em(line)
    for line in fragment_reads(0, 0, qmn):
        em(line)
    em(f"s_mov_b32 s{S_CNT}, s{S_NMID}")
    em("s_waitcnt lgkmcnt(0)")
    emit_stage(em, qmn, "first")
    top = em.label("stage")
    em(f"{top}:")
    emit_stage(em, qmn, "mid")
    em(f"s_sub_u32 s{S_CNT}, s{S_CNT}, 1")
    em(f"s_cmp_lg_u32 s{S_CNT}, 0")
    em(f"s_cbranch_scc1 {top}")
    emit_stage(em, qmn, "last")
    # the slots of the last stage are the ones the epilogue may use and the next entry refills
    em(f"s_mov_b32 s{S_PFILL}, s{S_PCUR}")
    em(f"s_mov_b32 s{S_QFILL}, s{S_QCUR}")
    # matrix results must not be read by the instructions that follow for 18 cycles
    em("s_nop 15")
    em("s_nop 7")
    return em.lines


# ---- the statement ------------------------------------------------------------------------------------------------------
def vrange(lo: int, n: int) -> str:
    return f"v{lo}" if n == 1 else f"v[{lo}:{lo + n - 1}]"


def srange(lo: int, n: int) -> str:
    return f"s{lo}" if n == 1 else f"s[{lo}:{lo + n - 1}]"


# ======================================================================================================================
# Weight-gradient loop ("MM"): dW[e][a][b] = sum over the expert's token rows m of R[row(m)][a] * S[row(m)][b].
# Both operands are token-major in memory, so both LDS stages are [64 token rows][256 columns] and both fragment kinds
# come from transpose reads.  P = R (output rows a), Q = S (output columns b).  One of the two is gathered through the
# index array (x resp. dout rows), the other is read in place (dz resp. y1s rows of the expert):
#   in place   per-lane byte offset fixed for the tile, the stage is a wave-uniform offset; the buffer resource ends at
#              the expert's last row, so rows past it are dropped by the range check and read as zeros
#   gathered   a wave's 16 token rows of a stage come with one scalar buffer load of 16 indices (range-checked against
#              the index array), requested right behind the previous stage's loads; entries past the expert's end are
#              replaced by -1, whose byte offset wraps to just below 4 GiB: out of range, zeros
# Same pipeline, ring and waits as above.  A tile has at least three stages (shorter experts are padded with stages
# past their end, which read nothing); a stream that has requested its tile's last stage takes over the next tile's
# offsets, extent, first stage and stage count, so the ring runs on across tiles of different length.
MV_PV, MV_QV, MV_PVN, MV_QVN = 128, 136, 144, 152  # in place: per-lane byte offsets of the 8 loads; gathered: column part
MV_PRA, MV_QRA = 160, 176        # 16 + 16 fragment read addresses: slot-relative outside the statement
MV_T, MV_HALF = 192, 194         # two scratch offsets; 1 in the upper half-wave (a load covers two token rows)
MV_LAST = 194
MS_PRSRC, MS_QRSRC, MS_GRSRC = 24, 28, 32
# state (in/out, one 8-tuple): offsets of the two streams, rows left at the next index run, stages left to request in
# the streams' tiles, the slots to refill
MS_ST = 36
MS_PSOFF, MS_QSOFF, MS_RLEFT, MS_PLEFT, MS_QLEFT, MS_PFILL, MS_QFILL = 36, 37, 38, 39, 40, 41, 42
# next tile (in, one 8-tuple): first offsets, extents of the operand read in place, rows at the first index run, stages
MS_NX = 44
MS_PSOFFN, MS_QSOFFN, MS_PEXTN, MS_QEXTN, MS_RLEFTN, MS_SNEXT = 44, 45, 46, 47, 48, 49
# geometry (in, one 8-tuple)
MS_GEO = 52
MS_PSTEP, MS_QSTEP, MS_NMID, MS_LDSP, MS_LDSQ, MS_WLDS = 52, 53, 54, 55, 56, 57
MS_PCUR, MS_QCUR, MS_PFW, MS_QFW, MS_QFWN, MS_CNT, MS_T0, MS_T1, MS_DP, MS_DQ = 60, 61, 62, 63, 64, 65, 66, 67, 68, 69
MS_A0, MS_A1 = 70, 71            # scratch of the gathered operand's address arithmetic
MS_TOK = 72
MS_LAST = MS_TOK + 15
RPW = 2 * P_INSTR  # token rows a wave requests per stage and operand


def mm_regs(which: str):
    if which == "p":
        return dict(v=MV_PV, vn=MV_PVN, rsrc=MS_PRSRC, soff=MS_PSOFF, soffn=MS_PSOFFN, extn=MS_PEXTN, step=MS_PSTEP,
                    fw=MS_PFW, left=MS_PLEFT)
    return dict(v=MV_QV, vn=MV_QVN, rsrc=MS_QRSRC, soff=MS_QSOFF, soffn=MS_QSOFFN, extn=MS_QEXTN, step=MS_QSTEP,
                fw=MS_QFW, left=MS_QLEFT)


def mm_fragment_reads(setno: int, ks: int) -> list[str]:
    out = []
    off = ks * KSTEP * ROWB
    for base, frag, n in ((MV_QRA, qfrag, FN), (MV_PRA, pfrag, FM)):
        for f in range(n):
            r = frag(setno, f)
            out.append(f"ds_read_b64_tr_b16 v[{r}:{r + 1}], v{base + 2 * f} offset:{off}")
            out.append(f"ds_read_b64_tr_b16 v[{r + 2}:{r + 3}], v{base + 2 * f + 1} offset:{off}")
    return out


def mm_next_slots() -> list[str]:
    """as next_slots; leaves the distance to the next stage's slots in MS_DP / MS_DQ for the read addresses"""
    return [
        f"s_add_u32 s{MS_PFW}, s{MS_PCUR}, s{MS_WLDS}",
        f"s_add_u32 s{MS_QFWN}, s{MS_QCUR}, s{MS_WLDS}",
        f"s_mov_b32 s{MS_PFILL}, s{MS_PCUR}",
        f"s_mov_b32 s{MS_QFILL}, s{MS_QCUR}",
        f"s_sub_u32 s{MS_T0}, s{MS_PCUR}, s{MS_LDSP}",
        f"s_xor_b32 s{MS_T0}, s{MS_T0}, {P_STAGE}",
        f"s_add_u32 s{MS_T0}, s{MS_T0}, s{MS_LDSP}",
        f"s_sub_u32 s{MS_DP}, s{MS_T0}, s{MS_PCUR}",
        f"s_mov_b32 s{MS_PCUR}, s{MS_T0}",
        f"s_add_u32 s{MS_T0}, s{MS_QCUR}, {Q_STAGE}",
        f"s_sub_u32 s{MS_T1}, s{MS_T0}, s{MS_LDSQ}",
        f"s_cmp_ge_u32 s{MS_T1}, {Q_SLOTS * Q_STAGE}",
        f"s_cselect_b32 s{MS_T1}, {Q_SLOTS * Q_STAGE}, 0",
        f"s_sub_u32 s{MS_T0}, s{MS_T0}, s{MS_T1}",
        f"s_sub_u32 s{MS_DQ}, s{MS_T0}, s{MS_QCUR}",
        f"s_mov_b32 s{MS_QCUR}, s{MS_T0}",
    ]


def mm_move_read_addresses() -> list[str]:
    out = [f"v_add_u32 v{MV_PRA + k}, s{MS_DP}, v{MV_PRA + k}" for k in range(2 * FM)]
    out += [f"v_add_u32 v{MV_QRA + k}, s{MS_DQ}, v{MV_QRA + k}" for k in range(2 * FN)]
    return out


def mm_ragged_fix(em: Emitter) -> list[str]:
    """index run just arrived: entries for rows past the expert's end become -1; account for the 64 rows of the stage"""
    lab = em.label("run")
    out = [f"s_cmp_ge_i32 s{MS_RLEFT}, {RPW}", f"s_cbranch_scc1 {lab}"]
    for j in range(RPW):
        out += [f"s_cmp_gt_i32 s{MS_RLEFT}, {j}", f"s_cselect_b32 s{MS_TOK + j}, s{MS_TOK + j}, -1"]
    out += [f"{lab}:", f"s_sub_i32 s{MS_RLEFT}, s{MS_RLEFT}, {BK}"]
    return out


def mm_load(which: str, i: int, gathered: bool) -> tuple[list[str], list[str], list[str]]:
    """this wave's i-th load of a stage of stream `which`: what goes two, one and no matrix instructions ahead of it"""
    r = mm_regs(which)
    m0 = f"s_add_u32 m0, s{r['fw']}, {i * 1024}"
    if not gathered:
        return [], [m0], [f"buffer_load_dwordx4 v{r['v'] + i}, s[{r['rsrc']}:{r['rsrc'] + 3}], s{r['soff']} offen lds"]
    vt = MV_T + (i & 1)
    pre2 = [f"s_mul_i32 s{MS_A0}, s{MS_TOK + 2 * i}, s{r['step']}",
            f"s_mul_i32 s{MS_A1}, s{MS_TOK + 2 * i + 1}, s{r['step']}",
            f"s_sub_u32 s{MS_A1}, s{MS_A1}, s{MS_A0}"]
    pre1 = [f"v_mul_lo_u32 v{vt}, v{MV_HALF}, s{MS_A1}",
            f"v_add3_u32 v{vt}, v{vt}, s{MS_A0}, v{r['v'] + i}", m0]
    return pre2, pre1, [f"buffer_load_dwordx4 v{vt}, s[{r['rsrc']}:{r['rsrc'] + 3}], 0 offen lds"]


def mm_after_issue(em: Emitter, which: str, gathered: bool, hand_over: bool = True) -> list[str]:
    """behind a stage's loads: move the stream along the rows; behind the tile's last stage take over the next tile"""
    r = mm_regs(which)
    out = []
    if not gathered:
        out.append(f"s_add_u32 s{r['soff']}, s{r['soff']}, s{r['step']}")
    if hand_over:
        lab = em.label("next")
        out += [f"s_sub_u32 s{r['left']}, s{r['left']}, 1", f"s_cmp_lg_u32 s{r['left']}, 0", f"s_cbranch_scc1 {lab}"]
        out += [f"v_mov_b32 v{r['v'] + i}, v{r['vn'] + i}" for i in range(P_INSTR)]
        out += [f"s_mov_b32 s{r['soff']}, s{r['soffn']}", f"s_mov_b32 s{r['left']}, s{MS_SNEXT}"]
        if gathered:
            out.append(f"s_mov_b32 s{MS_RLEFT}, s{MS_RLEFTN}")
        else:
            out.append(f"s_mov_b32 s{r['rsrc'] + 2}, s{r['extn']}")
        out.append(f"{lab}:")
    return out


def mm_request_run(which: str) -> list[str]:
    """request the 16 indices of the stage the gathered stream loads next.  Scalar loads share a counter with the LDS
    reads and return out of order with them, so the next wait for fragment reads is a wait for this load as well: it is
    issued right BEHIND such a wait, with a whole k-slice to land before the following one."""
    r = mm_regs(which)
    return [f"s_buffer_load_dwordx16 s[{MS_TOK}:{MS_TOK + 15}], s[{MS_GRSRC}:{MS_GRSRC + 3}], s{r['soff']}",
            f"s_add_u32 s{r['soff']}, s{r['soff']}, {4 * BK}"]


def mm_issue_now(em: Emitter, which: str, gathered: bool, hand_over: bool = True) -> None:
    """a whole stage of stream `which` into the slot its fill address names, outside the matrix-instruction stream"""
    if gathered:
        em("s_waitcnt lgkmcnt(0)")
        for ln in mm_ragged_fix(em):
            em(ln)
    for i in range(P_INSTR):
        pre2, pre1, ld = mm_load(which, i, gathered)
        for ln in pre2 + pre1:
            em(ln)
        em("s_nop 0")
        for ln in ld:
            em(ln)
    for ln in mm_after_issue(em, which, gathered, hand_over):
        em(ln)


MM_SCHED = dict(read_step=1, p_first=3, p_step=7, q_tail_first=3, q_tail_step=7)


def mm_emit_stage(em: Emitter, gp: bool, gq: bool, kind: str) -> None:
    rs = MM_SCHED["read_step"]
    nreads = 2 * (FN + FM)
    reads_at = [r * rs for r in range(nreads)]
    p_at = [MM_SCHED["p_first"] + MM_SCHED["p_step"] * i for i in range(P_INSTR)]
    q_at = [MM_SCHED["q_tail_first"] + MM_SCHED["q_tail_step"] * i for i in range(Q_INSTR)]
    assert p_at[0] >= 2 and q_at[0] >= 2 and p_at[-1] + 1 < 63 and q_at[-1] + 1 < 63
    # ---- k-slice 0 on set A
    ex: dict[int, list[str]] = {-1: ["s_waitcnt lgkmcnt(0)"]}
    for at, line in zip(reads_at, mm_fragment_reads(1, 1)):
        add_extra(ex, at, [line])
    if gp:
        # indices of the token-side stage this stage's k-slice 1 requests (the last stage: the next entry's)
        add_extra(ex, -1, mm_request_run("p"))
    if kind != "first":
        # the weight-side stage Q(s+2) goes into the slot the previous stage vacated
        if gq:
            add_extra(ex, -1, mm_ragged_fix(em))
        for j, at in enumerate(q_at):
            pre2, pre1, ld = mm_load("q", j, gq)
            add_extra(ex, at - 2, pre2)
            add_extra(ex, at - 1, pre1)
            add_extra(ex, at, ld)
        add_extra(ex, q_at[-1] + 1, mm_after_issue(em, "q", gq))
    if kind != "last":
        slots = mm_next_slots()
        at = max(reads_at) + 1
        for j in range(0, len(slots), 4):
            add_extra(ex, at, slots[j:j + 4])
            at += 1
        moves = mm_move_read_addresses()
        per = -(-len(moves) // (FN * FM - 1 - at))  # spread over what is left of the k-slice
        for j in range(0, len(moves), per):
            add_extra(ex, at, moves[j:j + per])
            at += 1
        assert at <= FN * FM - 1
        add_extra(ex, FN * FM - 1, [f"s_mov_b32 s{MS_QFW}, s{MS_QFWN}"])
    emit_kslice(em, 0, kind == "first", ex)
    em(f"s_waitcnt vmcnt({0 if kind == 'first' else Q_INSTR}) lgkmcnt(0)")
    em("s_barrier")
    # ---- k-slice 1 on set B
    ex = {}
    if gq:
        # indices of the weight-side stage the next stage's k-slice 0 requests (the last stage: the next entry's)
        add_extra(ex, -1, mm_request_run("q"))
    if kind != "last":
        for at, line in zip(reads_at, mm_fragment_reads(0, 0)):
            add_extra(ex, at, [line])
        if gp:
            add_extra(ex, -1, mm_ragged_fix(em))
        for i, at in enumerate(p_at):
            pre2, pre1, ld = mm_load("p", i, gp)
            add_extra(ex, at - 2, pre2)
            add_extra(ex, at - 1, pre1)
            add_extra(ex, at, ld)
        add_extra(ex, p_at[-1] + 1, mm_after_issue(em, "p", gp))
    emit_kslice(em, 1, False, ex)


def mm_emit_prologue(gp: bool, gq: bool) -> list[str]:
    """before the first statement of a workgroup: P(0) into token slot 1, Q(0), Q(1) into weight slots 1, 2 (the
    statement's entry then requests P(1), Q(2) into the slots 0 / 0 it is told are vacant); leaves the index run of the
    gathered stream's next stage requested and landed"""
    em = Emitter()
    req = lambda which: [em(ln) for ln in mm_request_run(which)]
    if gp:
        req("p")
    em(f"s_add_u32 s{MS_PFW}, s{MS_LDSP}, s{MS_WLDS}")
    em(f"s_add_u32 s{MS_PFW}, s{MS_PFW}, {P_STAGE}")
    mm_issue_now(em, "p", gp, False)
    if gp:
        req("p")
    if gq:
        req("q")
    em(f"s_add_u32 s{MS_QFW}, s{MS_LDSQ}, s{MS_WLDS}")
    em(f"s_add_u32 s{MS_QFW}, s{MS_QFW}, {Q_STAGE}")
    mm_issue_now(em, "q", gq, False)
    if gq:
        req("q")
    em(f"s_add_u32 s{MS_QFW}, s{MS_QFW}, {Q_STAGE}")
    mm_issue_now(em, "q", gq, False)
    if gq:
        req("q")
    em("s_waitcnt vmcnt(0) lgkmcnt(0)")
    return em.lines


def mm_emit_tile(gp: bool, gq: bool) -> list[str]:
    em = Emitter()
    em("s_barrier")
    em(f"s_add_u32 s{MS_PFW}, s{MS_PFILL}, s{MS_WLDS}")
    em(f"s_add_u32 s{MS_QFW}, s{MS_QFILL}, s{MS_WLDS}")
    mm_issue_now(em, "p", gp)
    mm_issue_now(em, "q", gq)
    # stage 0 sits in the other token slot and in the weight slot after the vacated one; the read addresses come in
    # slot-relative and leave slot-relative
    em(f"s_mov_b32 s{MS_PCUR}, s{MS_PFILL}")
    em(f"s_mov_b32 s{MS_QCUR}, s{MS_QFILL}")
    for line in mm_next_slots()[4:]:
        em(line)
    em(f"s_mov_b32 s{MS_DP}, s{MS_PCUR}")
    em(f"s_mov_b32 s{MS_DQ}, s{MS_QCUR}")
    for line in mm_move_read_addresses():
        em(line)
    for line in mm_fragment_reads(0, 0):
        em(line)
    em(f"s_mov_b32 s{MS_CNT}, s{MS_NMID}")
    em("s_waitcnt lgkmcnt(0)")
    mm_emit_stage(em, gp, gq, "first")
    top = em.label("stage")
    em(f"{top}:")
    mm_emit_stage(em, gp, gq, "mid")
    em(f"s_sub_u32 s{MS_CNT}, s{MS_CNT}, 1")
    em(f"s_cmp_lg_u32 s{MS_CNT}, 0")
    em(f"s_cbranch_scc1 {top}")
    mm_emit_stage(em, gp, gq, "last")
    em(f"s_mov_b32 s{MS_PFILL}, s{MS_PCUR}")
    em(f"s_mov_b32 s{MS_QFILL}, s{MS_QCUR}")
    em(f"s_sub_u32 s{MS_DP}, 0, s{MS_PCUR}")
    em(f"s_sub_u32 s{MS_DQ}, 0, s{MS_QCUR}")
    for line in mm_move_read_addresses():
        em(line)
    # the index run requested behind the last loads must not land in registers the compiler owns again
    em("s_waitcnt lgkmcnt(0)")
    em("s_nop 15")
    em("s_nop 7")
    return em.lines


def mm_operands():
    outs = [
        (vrange(MV_PRA, 2 * FM), "pra"), (vrange(MV_QRA, 2 * FN), "qra"), (vrange(MV_PV, P_INSTR), "pv"),
        (vrange(MV_QV, Q_INSTR), "qv"), (srange(MS_PRSRC, 4), "prsrc"), (srange(MS_QRSRC, 4), "qrsrc"),
        (srange(MS_ST, 8), "state"),
    ]
    ins = [
        (vrange(MV_PVN, P_INSTR), "pvn"), (vrange(MV_QVN, Q_INSTR), "qvn"), (vrange(MV_HALF, 1), "half"),
        (srange(MS_GRSRC, 4), "grsrc"), (srange(MS_NX, 8), "next"), (srange(MS_GEO, 8), "geo"),
    ]
    return outs, ins


def asm_text(line: str) -> str:
    """An instruction as it stands inside the asm statement's string literals: the matrix instructions take the suffix
    of the library's 16-bit element type (bf16 or f16) from the macro SMOE_ELEM_ASM."""
    return line.replace("v_mfma_f32_16x16x32_bf16", 'v_mfma_f32_16x16x32_" SMOE_ELEM_ASM "')


def mm_statement(name: str, lines: list[str], with_matrix: bool) -> str:
    outs, ins = mm_operands()
    clob = [f"v{i}" for i in range(MV_T, MV_T + 2)]
    if with_matrix:
        clob += [f"v{i}" for i in range(0, 128)] + [f"a{i}" for i in range(256)]
    clob += [f"s{i}" for i in range(MS_PCUR, MS_A1 + 1)] + [f"s{i}" for i in range(MS_TOK, MS_TOK + 16)]
    clob += ["scc", "memory"]
    params = ", ".join(n for _, n in outs + ins)
    body = [f"#define {name}({params}) \\", "  asm volatile( \\"]
    for ln in lines:
        body.append(f'    "{asm_text(ln)}\\n\\t" \\')
    body.append("    : " + ", ".join(f'"+{{{r}}}"({n})' for r, n in outs) + " \\")
    body.append("    : " + ", ".join(f'"{{{r}}}"({n})' for r, n in ins) + " \\")
    cl = [", ".join(f'"{c}"' for c in clob[i:i + 16]) for i in range(0, len(clob), 16)]
    body.append("    : " + ", \\\n      ".join(cl) + ")")
    return "\n".join(body)


def mm_layout_defines() -> list[str]:
    """positions inside the three scalar 8-tuples, for the C++ side"""
    names = dict(PSOFF=MS_PSOFF - MS_ST, QSOFF=MS_QSOFF - MS_ST, RLEFT=MS_RLEFT - MS_ST, PLEFT=MS_PLEFT - MS_ST,
                 QLEFT=MS_QLEFT - MS_ST, PFILL=MS_PFILL - MS_ST, QFILL=MS_QFILL - MS_ST,
                 PSOFFN=MS_PSOFFN - MS_NX, QSOFFN=MS_QSOFFN - MS_NX, PEXTN=MS_PEXTN - MS_NX, QEXTN=MS_QEXTN - MS_NX,
                 RLEFTN=MS_RLEFTN - MS_NX, SNEXT=MS_SNEXT - MS_NX,
                 PSTEP=MS_PSTEP - MS_GEO, QSTEP=MS_QSTEP - MS_GEO, NMID=MS_NMID - MS_GEO, LDSP=MS_LDSP - MS_GEO,
                 LDSQ=MS_LDSQ - MS_GEO, WLDS=MS_WLDS - MS_GEO)
    return [f"#define SMOE_MM_{k} {v}" for k, v in names.items()]


def statement(name: str, qmn: bool) -> str:
    lines = emit_tile(qmn)
    nq = n_qoff(qmn)
    outs = [
        (vrange(V_PV, P_INSTR), "pv"), (vrange(V_QV, Q_INSTR), "qv"), (srange(S_QRSRC, 4), "qrsrc"),
        (srange(S_PSOFF, 1), "psoff"), (srange(S_QSOFF, 1), "qsoff"), (srange(S_PFILL, 1), "pfill"),
        (srange(S_QFILL, 1), "qfill"),
    ]
    ins = [
        (vrange(V_PVN, P_INSTR), "pvn"), (vrange(V_QVN, Q_INSTR), "qvn"), (vrange(V_POFF, 2), "poff"),
        (vrange(V_QOFF, nq), "qoff"), (srange(S_PRSRC, 4), "prsrc"), (srange(S_QNB, 2), "qnb"),
        (srange(S_PEND, 1), "pend"), (srange(S_QEND, 1), "qend"), (srange(S_QSTEP, 1), "qstep"),
        (srange(S_NMID, 1), "nmid"), (srange(S_LDSP, 1), "ldsp"), (srange(S_LDSQ, 1), "ldsq"),
        (srange(S_WLDS, 1), "wlds"),
    ]
    clob = [f"v{i}" for i in range(0, 128)]
    clob += [f"v{i}" for i in range(V_PRA, V_PRA + 2)]
    clob += [f"v{i}" for i in range(V_QRA, V_QRA + nq)]
    clob += [f"a{i}" for i in range(256)]
    clob += [f"s{i}" for i in range(S_PCUR, S_LAST + 1)]
    clob += ["scc", "memory"]
    params = ", ".join(n for _, n in outs + ins)
    body = [f"#define {name}({params}) \\", "  asm volatile( \\"]
    for ln in lines:
        body.append(f'    "{asm_text(ln)}\\n\\t" \\')
    body.append("    : " + ", ".join(f'"+{{{r}}}"({n})' for r, n in outs) + " \\")
    body.append("    : " + ", ".join(f'"{{{r}}}"({n})' for r, n in ins) + " \\")
    # clobber list, a few per line
    cl = [", ".join(f'"{c}"' for c in clob[i:i + 16]) for i in range(0, len(clob), 16)]
    body.append("    : " + ", \\\n      ".join(cl) + ")")
    return "\n".join(body)


def header() -> str:
    parts = [
        "// GENERATED by gen_tile_loop.py - do not edit; regenerate with `python sonic-moe_amd/csrc/gen_tile_loop.py`.",
        "// The hand-scheduled contraction loop of one 256 x 256 output tile for four wavefronts (one per SIMD): see the",
        "// generator for the pipeline.  Operands are bound to fixed registers so that the text can name them.",
        "#pragma once",
        f"#define SMOE_TL_FM {FM}",
        f"#define SMOE_TL_FN {FN}",
        f"#define SMOE_TL_P_INSTR {P_INSTR}",
        f"#define SMOE_TL_Q_INSTR {Q_INSTR}",
        "// accumulator fragment (fn, fm) lives in a[SMOE_TL_ACC(fn, fm) .. + 3]",
        f"#define SMOE_TL_ACC(fn, fm) (4 * ((fn) * {FM} + (fm)))",
        "",
        statement("SMOE_TILE_LOOP_KK", False),
        "",
        statement("SMOE_TILE_LOOP_KM", True),
        "",
        "// weight-gradient loop: token operand in place, weight-side operand gathered (dW1) and the other way round (dW2);",
        "// state / next / geo are 8-tuples of scalars, SMOE_MM_* name their elements",
        *mm_layout_defines(),
        mm_statement("SMOE_TILE_PROLOGUE_MM_QG", mm_emit_prologue(False, True), False),
        "",
        mm_statement("SMOE_TILE_LOOP_MM_QG", mm_emit_tile(False, True), True),
        "",
        mm_statement("SMOE_TILE_PROLOGUE_MM_PG", mm_emit_prologue(True, False), False),
        "",
        mm_statement("SMOE_TILE_LOOP_MM_PG", mm_emit_tile(True, False), True),
        "",
    ]
    return "\n".join(parts)


OUT = Path(__file__).resolve().parent / "tile_loop_gen.h"

if __name__ == "__main__":
    text = header()
    if len(sys.argv) > 1 and sys.argv[1] == "--check":
        sys.exit(0 if OUT.exists() and OUT.read_text() == text else 1)
    OUT.write_text(text)
    print(OUT, len(text.splitlines()), "lines")
