"""Host-side replay of the hand-scheduled tile loop (sonic-moe_amd/csrc/gen_tile_loop.py).

The generated assembly text is EXECUTED here, instruction by instruction, for the four wavefronts of a workgroup in
lock step between barriers, on a symbolic machine: every 2-byte LDS element and every fragment register half carries
the identity (stream, global element index) of the value a direct-to-LDS load would have put there.  That checks, for
every wave, lane, stage and tile of a run,

  * global side: every load's per-lane byte offset + scalar offset lies inside the buffer extent;
  * LDS side: every load lands in a whole 1 KiB piece of the right ring, every fragment read is aligned and inside LDS;
  * synchronisation: a piece is read only after the load that filled it was waited for by its issuer AND (for other
    waves) a barrier lies in between; a piece is overwritten only after every wave's reads of it have returned and a
    barrier lies in between; all waves execute the same number of barriers;
  * arithmetic: every matrix instruction multiplies exactly the (feature row, k) and (token row, k) elements its
    accumulator fragment stands for, each accumulator sees every k-slice of the tile once, and the first k-slice starts
    from zero.

The driver below restates what the C++ kernel does around the statement (varlen_m_asm_kernel): the first tile's
prologue loads, the per-lane source offsets, the hand-over of the next tile's offsets, the epilogue's use of the two
vacated slots.
"""

from __future__ import annotations

import re
import sys
from dataclasses import dataclass, field
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "sonic-moe_amd" / "csrc"))
import gen_tile_loop as G  # noqa: E402

LDS_BYTES = 160 * 1024
PIECE = 1024
NPIECE = LDS_BYTES // PIECE
P_STREAM, Q_STREAM = 0, 1
ZERO = -3  # identity of a value a range-checked load replaced by zero


def kswz(row):  # kswz<64, 16> of gemm_common.h
    return ((row >> 1) & 7) ^ (((row >> 2) ^ (row >> 3)) & 1)


def mnswz(k):
    return ((k & 3) << 1) ^ ((k >> 3) & 1)


@dataclass
class Problem:
    qmn: bool
    S: int  # stages of 64 along the contraction
    N: int  # accumulator columns
    p_stride: int  # elements per row of the token operand
    p_rows: int
    q_stride_e: int
    q_stride_row: int
    gidx: np.ndarray | None  # grouped row -> token row (None: rows in place)
    tiles: list  # (expert, row0, row_end, n0) this workgroup walks through, in order

    @property
    def K(self):
        return self.S * G.BK


class SimError(AssertionError):
    pass


class Lds:
    def __init__(self):
        self.tag = np.full(LDS_BYTES // 2, -1, dtype=np.int64)
        self.pending = [None] * NPIECE  # wave that has a load into the piece in flight
        self.retire_phase = [-1] * NPIECE
        self.retired_by = [None] * NPIECE
        self.last_read = [[-1] * NPIECE for _ in range(G.NW)]  # phase of each wave's last read of the piece


class Wave:
    def __init__(self, wid, lds, prob):
        self.w = wid
        self.lds = lds
        self.prob = prob
        self.v = np.zeros((256, 64), dtype=np.int64)
        self.vt = np.full((256, 64, 2), -1, dtype=np.int64)  # identities held by fragment registers
        self.s = [0] * 128
        self.m0 = 0
        self.scc = 0
        self.vmq = []  # loads in flight: (piece, tags[512])
        self.reads_out = []  # pieces read whose data has not been waited for
        self.regs_out = set()  # registers such reads will write
        self.phase = 0
        self.nbarrier = 0
        self.mfma_count = 0
        self.acc_seen = {}
        self.tile = None  # (expert, row0, row_end, n0) the matrix instructions work on
        self.ldsp_reg = G.S_LDSP  # register that holds the LDS address of the token operand's ring
        self.rsrc_regs = (G.S_PRSRC, G.S_QRSRC)  # first registers of the two streams' buffer resources
        self.oob_zero = False  # loads beyond the extent write zeros (the weight-gradient loop relies on it)
        self.oob_zero_p = False  # the same for the token stream only: dropped rows of a ragged tile
        self.smem_out = set()  # scalar registers a scalar load in flight will write
        self.expect = None  # callable(wave, fn, fm, stage, ks) -> (want_q, want_p); default: the varlen-M operands

    # ---- memory side
    def issue_load(self, voff_reg, rsrc, soff_reg):
        lds = self.lds
        if rsrc == self.rsrc_regs[0]:
            stream = P_STREAM
        elif rsrc == self.rsrc_regs[1]:
            stream = Q_STREAM
        else:
            raise SimError(f"load through unknown resource s{rsrc}")
        base = self.s[rsrc] | ((self.s[rsrc + 1] & 0xffff) << 32)
        extent = self.s[rsrc + 2] & 0xffffffff
        soff = self.s[soff_reg] if soff_reg is not None else 0
        off = (self.v[voff_reg] + soff) & 0xffffffff
        oob = off + 16 > extent
        if oob.any() and not (self.oob_zero or (self.oob_zero_p and stream == P_STREAM)):
            raise SimError(f"wave {self.w}: load offset {int(off.max())} + 16 beyond extent {extent} (stream {stream})")
        if (off % 16).any():
            raise SimError("unaligned global piece")
        if self.m0 % PIECE or not (0 <= self.m0 < LDS_BYTES):
            raise SimError(f"wave {self.w}: M0 = {self.m0}")
        piece = self.m0 // PIECE
        ring_lo, ring_hi = (0, G.P_SLOTS * G.P_STAGE) if stream == P_STREAM else (G.P_SLOTS * G.P_STAGE, LDS_BYTES)
        if not (ring_lo <= self.m0 - self.s[self.ldsp_reg] < ring_hi):
            raise SimError(f"wave {self.w}: stream {stream} load lands outside its ring (M0 = {self.m0})")
        if lds.pending[piece] is not None:
            raise SimError(f"piece {piece} requested twice")
        for w in range(G.NW):
            if lds.last_read[w][piece] >= self.phase and w != self.w:
                raise SimError(f"wave {self.w} overwrites piece {piece} in phase {self.phase}; wave {w} read it in "
                               f"phase {lds.last_read[w][piece]}")
        if piece in self.reads_out:
            raise SimError(f"wave {self.w} overwrites piece {piece} while its own read is in flight")
        elem = (base + off) // 2
        tags = (elem[:, None] + np.arange(8)[None, :]) | (stream << 60)
        tags[oob] = ZERO
        tags = tags.reshape(-1)
        lds.pending[piece] = self.w
        self.vmq.append((piece, tags))

    def wait_vm(self, n):
        while len(self.vmq) > n:
            piece, tags = self.vmq.pop(0)
            self.lds.tag[piece * 512:(piece + 1) * 512] = tags
            self.lds.pending[piece] = None
            self.lds.retire_phase[piece] = self.phase
            self.lds.retired_by[piece] = self.w

    def check_readable(self, byte_addr, nbytes):
        lds = self.lds
        if (byte_addr < 0).any() or (byte_addr + nbytes > LDS_BYTES).any():
            raise SimError(f"wave {self.w}: LDS read outside the allocation")
        for piece in np.unique(np.concatenate([byte_addr // PIECE, (byte_addr + nbytes - 1) // PIECE])):
            piece = int(piece)
            if lds.pending[piece] is not None:
                raise SimError(f"wave {self.w} reads piece {piece} while a load into it is in flight")
            if lds.retired_by[piece] != self.w and lds.retire_phase[piece] >= self.phase:
                raise SimError(f"wave {self.w} reads piece {piece} in phase {self.phase}: landed for wave "
                               f"{lds.retired_by[piece]} in phase {lds.retire_phase[piece]}, no barrier between")
            lds.last_read[self.w][piece] = max(lds.last_read[self.w][piece], self.phase)
            if piece not in self.reads_out:
                self.reads_out.append(piece)

    def ds_read_b128(self, dst, areg, offset):
        addr = self.v[areg] + offset
        if (addr % 16).any():
            raise SimError("unaligned ds_read_b128")
        self.check_readable(addr, 16)
        self.regs_out.update(range(dst, dst + 4))
        e = addr // 2
        t = self.lds.tag[e[:, None] + np.arange(8)[None, :]]
        for r in range(4):
            self.vt[dst + r, :, 0] = t[:, 2 * r]
            self.vt[dst + r, :, 1] = t[:, 2 * r + 1]

    def ds_read_tr(self, dst, areg, offset):
        addr = self.v[areg] + offset
        if (addr % 8).any():
            raise SimError("unaligned transpose read")
        self.check_readable(addr, 8)
        self.regs_out.update(range(dst, dst + 2))
        lane = np.arange(64)
        grp, i = lane // 16, lane % 16
        for r in range(4):
            src = 16 * grp + 4 * r + i // 4
            e = (addr[src] + 2 * (i % 4)) // 2
            self.vt[dst + r // 2, :, r % 2] = self.lds.tag[e]

    # ---- matrix side
    def mfma(self, acc, qreg, preg, fresh):
        prob = self.prob
        e, row0, row_end, n0 = self.tile
        idx = acc // 4
        fn, fm = idx // G.FM, idx % G.FM
        if acc != G.acc_reg(fn, fm):
            raise SimError("accumulator register does not name a fragment")
        n_done = self.acc_seen.get(acc, 0)
        stage, ks = n_done // 2, n_done % 2
        if fresh != (n_done == 0):
            raise SimError(f"fragment ({fn},{fm}): k-slice {n_done} of the tile {'starts from zero' if fresh else 'accumulates'}")
        self.acc_seen[acc] = n_done + 1
        lane = np.arange(64)
        wm, wn = self.w % 2, self.w // 2
        if self.expect is not None:
            want_q, want_p = self.expect(self, fn, fm, stage, ks)
            self._compare(qreg, preg, want_q, want_p, stage, ks, fn, fm)
            return
        k = stage * G.BK + ks * G.KSTEP + 8 * (lane // 16)[:, None] + np.arange(8)[None, :]
        # weight fragment: feature row n
        n = n0 + wn * G.TN + fn * G.FR + lane % 16
        if not prob.qmn:
            nc = np.minimum(n, prob.N - 1)
            want_q = e * prob.q_stride_e + nc[:, None] * prob.q_stride_row + k
        else:
            start = np.minimum(n - n % 8, prob.N - 8)
            nc = start + n % 8
            want_q = e * prob.q_stride_e + k * prob.q_stride_row + nc[:, None]
        want_q = want_q | (Q_STREAM << 60)
        m0 = row0 + wm * G.TM + fm * G.FR + lane % 16
        m = np.minimum(m0, row_end - 1)
        row = prob.gidx[m] if prob.gidx is not None else m
        want_p = (row[:, None] * prob.p_stride + k) | (P_STREAM << 60)
        if drop_rows(prob):
            want_p = np.where((m0 >= row_end)[:, None], ZERO, want_p)
        self._compare(qreg, preg, want_q, want_p, stage, ks, fn, fm)

    def _compare(self, qreg, preg, want_q, want_p, stage, ks, fn, fm):
        got_q = self.vt[qreg:qreg + 4].transpose(1, 0, 2).reshape(64, 8)
        got_p = self.vt[preg:preg + 4].transpose(1, 0, 2).reshape(64, 8)
        if not (got_q == want_q).all():
            bad = np.argwhere(got_q != want_q)[0]
            raise SimError(f"wave {self.w} tile {self.tile} stage {stage} k-slice {ks} fragment ({fn},{fm}): weight "
                           f"operand lane {bad[0]} element {bad[1]} holds {int(got_q[bad[0], bad[1]]):#x}, "
                           f"expected {int(want_q[bad[0], bad[1]]):#x}")
        if not (got_p == want_p).all():
            bad = np.argwhere(got_p != want_p)[0]
            raise SimError(f"wave {self.w} tile {self.tile} stage {stage} k-slice {ks} fragment ({fn},{fm}): token "
                           f"operand lane {bad[0]} element {bad[1]} holds {int(got_p[bad[0], bad[1]]):#x}, "
                           f"expected {int(want_p[bad[0], bad[1]]):#x}")
        self.mfma_count += 1


# ---- interpreter ----------------------------------------------------------------------------------------------------
_RE_VR = re.compile(r"v\[(\d+):(\d+)\]|v(\d+)")
_RE_SR = re.compile(r"s\[(\d+):(\d+)\]|s(\d+)")


def _first(m):
    return int(m.group(1) if m.group(1) is not None else m.group(3))


def asm_lines(qmn: bool) -> list[str]:
    return G.emit_tile(qmn)


def _signed(x: int) -> int:
    x &= 0xffffffff
    return x - (1 << 32) if x & 0x80000000 else x


def _sval(w: Wave, tok: str) -> int:
    tok = tok.strip()
    if tok == "m0":
        return w.m0
    if tok.startswith("s"):
        return w.s[int(tok[1:])]
    return int(tok, 0)


def run_wave(w: Wave, lines: list[str]):
    """generator: executes the statement for one wave, yields at every barrier"""
    labels = {ln[:-1]: i for i, ln in enumerate(lines) if ln.endswith(":")}
    pc = 0
    steps = 0
    while pc < len(lines):
        steps += 1
        if steps > 2_000_000:
            raise SimError("runaway loop")
        ln = lines[pc]
        pc += 1
        if ln.endswith(":"):
            continue
        op, _, rest = ln.partition(" ")
        args = [a.strip() for a in rest.split(",")] if rest else []
        if op == "s_barrier":
            if w.reads_out:
                pass  # reads still in flight cross the barrier: they count for the next phase as well
            w.nbarrier += 1
            yield
            w.phase += 1
            for piece in w.reads_out:
                w.lds.last_read[w.w][piece] = w.phase
        elif op == "s_nop":
            pass
        elif op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", rest)
            if m:
                w.wait_vm(int(m.group(1)))
            m = re.search(r"lgkmcnt\((\d+)\)", rest)
            if m:
                assert int(m.group(1)) == 0
                w.reads_out = []
                w.regs_out = set()
                w.smem_out = set()
        elif op in ("s_add_u32", "s_sub_u32", "s_xor_b32"):
            a, b = _sval(w, args[1]), _sval(w, args[2])
            r = a + b if op == "s_add_u32" else (a - b if op == "s_sub_u32" else a ^ b)
            r &= 0xffffffff
            if args[0] == "m0":
                w.m0 = r
            else:
                w.s[int(args[0][1:])] = r
        elif op == "s_mul_i32":
            for a in args[1:]:
                if a.startswith("s") and int(a[1:]) in w.smem_out:
                    raise SimError("scalar register read while a scalar load into it is in flight")
            w.s[int(args[0][1:])] = (_sval(w, args[1]) * _sval(w, args[2])) & 0xffffffff
        elif op == "s_sub_i32":
            w.s[int(args[0][1:])] = (_sval(w, args[1]) - _sval(w, args[2])) & 0xffffffff
        elif op in ("s_cmp_ge_i32", "s_cmp_gt_i32"):
            a, b = _signed(_sval(w, args[0])), _signed(_sval(w, args[1]))
            w.scc = int(a >= b) if op == "s_cmp_ge_i32" else int(a > b)
        elif op == "s_buffer_load_dwordx16":
            dst = _first(_RE_SR.match(args[0]))
            rs = _first(_RE_SR.match(args[1]))
            off = _sval(w, args[2])
            extent = w.s[rs + 2] & 0xffffffff
            base = w.s[rs] | ((w.s[rs + 1] & 0xffff) << 32)
            assert base == 0 and off % 4 == 0
            for j in range(16):
                o = off + 4 * j
                w.s[dst + j] = int(w.prob.gidx_flat[o // 4]) & 0xffffffff if o + 4 <= extent else 0
            w.smem_out = set(range(dst, dst + 16))
        elif op == "v_mul_lo_u32":
            w.v[int(args[0][1:])] = (w.v[int(args[1][1:])] * _sval(w, args[2])) & 0xffffffff
        elif op == "v_add3_u32":
            w.v[int(args[0][1:])] = (w.v[int(args[1][1:])] + _sval(w, args[2]) + w.v[int(args[3][1:])]) & 0xffffffff
        elif op == "s_mov_b32":
            w.s[int(args[0][1:])] = _sval(w, args[1])
        elif op == "s_cmp_lg_u32":
            w.scc = int(_sval(w, args[0]) != _sval(w, args[1]))
        elif op == "s_cmp_ge_u32":
            w.scc = int(_sval(w, args[0]) >= _sval(w, args[1]))
        elif op == "s_cselect_b32":
            if any(a.startswith("s") and int(a[1:]) in w.smem_out for a in args[1:]):
                raise SimError("scalar register read while a scalar load into it is in flight")
            w.s[int(args[0][1:])] = (_sval(w, args[1]) if w.scc else _sval(w, args[2])) & 0xffffffff
        elif op == "s_cbranch_scc1":
            if w.scc:
                pc = labels[args[0]]
        elif op == "v_add_u32":
            w.v[int(args[0][1:])] = (_sval(w, args[1]) + w.v[int(args[2][1:])]) & 0xffffffff
        elif op == "v_mov_b32":
            w.v[int(args[0][1:])] = w.v[int(args[1][1:])]
        elif op in ("ds_read_b128", "ds_read_b64_tr_b16"):
            dst = _first(_RE_VR.match(args[0]))
            addr_tok, off_tok = args[1].split()
            off = int(off_tok.split(":")[1])
            if op == "ds_read_b128":
                w.ds_read_b128(dst, int(addr_tok[1:]), off)
            else:
                w.ds_read_tr(dst, int(addr_tok[1:]), off)
        elif op == "buffer_load_dwordx4":
            soff = args[2].split()[0]
            assert args[2].split()[1:] == ["offen", "lds"]
            w.issue_load(int(args[0][1:]), _first(_RE_SR.match(args[1])), int(soff[1:]) if soff.startswith("s") else None)
        elif op == "v_mfma_f32_16x16x32_bf16":
            # operands: a[..], v[..], v[..], (0 | a[..]) - the vector ranges contain commas only between operands
            m = re.match(r"a\[(\d+):(\d+)\], v\[(\d+):(\d+)\], v\[(\d+):(\d+)\], (0|a\[(\d+):(\d+)\])$", rest)
            if not m:
                raise SimError("cannot parse " + ln)
            acc = int(m.group(1))
            fresh = m.group(7) == "0"
            if not fresh and int(m.group(8)) != acc:
                raise SimError("accumulates into a different fragment")
            qreg, preg = int(m.group(3)), int(m.group(5))
            if w.regs_out & (set(range(qreg, qreg + 4)) | set(range(preg, preg + 4))):
                raise SimError(f"wave {w.w}: matrix instruction reads a fragment whose LDS read has not been waited for")
            w.mfma(acc, qreg, preg, fresh)
        else:
            raise SimError("unknown instruction: " + ln)


# ---- the C++ side, restated ------------------------------------------------------------------------------------------
def p_extent(prob: Problem) -> int:
    return prob.p_rows * prob.p_stride * 2


def drop_rows(prob: Problem) -> bool:
    """rows behind an expert's end are not fetched (offset = the tensor's end: dropped by the range check) when that
    offset plus the longest stage offset cannot wrap around 32 bits; otherwise they re-read the expert's last row"""
    return p_extent(prob) + prob.K * 2 + 16 <= 0xffffffff


def token_rows(prob: Problem, wave: int, tile):
    e, row0, row_end, n0 = tile
    lane = np.arange(64)
    rows = []
    for i in range(G.P_INSTR):
        m0 = row0 + (wave * G.P_INSTR + i) * 8 + lane // 8
        m = np.minimum(m0, row_end - 1)
        row = prob.gidx[m] if prob.gidx is not None else m
        rows.append(np.where(m0 >= row_end, -1, row) if drop_rows(prob) else row)
    return rows


def point_p(prob: Problem, wave: int, rows):
    lane = np.arange(64)
    out = []
    for i in range(G.P_INSTR):
        r = (wave * G.P_INSTR + i) * 8 + lane // 8
        off = rows[i] * (prob.p_stride * 2) + (((lane % 8) ^ kswz(r)) << 4)
        out.append(np.where(rows[i] < 0, p_extent(prob), off))
    return out


def point_q(prob: Problem, wave: int, tile):
    e, row0, row_end, n0 = tile
    lane = np.arange(64)
    out = []
    qrb = prob.q_stride_row * 2
    for i in range(G.Q_INSTR):
        if not prob.qmn:
            r = (wave * G.Q_INSTR + i) * 8 + lane // 8
            n = np.minimum(n0 + r, prob.N - 1)
            out.append(n * qrb + (((lane % 8) ^ kswz(r)) << 4))
        else:
            kl = (wave * G.Q_INSTR + i) * 2 + lane // 32
            phys16 = lane % 32
            log32 = (phys16 >> 1) ^ mnswz(kl)
            n = np.minimum(n0 + ((log32 << 1) | (phys16 & 1)) * 8, prob.N - 8)
            out.append(kl * qrb + n * 2)
    return out


def fragment_offsets(prob: Problem, wave: int):
    lane = np.arange(64)
    wm, wn = wave % 2, wave // 2
    row = wm * G.TM + (lane & 15)
    p_off = [row * G.KROW + (((4 * ks + lane // 16) ^ kswz(row)) << 4) for ks in range(2)]
    if not prob.qmn:
        row = wn * G.TN + (lane & 15)
        q_off = [row * G.KROW + (((4 * ks + lane // 16) ^ kswz(row)) << 4) for ks in range(2)]
    else:
        grp, i16 = lane >> 4, lane & 15
        kk = 8 * grp + (i16 >> 2)
        q_off = []
        for fn in range(G.FN):
            c16 = (wn * G.TN) // 16 + fn
            for h in range(2):
                k = kk + 4 * h
                q_off.append(k * G.ROWB + ((c16 ^ mnswz(k)) << 5) + ((i16 & 3) << 3))
    return p_off, q_off


def q_extent(prob: Problem) -> int:
    qrb = prob.q_stride_row * 2
    return (prob.K - 1) * qrb + prob.N * 2 if prob.qmn else (prob.N - 1) * qrb + prob.K * 2


def simulate(prob: Problem, lds_base: int = 0) -> dict:
    """Runs the workgroup through prob.tiles; returns counters.  Raises SimError at the first violation."""
    assert prob.S >= 3
    lines = asm_lines(prob.qmn)
    lds = Lds()
    waves = [Wave(w, lds, prob) for w in range(G.NW)]
    for w in waves:
        w.oob_zero_p = drop_rows(prob)
    tiles = prob.tiles
    q_step = G.BK * prob.q_stride_row * 2 if prob.qmn else G.BK * 2
    q_ring = G.P_SLOTS * G.P_STAGE

    def tile_or_last(i):
        return tiles[min(i, len(tiles) - 1)]

    def set_vec(w, reg, vals):
        for i, v in enumerate(vals):
            w.v[reg + i] = np.asarray(v, dtype=np.int64) & 0xffffffff

    def q_base_words(tile):
        b = tile[0] * prob.q_stride_e * 2
        return b & 0xffffffff, (b >> 32) & 0xffff

    # ---- what the kernel does before the first statement
    for w in waves:
        s = w.s
        s[G.S_PRSRC:G.S_PRSRC + 4] = [0, 0, prob.p_rows * prob.p_stride * 2, 0x20000]
        lo, hi = q_base_words(tiles[0])
        s[G.S_QRSRC:G.S_QRSRC + 4] = [lo, hi, q_extent(prob), 0x20000]
        set_vec(w, G.V_PV, point_p(prob, w.w, token_rows(prob, w.w, tiles[0])))
        set_vec(w, G.V_QV, point_q(prob, w.w, tiles[0]))
        set_vec(w, G.V_PVN, point_p(prob, w.w, token_rows(prob, w.w, tile_or_last(1))))
        set_vec(w, G.V_QVN, point_q(prob, w.w, tile_or_last(1)))
        s[G.S_QNB], s[G.S_QNB + 1] = q_base_words(tile_or_last(1))
        p_off, q_off = fragment_offsets(prob, w.w)
        set_vec(w, G.V_POFF, p_off)
        set_vec(w, G.V_QOFF, q_off)
        s[G.S_LDSP], s[G.S_LDSQ], s[G.S_WLDS] = lds_base, lds_base + q_ring, w.w * G.P_INSTR * 1024
        s[G.S_PEND], s[G.S_QEND], s[G.S_QSTEP], s[G.S_NMID] = prob.S * G.BK * 2, prob.S * q_step, q_step, prob.S - 2
        s[G.S_PFILL], s[G.S_QFILL] = lds_base, lds_base + q_ring
        # prologue: P(0) into token slot 1, Q(0), Q(1) into weight slots 1, 2
        s[G.S_PSOFF] = 0
        for i in range(G.P_INSTR):
            w.m0 = lds_base + G.P_STAGE + s[G.S_WLDS] + i * 1024
            w.issue_load(G.V_PV + i, G.S_PRSRC, G.S_PSOFF)
        for st in range(2):
            s[G.S_QSOFF] = st * q_step
            for i in range(G.Q_INSTR):
                w.m0 = lds_base + q_ring + (1 + st) * G.Q_STAGE + s[G.S_WLDS] + i * 1024
                w.issue_load(G.V_QV + i, G.S_QRSRC, G.S_QSOFF)
        s[G.S_PSOFF], s[G.S_QSOFF] = G.BK * 2, 2 * q_step
        w.wait_vm(0)

    nbar = 0
    for ti, tile in enumerate(tiles):
        for w in waves:
            w.tile = tile
            w.acc_seen = {}
        gens = [run_wave(w, lines) for w in waves]
        alive = [True] * G.NW
        while any(alive):
            state = []
            for i, g in enumerate(gens):
                try:
                    next(g)
                    state.append("barrier")
                except StopIteration:
                    alive[i] = False
                    state.append("done")
            if len(set(state)) != 1:
                raise SimError(f"waves disagree at a barrier: {state}")
        for w in waves:
            if len(w.acc_seen) != G.FN * G.FM or any(v != 2 * prob.S for v in w.acc_seen.values()):
                raise SimError(f"wave {w.w}: accumulators saw {sorted(set(w.acc_seen.values()))} k-slices, want {2 * prob.S}")
            if w.reads_out:
                raise SimError("fragment reads in flight at the end of the statement")
        nb = {w.nbarrier for w in waves}
        if len(nb) != 1:
            raise SimError("barrier counts differ")
        # ---- epilogue: waves 0, 1 park rows in the vacated token slot, waves 2, 3 in the vacated weight slot
        for w in waves:
            slot = w.s[G.S_PFILL] if w.w < 2 else w.s[G.S_QFILL]
            size = G.P_STAGE
            for piece in range(slot // PIECE, (slot + size) // PIECE):
                if lds.pending[piece] is not None:
                    raise SimError(f"epilogue parks in piece {piece} with a load in flight")
                for o in waves:
                    if o.w != w.w and lds.last_read[o.w][piece] >= w.phase:
                        raise SimError(f"epilogue of wave {w.w} parks in piece {piece} wave {o.w} may still read")
                lds.tag[piece * 512:(piece + 1) * 512] = -2
        # ---- hand the offsets of the tile after next to the streams
        for w in waves:
            nn = tile_or_last(ti + 2)
            set_vec(w, G.V_PVN, point_p(prob, w.w, token_rows(prob, w.w, nn)))
            set_vec(w, G.V_QVN, point_q(prob, w.w, nn))
            w.s[G.S_QNB], w.s[G.S_QNB + 1] = q_base_words(nn)
    for w in waves:
        w.wait_vm(0)
    return dict(mfma=sum(w.mfma_count for w in waves), barriers=waves[0].nbarrier)


# ---- weight-gradient loop --------------------------------------------------------------------------------------------
@dataclass
class ProblemMM:
    gp: bool  # the token-side operand R is gathered (dW2); otherwise the weight-side operand S is (dW1)
    NA: int
    NB: int
    r_stride: int
    s_stride: int
    gather_rows: int
    gidx_flat: np.ndarray  # (total_rows,) grouped row -> row of the gathered tensor
    tiles: list  # (row_begin, row_end, a0, b0) this workgroup walks through, in order

    @property
    def total_rows(self):
        return len(self.gidx_flat)


def simulate_mm(prob: ProblemMM) -> dict:
    gp, gq = prob.gp, not prob.gp
    pro, lines = G.mm_emit_prologue(gp, gq), G.mm_emit_tile(gp, gq)
    lds = Lds()
    waves = [Wave(w, lds, prob) for w in range(G.NW)]
    rrb, srb = prob.r_stride * 2, prob.s_stride * 2
    lane = np.arange(64)
    tiles = prob.tiles

    def stages(tile):
        return max(3, -(-(tile[1] - tile[0]) // G.BK))

    def clamp8(c, n):
        return np.minimum(c - c % 8, n - 8) + c % 8

    def expect(w, fn, fm, stage, ks):
        row_begin, row_end, a0, b0 = w.tile
        wa, wb = w.w % 2, w.w // 2
        m = row_begin + stage * G.BK + ks * G.KSTEP + 8 * (lane // 16)[:, None] + np.arange(8)[None, :]
        valid = m < row_end
        mc = np.minimum(m, prob.total_rows - 1)
        b = clamp8(b0 + wb * G.TN + fn * G.FR + lane % 16, prob.NB)
        a = clamp8(a0 + wa * G.TM + fm * G.FR + lane % 16, prob.NA)
        rq = prob.gidx_flat[mc] if gq else mc
        rp = prob.gidx_flat[mc] if gp else mc
        want_q = np.where(valid, (rq * prob.s_stride + b[:, None]) | (Q_STREAM << 60), ZERO)
        want_p = np.where(valid, (rp * prob.r_stride + a[:, None]) | (P_STREAM << 60), ZERO)
        return want_q, want_p

    def lane_offsets(wv, tile):
        row_begin, row_end, a0, b0 = tile
        pv, qv = [], []
        for i in range(G.P_INSTR):
            kl = (wv * G.P_INSTR + i) * 2 + lane // 32
            phys16 = lane % 32
            log32 = (phys16 >> 1) ^ mnswz(kl)
            c = ((log32 << 1) | (phys16 & 1)) * 8
            a = np.minimum(a0 + c, prob.NA - 8)
            b = np.minimum(b0 + c, prob.NB - 8)
            pv.append((0 if gp else kl * rrb) + a * 2)
            qv.append((0 if gq else kl * srb) + b * 2)
        return pv, qv

    def first_offsets(wv, tile):
        row_begin = tile[0]
        run = (row_begin + wv * 16) * 4
        return (run if gp else row_begin * rrb), (run if gq else row_begin * srb)

    NULL = (0, 0, 0, 0)  # behind the last tile: an empty expert, every load out of range

    def set_next(w, tile):
        pvn, qvn = lane_offsets(w.w, tile)
        for i in range(G.P_INSTR):
            w.v[G.MV_PVN + i] = pvn[i]
            w.v[G.MV_QVN + i] = qvn[i]
        s = w.s
        s[G.MS_PSOFFN], s[G.MS_QSOFFN] = first_offsets(w.w, tile)
        s[G.MS_PEXTN], s[G.MS_QEXTN] = tile[1] * rrb, tile[1] * srb
        s[G.MS_RLEFTN] = (tile[1] - (tile[0] + w.w * 16)) & 0xffffffff
        s[G.MS_SNEXT] = stages(tile)

    for w in waves:
        w.ldsp_reg = G.MS_LDSP
        w.rsrc_regs = (G.MS_PRSRC, G.MS_QRSRC)
        w.oob_zero = True
        w.expect = expect
        t0 = tiles[0]
        s = w.s
        s[G.MS_PRSRC:G.MS_PRSRC + 4] = [0, 0, (prob.gather_rows if gp else t0[1]) * rrb, 0x20000]
        s[G.MS_QRSRC:G.MS_QRSRC + 4] = [0, 0, (prob.gather_rows if gq else t0[1]) * srb, 0x20000]
        s[G.MS_GRSRC:G.MS_GRSRC + 4] = [0, 0, prob.total_rows * 4, 0x20000]
        pv, qv = lane_offsets(w.w, t0)
        for i in range(G.P_INSTR):
            w.v[G.MV_PV + i] = pv[i]
            w.v[G.MV_QV + i] = qv[i]
        wa, wb = w.w % 2, w.w // 2
        grp, i16 = lane >> 4, lane & 15
        kk = 8 * grp + (i16 >> 2)
        for f in range(8):
            for h in range(2):
                k = kk + 4 * h
                w.v[G.MV_PRA + 2 * f + h] = k * G.ROWB + ((((wa * G.TM) // 16 + f) ^ mnswz(k)) << 5) + ((i16 & 3) << 3)
                w.v[G.MV_QRA + 2 * f + h] = k * G.ROWB + ((((wb * G.TN) // 16 + f) ^ mnswz(k)) << 5) + ((i16 & 3) << 3)
        w.v[G.MV_HALF] = lane >> 5
        s[G.MS_PSOFF], s[G.MS_QSOFF] = first_offsets(w.w, t0)
        s[G.MS_PSTEP] = rrb if gp else G.BK * rrb
        s[G.MS_QSTEP] = srb if gq else G.BK * srb
        s[G.MS_RLEFT] = (t0[1] - (t0[0] + w.w * 16)) & 0xffffffff
        s[G.MS_LDSP], s[G.MS_LDSQ], s[G.MS_WLDS] = 0, G.P_SLOTS * G.P_STAGE, w.w * G.P_INSTR * 1024
        s[G.MS_PFILL], s[G.MS_QFILL] = 0, G.P_SLOTS * G.P_STAGE
        for _ in run_wave(w, pro):
            raise SimError("barrier in the prologue")
        if w.vmq or w.smem_out:
            raise SimError("the prologue leaves operations in flight")
        # the prologue has requested one token stage and two weight stages of the first tile
        s[G.MS_PLEFT], s[G.MS_QLEFT] = stages(t0) - 1, stages(t0) - 2
    saved = [(w.v[G.MV_PRA:G.MV_PRA + 16].copy(), w.v[G.MV_QRA:G.MV_QRA + 16].copy()) for w in waves]
    total_mfma = 0
    for ti, tile in enumerate(tiles):
        nxt = tiles[ti + 1] if ti + 1 < len(tiles) else NULL
        for w in waves:
            w.tile = tile
            w.acc_seen = {}
            w.s[G.MS_NMID] = stages(tile) - 2
            set_next(w, nxt)
        gens = [run_wave(w, lines) for w in waves]
        alive = [True] * G.NW
        while any(alive):
            state = []
            for i, g in enumerate(gens):
                try:
                    next(g)
                    state.append("barrier")
                except StopIteration:
                    alive[i] = False
                    state.append("done")
            if len(set(state)) != 1:
                raise SimError(f"waves disagree at a barrier: {state}")
        for w, (pra, qra) in zip(waves, saved):
            if len(w.acc_seen) != G.FN * G.FM or any(v != 2 * stages(tile) for v in w.acc_seen.values()):
                raise SimError(f"wave {w.w}: accumulators saw {sorted(set(w.acc_seen.values()))} k-slices, want {2 * stages(tile)}")
            if w.reads_out or w.smem_out:
                raise SimError("LDS or scalar reads in flight at the end of the statement")
            if not ((w.v[G.MV_PRA:G.MV_PRA + 16] == pra).all() and (w.v[G.MV_QRA:G.MV_QRA + 16] == qra).all()):
                raise SimError("read addresses do not come back slot-relative")
        total_mfma += G.NW * 64 * 2 * stages(tile)
        # epilogue: parks rows in the two vacated slots
        for w in waves:
            slot = w.s[G.MS_PFILL] if w.w < 2 else w.s[G.MS_QFILL]
            for piece in range(slot // PIECE, (slot + G.P_STAGE) // PIECE):
                if lds.pending[piece] is not None:
                    raise SimError(f"epilogue parks in piece {piece} with a load in flight")
                for o in waves:
                    if o.w != w.w and lds.last_read[o.w][piece] >= w.phase:
                        raise SimError(f"epilogue of wave {w.w} parks in piece {piece} wave {o.w} may still read")
                lds.tag[piece * 512:(piece + 1) * 512] = -2
    for w in waves:
        w.wait_vm(0)
    got = sum(w.mfma_count for w in waves)
    if got != total_mfma:
        raise SimError(f"{got} matrix instructions, want {total_mfma}")
    return dict(mfma=got, barriers=waves[0].nbarrier)
