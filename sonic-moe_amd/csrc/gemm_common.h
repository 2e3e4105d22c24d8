// Building blocks shared by the grouped GEMM kernels (gfx950, wave64, bf16 MFMA 32x32x16, fp32 accumulate).
//
// Vocabulary.  A GEMM tile multiplies a "P" operand (token side) with a "Q" operand (weight side) over a
// contraction index k.  Both live in LDS as a ring of NSTAGE stages, BK = 32 deep each, filled by direct-to-LDS loads
// (global_load_lds_dwordx4: every lane names its own 16 global bytes, the wavefront's 64 pieces land in 1024
// consecutive LDS bytes), so the LDS position of a piece is fixed by (wave, instruction, lane) and swizzling is
// done by choosing WHICH global piece a lane fetches.
//
//   K-major stage : [rows][BK k]   row = BK*2 B = BK/8 pieces; piece c of row r sits at c ^ kswz(r).
//                   MFMA operand fragment = one ds_read_b128 per lane (row l%32, pieces 2*ks + l/32).
//   MN-major stage: [BK k][cols]   row = cols*2 B; 32-byte group g of k-row k sits at g ^ mnswz(k).
//                   MFMA operand fragment = two ds_read_b64_tr_b16 per lane (the transpose load hands lane i of a
//                   16-lane group column i of a 4 x 16 block whose rows are named by the lanes' addresses).
//
// The MFMA is issued as D[n][m] += Q[n][k] P[k][m]: lane l of the accumulator owns token column m = l % 32 and,
// in register r, feature n = 8*(r/4) + 4*(l/32) + r%4, so four consecutive features (two gate/up pairs) sit in
// one lane and per-token scalars are per-lane.
#pragma once
#include <type_traits>

#include "common.h"

namespace smoe {


typedef __attribute__((address_space(3))) void* lds_ptr_t;

// byte address inside the workgroup's LDS allocation of a generic pointer into __shared__ memory
SMOE_DEV uint32_t lds_address(const void* p) { return (uint32_t)(uintptr_t)(lds_ptr_t)p; }

// Direct-to-LDS load: every lane fetches its own 16 global bytes; the 64 pieces of the wavefront land in the 1024
// LDS bytes starting at the wave-uniform address lds_wave_base (M0).  Issued through inline assembly on purpose:
// when the compiler knows an instruction writes LDS from memory it protects every later LDS read with
// s_waitcnt vmcnt(0), which would allow only one stage in flight.  The kernels wait by hand (wait_vmem_upto) for
// exactly the stage they are about to read.
SMOE_DEV void load16_to_lds(const void* g, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(lds_wave_base) : "memory");
}

// The same through a buffer resource: source = resource base + per-lane byte offset `voff` + wave-uniform byte offset
// `soff`.  The address arithmetic of a stage is then one scalar add (soff moves along the contraction) instead of a
// 64-bit vector add per load, and a lane keeps one 32-bit offset per load instead of a pointer.
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
SMOE_DEV i32x4 make_buffer_resource(const void* base) {
  const uint64_t b = (uint64_t)base;
  i32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((uint32_t)b);
  r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32) & 0xffffu);  // 48-bit base, stride 0 (raw buffer)
  r[2] = -1;                                                                // no range limit: the kernels clamp rows
  r[3] = 0x00020000;                                                        // 32-bit untyped data
  return r;
}
// with a range limit: loads whose byte offset (per-lane + wave-uniform) reaches `bytes` are dropped by the hardware
SMOE_DEV i32x4 make_buffer_resource(const void* base, uint32_t bytes) {
  i32x4 r = make_buffer_resource(base);
  r[2] = (int32_t)bytes;
  return r;
}
SMOE_DEV void buffer_load16_to_lds(i32x4 rsrc, uint32_t voff, uint32_t soff, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
               :
               : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_wave_base)
               : "memory");
}

// Piece swizzle of a K-major stage with BK_ of the contraction per row (BK_*2/16 pieces).  The LDS has 64 banks and
// serves a ds_read_b128 16 lanes at a time, in the groups {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31} and the
// same of the upper half-wave: the 16 pieces of a group have to fall into the 16 different 16-byte bank groups (row
// parity, piece).  With 32-row fragments (FR_ = 32: lane l reads row l % 32) a group holds 16 rows of one piece; with
// 16-row fragments (FR_ = 16: row l % 16, piece c + l / 16) it holds rows 0-3 and 12-15 of piece c and rows 4-11 of
// piece c ^ 1, which the first swizzle sends to the same banks twice (SQ_LDS_BANK_CONFLICT equal to half of
// SQ_LDS_IDX_ACTIVE); the second one is row / 2 with the low bit flipped for the rows 4-11.
template <int BK_, int FR_ = 32>
SMOE_DEV int kswz(int row) {
  if constexpr (BK_ == 32) return (row >> 2) & 3;
  else if constexpr (FR_ == 16) return ((row >> 1) & 7) ^ (((row >> 2) ^ (row >> 3)) & 1);
  else return (row & 7) ^ ((row >> 3) & 1);
}

// 32-byte-group swizzle of an MN-major stage: group g of contraction row k sits at g ^ mnswz(k).  A transpose load
// makes the 32 lanes of a half-wave read eight k-rows (k & 3 = 0..3, twice) of one or two neighbouring groups; the
// swizzle sends the eight 32-byte pieces to the eight different 32-byte bank groups of the 64 banks for both fragment
// shapes (32-row fragments: rows k..k+3 of two neighbouring groups; 16-row fragments: rows k..k+3 and k+8..k+11 of one).
SMOE_DEV int mnswz(int k) { return ((k & 3) << 1) ^ ((k >> 3) & 1); }

SMOE_DEV bf16x8 lds_read_b128(const char* p) { return *(const bf16x8*)p; }

SMOE_DEV bf16x8 lds_read_tr2(const char* p0, const char* p1) {
  typedef __attribute__((address_space(3))) s16x4* tr_ptr_t;
  s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)p0);
  s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)p1);
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
  s16x8 r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

// compile-time loop: f(std::integral_constant<int, i>) for i in [0, N); keeps register-array indices static
template <int I, int N, class F>
SMOE_DEV void static_for_impl(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for_impl<I + 1, N>(f);
  }
}
template <int N, class F>
SMOE_DEV void static_for(F&& f) {
  static_for_impl<0, N>(f);
}

// s_waitcnt vmcnt(N) lgkmcnt(0): at most N of this wave's vector-memory operations (oldest first) may still be
// outstanding, and all of its LDS operations have completed
template <int N>
SMOE_DEV void wait_vmem_upto() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 15) | ((N >> 4) << 14));
}
SMOE_DEV void wait_vmem_all() { wait_vmem_upto<0>(); }
// s_waitcnt lgkmcnt(0) only: all of this wave's LDS operations have completed, vector memory untouched
SMOE_DEV void wait_lds_all() { __builtin_amdgcn_s_waitcnt(0xC07F); }

// Workgroup barrier WITHOUT the memory fence of __syncthreads(): a fence would wait for every outstanding
// direct-to-LDS load (vmcnt(0)) and collapse the ring to one stage in flight.  The waits that make LDS contents
// visible are placed by hand (wait_vmem_upto before the barrier); the empty asm statements keep the compiler from
// moving LDS accesses across the barrier.
SMOE_DEV void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// ---- matrix instruction policies ---------------------------------------------------------------------------------
// A main loop works in STEPS per LDS stage.  A step issues NQ x NP matrix instructions on fragments that the previous
// step read from LDS: two register sets of weight-side (Q) fragments and two of token-side (P) fragments alternate.
//   Bf16Mma32  v_mfma_f32_32x32x16_bf16: a step is one k-slice of 16; it reads all of the wave's fragments.
//   Bf16Mma16  v_mfma_f32_16x16x32_bf16: a k-slice is 32 deep and is worked through in PH = 2 steps over the two halves
//              of the wave's token fragments; the Q fragments are read on the even step and serve both.  Same bytes
//              from LDS per FLOP, four times the instructions, and markedly less power per FLOP on random data (a
//              register-only loop of these instructions sustains 2.07 PFLOP/s under the chip's power limit where
//              the 32x32x16 form sustains 1.8), which is what bounds these kernels.
// Accumulator layout (operands are issued as D[n][m] += Q[n][k] P[k][m]): lane l owns token column m = l % FR of the
// fragment and, per group of four registers, four consecutive features.
struct Bf16Mma32 {
  typedef bf16x8 Frag;
  typedef f32x16 Acc;
  static constexpr int FR = 32, KSTEP = 16, PH = 1, ACC_REGS = 16, FRAG_REGS = 4;
  static constexpr int qset(int step) { return step & 1; }
  static constexpr int phalf(int) { return 0; }
  static constexpr bool reads_q(int) { return true; }
  static constexpr int kslice(int step) { return step; }
  static __device__ __forceinline__ Acc run(const Frag& q, const Frag& p, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(q, p, c, 0, 0, 0);
  }
};
struct Bf16Mma16 {
  typedef bf16x8 Frag;
  typedef f32x4 Acc;
  static constexpr int FR = 16, KSTEP = 32, PH = 2, ACC_REGS = 4, FRAG_REGS = 4;
  static constexpr int qset(int step) { return (step >> 1) & 1; }
  static constexpr int phalf(int step) { return step & 1; }
  static constexpr bool reads_q(int step) { return (step & 1) == 0; }
  static constexpr int kslice(int step) { return step >> 1; }
  static __device__ __forceinline__ Acc run(const Frag& q, const Frag& p, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(q, p, c, 0, 0, 0);
  }
};
// the bf16 kernels' instruction
typedef Bf16Mma16 Bf16Mma;

template <class Mma, int NQ, int NPT>
SMOE_DEV void clear_accumulators(typename Mma::Acc (&acc)[NQ][NPT]) {
#pragma unroll
  for (int q = 0; q < NQ; q++)
#pragma unroll
    for (int pp = 0; pp < NPT; pp++)
#pragma unroll
      for (int r = 0; r < Mma::ACC_REGS; r++) acc[q][pp][r] = 0.f;
}

// The matrix instructions of one step, with the LDS reads issued just before them (for the NEXT step) slotted in
// RPM per instruction, starting after the first so that the wait in front of it covers only reads of the previous step.
template <class Mma, int NQ, int NP, int NREADS, int RPM, int STEP, bool FRESH>
SMOE_DEV void mma_step(typename Mma::Acc (&acc)[NQ][NP * Mma::PH], typename Mma::Frag (&qf)[2][NQ],
                       typename Mma::Frag (&pf)[2][NP]) {
  constexpr int qs = Mma::qset(STEP), ps = STEP & 1, ph = Mma::phalf(STEP), NM = NQ * NP;
  typename Mma::Acc zero;
#pragma unroll
  for (int r = 0; r < Mma::ACC_REGS; r++) zero[r] = 0.f;
#pragma unroll
  for (int q = 0; q < NQ; q++)
#pragma unroll
    for (int pp = 0; pp < NP; pp++)
      acc[q][ph * NP + pp] = Mma::run(qf[qs][q], pf[ps][pp], FRESH ? zero : acc[q][ph * NP + pp]);
  constexpr int NG0 = (NREADS + RPM - 1) / RPM, NR = NG0 < NM ? NG0 : NM - 1;
#pragma unroll
  for (int i = 0; i < NR; i++) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, RPM, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, NM - NR, 0);
  // large fragments: keep the scheduler from pulling the reads of later steps up in front of this one (more than two
  // fragment sets do not fit beside the accumulators)
  if constexpr (Mma::FRAG_REGS > 4) __builtin_amdgcn_sched_barrier(0);
}

// The last step of a stage whose ring slots are refilled: `deal(i)` is called behind the i-th matrix instruction and
// issues the refill's load instructions that fall there, so they are dealt out between the matrix instructions instead
// of standing in front of them (the matrix pipe does not idle while every wave issues its loads behind the barrier).
template <class Mma, int NQ, int NP, int STEP, class Deal>
SMOE_DEV void mma_step_refill(typename Mma::Acc (&acc)[NQ][NP * Mma::PH], typename Mma::Frag (&qf)[2][NQ],
                              typename Mma::Frag (&pf)[2][NP], Deal&& deal) {
  constexpr int qs = Mma::qset(STEP), ps = STEP & 1, ph = Mma::phalf(STEP), NM = NQ * NP;
  static_for<NM>([&](auto i_c) {
    constexpr int i = decltype(i_c)::value;
    acc[i / NP][ph * NP + i % NP] = Mma::run(qf[qs][i / NP], pf[ps][i % NP], acc[i / NP][ph * NP + i % NP]);
    deal(i_c);
    __builtin_amdgcn_sched_barrier(0);
  });
}

// ---- software-pipelined main loop ------------------------------------------------------------------------------
// LDS holds a ring of NSTAGE stages; a stage is worked through in STEPS steps.  One stage is consumed while up to
// NSTAGE-1 are in flight from L2/HBM.  Per stage:
//   steps 0..STEPS-2: read the fragments of the next step from LDS while the matrix instructions of the current run;
//   last step: wait until this wave's pieces of the NEXT stage have landed (vmcnt leaves the younger stages in
//            flight), workgroup barrier (everyone's pieces landed; everyone drained the current stage), refill the
//            current stage's slot with stage s+NSTAGE, read step 0 of the next stage while the last instructions run.
//   issue(buf, s, i)              start the i-th (compile-time index, 0 <= i < LPS) of this wave's direct-to-LDS loads of
//                                 stage s into ring slot buf; called with i ascending, stages in order
//   load(buf, s, step, qf, pf)    read the fragments step `step` (a compile-time constant) needs from ring slot buf
//                                 into the fragment sets handed in
template <int NQ, int NP, int NREADS, int LPS, int STEPS, int NSTAGE, class Mma = Bf16Mma, int RPM = 1, class Issue,
          class Load>
SMOE_DEV void gemm_mainloop(const int S, typename Mma::Acc (&acc)[NQ][NP * Mma::PH], Issue&& issue, Load&& load) {
  if (S <= 0) return;
  static_assert((NSTAGE - 1) * LPS < 64, "too many loads in flight for vmcnt");
  static_assert(STEPS % 2 == 0 && NSTAGE >= 2 && NSTAGE <= 6, "unsupported pipeline shape");
  typename Mma::Frag qf[2][NQ], pf[2][NP];
  constexpr int NM = NQ * NP, LAST = STEPS - 1;
  auto issue_all = [&](int buf, int s) { static_for<LPS>([&](auto i_c) { issue(buf, s, i_c); }); };
  const int pre = S < NSTAGE ? S : NSTAGE;
  for (int s = 0; s < pre; s++) issue_all(s, s);

  auto wait_next_stage = [&](int younger) {  // `younger` stages were issued after the one we need
    if constexpr (NSTAGE >= 6) if (younger >= 4) { wait_vmem_upto<4 * LPS>(); return; }
    if constexpr (NSTAGE >= 5) if (younger == 3) { wait_vmem_upto<3 * LPS>(); return; }
    if constexpr (NSTAGE >= 4) if (younger == 2) { wait_vmem_upto<2 * LPS>(); return; }
    if constexpr (NSTAGE >= 3) if (younger == 1) { wait_vmem_upto<LPS>(); return; }
    wait_vmem_all();
  };
  auto read_step = [&](int buf, int s, auto step_c) {
    constexpr int step = decltype(step_c)::value;
    load(buf, s, step_c, qf[Mma::qset(step)], pf[step & 1]);
  };
  auto inner_steps = [&](int buf, int s) {
    static_for<STEPS - 1>([&](auto k_c) {
      constexpr int k = decltype(k_c)::value;
      read_step(buf, s, std::integral_constant<int, k + 1>{});
      mma_step<Mma, NQ, NP, NREADS, RPM, k, false>(acc, qf, pf);
    });
  };
  constexpr std::integral_constant<int, 0> step0{};

  wait_next_stage(pre - 1);
  lds_barrier();
  read_step(0, 0, step0);
  int buf = 0;
  int s = 0;
  for (; s + NSTAGE < S; s++) {  // steady state: every stage boundary refills the slot it frees
    inner_steps(buf, s);
    wait_next_stage(NSTAGE - 2);
    lds_barrier();
    const int next = buf + 1 == NSTAGE ? 0 : buf + 1;
    read_step(next, s + 1, step0);
    __builtin_amdgcn_sched_barrier(0);
    const int s_new = s + NSTAGE;
    mma_step_refill<Mma, NQ, NP, LAST>(acc, qf, pf, [&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      static_for<LPS>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        if constexpr (j * NM / LPS == i) issue(buf, s_new, j_c);
      });
    });
    buf = next;
  }
  for (; s < S - 1; s++) {  // drain: nothing left to fetch
    inner_steps(buf, s);
    const int younger = S - 2 - s < NSTAGE - 2 ? S - 2 - s : NSTAGE - 2;
    wait_next_stage(younger);
    lds_barrier();
    buf = buf + 1 == NSTAGE ? 0 : buf + 1;
    read_step(buf, s + 1, step0);
    mma_step<Mma, NQ, NP, NREADS, RPM, LAST, false>(acc, qf, pf);
  }
  inner_steps(buf, S - 1);
  mma_step<Mma, NQ, NP, NREADS, RPM, LAST, false>(acc, qf, pf);
}

// ---- main loop with an asymmetric ring -------------------------------------------------------------------------------
// Same pipeline, but the two operands have rings of different depth: the token operand P has 2 slots, the weight
// operand Q has 3 (2 + 3 slots of 32 KiB are the whole 160 KiB of LDS for a 256 x 256 x 64 tile).  At the boundary
// behind stage s the loads of P(s+2) and Q(s+3) are issued, in that order, so the wait for stage s+1 leaves only the
// QI loads of Q(s+2) outstanding: half of a stage's bytes are requested two stages ahead, and only the other half has
// to come back within one.
//   issue_p(slot, i) / issue_q(slot, j)   start the i-th / j-th load of this wave into that operand's ring slot; stages
//                                          are issued in order, so the callee advances its own source pointers
//   load(p_slot, q_slot, step, qf, pf)    read the fragments of step `step`
template <int NQ, int NP, int NREADS, int PI, int QI, int STEPS, class Mma = Bf16Mma, int RPM = 1, class IssueP,
          class IssueQ, class Load>
SMOE_DEV void gemm_mainloop_asym(const int S, typename Mma::Acc (&acc)[NQ][NP * Mma::PH], IssueP&& issue_p,
                                 IssueQ&& issue_q, Load&& load) {
  if (S <= 0) return;
  static_assert(STEPS % 2 == 0 && PI + 2 * QI < 64, "unsupported pipeline shape");
  typename Mma::Frag qf[2][NQ], pf[2][NP];
  constexpr int NM = NQ * NP, LPS = PI + QI, LAST = STEPS - 1;
  auto all_p = [&](int slot) { static_for<PI>([&](auto i_c) { issue_p(slot, i_c); }); };
  auto all_q = [&](int slot) { static_for<QI>([&](auto j_c) { issue_q(slot, j_c); }); };
  all_p(0);
  all_q(0);
  if (S > 1) {
    all_p(1);
    all_q(1);
  }
  if (S > 2) all_q(2);

  auto read_step = [&](int bp, int bq, auto step_c) {
    constexpr int step = decltype(step_c)::value;
    load(bp, bq, step_c, qf[Mma::qset(step)], pf[step & 1]);
  };
  auto inner_steps = [&](int bp, int bq) {
    static_for<STEPS - 1>([&](auto k_c) {
      constexpr int k = decltype(k_c)::value;
      read_step(bp, bq, std::integral_constant<int, k + 1>{});
      mma_step<Mma, NQ, NP, NREADS, RPM, k, false>(acc, qf, pf);
    });
  };
  constexpr std::integral_constant<int, 0> step0{};

  if (S > 2) wait_vmem_upto<PI + 2 * QI>();  // stage 0 has landed; P1, Q1, Q2 may still be on their way
  else wait_vmem_all();
  lds_barrier();
  read_step(0, 0, step0);
  int bp = 0, bq = 0, s = 0;
  for (; s + 3 < S; s++) {  // steady state: P(s+2) and Q(s+3) exist
    inner_steps(bp, bq);
    wait_vmem_upto<QI>();  // P(s+1) and Q(s+1) have landed; only Q(s+2) may still be on its way
    lds_barrier();
    const int np = bp ^ 1, nq = bq == 2 ? 0 : bq + 1;
    read_step(np, nq, step0);
    __builtin_amdgcn_sched_barrier(0);
    // the slots stage s leaves behind: P pieces first, then Q pieces
    mma_step_refill<Mma, NQ, NP, LAST>(acc, qf, pf, [&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      static_for<LPS>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        if constexpr (j * NM / LPS == i) {
          if constexpr (j < PI) issue_p(bp, j_c);
          else issue_q(bq, std::integral_constant<int, j - PI>{});
        }
      });
    });
    bp = np;
    bq = nq;
  }
  for (; s < S - 1; s++) {  // drain: at most P(s+2) is left to request
    inner_steps(bp, bq);
    wait_vmem_all();
    lds_barrier();
    if (s + 2 < S) all_p(bp);
    bp ^= 1;
    bq = bq == 2 ? 0 : bq + 1;
    read_step(bp, bq, step0);
    mma_step<Mma, NQ, NP, NREADS, RPM, LAST, false>(acc, qf, pf);
  }
  inner_steps(bp, bq);
  mma_step<Mma, NQ, NP, NREADS, RPM, LAST, false>(acc, qf, pf);
}


// ---- main loop over a STREAM of tiles ------------------------------------------------------------------------------
// A workgroup that works through several output tiles keeps the asymmetric ring running across the tile boundary: the
// stages of the next tile follow the last stage of the current one in the P and Q streams, so the first stages of the
// next tile are already in LDS when the current tile's epilogue starts, and the epilogue's stores drain while the next
// tile computes.  Only the epilogue itself (accumulators -> LDS -> global stores) is not overlapped.  It parks its rows
// in the two ring slots the tile's last stage has just vacated; the refill of those slots waits for the epilogue.
//   issue_p / issue_q / load   as in gemm_mainloop_asym
//   issued_p() / issued_q()    called after every stage issued to a stream: the callee counts stages and moves the
//                              stream's source pointers on to the next tile behind the S-th
//   first_boundary()           called once per tile behind the wait of its first stage, where no vector-memory
//                              operation of the wave is outstanding: the place to pick up ordinary loads issued in
//                              tile_end (a wait for them anywhere else would also wait for the ring)
//   tile_end(p_slot, q_slot)   epilogue of the finished tile; may use the two slots as scratch (every wave is past the
//                              barrier behind the last stage); advances the caller's tile state and returns false if
//                              the tile was the workgroup's last.  The accumulators need no clearing: the first
//                              k-slice of every tile starts them from zero
// QS = 3 is that asymmetric ring and needs S >= 3 (stage 0 of the next tile is requested at the latest behind stage S-3
// of the current one); QS = 2 is a plain double buffer (both operands two slots, one stage in flight, every wait is
// for everything) and needs S >= 2.  Stores and loads share one counter and may retire out of order with respect to
// each other, so the first wait of a tile is for everything; from then on only loads are outstanding and the counted
// waits are exact again.
template <int NQ, int NP, int NREADS, int PI, int QI, int STEPS, class Mma = Bf16Mma, int RPM = 1, int QS = 3,
          class IssueP, class IssueQ, class Load, class IssuedP, class IssuedQ, class First, class TileEnd>
SMOE_DEV void gemm_stream_loop(const int S, typename Mma::Acc (&acc)[NQ][NP * Mma::PH], IssueP&& issue_p,
                               IssueQ&& issue_q, Load&& load, IssuedP&& issued_p, IssuedQ&& issued_q,
                               First&& first_boundary, TileEnd&& tile_end) {
  static_assert(STEPS % 2 == 0 && PI + 2 * QI < 64, "unsupported pipeline shape");
  static_assert(STEPS > Mma::PH, "a stage holds more than one k-slice");
  static_assert(QS == 2 || QS == 3, "the weight operand's ring has two or three slots");
  constexpr int AHEAD = (QS - 2) * QI;  // loads of the stage after next that may be outstanding behind a stage
  typename Mma::Frag qf[2][NQ], pf[2][NP];
  constexpr int NM = NQ * NP, LPS = PI + QI, LAST = STEPS - 1;
  auto all_p = [&](int slot) {
    static_for<PI>([&](auto i_c) { issue_p(slot, i_c); });
    issued_p();
  };
  auto all_q = [&](int slot) {
    static_for<QI>([&](auto j_c) { issue_q(slot, j_c); });
    issued_q();
  };
  auto read_step = [&](int bp, int bq, auto step_c) {
    constexpr int step = decltype(step_c)::value;
    load(bp, bq, step_c, qf[Mma::qset(step)], pf[step & 1]);
  };
  // first_stage: the steps of the tile's first k-slice start the accumulators from the constant 0 operand instead of
  // reading them, so nobody has to clear 128 registers per lane between tiles
  auto inner_steps = [&](int bp, int bq, auto first_stage_c) {
    static_for<STEPS - 1>([&](auto k_c) {
      constexpr int k = decltype(k_c)::value;
      read_step(bp, bq, std::integral_constant<int, k + 1>{});
      mma_step<Mma, NQ, NP, NREADS, RPM, k, decltype(first_stage_c)::value && (k < Mma::PH)>(acc, qf, pf);
    });
  };
  constexpr std::false_type later{};
  constexpr std::integral_constant<int, 0> step0{};

  all_p(0);
  all_q(0);
  all_p(1);
  all_q(1);
  if constexpr (QS == 3) all_q(2);
  wait_vmem_upto<PI + QI + AHEAD>();
  lds_barrier();
  read_step(0, 0, step0);
  int bp = 0, bq = 0;
  // Branching code follows the last step of every stage (stream bookkeeping, the epilogue).  Without a use of the
  // accumulators in front of it the compiler sinks that step's matrix instructions past the branches to where their
  // results are first read (seen with the 16-register fragments): the matrix pipe idles and the step's operand
  // fragments stay alive into the epilogue.
  auto pin_accumulators = [&]() {
    if constexpr (Mma::FRAG_REGS > 4) {
#pragma unroll
      for (int q = 0; q < NQ; q++)
#pragma unroll
        for (int pp = 0; pp < NP * Mma::PH; pp++) asm volatile("" : "+v"(acc[q][pp]));
    }
  };
  // boundary behind a stage that is not the tile's last: read step 0 of the next stage, refill the vacated slots
  auto boundary = [&]() {
    lds_barrier();
    const int np = bp ^ 1, nq = bq == QS - 1 ? 0 : bq + 1;
    read_step(np, nq, step0);
    __builtin_amdgcn_sched_barrier(0);
    // P(s+2), Q(s+QS) into the slots stage s leaves behind
    mma_step_refill<Mma, NQ, NP, LAST>(acc, qf, pf, [&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      static_for<LPS>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        if constexpr (j * NM / LPS == i) {
          if constexpr (j < PI) issue_p(bp, j_c);
          else issue_q(bq, std::integral_constant<int, j - PI>{});
        }
      });
    });
    pin_accumulators();
    issued_p();
    issued_q();
    bp = np;
    bq = nq;
  };
  // 16-register accumulator fragments: a zero operand would occupy 16 registers through the whole loop, so the tile
  // is started by clearing the accumulators instead
  constexpr bool CLEAR = Mma::ACC_REGS > 4;
  constexpr std::integral_constant<bool, !CLEAR> first{};
  for (;;) {
    // stage 0: stores of the previous epilogue may still be outstanding, wait for everything
    if constexpr (CLEAR) clear_accumulators<Mma>(acc);
    inner_steps(bp, bq, first);
    wait_vmem_all();
    first_boundary();
    boundary();
    for (int s = 1; s + 1 < S; s++) {
      inner_steps(bp, bq, later);
      wait_vmem_upto<AHEAD>();  // P(s+1) and Q(s+1) have landed; only Q(s+2) may still be on its way
      boundary();
    }
    // last stage: the stages of the next tile that are due are already requested; its own slots become scratch
    inner_steps(bp, bq, later);
    wait_vmem_upto<AHEAD>();
    lds_barrier();
    mma_step<Mma, NQ, NP, NREADS, RPM, LAST, false>(acc, qf, pf);
    pin_accumulators();
    if (!tile_end(bp, bq)) break;
    wait_lds_all();
    lds_barrier();  // every wave has read its parked rows back: the two slots may be refilled
    all_p(bp);
    all_q(bq);
    bp ^= 1;
    bq = bq == QS - 1 ? 0 : bq + 1;
    read_step(bp, bq, step0);
  }
  wait_vmem_all();  // the streams ran ahead into ring slots nobody reads any more: let those loads land before the end
}

// ---- epilogue through LDS ----------------------------------------------------------------------------------------
// A wavefront parks its TR x TC accumulator tile (lane = tile row l%32, register quad = 4 consecutive columns) as
// bf16 in its own LDS region with padded rows, then reads it back row-contiguous and writes 16 bytes per lane.
template <int TC>
struct EpiLayout {
  static constexpr int ROW_BYTES = TC * 2 + 16;  // +16: quads of different rows fall into different banks
  static constexpr int LANES_PER_ROW = TC * 2 / 16;
  static constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
};

// store rows [0, TR) of the parked tile: global row = row_base + r (valid below row_limit), col = col_base + c.
// The LDS reads of a batch are issued together ahead of its stores: one LDS round trip per batch, not per store.
template <int TR, int TC>
SMOE_DEV void epilogue_flush(const char* region, int lane, uint16_t* out, int64_t out_stride, int row_base,
                             int row_limit, int col_base, int col_limit) {
  using L = EpiLayout<TC>;
  constexpr int NIT = TR / L::ROWS_PER_PASS, BATCH = NIT < 8 ? NIT : 8;
  static_assert(NIT % BATCH == 0, "passes come in whole batches");
  const int rr = lane / L::LANES_PER_ROW, cc = lane % L::LANES_PER_ROW;
  const int col = col_base + cc * 8;
  uint16_t* dst = out + (int64_t)(row_base + rr) * out_stride + col;
#pragma unroll
  for (int b0 = 0; b0 < NIT; b0 += BATCH) {
    u32x4 v[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; j++)
      v[j] = *(const u32x4*)(region + ((b0 + j) * L::ROWS_PER_PASS + rr) * L::ROW_BYTES + cc * 16);
#pragma unroll
    for (int j = 0; j < BATCH; j++) {
      const int r = (b0 + j) * L::ROWS_PER_PASS + rr;
      if (row_base + r < row_limit && col < col_limit)
        *(u32x4*)(dst + (int64_t)((b0 + j) * L::ROWS_PER_PASS) * out_stride) = v[j];
    }
  }
}

// 256 zero bytes: clamped (out-of-range) token rows of the weight-gradient GEMMs are fetched from here
static __device__ __attribute__((aligned(256))) const uint32_t smoe_zero_page[64] = {};

// park a few bytes of row `row` of an unpadded [32][RB-byte] LDS area; 16-byte chunk c sits at c ^ ((row >> 1) & 7)
template <int RB, class V>
SMOE_DEV void epi_park_y(char* area, int row, int col_bytes, V v) {
  constexpr int CH = RB / 16;
  const int chunk = (col_bytes >> 4) ^ ((row >> 1) & (CH < 8 ? CH - 1 : 7));
  *(V*)(area + row * RB + (chunk << 4) + (col_bytes & 15)) = v;
}

// ---- activations -------------------------------------------------------------------------------------------------
// The seven activation codes (smoe_activation) are four pointwise functions, gated (y = f(gate) * up, codes 0-2) or
// not (y = f(z)).  GELU is the exact erf form, the one the reference's torch backend evaluates.
enum Pointwise { PW_SILU = 0, PW_GELU = 1, PW_RELU = 2, PW_RELU_SQ = 3 };
constexpr bool act_is_glu(int act) { return act <= SMOE_ACT_REGLU; }
constexpr int act_pointwise(int act) {
  return act == SMOE_ACT_SWIGLU || act == SMOE_ACT_SILU ? PW_SILU
         : act == SMOE_ACT_GEGLU || act == SMOE_ACT_GELU ? PW_GELU
         : act == SMOE_ACT_REGLU || act == SMOE_ACT_RELU ? PW_RELU
                                                         : PW_RELU_SQ;
}

template <int PW>
SMOE_DEV float pointwise(float t) {
  if constexpr (PW == PW_SILU) return t * fast_sigmoid(t);
  else if constexpr (PW == PW_GELU) return t * (0.5f + 0.5f * erff(t * 0.70710678f));
  else if constexpr (PW == PW_RELU) return fmaxf(t, 0.f);
  else { const float r = fmaxf(t, 0.f); return r * r; }
}

// f(t) and f'(t)
template <int PW>
SMOE_DEV void pointwise_grad(float t, float& f, float& fp) {
  if constexpr (PW == PW_SILU) {
    const float sig = fast_sigmoid(t);
    f = t * sig;
    fp = f * (1.f - sig) + sig;
  } else if constexpr (PW == PW_GELU) {
    const float cdf = 0.5f + 0.5f * erff(t * 0.70710678f);
    f = t * cdf;
    fp = cdf + t * (0.39894228f * __expf(-0.5f * t * t));
  } else if constexpr (PW == PW_RELU) {
    f = fmaxf(t, 0.f);
    fp = t > 0.f ? 1.f : 0.f;
  } else {
    const float r = fmaxf(t, 0.f);
    f = r * r;
    fp = 2.f * r;
  }
}

// ---- epilogue of the forward GEMMs ---------------------------------------------------------------------------------
struct FwdEpilogueArgs {
  const uint16_t* bias;  // this expert's bias row (N values) or null
  uint16_t* out0;        // accumulator (+bias) as bf16: z resp. y2; null = not stored
  int64_t out0_stride;
  uint16_t* out1;        // activation output y1 (WITH_ACT only); null = not stored
  int64_t out1_stride;
  int m_base, row_end;   // first grouped row of this wave's tile, end of the expert's rows
  int n_base, N;         // first accumulator column of this wave's tile, number of accumulator columns
};

// Where a lane's accumulator registers sit in the wave's TM x TN tile: acc[fn][fm] is fragment (fn, fm) of FR x FR
// values; a lane owns token row fm * FR + l % FR and, in register group rg (QPF groups of four per fragment), the four
// consecutive features fn * FR + rg * 4 * (64 / FR) + 4 * (l / FR) + 0..3.
template <class Mma>
struct AccLayout {
  static constexpr int FR = Mma::FR, QPF = Mma::ACC_REGS / 4, NGRP = 64 / FR;
  static __device__ __forceinline__ int row(int lane) { return lane & (FR - 1); }
  static __device__ __forceinline__ int col(int rg, int lane) { return rg * (4 * NGRP) + 4 * (lane / FR); }
};

// acc is the wave's TM x TN tile.  Adds the bias, stores out0, and with WITH_ACT evaluates activation ACT from the
// un-rounded accumulator into out1 (TN/2 columns for the gated activations, TN otherwise).  The caller has made sure
// that no wave still reads the LDS ring: every wave parks its tile in its own region of it.
template <class Mma, int TM, int TN, bool WITH_ACT, int ACT>
SMOE_DEV void forward_epilogue(typename Mma::Acc (&acc)[TN / Mma::FR][TM / Mma::FR], char* smem, int wave, int lane,
                               const FwdEpilogueArgs& a) {
  using AL = AccLayout<Mma>;
  constexpr int FR = Mma::FR, FM = TM / FR, FN = TN / FR, QPF = AL::QPF;
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int PW = act_pointwise(ACT);
  if (a.bias != nullptr) {
    static_for<FN * QPF>([&](auto q_c) {
      constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
      int n = a.n_base + fn * FR + AL::col(rg, lane);
      n = n <= a.N - 4 ? n : a.N - 4;
      const u32x2 b = *(const u32x2*)(a.bias + n);
      const float b0 = bf16_lo(b[0]), b1 = bf16_hi(b[0]), b2 = bf16_lo(b[1]), b3 = bf16_hi(b[1]);
      static_for<FM>([&](auto fm_c) {
        constexpr int fm = decltype(fm_c)::value;
        acc[fn][fm][4 * rg + 0] += b0;
        acc[fn][fm][4 * rg + 1] += b1;
        acc[fn][fm][4 * rg + 2] += b2;
        acc[fn][fm][4 * rg + 3] += b3;
      });
    });
  }
  using LZ = EpiLayout<TN>;
  using LY = EpiLayout<TN / 2>;
  char* region = smem + wave * (TM * LZ::ROW_BYTES);
  const int lrow = AL::row(lane);
  if (!WITH_ACT || a.out0 != nullptr) {
    static_for<FM>([&](auto fm_c) {
      constexpr int fm = decltype(fm_c)::value;
      static_for<FN * QPF>([&](auto q_c) {
        constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
        u32x2 v = {pack_bf16x2(acc[fn][fm][4 * rg + 0], acc[fn][fm][4 * rg + 1]),
                   pack_bf16x2(acc[fn][fm][4 * rg + 2], acc[fn][fm][4 * rg + 3])};
        *(u32x2*)(region + (fm * FR + lrow) * LZ::ROW_BYTES + (fn * FR + AL::col(rg, lane)) * 2) = v;
      });
    });
    epilogue_flush<TM, TN>(region, lane, a.out0, a.out0_stride, a.m_base, a.row_end, a.n_base, a.N);
  }
  if constexpr (WITH_ACT && GLU) {
    if (a.out1 != nullptr) {
      static_for<FM>([&](auto fm_c) {
        constexpr int fm = decltype(fm_c)::value;
        static_for<FN * QPF>([&](auto q_c) {
          constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
          const float g0 = acc[fn][fm][4 * rg + 0], u0 = acc[fn][fm][4 * rg + 1];
          const float g1 = acc[fn][fm][4 * rg + 2], u1 = acc[fn][fm][4 * rg + 3];
          const uint32_t v = pack_bf16x2(pointwise<PW>(g0) * u0, pointwise<PW>(g1) * u1);
          *(uint32_t*)(region + (fm * FR + lrow) * LY::ROW_BYTES + (fn * FR + AL::col(rg, lane))) = v;
        });
      });
      epilogue_flush<TM, TN / 2>(region, lane, a.out1, a.out1_stride, a.m_base, a.row_end, a.n_base / 2, a.N / 2);
    }
  } else if constexpr (WITH_ACT) {
    if (a.out1 != nullptr) {
      static_for<FM>([&](auto fm_c) {
        constexpr int fm = decltype(fm_c)::value;
        static_for<FN * QPF>([&](auto q_c) {
          constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
          u32x2 v = {pack_bf16x2(pointwise<PW>(acc[fn][fm][4 * rg + 0]), pointwise<PW>(acc[fn][fm][4 * rg + 1])),
                     pack_bf16x2(pointwise<PW>(acc[fn][fm][4 * rg + 2]), pointwise<PW>(acc[fn][fm][4 * rg + 3]))};
          *(u32x2*)(region + (fm * FR + lrow) * LZ::ROW_BYTES + (fn * FR + AL::col(rg, lane)) * 2) = v;
        });
      });
      epilogue_flush<TM, TN>(region, lane, a.out1, a.out1_stride, a.m_base, a.row_end, a.n_base, a.N);
    }
  }
}

// One 32-row batch of that epilogue, parked in a caller-chosen LDS region of 32 padded rows
// (32 * EpiLayout<TN>::ROW_BYTES bytes per wave): for kernels whose ring keeps running during the epilogue.
// frag(fn_c, sub_c) names the accumulator fragment (fn, sub) of the batch (sub = fragment row inside the batch);
// m0 = first grouped row of the batch.
template <class Mma, int TN, bool WITH_ACT, int ACT, class FragAt>
SMOE_DEV void forward_epilogue_batch(FragAt&& frag, char* region, int lane, const FwdEpilogueArgs& a, int m0) {
  using AL = AccLayout<Mma>;
  constexpr int FR = Mma::FR, FN = TN / FR, QPF = AL::QPF, RB = 32 / FR;  // RB fragment rows make a 32-row batch
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int PW = act_pointwise(ACT);
  using LZ = EpiLayout<TN>;
  using LY = EpiLayout<TN / 2>;
  const int lrow = AL::row(lane);
  if (a.bias != nullptr) {  // re-read per batch (a few cached words) rather than held in registers across the batches
    static_for<FN * QPF>([&](auto q_c) {
      constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
      int n = a.n_base + fn * FR + AL::col(rg, lane);
      n = n <= a.N - 4 ? n : a.N - 4;
      const u32x2 b = *(const u32x2*)(a.bias + n);
      static_for<RB>([&](auto sub_c) {
        auto& f = frag(std::integral_constant<int, fn>{}, sub_c);
        f[4 * rg + 0] += bf16_lo(b[0]);
        f[4 * rg + 1] += bf16_hi(b[0]);
        f[4 * rg + 2] += bf16_lo(b[1]);
        f[4 * rg + 3] += bf16_hi(b[1]);
      });
    });
  }
  if (!WITH_ACT || a.out0 != nullptr) {
    static_for<RB>([&](auto sub_c) {
      constexpr int sub = decltype(sub_c)::value;
      static_for<FN * QPF>([&](auto q_c) {
        constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
        const auto& f = frag(std::integral_constant<int, fn>{}, sub_c);
        u32x2 v = {pack_bf16x2(f[4 * rg + 0], f[4 * rg + 1]), pack_bf16x2(f[4 * rg + 2], f[4 * rg + 3])};
        *(u32x2*)(region + (sub * FR + lrow) * LZ::ROW_BYTES + (fn * FR + AL::col(rg, lane)) * 2) = v;
      });
    });
    epilogue_flush<32, TN>(region, lane, a.out0, a.out0_stride, m0, a.row_end, a.n_base, a.N);
  }
  if constexpr (WITH_ACT && GLU) {
    if (a.out1 != nullptr) {
      static_for<RB>([&](auto sub_c) {
        constexpr int sub = decltype(sub_c)::value;
        static_for<FN * QPF>([&](auto q_c) {
          constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
          const auto& f = frag(std::integral_constant<int, fn>{}, sub_c);
          const float g0 = f[4 * rg + 0], u0 = f[4 * rg + 1];
          const float g1 = f[4 * rg + 2], u1 = f[4 * rg + 3];
          const uint32_t v = pack_bf16x2(pointwise<PW>(g0) * u0, pointwise<PW>(g1) * u1);
          *(uint32_t*)(region + (sub * FR + lrow) * LY::ROW_BYTES + (fn * FR + AL::col(rg, lane))) = v;
        });
      });
      epilogue_flush<32, TN / 2>(region, lane, a.out1, a.out1_stride, m0, a.row_end, a.n_base / 2, a.N / 2);
    }
  } else if constexpr (WITH_ACT) {
    if (a.out1 != nullptr) {
      static_for<RB>([&](auto sub_c) {
        constexpr int sub = decltype(sub_c)::value;
        static_for<FN * QPF>([&](auto q_c) {
          constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
          const auto& f = frag(std::integral_constant<int, fn>{}, sub_c);
          u32x2 v = {pack_bf16x2(pointwise<PW>(f[4 * rg + 0]), pointwise<PW>(f[4 * rg + 1])),
                     pack_bf16x2(pointwise<PW>(f[4 * rg + 2]), pointwise<PW>(f[4 * rg + 3]))};
          *(u32x2*)(region + (sub * FR + lrow) * LZ::ROW_BYTES + (fn * FR + AL::col(rg, lane)) * 2) = v;
        });
      });
      epilogue_flush<32, TN>(region, lane, a.out1, a.out1_stride, m0, a.row_end, a.n_base, a.N);
    }
  }
}

// The whole wave tile, 32 rows at a time, from accumulators the compiler holds
template <class Mma, int TM, int TN, bool WITH_ACT, int ACT>
SMOE_DEV void forward_epilogue_rows(typename Mma::Acc (&acc)[TN / Mma::FR][TM / Mma::FR], char* region, int lane,
                                    const FwdEpilogueArgs& a) {
  constexpr int RB = 32 / Mma::FR;
  static_for<TM / 32>([&](auto blk_c) {
    constexpr int blk = decltype(blk_c)::value;
    forward_epilogue_batch<Mma, TN, WITH_ACT, ACT>(
        [&](auto fn_c, auto sub_c) -> typename Mma::Acc& {
          return acc[decltype(fn_c)::value][blk * RB + decltype(sub_c)::value];
        },
        region, lane, a, a.m_base + blk * 32);
  });
}

// ---- accumulators of the hand-scheduled loop -------------------------------------------------------------------------
// The tile loop of tile_loop_gen.h leaves its results in the accumulation registers a[0:255], which the compiler does
// not know about: they are read out four at a time, in program order (volatile), while the epilogue runs.
template <int R>
SMOE_DEV f32x4 agpr_read4() {
  f32x4 r;
  asm volatile(
      "v_accvgpr_read_b32 %0, a[%4]\n\tv_accvgpr_read_b32 %1, a[%5]\n\tv_accvgpr_read_b32 %2, a[%6]\n\t"
      "v_accvgpr_read_b32 %3, a[%7]"
      : "=v"(r[0]), "=v"(r[1]), "=v"(r[2]), "=v"(r[3])
      : "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
  return r;
}

// forward epilogue of a wave tile whose FN x FM fragments of 16 x 16 sit in a[4 * (fn * FM + fm) ..]
template <class Mma, int TM, int TN, bool WITH_ACT, int ACT>
SMOE_DEV void forward_epilogue_rows_agpr(char* region, int lane, const FwdEpilogueArgs& a) {
  static_assert(Mma::ACC_REGS == 4, "four accumulator registers per fragment");
  constexpr int FR = Mma::FR, FN = TN / FR, FM = TM / FR, RB = 32 / FR;
  static_for<TM / 32>([&](auto blk_c) {
    constexpr int blk = decltype(blk_c)::value;
    f32x4 loc[FN][RB];
    static_for<RB>([&](auto sub_c) {
      constexpr int sub = decltype(sub_c)::value;
      static_for<FN>([&](auto fn_c) {
        constexpr int fn = decltype(fn_c)::value;
        loc[fn][sub] = agpr_read4<4 * (fn * FM + blk * RB + sub)>();
      });
    });
    forward_epilogue_batch<Mma, TN, WITH_ACT, ACT>(
        [&](auto fn_c, auto sub_c) -> f32x4& { return loc[decltype(fn_c)::value][decltype(sub_c)::value]; }, region,
        lane, a, a.m_base + blk * 32);
  });
}

// ---- epilogue of the activation-gradient GEMM of the down projection (dz) -------------------------------------------
// acc = dy1 (token rows x I columns) of the wave's TM x TN tile.  32 token rows at a time the wavefront stages its z
// sub-tile (32 rows x ZW*TN bf16; ZW = 2 interleaved (gate, up) columns per dy1 column for gated activations, 1
// otherwise) through LDS: row-contiguous 16-byte global loads (PF batches in flight in registers) -> LDS -> each lane
// picks the z values of its four dy1 columns of its token rows, computes dz in place and y1s into a second area -> both
// are written back row-contiguous.  All global traffic of the epilogue is full 128-byte lines.
struct DzEpilogueArgs {
  const uint16_t* zin;
  int64_t zin_stride;
  uint16_t* dz;  // (rows, ZW * N) bf16
  int64_t dz_stride;
  uint16_t* y1s;  // (rows, N) bf16: score * act(z)
  int64_t y1s_stride;
  const float* scores;
  const int32_t* sidx;
  float* ds_partial;  // (rows, ds_cols) fp32: this wave writes column ds_col, sum_i dy1 * y1 over its columns
  int ds_cols, ds_col;
  int ds_pad_col1;  // 1 + a second column of this wave's rows that is written as zero (0: none): the table's pitch is
                    // fixed by the widest kernel, a kernel with fewer waves per tile fills the columns it has no sum for
  int m_base, row_end;  // first grouped row of this wave's tile, end of the expert's rows
  int n_base, N;        // first dy1 column of this wave's tile, number of dy1 columns (I)
  // with QUANT: dz once more as e4m3 bytes (rows, ZW * N) with one power-of-two scale per 32 columns, the operand format
  // of the fp8 GEMMs: scale word [c / 128][row] of a (ZW * N / 128, dzq_rows) table, byte (c / 32) % 4.  Quantised
  // from the bf16-rounded values, so it equals quantising the stored dz.
  uint8_t* dzq;
  uint32_t* dzq_scales;
  int64_t dzq_rows;
};

template <int TN, int ACT, int BR = 32>
struct DzStaging {
  static constexpr int ZW = act_is_glu(ACT) ? 2 : 1;
  static constexpr int ZB = TN * 2 * ZW, YB = TN * 2;  // bytes per staged z / dz row, y1s row
  static constexpr int BYTES = BR * (ZB + YB);         // per wavefront: BR token rows are staged at a time
};

// e8m0 exponent of the smallest power of two s with amax / s <= 448 (the largest e4m3 value): no element saturates
SMOE_DEV int mx_scale_exponent(float amax) {
  if (!(amax > 0.f)) return 0;
  // amax = m * 2^e with m in [1, 2): 448 = 1.75 * 2^8 -> need 2^k >= amax / 448
  const uint32_t bits = __float_as_uint(amax);
  const int e = (int)((bits >> 23) & 0xff) - 127;
  const uint32_t mant = bits & 0x7fffffu;
  int k = e - 8;                      // 2^(e-8) * 448 = 1.75 * 2^e
  if (mant > 0x600000u) k += 1;       // m > 1.75
  k += 127;
  return k < 0 ? 0 : (k > 254 ? 254 : k);
}

// frag(fn_c, fm_c) hands out the accumulator fragment (fn, fm) of the wave tile, by reference or by value; every
// fragment is asked for once per register group, in the order the batches consume them.
template <class Mma, int TM, int TN, int ACT, int PF = 2, bool QUANT = false, int BR = 32, class FragAt, class RingIdle>
SMOE_DEV void dz_epilogue_at(FragAt&& frag, char* zbuf, int lane, const DzEpilogueArgs& a, RingIdle&& ring_idle) {
  using AL = AccLayout<Mma>;
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int PW = act_pointwise(ACT);
  constexpr int FR = Mma::FR, FN = TN / FR, QPF = AL::QPF;
  constexpr int ZW = DzStaging<TN, ACT>::ZW, ZB = DzStaging<TN, ACT>::ZB, YB = DzStaging<TN, ACT>::YB;
  constexpr int ZL = ZB / 16, ZR = 64 / ZL, ZN = BR / ZR;  // lanes per row, rows per instruction, instructions
  constexpr int YL = YB / 16, YR = 64 / YL, YN = BR / YR;
  constexpr int ZSW = ZL < 16 ? ZL - 1 : 15;  // row swizzle of the staged z chunks
  constexpr int NB = TM / BR, RB = BR / FR;   // batches of BR rows; fragment rows per batch
  static_assert(BR % FR == 0 && ZN >= 1 && YN >= 1, "a batch is whole fragment rows and whole load instructions");
  static_assert(PF >= 1 && PF <= 4, "one to four batches of z are prefetched");
  // N is a multiple of 64 (checked by the entry points): a wave tile of at most 64 columns lies wholly inside or wholly
  // outside the matrix, so the column test of the score-gradient sum is made once per row instead of once per value
  constexpr bool COLS_WHOLE = 64 % TN == 0;
  char* ybuf = zbuf + BR * ZB;
  const int zr = lane / ZL, zc = lane % ZL, yr = lane / YL, yc = lane % YL;
  const int zlimit = ZW * a.N;
  const int zcol = ZW * a.n_base + zc * 8;  // first z column of this lane's 16-byte chunk
  const int zcol_c = zcol <= zlimit - 8 ? zcol : zlimit - 8;
  // Global addresses are a wave-uniform anchor (the wave's first row; for the loads, which clamp rows behind the
  // expert's end to its last row, the earlier of the two) plus a 32-bit byte offset whose per-lane part is fixed for the
  // whole epilogue: an access costs at most two vector instructions of address arithmetic instead of a 64-bit
  // multiply-add, and the epilogue is bound by its vector instructions (a wave evaluates the activation's derivative for
  // TM x TN values per tile).
  const int m_base = __builtin_amdgcn_readfirstlane(a.m_base), m_last = __builtin_amdgcn_readfirstlane(a.row_end) - 1;
  const int m_anchor = m_base < m_last ? m_base : m_last;
  const int rows_left = m_last + 1 - m_base;  // valid rows from the wave's first row on (may be <= 0)
  const uint32_t zin_rb = (uint32_t)a.zin_stride * 2u, dz_rb = (uint32_t)a.dz_stride * 2u, y_rb = (uint32_t)a.y1s_stride * 2u;
  const char* zin_anchor = (const char*)(a.zin + (int64_t)m_anchor * a.zin_stride);
  char* dz_anchor = (char*)(a.dz + (int64_t)m_base * a.dz_stride);
  char* y_anchor = (char*)(a.y1s + (int64_t)m_base * a.y1s_stride);
  const uint32_t zin_lane = (uint32_t)zr * zin_rb + (uint32_t)zcol_c * 2u;
  const uint32_t zin_max = (uint32_t)(m_last - m_anchor) * zin_rb + (uint32_t)zcol_c * 2u;
  const uint32_t dz_lane = (uint32_t)zr * dz_rb + (uint32_t)zcol * 2u;
  const uint32_t y_lane = (uint32_t)yr * y_rb + (uint32_t)(a.n_base + yc * 8) * 2u;
  u32x4 zreg[PF][ZN];
  auto fetch_z = [&](int blk, u32x4(&dst)[ZN]) {
#pragma unroll
    for (int it = 0; it < ZN; it++) {
      uint32_t off = zin_lane + (uint32_t)(blk * BR + it * ZR + (m_base - m_anchor)) * zin_rb;
      off = off < zin_max ? off : zin_max;
      dst[it] = *(const u32x4*)(zin_anchor + off);
    }
  };
  static_for<(PF < NB ? PF : NB)>([&](auto i_c) { fetch_z(decltype(i_c)::value, zreg[decltype(i_c)::value]); });
  ring_idle();  // the staging areas lie in the ring: every wave must be done reading it
  static_for<NB>([&](auto blk_c) {
    constexpr int blk = decltype(blk_c)::value;
#pragma unroll
    for (int it = 0; it < ZN; it++) {
      const int r = it * ZR + zr;
      *(u32x4*)(zbuf + r * ZB + ((zc ^ (r & ZSW)) << 4)) = zreg[blk % PF][it];
    }
    if constexpr (blk + PF < NB) fetch_z(blk + PF, zreg[blk % PF]);
    static_for<RB>([&](auto sub_c) {
      constexpr int sub = decltype(sub_c)::value, fm = blk * RB + sub;
      const int mrow = sub * FR + AL::row(lane);  // row inside the staged batch
      const int m = a.m_base + blk * BR + mrow;
      const bool mvalid = m < a.row_end;
      float sc = 0.f, dsum = 0.f;
      if (mvalid) sc = a.scores[a.sidx[m]];
      static_for<FN * QPF>([&](auto q_c) {
        constexpr int fn = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
        const int il = fn * FR + AL::col(rg, lane);  // first of this lane's 4 dy1 columns (wave-local)
        const int zbyte = il * 2 * ZW;                // their z bytes inside the staged row
        char* zaddr = zbuf + mrow * ZB + (((zbyte >> 4) ^ (mrow & ZSW)) << 4) + (zbyte & 15);
        float ys[4];
        const auto& dyf = frag(std::integral_constant<int, fn>{}, std::integral_constant<int, fm>{});
        if constexpr (GLU) {
          const u32x4 zz = *(const u32x4*)zaddr;
          u32x4 dzv;
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float dy = dyf[4 * rg + q];
            const float g = bf16_lo(zz[q]), u = bf16_hi(zz[q]);
            float f, fp;
            pointwise_grad<PW>(g, f, fp);
            const float y1v = f * u;
            if (COLS_WHOLE || a.n_base + il + q < a.N) dsum += dy * y1v;
            const float sd = sc * dy;
            dzv[q] = pack_bf16x2(sd * u * fp, sd * f);
            ys[q] = sc * y1v;
          }
          *(u32x4*)zaddr = dzv;
        } else {
          const u32x2 zz = *(const u32x2*)zaddr;
          float dzf[4];
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float dy = dyf[4 * rg + q];
            const float t = (q & 1) ? bf16_hi(zz[q >> 1]) : bf16_lo(zz[q >> 1]);
            float f, fp;
            pointwise_grad<PW>(t, f, fp);
            if (COLS_WHOLE || a.n_base + il + q < a.N) dsum += dy * f;
            dzf[q] = sc * dy * fp;
            ys[q] = sc * f;
          }
          *(u32x2*)zaddr = u32x2{pack_bf16x2(dzf[0], dzf[1]), pack_bf16x2(dzf[2], dzf[3])};
        }
        u32x2 yv = {pack_bf16x2(ys[0], ys[1]), pack_bf16x2(ys[2], ys[3])};
        epi_park_y<YB>(ybuf, mrow, il * 2, yv);
      });
      if (COLS_WHOLE && a.n_base >= a.N) dsum = 0.f;
      // the 64 / FR lanes that share a token row hold disjoint columns: add their partial sums
      dsum += __shfl_xor(dsum, 32, 64);
      if constexpr (FR == 16) dsum += __shfl_xor(dsum, 16, 64);
      if (mvalid && lane < FR) {
        a.ds_partial[(int64_t)m * a.ds_cols + a.ds_col] = dsum;
        if (a.ds_pad_col1 > 0) a.ds_partial[(int64_t)m * a.ds_cols + a.ds_pad_col1 - 1] = 0.f;
      }
    });
#pragma unroll
    for (int it = 0; it < ZN; it++) {
      const int r = it * ZR + zr;
      const u32x4 v = *(const u32x4*)(zbuf + r * ZB + ((zc ^ (r & ZSW)) << 4));
      const int r0 = blk * BR + it * ZR;  // first row of this store instruction, relative to the wave's first row
      const int mm = m_base + r0 + zr;
      const bool live = zr < rows_left - r0 && zcol < zlimit;
      if (live) *(u32x4*)(dz_anchor + (size_t)r0 * dz_rb + dz_lane) = v;
      if constexpr (QUANT) {
        // 32 columns = the 16-byte chunks of 4 consecutive lanes
        float x[8];
        float amax = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          x[2 * q] = bf16_lo(v[q]);
          x[2 * q + 1] = bf16_hi(v[q]);
          amax = fmaxf(amax, fmaxf(fabsf(x[2 * q]), fabsf(x[2 * q + 1])));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        const int ex = mx_scale_exponent(amax);
        const float inv = __uint_as_float((uint32_t)(254 - ex) << 23);
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(x[0] * inv, x[1] * inv, 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(x[2] * inv, x[3] * inv, w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(x[4] * inv, x[5] * inv, 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(x[6] * inv, x[7] * inv, w1, true);
        if (live) {
          *(u32x2*)(a.dzq + (int64_t)mm * zlimit + zcol) = u32x2{(uint32_t)w0, (uint32_t)w1};
          if ((zc & 3) == 0)
            ((uint8_t*)a.dzq_scales)[((int64_t)(zcol >> 7) * a.dzq_rows + mm) * 4 + ((zcol >> 5) & 3)] = (uint8_t)ex;
        }
      }
    }
#pragma unroll
    for (int it = 0; it < YN; it++) {
      const int r = it * YR + yr;
      const u32x4 v = *(const u32x4*)(ybuf + r * YB + ((yc ^ ((r >> 1) & (YL < 8 ? YL - 1 : 7))) << 4));
      const int r0 = blk * BR + it * YR;
      if (yr < rows_left - r0 && a.n_base + yc * 8 < a.N) *(u32x4*)(y_anchor + (size_t)r0 * y_rb + y_lane) = v;
    }
  });
}

// accumulators the compiler holds
template <class Mma, int TM, int TN, int ACT, int PF = 2, bool QUANT = false, int BR = 32, class RingIdle>
SMOE_DEV void dz_epilogue(typename Mma::Acc (&acc)[TN / Mma::FR][TM / Mma::FR], char* zbuf, int lane,
                          const DzEpilogueArgs& a, RingIdle&& ring_idle) {
  dz_epilogue_at<Mma, TM, TN, ACT, PF, QUANT, BR>(
      [&](auto fn_c, auto fm_c) -> const typename Mma::Acc& { return acc[decltype(fn_c)::value][decltype(fm_c)::value]; },
      zbuf, lane, a, ring_idle);
}

// ---- tuning knobs ----------------------------------------------------------------------------------------------
// Read from the environment ONCE, at the first launch that asks (variable = "SMOE_" + the upper-cased field name);
// smoe_set_tuning() overrides a knob afterwards (tests walk through the alternative kernels with it).
struct Tuning {
  int gemm_stream;          // 1 (default): up-projection forward, down-projection forward and dx run as tile streams
  int gemm_stream_grid;     // workgroups of the tile-stream kernels; 0 (default) = one per compute unit
  int varlen_k_tile_order;  // 2 blocked (default), 0 single tiles round-robin over the XCDs, 1 whole experts per XCD
  int dz_stream;            // 1: dz runs as a tile stream too (with gemm_stream); 0: one tile per workgroup
  int gemm_asm;             // 1: the tile streams run on the hand-scheduled four-wavefront loop (tile_loop_gen.h)
};
const Tuning& tuning();

// number of compute units of the current device (looked up once per device)
int device_compute_units(int* out);

// ---- launch helper -------------------------------------------------------------------------------------------------
// Raise a kernel's dynamic-LDS limit once per device (the attribute is per device; a repeated call is harmless, so the
// flags need no lock).
struct LdsLimitOnce {
  bool done[64] = {};
  int ensure(const void* kernel, int bytes) {
    int dev = 0;
    SMOE_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64 || !done[dev]) {
      SMOE_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
      if (dev >= 0 && dev < 64) done[dev] = true;
    }
    return SMOE_OK;
  }
};

// ---- tile map ------------------------------------------------------------------------------------------------
// Built on the device from the expert offsets; header[0] = number of token tiles.  Entry i = (expert, first row).
struct TileMap {
  int32_t* header;  // [4]
  int32_t* expert;  // [max_tiles]
  int32_t* row0;    // [max_tiles]
};

static inline int64_t max_token_tiles(int64_t TK, int E, int BM) { return TK / BM + E; }

static inline size_t tile_map_bytes(int64_t TK, int E) {
  // sized for the smallest token tile any kernel uses (64 rows)
  return (size_t)(4 + 2 * max_token_tiles(TK, E, 64)) * sizeof(int32_t);
}

static inline TileMap carve_tile_map(void* ws, int64_t TK, int E, int BM) {
  TileMap t;
  t.header = (int32_t*)ws;
  t.expert = t.header + 4;
  t.row0 = t.expert + max_token_tiles(TK, E, BM);
  return t;
}

// single workgroup of 1024 threads
__global__ void build_tile_map_kernel(const int32_t* __restrict__ off, int E, int BM, TileMap tm);

int launch_build_tile_map(const int32_t* off, const int32_t* order, int E, int BM, TileMap tm, hipStream_t st);

// XCD-aware linear tile id: workgroups are dealt round-robin to the 8 XCDs, so workgroup b runs on XCD b % 8;
// give every XCD one contiguous range of the tile space so that tiles sharing operands share an L2.
SMOE_DEV int64_t xcd_linear_tile_of(int64_t b, int64_t total) {
  const int64_t per = (total + 7) >> 3;
  const int64_t slot = b >> 3;
  if (slot >= per) return -1;
  const int64_t lin = (b & 7) * per + slot;
  return lin < total ? lin : -1;
}
SMOE_DEV int64_t xcd_linear_tile(int64_t total) { return xcd_linear_tile_of(blockIdx.x, total); }

// The tiles a persistent workgroup of a tile-stream kernel walks through: virtual workgroup vb = b, b + gridDim.x, ...
// of the XCD-aware order of the one-tile-per-workgroup kernels (groups of GM token tiles share a feature panel).  The
// bookkeeping is read through the constant address space: uniform addresses then become scalar loads, which do not
// touch the vector-memory counter the ring is timed with.
struct StreamTile {
  int e, row0, row_end, n0;
  bool valid;
};
struct StreamTiles {
  typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
  const_i32_ptr expert, row0, off;
  int num_m_tiles, n_tiles, bn;
  int64_t total, per_xcd;
  __device__ __forceinline__ StreamTiles(const TileMap& tm, const int32_t* off_, int n_tiles_, int bn_)
      : expert((const_i32_ptr)tm.expert), row0((const_i32_ptr)tm.row0), off((const_i32_ptr)off_), n_tiles(n_tiles_),
        bn(bn_) {
    num_m_tiles = ((const_i32_ptr)tm.header)[0];
    total = (int64_t)num_m_tiles * n_tiles;
    per_xcd = (total + 7) >> 3;
  }
  __device__ __forceinline__ StreamTile at(int64_t vb) const {
    StreamTile t = {0, 0, 1, 0, false};
    const int64_t slot = vb >> 3;
    const int64_t lin = (vb & 7) * per_xcd + slot;
    if (slot < per_xcd && lin < total) {
      constexpr int GM = 8;
      const int64_t per_group = (int64_t)GM * n_tiles;
      const int group = (int)(lin / per_group);
      const int first_m = group * GM;
      const int gm = num_m_tiles - first_m < GM ? num_m_tiles - first_m : GM;
      const int within = (int)(lin - (int64_t)group * per_group);
      const int mt = first_m + within % gm;
      t.e = expert[mt];
      t.row0 = row0[mt];
      t.row_end = off[t.e + 1];
      t.n0 = (within / gm) * bn;
      t.valid = true;
    }
    return t;
  }
};

int launch_ds_finalize(const float* ds_partial, int ncols, const int32_t* sidx, float* ds, int64_t TK, hipStream_t st);

// out[e][c] = sum_{m in [off[e], off[e+1])} w_m * src[row(m)][c]  (bf16 out, fp32 accumulate, zeros for empty experts);
// row(m) = gidx[m] or m, w_m = scores[sidx[m]] or 1.  The per-expert bias gradients db1 (src = dz) and db2 (src = dout).
int launch_expert_colsum(const uint16_t* src, int64_t src_stride, int ncols, const int32_t* gidx, const float* scores,
                         const int32_t* sidx, const int32_t* off, int E, uint16_t* out, hipStream_t st);
// ds[sidx[m]] += <dout[gidx[m]], b2[e(m)]>: the bias term of the score gradient
int launch_ds_bias_term(const uint16_t* dout, const uint16_t* b2, const int32_t* gidx, const int32_t* sidx,
                        const int32_t* off, int E, int H, float* ds, int64_t TK, hipStream_t st);

}  // namespace smoe
