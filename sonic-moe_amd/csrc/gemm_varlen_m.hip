// Grouped GEMM over ragged token groups ("varlen-M"): for every expert e and every grouped row m of that expert
//     C[m, n] = sum_k P[row(m), k] * Q_e[n, k]
// with fused epilogues.  Four roles of the MoE layer share the main loop:
//   up-projection forward    P = x rows gathered by x_gather_idx, Q = W1[e] (K-major)   -> z (+b1), y1 = act(z)
//   down-projection forward  P = y1 rows,                          Q = W2[e] (K-major)   -> y2 (+b2)
//   down-proj activation grad P = dout rows gathered,              Q = W2[e] (MN-major)  -> dz, y1s, ds partials
//   up-proj activation grad  P = dz rows,                          Q = W1[e] (MN-major)  -> dx_expanded
#include "gemm_common.h"
#include "tile_loop_gen.h"

namespace smoe {

// ROLE_COMBINE: the down-projection forward that adds its score-weighted rows onto the tokens' output rows instead of
// storing y2 (opt-in, atomic: combine_epilogue_batch)
enum Role { ROLE_UP_FWD = 0, ROLE_PLAIN = 1, ROLE_DZ = 2, ROLE_COMBINE = 3 };

struct VarlenMParams {
  const uint16_t* P;
  int64_t p_stride;
  const int32_t* gidx;  // nullable: P rows are the grouped rows themselves
  int64_t p_rows;       // rows of P when gathered (the range of gidx)
  const uint16_t* Q;
  int64_t q_stride_e, q_stride_row;
  const int32_t* off;
  const int32_t* order;  // nullable: the tile map lists the experts in this order (a permutation of 0 .. E-1)
  TileMap tm;
  int N, Kdim, n_tiles;
  uint16_t* out0;
  int64_t out0_stride;
  uint16_t* out1;
  int64_t out1_stride;
  const uint16_t* bias;  // nullable: (E, N) added to the accumulator before the epilogue
  const uint16_t* zin;
  int64_t zin_stride;
  const float* scores;
  const int32_t* sidx;
  float* ds_partial;
  int ds_cols;
  const int32_t* out_rows;  // ROLE_COMBINE: grouped row -> row of out0 (the token)
};

template <int BM_, int BN_, int WM_, int WN_, bool QMN_, int BK_, int NSTAGE_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, BK = BK_, NSTAGE = NSTAGE_;
  static constexpr bool QMN = QMN_;
  static constexpr int NW = WM * WN, NT = NW * 64;
  typedef ElemMma Mma;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int FR = Mma::FR;                       // rows / columns of a matrix-instruction fragment
  static constexpr int FM = TM / FR, FN = TN / FR;         // fragments of the wave tile
  static constexpr int NP = FM / Mma::PH;                  // token fragments a step works on
  static constexpr int KSL = BK / Mma::KSTEP;              // k-slices per stage
  static constexpr int STEPS = KSL * Mma::PH;              // steps per stage
  static constexpr int P_STAGE = BM * BK * 2, Q_STAGE = BN * BK * 2;  // bytes
  static constexpr int STAGE = P_STAGE + Q_STAGE;
  static constexpr int P_INSTR = P_STAGE / 1024 / NW;  // direct-to-LDS loads per wave and stage
  static constexpr int Q_INSTR = Q_STAGE / 1024 / NW;
  static constexpr int KROW = BK * 2;                   // bytes per row of a K-major stage
  static constexpr int EPI = NW * TM * (TN * 2 + 16);   // per-wave parking regions of the LDS epilogue
  // ring: 2 slots of the token operand, then 3 slots of the weight operand (NSTAGE is not used by this kernel)
  static constexpr int P_SLOTS = 2, Q_SLOTS = 3;
  static constexpr int RING = P_SLOTS * P_STAGE + Q_SLOTS * Q_STAGE;
  static constexpr int SMEM = RING > EPI ? RING : EPI;
  // MN-major Q stage geometry
  static constexpr int ROWB = BN * 2;     // bytes per k-row
  static constexpr int LPR = ROWB / 16;   // lanes (16-byte pieces) per k-row
  static constexpr int RPI = 64 / LPR;    // k-rows per load instruction
  static constexpr int KPR = KROW / 16;   // 16-byte pieces per row of a K-major stage
  static constexpr int KRPI = 64 / KPR;   // rows per load instruction of a K-major stage
  static constexpr int NG = ROWB / 32;    // 32-byte groups per k-row
  static_assert(P_INSTR >= 1 && Q_INSTR >= 1, "tile too small for the wave count");
  static_assert(TM % 32 == 0 && TN % 32 == 0 && FM % Mma::PH == 0, "wave tile must be a multiple of 32 x 32");
  static_assert(SMEM <= 160 * 1024, "LDS budget of a CU");
};

// Per-lane LDS fragment offsets (bytes inside a ring slot) of wave (wm, wn): p_off[ksl] / q_off[ksl] for K-major
// stages (one 16-byte piece per k-slice ksl; fragment f of the wave lies f * FR rows further), q_off[2 * fn + h] for an
// MN-major weight stage (two transpose loads per fragment; k-slice ksl lies ksl * KSTEP k-rows further).
// A fragment lane supplies row (K-major) or column (MN-major) l % FR and the 8 contraction elements 8 * (l / FR) + 0..7
// of the k-slice.
template <class C>
SMOE_DEV void fragment_offsets(int wm, int wn, int lane, int (&p_off)[C::KSL], int (&q_off)[C::QMN ? 2 * C::FN : C::KSL]) {
  constexpr int FR = C::FR, PPS = C::Mma::KSTEP / 8;  // 16-byte pieces per row and k-slice
  {
    const int row = wm * C::TM + (lane & (FR - 1));
    const int sw = kswz<C::BK, C::FR>(row);
#pragma unroll
    for (int ks = 0; ks < C::KSL; ks++) p_off[ks] = row * C::KROW + (((PPS * ks + lane / FR) ^ sw) << 4);
  }
  if constexpr (!C::QMN) {
    const int row = wn * C::TN + (lane & (FR - 1));
    const int sw = kswz<C::BK, C::FR>(row);
#pragma unroll
    for (int ks = 0; ks < C::KSL; ks++) q_off[ks] = row * C::KROW + (((PPS * ks + lane / FR) ^ sw) << 4);
  } else {
    // the transpose load hands lane i of a 16-lane group column i of a 4 (k) x 16 (n) block; the lanes' addresses name
    // its four k-rows, 4 lanes x 8 bytes each
    const int grp = lane >> 4, i16 = lane & 15;
    const int kk = (FR == 32 ? 8 * (grp >> 1) : 8 * grp) + (i16 >> 2);
#pragma unroll
    for (int fn = 0; fn < C::FN; fn++) {
      const int c16 = (wn * C::TN) / 16 + (FR == 32 ? fn * 2 + (grp & 1) : fn);  // 16-column block = 32-byte group
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = kk + 4 * h;
        q_off[fn * 2 + h] = k * C::ROWB + ((c16 ^ mnswz(k)) << 5) + ((i16 & 3) << 3);
      }
    }
  }
}

// the LDS reads of one step: the step's half of the token fragments, and the weight fragments when the step starts a
// k-slice
template <class C, int STEP>
SMOE_DEV void read_fragments(const char* sp, const char* sq, const int (&p_off)[C::KSL],
                             const int (&q_off)[C::QMN ? 2 * C::FN : C::KSL], elemx8 (&qf)[C::FN], elemx8 (&pf)[C::NP]) {
  using Mma = typename C::Mma;
  constexpr int ksl = Mma::kslice(STEP), ph = Mma::phalf(STEP);
#pragma unroll
  for (int pp = 0; pp < C::NP; pp++) pf[pp] = lds_read_b128(sp + p_off[ksl] + (ph * C::NP + pp) * C::FR * C::KROW);
  if constexpr (Mma::reads_q(STEP)) {
#pragma unroll
    for (int fn = 0; fn < C::FN; fn++) {
      if constexpr (!C::QMN) {
        qf[fn] = lds_read_b128(sq + q_off[ksl] + fn * C::FR * C::KROW);
      } else {
        qf[fn] = lds_read_tr2(sq + q_off[fn * 2] + ksl * Mma::KSTEP * C::ROWB,
                              sq + q_off[fn * 2 + 1] + ksl * Mma::KSTEP * C::ROWB);
      }
    }
  }
}

// ACT (an smoe_activation) matters to ROLE_UP_FWD and ROLE_DZ only.  p.N counts accumulator columns: the z columns
// (2I gated, I otherwise) for ROLE_UP_FWD, the y1 columns I for ROLE_DZ.
template <class C, int ROLE, int ACT>
__global__ __launch_bounds__(C::NT) void varlen_m_kernel(const VarlenMParams p) {
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int PW = act_pointwise(ACT);
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  using Mma = typename C::Mma;
  using AL = AccLayout<Mma>;
  constexpr int BN = C::BN, FM = C::FM, FN = C::FN, BK = C::BK, FR = C::FR, QPF = AL::QPF;
  const uint32_t smem_base = lds_address(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % C::WM, wn = wave / C::WM;

  const int num_m_tiles = p.tm.header[0];
  const int64_t total = (int64_t)num_m_tiles * p.n_tiles;
  const int64_t lin = xcd_linear_tile(total);
  if (lin < 0) return;
  constexpr int GM = 8;
  const int64_t per_group = (int64_t)GM * p.n_tiles;
  const int group = (int)(lin / per_group);
  const int first_m = group * GM;
  const int gm = num_m_tiles - first_m < GM ? num_m_tiles - first_m : GM;
  const int within = (int)(lin - (int64_t)group * per_group);
  const int mt = first_m + within % gm;
  const int nt = within / gm;
  const int e = p.tm.expert[mt];
  const int row0 = p.tm.row0[mt];
  const int row_end = p.off[e + 1];
  const int n0 = nt * BN;

  // ---- per-lane global source pointers (advance by one stage per k-step) ----
  const uint16_t* p_src[C::P_INSTR];
#pragma unroll
  for (int i = 0; i < C::P_INSTR; i++) {
    const int r = (wave * C::P_INSTR + i) * C::KRPI + lane / C::KPR;
    int m = row0 + r;
    m = m < row_end ? m : row_end - 1;
    const int64_t src_row = p.gidx ? (int64_t)p.gidx[m] : (int64_t)m;
    p_src[i] = p.P + src_row * p.p_stride + (((lane % C::KPR) ^ kswz<BK, C::FR>(r)) << 3);
  }
  const uint16_t* q_src[C::Q_INSTR];
  const uint16_t* qe = p.Q + (int64_t)e * p.q_stride_e;
  int64_t q_step;
  if constexpr (!C::QMN) {
#pragma unroll
    for (int i = 0; i < C::Q_INSTR; i++) {
      const int r = (wave * C::Q_INSTR + i) * C::KRPI + lane / C::KPR;
      int n = n0 + r;
      n = n < p.N ? n : p.N - 1;
      q_src[i] = qe + (int64_t)n * p.q_stride_row + (((lane % C::KPR) ^ kswz<BK, C::FR>(r)) << 3);
    }
    q_step = BK;
  } else {
#pragma unroll
    for (int i = 0; i < C::Q_INSTR; i++) {
      const int kl = (wave * C::Q_INSTR + i) * C::RPI + lane / C::LPR;
      const int phys16 = lane % C::LPR;
      const int log32 = (phys16 >> 1) ^ mnswz(kl);
      int n = n0 + ((log32 << 1) | (phys16 & 1)) * 8;
      n = n <= p.N - 8 ? n : p.N - 8;
      q_src[i] = qe + (int64_t)kl * p.q_stride_row + n;
    }
    q_step = (int64_t)BK * p.q_stride_row;
  }

  const int S_total = p.Kdim / BK;

  // ---- per-lane LDS fragment offsets (bytes inside a ring slot) ----
  int p_off[C::KSL];
  int q_off[C::QMN ? 2 * FN : C::KSL];
  fragment_offsets<C>(wm, wn, lane, p_off, q_off);

  typename Mma::Acc acc[FN][FM];
  clear_accumulators<Mma>(acc);

  constexpr int Q_RING = C::P_SLOTS * C::P_STAGE;  // byte offset of the weight operand's slots
  auto issue_p = [&](int slot, auto i_c) {
    constexpr int i = decltype(i_c)::value;
    load16_to_lds(p_src[i], smem_base + slot * C::P_STAGE + (wave * C::P_INSTR + i) * 1024);
    p_src[i] += BK;
  };
  auto issue_q = [&](int slot, auto j_c) {
    constexpr int j = decltype(j_c)::value;
    load16_to_lds(q_src[j], smem_base + Q_RING + slot * C::Q_STAGE + (wave * C::Q_INSTR + j) * 1024);
    q_src[j] += q_step;
  };
  auto load = [&](int p_slot, int q_slot, auto step_c, elemx8(&qf)[FN], elemx8(&pf)[C::NP]) {
    read_fragments<C, decltype(step_c)::value>(smem + p_slot * C::P_STAGE, smem + Q_RING + q_slot * C::Q_STAGE, p_off,
                                               q_off, qf, pf);
  };
  gemm_mainloop_asym<FN, C::NP, (C::QMN ? 2 * FN : FN) + C::NP, C::P_INSTR, C::Q_INSTR, C::STEPS, Mma>(
      S_total, acc, issue_p, issue_q, load);

  const int m_base = row0 + wm * C::TM, n_base = n0 + wn * C::TN;

  if constexpr (ROLE == ROLE_PLAIN || ROLE == ROLE_UP_FWD) {
    FwdEpilogueArgs ea;
    ea.bias = p.bias ? p.bias + (int64_t)e * p.N : nullptr;
    ea.out0 = p.out0;
    ea.out0_stride = p.out0_stride;
    ea.out1 = p.out1;
    ea.out1_stride = p.out1_stride;
    ea.m_base = m_base;
    ea.row_end = row_end;
    ea.n_base = n_base;
    ea.N = p.N;
    wait_vmem_all();
    lds_barrier();  // all waves are done reading the last stage
    forward_epilogue<Mma, C::TM, C::TN, ROLE == ROLE_UP_FWD, ACT>(acc, smem, wave, lane, ea);
  } else if constexpr (ROLE == ROLE_COMBINE) {
    CombineEpilogueArgs ca;
    ca.bias = p.bias ? p.bias + (int64_t)e * p.N : nullptr;
    ca.o = p.out0;
    ca.o_stride = p.out0_stride;
    ca.out_rows = p.out_rows;
    ca.scores = p.scores;
    ca.sidx = p.sidx;
    ca.m_base = m_base;
    ca.row_end = row_end;
    ca.n_base = n_base;
    ca.N = p.N;
    wait_vmem_all();
    lds_barrier();  // all waves are done reading the last stage
    combine_epilogue_rows<Mma, C::TM, C::TN>(acc, smem + wave * (32 * EpiLayout<C::TN>::ROW_BYTES), lane, ca);
  } else {
    // ---- dz epilogue (dz_epilogue in gemm_common.h) ----
    DzEpilogueArgs da = {};
    da.zin = p.zin;
    da.zin_stride = p.zin_stride;
    da.dz = p.out0;
    da.dz_stride = p.out0_stride;
    da.y1s = p.out1;
    da.y1s_stride = p.out1_stride;
    da.scores = p.scores;
    da.sidx = p.sidx;
    da.ds_partial = p.ds_partial;
    da.ds_cols = p.ds_cols;
    da.ds_col = nt * C::WN + wn;
    da.m_base = m_base;
    da.row_end = row_end;
    da.n_base = n_base;
    da.N = p.N;
    static_assert(C::NW * DzStaging<C::TN, ACT>::BYTES <= C::RING, "dz staging must fit into the idle ring");
    // (GEGLU: one batch of z in flight instead of two, its erf needs the registers)
    dz_epilogue<Mma, C::TM, C::TN, ACT, act_pointwise(ACT) == PW_GELU ? 1 : 2>(acc, smem + wave * DzStaging<C::TN, ACT>::BYTES, lane, da, [&]() {
      wait_lds_all();
      lds_barrier();  // every wave has finished reading the ring
    });
  }
}

// ---- the same GEMM as a stream of tiles per workgroup -----------------------------------------------------------------
// One workgroup per compute unit walks through the tiles b, b + gridDim.x, ... of the XCD-aware tile order and keeps
// the ring running across tile boundaries (gemm_stream_loop).  ROLE_UP_FWD and ROLE_PLAIN only; needs Kdim >= 3 * BK.
template <class C, int ROLE, int ACT>
__global__ __launch_bounds__(C::NT) void varlen_m_stream_kernel(const VarlenMParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  using Mma = typename C::Mma;
  constexpr int BN = C::BN, FM = C::FM, FN = C::FN, BK = C::BK;
  const uint32_t smem_base = lds_address(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % C::WM, wn = wave / C::WM;

  const StreamTiles tiles(p.tm, p.off, p.n_tiles, BN);
  using Tile = StreamTile;
  auto tile_at = [&](int64_t vb) { return tiles.at(vb); };
  int64_t vb = blockIdx.x;
  Tile cur = tile_at(vb);
  if (!cur.valid) return;
  Tile nxt = tile_at(vb += gridDim.x);
  bool more = nxt.valid;  // a tile follows the current one
  if (!more) nxt = cur;   // the streams always run on: past the last tile they re-read it into slots nobody reads
  Tile nn = tile_at(vb += gridDim.x);

  // ---- global source addresses ----
  // Everything a tile switch computes from the lane number starts from a copy of it the compiler cannot see through:
  // otherwise the per-lane parts are hoisted out of the tile loop and occupy registers the main loop needs.
  auto opaque_lane = [&]() {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  // source rows of a tile's token operand (ordinary vector loads when gathered)
  auto token_rows = [&](const Tile& t, int(&rows)[C::P_INSTR]) {
    const int ln = opaque_lane();
#pragma unroll
    for (int i = 0; i < C::P_INSTR; i++) {
      int m = t.row0 + (wave * C::P_INSTR + i) * C::KRPI + ln / C::KPR;
      m = m < t.row_end ? m : t.row_end - 1;
      rows[i] = p.gidx ? p.gidx[m] : m - t.row0;
    }
  };
  // Operands are fetched through buffer resources: a lane keeps one 32-bit byte offset per load (fixed for a tile),
  // the position along the contraction is a wave-uniform offset.  The token operand's resource starts at the tensor
  // (gathered rows: row * stride has to fit 32 bits, checked on the host) or at the tile's first row (rows in place);
  // the weight operand's resource starts at the tile's expert.
  uint32_t p_voff[C::P_INSTR], q_voff[C::Q_INSTR];
  i32x4 p_rsrc = make_buffer_resource(p.P), q_rsrc = make_buffer_resource(p.Q);
  const uint32_t p_row_bytes = (uint32_t)p.p_stride * 2u, q_row_bytes = (uint32_t)p.q_stride_row * 2u;
  const uint32_t q_step = C::QMN ? (uint32_t)BK * q_row_bytes : (uint32_t)BK * 2u;
  // rows: token indices (gathered) or grouped rows relative to the tile's first row
  auto point_p = [&](const int(&rows)[C::P_INSTR], const Tile& t) {
    const int ln = opaque_lane();
    if (!p.gidx) p_rsrc = make_buffer_resource(p.P + (int64_t)t.row0 * p.p_stride);
#pragma unroll
    for (int i = 0; i < C::P_INSTR; i++) {
      const int r = (wave * C::P_INSTR + i) * C::KRPI + ln / C::KPR;
      p_voff[i] = (uint32_t)rows[i] * p_row_bytes + ((((uint32_t)ln % C::KPR) ^ kswz<BK, C::FR>(r)) << 4);
    }
  };
  auto point_q = [&](const Tile& t) {
    const int ln = opaque_lane();
    q_rsrc = make_buffer_resource(p.Q + (int64_t)t.e * p.q_stride_e);
#pragma unroll
    for (int i = 0; i < C::Q_INSTR; i++) {
      if constexpr (!C::QMN) {
        const int r = (wave * C::Q_INSTR + i) * C::KRPI + ln / C::KPR;
        int n = t.n0 + r;
        n = n < p.N ? n : p.N - 1;
        q_voff[i] = (uint32_t)n * q_row_bytes + ((((uint32_t)ln % C::KPR) ^ kswz<BK, C::FR>(r)) << 4);
      } else {
        const int kl = (wave * C::Q_INSTR + i) * C::RPI + ln / C::LPR;
        const int phys16 = ln % C::LPR;
        const int log32 = (phys16 >> 1) ^ mnswz(kl);
        int n = t.n0 + ((log32 << 1) | (phys16 & 1)) * 8;
        n = n <= p.N - 8 ? n : p.N - 8;
        q_voff[i] = (uint32_t)kl * q_row_bytes + (uint32_t)n * 2u;
      }
    }
  };
  int rows_next[C::P_INSTR];  // token rows of nxt: loaded at the start of a tile, picked up behind its first stage
  {
    int rows_cur[C::P_INSTR];
    token_rows(cur, rows_cur);
    point_p(rows_cur, cur);
    point_q(cur);
    token_rows(nxt, rows_next);
  }

  const int S_total = p.Kdim / BK;

  // ---- per-lane LDS fragment offsets (bytes inside a ring slot) ----
  int p_off[C::KSL];
  int q_off[C::QMN ? 2 * FN : C::KSL];
  fragment_offsets<C>(wm, wn, lane, p_off, q_off);

  typename Mma::Acc acc[FN][FM];  // started from zero by the first k-slice of every tile

  constexpr int Q_RING = C::P_SLOTS * C::P_STAGE;
  int p_stage = 0, q_stage = 0;  // stages issued to each stream for the tile it is on
  auto issue_p = [&](int slot, auto i_c) {
    constexpr int i = decltype(i_c)::value;
    buffer_load16_to_lds(p_rsrc, p_voff[i], (uint32_t)p_stage * (BK * 2u),
                         smem_base + slot * C::P_STAGE + (wave * C::P_INSTR + i) * 1024);
  };
  auto issue_q = [&](int slot, auto j_c) {
    constexpr int j = decltype(j_c)::value;
    buffer_load16_to_lds(q_rsrc, q_voff[j], (uint32_t)q_stage * q_step,
                         smem_base + Q_RING + slot * C::Q_STAGE + (wave * C::Q_INSTR + j) * 1024);
  };
  auto issued_p = [&]() {
    if (++p_stage == S_total) {
      p_stage = 0;
      point_p(rows_next, nxt);
    }
  };
  auto issued_q = [&]() {
    if (++q_stage == S_total) {
      q_stage = 0;
      point_q(nxt);
    }
  };
  auto load = [&](int p_slot, int q_slot, auto step_c, elemx8(&qf)[FN], elemx8(&pf)[C::NP]) {
    read_fragments<C, decltype(step_c)::value>(smem + p_slot * C::P_STAGE, smem + Q_RING + q_slot * C::Q_STAGE, p_off,
                                               q_off, qf, pf);
  };
  // the rows loaded in tile_end are complete here; naming them in an asm statement makes this the place where the
  // compiler waits for them
  auto first_boundary = [&]() {
#pragma unroll
    for (int i = 0; i < C::P_INSTR; i++) asm volatile("" : "+v"(rows_next[i]));
  };
  // what a wave parks in the two ring slots the tile's last stage vacates: a 32-row fragment row of its output, or (dz)
  // 16 staged rows of z / dz and of y1s
  constexpr int PARK = ROLE == ROLE_DZ ? DzStaging<C::TN, ACT, 16>::BYTES : 32 * EpiLayout<C::TN>::ROW_BYTES;
  static_assert((C::NW / 2) * PARK <= C::P_STAGE && (C::NW / 2) * PARK <= C::Q_STAGE, "parking must fit into a ring slot");
  auto advance_tile = [&]() {
    if (!more) return false;
    cur = nxt;
    nxt = nn;
    more = nxt.valid;
    if (!more) nxt = cur;
    nn = tile_at(vb += gridDim.x);
    token_rows(nxt, rows_next);
    return true;
  };
  auto tile_end = [&](int p_slot, int q_slot) {
    // waves 0..NW/2-1 park in the vacated P slot, the others in the vacated Q slot
    char* region = wave < C::NW / 2 ? smem + p_slot * C::P_STAGE + wave * PARK
                                    : smem + Q_RING + q_slot * C::Q_STAGE + (wave - C::NW / 2) * PARK;
    if constexpr (ROLE == ROLE_DZ) {
      DzEpilogueArgs da = {};
      da.zin = p.zin;
      da.zin_stride = p.zin_stride;
      da.dz = p.out0;
      da.dz_stride = p.out0_stride;
      da.y1s = p.out1;
      da.y1s_stride = p.out1_stride;
      da.scores = p.scores;
      da.sidx = p.sidx;
      da.ds_partial = p.ds_partial;
      da.ds_cols = p.ds_cols;
      da.ds_col = (cur.n0 / BN) * C::WN + wn;
      da.m_base = cur.row0 + wm * C::TM;
      da.row_end = cur.row_end;
      da.n_base = cur.n0 + wn * C::TN;
      da.N = p.N;
      // every wave has issued its reads of the last stage ahead of the barrier in front of the last step
      dz_epilogue<Mma, C::TM, C::TN, ACT, act_is_glu(ACT) && act_pointwise(ACT) != PW_GELU ? 2 : 1, false, 16>(acc, region, opaque_lane(), da, [] {});
      return advance_tile();
    }
    FwdEpilogueArgs ea;
    ea.bias = p.bias ? p.bias + (int64_t)cur.e * p.N : nullptr;
    ea.out0 = p.out0;
    ea.out0_stride = p.out0_stride;
    ea.out1 = p.out1;
    ea.out1_stride = p.out1_stride;
    ea.m_base = cur.row0 + wm * C::TM;
    ea.row_end = cur.row_end;
    ea.n_base = cur.n0 + wn * C::TN;
    ea.N = p.N;
    forward_epilogue_rows<Mma, C::TM, C::TN, ROLE == ROLE_UP_FWD, ACT>(acc, region, opaque_lane(), ea);
    return advance_tile();
  };
  gemm_stream_loop<FN, C::NP, (C::QMN ? 2 * FN : FN) + C::NP, C::P_INSTR, C::Q_INSTR, C::STEPS, Mma>(
      S_total, acc, issue_p, issue_q, load, issued_p, issued_q, first_boundary, tile_end);
}

// ---- the tile stream on the hand-scheduled loop ----------------------------------------------------------------------
// Four wavefronts (one per SIMD) as 2 x 2 wave tiles of 128 x 128; the contraction of a tile is the single assembly
// statement of tile_loop_gen.h, which leaves the tile in a[0:255].  This kernel does what happens once per tile: picks
// the tiles, forms the per-lane source offsets of the current and the next tile for the two load streams (the streams
// run across tile boundaries), and runs the epilogue out of the accumulation registers.  Source offsets are 32-bit byte
// offsets from the token tensor's start and from the expert's weight matrix (the host checks that they fit).
typedef int32_t i32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x8 __attribute__((ext_vector_type(8)));
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));

constexpr int DS_COLS_PER_TILE = 4;  // pitch of the score-gradient partials per 256-column tile

template <class C, int ROLE, int ACT>
__global__ __launch_bounds__(C::NT) void varlen_m_asm_kernel(const VarlenMParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  using Mma = typename C::Mma;
  constexpr int BN = C::BN, FN = C::FN, BK = C::BK;
  static_assert(C::NW == 4 && C::WM == 2 && C::FM == SMOE_TL_FM && FN == SMOE_TL_FN && C::P_INSTR == SMOE_TL_P_INSTR &&
                    C::Q_INSTR == SMOE_TL_Q_INSTR && Mma::FR == 16 && BK == 64,
                "the generated loop is written for this tile shape");
  const uint32_t smem_base = lds_address(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % C::WM, wn = wave / C::WM;

  const StreamTiles tiles(p.tm, p.off, p.n_tiles, BN);
  int64_t vb = blockIdx.x;
  StreamTile cur = tiles.at(vb);
  if (!cur.valid) return;
  StreamTile nxt = tiles.at(vb += gridDim.x);
  bool more = nxt.valid;  // a tile follows the current one
  if (!more) nxt = cur;   // the streams always run on: past the last tile they re-read it into slots nobody reads
  StreamTile nn = tiles.at(vb += gridDim.x);
  bool more2 = nn.valid;
  if (!more2) nn = nxt;

  auto opaque_lane = [&]() {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  const uint32_t p_row_bytes = (uint32_t)p.p_stride * 2u, q_row_bytes = (uint32_t)p.q_stride_row * 2u;
  // extents: what the streams may touch (anything beyond is dropped by the range check instead of faulting)
  const uint32_t p_bytes = (uint32_t)(p.p_rows * p.p_stride * 2);
  // Rows of a ragged last tile behind the expert's end are not fetched at all when the tensor's end plus the longest
  // stage offset still fits 32 bits: their loads get the tensor's end as offset, the range check drops them and the LDS
  // receives zeros.  Otherwise they re-read the expert's last row.
  const bool drop_rows = (uint64_t)p_bytes + (uint64_t)p.Kdim * 2u + 16u <= 0xffffffffull;
  // source rows of a tile's token operand: token indices (gathered) or the grouped rows themselves; -1 = dropped
  auto token_rows = [&](const StreamTile& t, int(&rows)[C::P_INSTR]) {
    const int ln = opaque_lane();
#pragma unroll
    for (int i = 0; i < C::P_INSTR; i++) {
      const int m0 = t.row0 + (wave * C::P_INSTR + i) * C::KRPI + ln / C::KPR;
      const int m = m0 < t.row_end ? m0 : t.row_end - 1;
      const int row = p.gidx ? p.gidx[m] : m;
      rows[i] = drop_rows && m0 >= t.row_end ? -1 : row;
    }
  };
  auto point_p = [&](const int(&rows)[C::P_INSTR]) {
    const int ln = opaque_lane();
    i32x8 v;
#pragma unroll
    for (int i = 0; i < C::P_INSTR; i++) {
      const int r = (wave * C::P_INSTR + i) * C::KRPI + ln / C::KPR;
      const uint32_t off = (uint32_t)rows[i] * p_row_bytes + ((((uint32_t)ln % C::KPR) ^ kswz<BK, C::FR>(r)) << 4);
      v[i] = (int32_t)(rows[i] < 0 ? p_bytes : off);
    }
    return v;
  };
  auto point_q = [&](const StreamTile& t) {
    const int ln = opaque_lane();
    i32x8 v;
#pragma unroll
    for (int i = 0; i < C::Q_INSTR; i++) {
      if constexpr (!C::QMN) {
        const int r = (wave * C::Q_INSTR + i) * C::KRPI + ln / C::KPR;
        int n = t.n0 + r;
        n = n < p.N ? n : p.N - 1;
        v[i] = (int32_t)((uint32_t)n * q_row_bytes + ((((uint32_t)ln % C::KPR) ^ kswz<BK, C::FR>(r)) << 4));
      } else {
        const int kl = (wave * C::Q_INSTR + i) * C::RPI + ln / C::LPR;
        const int phys16 = ln % C::LPR;
        const int log32 = (phys16 >> 1) ^ mnswz(kl);
        int n = t.n0 + ((log32 << 1) | (phys16 & 1)) * 8;
        n = n <= p.N - 8 ? n : p.N - 8;
        v[i] = (int32_t)((uint32_t)kl * q_row_bytes + (uint32_t)n * 2u);
      }
    }
    return v;
  };
  // base (48 bits) of an expert's weight matrix, as the first two words of a buffer resource
  auto q_base = [&](const StreamTile& t) {
    const uint64_t b = (uint64_t)(p.Q + (int64_t)t.e * p.q_stride_e);
    i32x2 r;
    r[0] = __builtin_amdgcn_readfirstlane((uint32_t)b);
    r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32) & 0xffffu);
    return r;
  };
  const uint32_t q_bytes = C::QMN ? (uint32_t)(p.Kdim - 1) * q_row_bytes + (uint32_t)p.N * 2u
                                  : (uint32_t)(p.N - 1) * q_row_bytes + (uint32_t)p.Kdim * 2u;
  const i32x4 p_rsrc = make_buffer_resource(p.P, p_bytes);
  i32x4 q_rsrc = make_buffer_resource(p.Q + (int64_t)cur.e * p.q_stride_e, q_bytes);

  i32x8 pv, qv, pvn, qvn;
  i32x2 qnb;
  int rows_nn[C::P_INSTR];  // token rows of nn: requested one tile ahead of the offsets made from them
  {
    int rows[C::P_INSTR];
    token_rows(cur, rows);
    pv = point_p(rows);
    qv = point_q(cur);
    token_rows(nxt, rows);
    pvn = point_p(rows);
    qvn = point_q(nxt);
    qnb = q_base(nxt);
    token_rows(nn, rows_nn);
  }

  const int S_total = p.Kdim / BK;
  int p_off_a[C::KSL];
  int q_off_a[C::QMN ? 2 * FN : C::KSL];
  fragment_offsets<C>(wm, wn, lane, p_off_a, q_off_a);
  i32x2 poff = {p_off_a[0], p_off_a[1]};

  constexpr int Q_RING = C::P_SLOTS * C::P_STAGE;
  const uint32_t q_step = C::QMN ? (uint32_t)BK * q_row_bytes : (uint32_t)BK * 2u;
  const uint32_t lds_p = smem_base, lds_q = smem_base + Q_RING, wave_lds = (uint32_t)wave * (C::P_INSTR * 1024);
  const uint32_t p_end = (uint32_t)S_total * (BK * 2u), q_end = (uint32_t)S_total * q_step;
  const uint32_t n_mid = (uint32_t)S_total - 2u;
  // the first tile's stage 0 and the weight stage after it; the loop's entry requests P(1) and Q(2) into the "vacated"
  // slots 0 / 0 and finds stage 0 in the slots after them
  uint32_t p_soff = 0, q_soff = 0, p_fill = lds_p, q_fill = lds_q;
  static_for<C::P_INSTR>([&](auto i_c) {
    constexpr int i = decltype(i_c)::value;
    buffer_load16_to_lds(p_rsrc, (uint32_t)pv[i], 0u, lds_p + C::P_STAGE + wave_lds + i * 1024);
  });
  static_for<2>([&](auto s_c) {
    constexpr int s = decltype(s_c)::value;
    static_for<C::Q_INSTR>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      buffer_load16_to_lds(q_rsrc, (uint32_t)qv[i], (uint32_t)s * q_step, lds_q + (1 + s) * C::Q_STAGE + wave_lds + i * 1024);
    });
  });
  p_soff = BK * 2u;
  q_soff = 2u * q_step;
  wait_vmem_all();

  constexpr int PARK = ROLE == ROLE_DZ ? DzStaging<C::TN, ACT, 16>::BYTES : 32 * EpiLayout<C::TN>::ROW_BYTES;
  static_assert((C::NW / 2) * PARK <= C::P_STAGE && (C::NW / 2) * PARK <= C::Q_STAGE, "parking must fit into a ring slot");

  for (;;) {
    if constexpr (!C::QMN) {
      i32x2 qoff = {q_off_a[0], q_off_a[1]};
      SMOE_TILE_LOOP_KK(pv, qv, q_rsrc, p_soff, q_soff, p_fill, q_fill, pvn, qvn, poff, qoff, p_rsrc, qnb, p_end, q_end,
                        q_step, n_mid, lds_p, lds_q, wave_lds);
    } else {
      i32x16 qoff;
#pragma unroll
      for (int i = 0; i < 2 * FN; i++) qoff[i] = q_off_a[i];
      SMOE_TILE_LOOP_KM(pv, qv, q_rsrc, p_soff, q_soff, p_fill, q_fill, pvn, qvn, poff, qoff, p_rsrc, qnb, p_end, q_end,
                        q_step, n_mid, lds_p, lds_q, wave_lds);
    }
    // Offsets of the tile after next, from the rows requested a tile ago.  Formed here, in front of the epilogue's
    // stores: the wait for those rows then finds only loads outstanding.
    const i32x8 pvn_new = point_p(rows_nn);
    const i32x8 qvn_new = point_q(nn);
    const i32x2 qnb_new = q_base(nn);

    // waves 0, 1 park in the vacated token slot, waves 2, 3 in the vacated weight slot
    char* region = smem + ((wave < C::NW / 2 ? p_fill : q_fill) - smem_base) + (wave & (C::NW / 2 - 1)) * PARK;
    if constexpr (ROLE == ROLE_DZ) {
      DzEpilogueArgs da = {};
      da.zin = p.zin;
      da.zin_stride = p.zin_stride;
      da.dz = p.out0;
      da.dz_stride = p.out0_stride;
      da.y1s = p.out1;
      da.y1s_stride = p.out1_stride;
      da.scores = p.scores;
      da.sidx = p.sidx;
      da.ds_partial = p.ds_partial;
      da.ds_cols = p.ds_cols;
      // the table has the pitch of the eight-wave kernels (four columns per tile): two sums, two zeros
      da.ds_col = (cur.n0 / BN) * DS_COLS_PER_TILE + wn;
      da.ds_pad_col1 = da.ds_col + C::WN + 1;
      da.m_base = cur.row0 + wm * C::TM;
      da.row_end = cur.row_end;
      da.n_base = cur.n0 + wn * C::TN;
      da.N = p.N;
      // z and dz do not pass through LDS here (dz_epilogue_direct); only y1s is parked, in the first 4 KiB of the region
      // (two fragment rows of z in flight for the gated activations; one for GEGLU, whose erf needs the registers)
      dz_epilogue_direct<Mma, C::TM, C::TN, ACT, act_is_glu(ACT) && act_pointwise(ACT) != PW_GELU ? 2 : 1>(
          [&](auto fn_c, auto fm_c) { return agpr_read4<SMOE_TL_ACC(decltype(fn_c)::value, decltype(fm_c)::value)>(); },
          region, opaque_lane(), da);
    } else if constexpr (ROLE == ROLE_COMBINE) {
      CombineEpilogueArgs ca;
      ca.bias = p.bias ? p.bias + (int64_t)cur.e * p.N : nullptr;
      ca.o = p.out0;
      ca.o_stride = p.out0_stride;
      ca.out_rows = p.out_rows;
      ca.scores = p.scores;
      ca.sidx = p.sidx;
      ca.m_base = cur.row0 + wm * C::TM;
      ca.row_end = cur.row_end;
      ca.n_base = cur.n0 + wn * C::TN;
      ca.N = p.N;
      combine_epilogue_rows_agpr<Mma, C::TM, C::TN>(region, opaque_lane(), ca);
    } else {
      FwdEpilogueArgs ea;
      ea.bias = p.bias ? p.bias + (int64_t)cur.e * p.N : nullptr;
      ea.out0 = p.out0;
      ea.out0_stride = p.out0_stride;
      ea.out1 = p.out1;
      ea.out1_stride = p.out1_stride;
      ea.m_base = cur.row0 + wm * C::TM;
      ea.row_end = cur.row_end;
      ea.n_base = cur.n0 + wn * C::TN;
      ea.N = p.N;
      forward_epilogue_rows_agpr<Mma, C::TM, C::TN, ROLE == ROLE_UP_FWD, ACT>(region, opaque_lane(), ea);
    }
    if (!more) break;
    cur = nxt;
    nxt = nn;
    more = more2;
    nn = tiles.at(vb += gridDim.x);
    more2 = nn.valid;
    if (!more2) nn = nxt;
    token_rows(nn, rows_nn);
    pvn = pvn_new;
    qvn = qvn_new;
    qnb = qnb_new;
    wait_lds_all();  // this wave has read its parked rows back; the loop's entry barrier then frees the two slots
  }
  wait_vmem_all();  // the streams ran ahead into ring slots nobody reads any more: let those loads land before the end
}

// the four-wavefront shape of the hand-scheduled loop: 2 x 2 wave tiles of 128 x 128
template <bool QMN>
using AsmCfg = Cfg<256, 256, 2, 2, QMN, 64, 2>;

// 32-bit byte offsets: the tile streams address the token operand from the tensor's start when it is gathered (all of
// them on the hand-scheduled loop) and the weight operand from the expert's matrix
static bool offsets_fit32(const VarlenMParams& p, bool qmn, bool all_rows) {
  const int64_t lim = 0xffffffffll;
  if ((p.gidx != nullptr || all_rows) && p.p_rows * p.p_stride * 2 > lim) return false;
  const int64_t q_rows = qmn ? p.Kdim : p.N;
  return p.q_stride_row > 0 && q_rows * p.q_stride_row * 2 <= lim;
}

template <class C, int ROLE, int ACT>
static int launch_varlen_m(VarlenMParams& p, const int32_t* off, void* workspace, int64_t TK, int E, hipStream_t st) {
  static LdsLimitOnce lds_limit;
  auto kern = varlen_m_kernel<C, ROLE, ACT>;
  {
    const int rc_attr = lds_limit.ensure((const void*)kern, C::SMEM);
    if (rc_attr) return rc_attr;
  }
  if (p.gidx == nullptr) p.p_rows = TK;
  p.tm = carve_tile_map(workspace, TK, E, C::BM);
  int rc = launch_build_tile_map(off, p.order, E, C::BM, p.tm, st);
  if (rc) return rc;
  p.n_tiles = (int)ceil_div(p.N, C::BN);
  static_assert(C::WN == DS_COLS_PER_TILE, "pitch of the score-gradient partials");
  if (ROLE == ROLE_DZ) p.ds_cols = p.n_tiles * C::WN;
  const int64_t max_tiles = max_token_tiles(TK, E, C::BM) * p.n_tiles;
  const int64_t grid = ((max_tiles + 7) / 8) * 8;
  SMOE_REQUIRE(grid < (1ll << 31) && tile_map_fits(TK, E, C::BM), SMOE_ERR_UNSUPPORTED, "grouped gemm: too many tiles");
  {
    const Tuning& tune = tuning();
    if (tune.gemm_stream && (ROLE != ROLE_DZ || tune.dz_stream) && p.Kdim >= 3 * C::BK && offsets_fit32(p, C::QMN, false)) {
      int cus = 0;
      const int rc_cu = device_compute_units(&cus);
      if (rc_cu) return rc_cu;
      int64_t sgrid = ((int64_t)cus / 8) * 8;  // one resident workgroup per compute unit, the same number on every XCD
      // a smaller grid makes small problems run several tiles per workgroup (used by the tests)
      if (tune.gemm_stream_grid > 0) sgrid = ((int64_t)tune.gemm_stream_grid + 7) / 8 * 8;
      if (sgrid < 8) sgrid = 8;
      if (sgrid > grid) sgrid = grid;
      using CA = AsmCfg<C::QMN>;
      static_assert(CA::BM == C::BM && CA::BN == C::BN, "both shapes walk the same tile map");
      if (tune.gemm_asm && offsets_fit32(p, C::QMN, true)) {
        static LdsLimitOnce lds_limit_asm;
        auto akern = varlen_m_asm_kernel<CA, ROLE, ACT>;
        const int rc_a = lds_limit_asm.ensure((const void*)akern, CA::SMEM);
        if (rc_a) return rc_a;
        hipLaunchKernelGGL(akern, dim3((unsigned)sgrid), dim3(CA::NT), CA::SMEM, st, p);
        SMOE_LAUNCH_CHECK();
        return SMOE_OK;
      }
      if constexpr (ROLE != ROLE_COMBINE) {  // (the combining epilogue exists in the two other kernels only)
        static LdsLimitOnce lds_limit_stream;
        auto skern = varlen_m_stream_kernel<C, ROLE, ACT>;
        const int rc_s = lds_limit_stream.ensure((const void*)skern, C::SMEM);
        if (rc_s) return rc_s;
        hipLaunchKernelGGL(skern, dim3((unsigned)sgrid), dim3(C::NT), C::SMEM, st, p);
        SMOE_LAUNCH_CHECK();
        return SMOE_OK;
      }
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(C::NT), C::SMEM, st, p);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

// 256 x 256 tile, 8 wavefronts as 2 (token) x 4 (feature), 64 of the contraction per stage; the ring is 2 token-operand
// slots + 3 weight-operand slots (the last template argument is not used by these kernels)
template <bool QMN>
using TileCfg = Cfg<256, 256, 2, 4, QMN, 64, 2>;

// one kernel per activation: the epilogue math and (gated or not) the tile geometry of z / y1 depend on it
template <bool QMN, int ROLE>
static int launch_by_activation(int act, VarlenMParams& p, const int32_t* off, void* workspace, int64_t TK, int E,
                                hipStream_t st) {
  switch (act) {
    case SMOE_ACT_SWIGLU: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_SWIGLU>(p, off, workspace, TK, E, st);
    case SMOE_ACT_GEGLU: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_GEGLU>(p, off, workspace, TK, E, st);
    case SMOE_ACT_REGLU: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_REGLU>(p, off, workspace, TK, E, st);
    case SMOE_ACT_RELU_SQ: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_RELU_SQ>(p, off, workspace, TK, E, st);
    case SMOE_ACT_RELU: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_RELU>(p, off, workspace, TK, E, st);
    case SMOE_ACT_GELU: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_GELU>(p, off, workspace, TK, E, st);
    case SMOE_ACT_SILU: return launch_varlen_m<TileCfg<QMN>, ROLE, SMOE_ACT_SILU>(p, off, workspace, TK, E, st);
  }
  set_error("unknown activation code %d", act);
  return SMOE_ERR_INVALID;
}

int dz_wave_cols() { return TileCfg<true>::WN; }
int dz_tile_cols() { return TileCfg<true>::BN; }

}  // namespace smoe

using namespace smoe;

static int check_common(int64_t TK, int H, int I, int E, const void* ws, size_t ws_bytes, const char* who) {
  SMOE_REQUIRE(TK >= 0 && TK < (1ll << 31), SMOE_ERR_INVALID, "%s: TK out of range", who);
  SMOE_REQUIRE(E >= 1, SMOE_ERR_INVALID, "%s: E must be >= 1", who);
  SMOE_REQUIRE(H >= 64 && H % 64 == 0, SMOE_ERR_UNSUPPORTED, "%s: H=%d must be a multiple of 64", who, H);
  SMOE_REQUIRE(I >= 64 && I % 64 == 0, SMOE_ERR_UNSUPPORTED, "%s: I=%d must be a multiple of 64", who, I);
  SMOE_REQUIRE(ws != nullptr && ws_bytes >= smoe_gemm_workspace_bytes(TK, E), SMOE_ERR_WORKSPACE,
               "%s: workspace too small", who);
  return SMOE_OK;
}

extern "C" size_t smoe_gemm_workspace_bytes(int64_t TK, int E) {
  if (TK < 0 || E < 1) return 0;
  return tile_map_bytes(TK, E);
}

extern "C" int smoe_dz_partial_cols(int I) { return (int)ceil_div(I, dz_tile_cols()) * dz_wave_cols(); }

extern "C" int smoe_up_projection_forward(const void* x, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row,
                                          const void* b1, void* z, void* y1, const int32_t* off,
                                          const int32_t* expert_schedule_order, const int32_t* x_gather_idx, int64_t T,
                                          int64_t TK, int H, int I, int E, int activation, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  int rc = check_common(TK, H, I, E, workspace, workspace_bytes, "up_projection_forward");
  if (rc) return rc;
  SMOE_REQUIRE(activation >= SMOE_ACT_SWIGLU && activation <= SMOE_ACT_SILU, SMOE_ERR_INVALID,
               "up_projection_forward: unknown activation code %d", activation);
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(x && w1 && y1 && off && x_gather_idx, SMOE_ERR_INVALID, "up_projection_forward: null pointer");
  SMOE_REQUIRE(T > 0, SMOE_ERR_INVALID, "up_projection_forward: T must be positive");
  SMOE_REQUIRE_ALIGNED("up_projection_forward", x, w1, b1, z, y1);
  SMOE_REQUIRE(stride8(w1_stride_e) && stride8(w1_stride_row), SMOE_ERR_UNSUPPORTED,
               "up_projection_forward: weight strides must be multiples of 8 elements");
  hipStream_t st = (hipStream_t)stream;
  VarlenMParams p = {};
  p.P = (const uint16_t*)x;
  p.p_stride = H;
  p.gidx = x_gather_idx;
  p.p_rows = T;
  p.Q = (const uint16_t*)w1;
  p.q_stride_e = w1_stride_e;
  p.q_stride_row = w1_stride_row;
  p.off = off;
  p.order = expert_schedule_order;
  p.N = act_is_glu(activation) ? 2 * I : I;
  p.Kdim = H;
  p.bias = (const uint16_t*)b1;
  p.out0 = (uint16_t*)z;
  p.out0_stride = p.N;
  p.out1 = (uint16_t*)y1;
  p.out1_stride = I;
  return launch_by_activation<false, ROLE_UP_FWD>(activation, p, off, workspace, TK, E, st);
}

extern "C" int smoe_down_projection_forward(const void* y1, const void* w2, int64_t w2_stride_e, int64_t w2_stride_row,
                                            const void* b2, void* y2, const int32_t* off,
                                            const int32_t* expert_schedule_order, int64_t TK, int H, int I, int E,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_common(TK, H, I, E, workspace, workspace_bytes, "down_projection_forward");
  if (rc) return rc;
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(y1 && w2 && y2 && off, SMOE_ERR_INVALID, "down_projection_forward: null pointer");
  SMOE_REQUIRE_ALIGNED("down_projection_forward", y1, w2, b2, y2);
  SMOE_REQUIRE(stride8(w2_stride_e) && stride8(w2_stride_row), SMOE_ERR_UNSUPPORTED,
               "down_projection_forward: weight strides must be multiples of 8 elements");
  hipStream_t st = (hipStream_t)stream;
  VarlenMParams p = {};
  p.P = (const uint16_t*)y1;
  p.p_stride = I;
  p.Q = (const uint16_t*)w2;
  p.q_stride_e = w2_stride_e;
  p.q_stride_row = w2_stride_row;
  p.off = off;
  p.order = expert_schedule_order;
  p.N = H;
  p.Kdim = I;
  p.bias = (const uint16_t*)b2;
  p.out0 = (uint16_t*)y2;
  p.out0_stride = H;
  return launch_varlen_m<TileCfg<false>, ROLE_PLAIN, SMOE_ACT_SWIGLU>(p, off, workspace, TK, E, st);
}

extern "C" int smoe_down_projection_forward_combine(const void* y1, const void* w2, int64_t w2_stride_e,
                                                    int64_t w2_stride_row, const void* b2, void* o,
                                                    const float* scores, const int32_t* off,
                                                    const int32_t* expert_schedule_order,
                                                    const int32_t* x_gather_idx, const int32_t* s_scatter_idx,
                                                    int64_t T, int64_t TK, int H, int I, int E, void* workspace,
                                                    size_t workspace_bytes, void* stream) {
  int rc = check_common(TK, H, I, E, workspace, workspace_bytes, "down_projection_forward_combine");
  if (rc) return rc;
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(y1 && w2 && o && scores && off && x_gather_idx && s_scatter_idx && T > 0, SMOE_ERR_INVALID,
               "down_projection_forward_combine: null pointer");
  SMOE_REQUIRE_ALIGNED("down_projection_forward_combine", y1, w2, b2, o);
  SMOE_REQUIRE(stride8(w2_stride_e) && stride8(w2_stride_row), SMOE_ERR_UNSUPPORTED,
               "down_projection_forward_combine: weight strides must be multiples of 8 elements");
  hipStream_t st = (hipStream_t)stream;
  VarlenMParams p = {};
  p.P = (const uint16_t*)y1;
  p.p_stride = I;
  p.Q = (const uint16_t*)w2;
  p.q_stride_e = w2_stride_e;
  p.q_stride_row = w2_stride_row;
  p.off = off;
  p.order = expert_schedule_order;
  p.N = H;
  p.Kdim = I;
  p.bias = (const uint16_t*)b2;
  p.out0 = (uint16_t*)o;
  p.out0_stride = H;
  p.out_rows = x_gather_idx;
  p.scores = scores;
  p.sidx = s_scatter_idx;
  return launch_varlen_m<TileCfg<false>, ROLE_COMBINE, SMOE_ACT_SWIGLU>(p, off, workspace, TK, E, st);
}

// activation-gradient halves of the two backward operators; the weight-gradient halves live in gemm_varlen_k.hip
namespace smoe {

int launch_dz(const void* dout, const void* z, const void* w2, int64_t w2_stride_e, int64_t w2_stride_row, void* dz,
              void* y1s, float* ds_partial, const float* scores, const int32_t* off, const int32_t* order,
              const int32_t* gidx, const int32_t* sidx, int64_t T, int64_t TK, int H, int I, int E,
              int activation, void* workspace, hipStream_t st) {
  const int zw = act_is_glu(activation) ? 2 : 1;
  VarlenMParams p = {};
  p.P = (const uint16_t*)dout;
  p.p_stride = H;
  p.gidx = gidx;
  p.p_rows = T;  // the range of gidx
  p.Q = (const uint16_t*)w2;  // W2[e] is (H, I): k = h rows, n = i contiguous
  p.q_stride_e = w2_stride_e;
  p.q_stride_row = w2_stride_row;
  p.off = off;
  p.order = order;
  p.N = I;
  p.Kdim = H;
  p.out0 = (uint16_t*)dz;
  p.out0_stride = zw * I;
  p.out1 = (uint16_t*)y1s;
  p.out1_stride = I;
  p.zin = (const uint16_t*)z;
  p.zin_stride = zw * I;
  p.scores = scores;
  p.sidx = sidx;
  p.ds_partial = ds_partial;
  return launch_by_activation<true, ROLE_DZ>(activation, p, off, workspace, TK, E, st);
}

int launch_dx(const void* dz, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row, void* dx_expanded,
              const int32_t* off, const int32_t* order, int64_t TK, int H, int N1, int E, void* workspace,
              hipStream_t st) {
  VarlenMParams p = {};
  p.P = (const uint16_t*)dz;
  p.p_stride = N1;
  p.Q = (const uint16_t*)w1;  // W1[e] is (N1, H): k = j rows, n = h contiguous
  p.q_stride_e = w1_stride_e;
  p.q_stride_row = w1_stride_row;
  p.off = off;
  p.order = order;
  p.N = H;
  p.Kdim = N1;
  p.out0 = (uint16_t*)dx_expanded;
  p.out0_stride = H;
  return launch_varlen_m<TileCfg<true>, ROLE_PLAIN, SMOE_ACT_SWIGLU>(p, off, workspace, TK, E, st);
}

}  // namespace smoe

