// Weight-gradient grouped GEMMs ("varlen-K"): for every expert e
//     dW[e][a][b] = sum_{m in [off[e], off[e+1])} R[rowR(m)][a] * S[rowS(m)][b]
// The contraction runs over the expert's ragged token range; both operands are token-major in memory (a token row
// is contiguous along a resp. b), so both LDS stages are MN-major and both MFMA operands come from transpose loads.
// Either operand may be gathered through x_gather_idx, which re-reads the original activation rows instead of a
// materialised gathered copy.  Experts without tokens still get their zeros written.
//   dW1[e] (2I, H): R = dz rows,              S = x rows gathered
//   dW2[e] (H, I) : R = dout rows gathered,   S = y1s rows
#include "gemm_common.h"
#include "tile_loop_gen.h"

namespace smoe {

struct VarlenKParams {
  const uint16_t* R;
  int64_t r_stride;
  const uint16_t* S;
  int64_t s_stride;
  const int32_t* gidx;
  const int32_t* off;
  uint16_t* out;
  int64_t out_stride_e, out_stride_row;
  int NA, NB;  // output rows / cols
  int tiles_a, tiles_b;
  int E;
  const int32_t* order;  // nullable: position i of the tile order works on expert order[i]
  int64_t gather_rows;  // rows of the gathered operand's tensor (the range of gidx)
  int uniform_rows;  // off == nullptr: group e is rows [e * uniform_rows, min((e + 1) * uniform_rows, total_rows))
  int64_t total_rows;
  int xcd_chunked;  // tile order: 2 blocked, 1 contiguous tile range per XCD (probe: unbalanced on skewed experts), 0 round-robin
};

template <int BA_, int BB_, int WA_, int WB_, bool R_GATHER_, bool S_GATHER_, int BK_, int NSTAGE_>
struct KCfg {
  static constexpr int BA = BA_, BB = BB_, WA = WA_, WB = WB_, BK = BK_, NSTAGE = NSTAGE_;
  static constexpr bool R_GATHER = R_GATHER_, S_GATHER = S_GATHER_;
  static constexpr int NW = WA * WB, NT = NW * 64;
  typedef ElemMma Mma;
  static constexpr int TA = BA / WA, TB = BB / WB;
  static constexpr int FR = Mma::FR;                   // rows / columns of a matrix-instruction fragment
  static constexpr int FA = TA / FR, FB = TB / FR;     // fragments of the wave tile
  static constexpr int NP = FA / Mma::PH;              // R fragments a step works on
  static constexpr int STEPS = BK / Mma::KSTEP * Mma::PH;
  static constexpr int R_STAGE = BA * BK * 2, S_STAGE = BB * BK * 2;
  static constexpr int STAGE = R_STAGE + S_STAGE;
  static constexpr int EPI = NW * TA * (TB * 2 + 16);
  static constexpr int SMEM = NSTAGE * STAGE > EPI ? NSTAGE * STAGE : EPI;
  static constexpr int R_ROWB = BA * 2, S_ROWB = BB * 2;
  static constexpr int R_LPR = R_ROWB / 16, S_LPR = S_ROWB / 16;
  static constexpr int R_RPI = 64 / R_LPR, S_RPI = 64 / S_LPR;
  static constexpr int R_INSTR = R_STAGE / 1024 / NW, S_INSTR = S_STAGE / 1024 / NW;
  static_assert(SMEM <= 160 * 1024, "LDS budget of a CU");
};

// Tile order.  Workgroup slot v runs on XCD v % 8 and every XCD runs 32 slots side by side.  An expert's cost is its
// token count, so every expert is spread over several XCDs (skewed loads stay balanced), in blocks that share operand
// panels in the XCD's L2 (the blocked order); order 0 deals single tiles round-robin instead, order 1 gives every XCD
// one contiguous range of tiles.  Returns false when slot v holds no tile (then no later slot does either).
SMOE_DEV bool decode_tile(const VarlenKParams& p, int64_t v, int& e, int& ta, int& tb) {
  const int64_t per_e = (int64_t)p.tiles_a * p.tiles_b;
  if (p.xcd_chunked == 2) {
    // Blocked order: the 32 tiles an XCD runs side by side are one ba x bb block of ONE expert's output (8 blocks of
    // 32 consecutive workgroup slots per round of 256 slots), so per stage they fetch ba + bb operand panels
    // instead of one or two panels each.  Block B runs on XCD (B + B/8) % 8: an expert's blocks go to neighbouring
    // XCDs, and the rotation keeps any XCD from always getting the same experts.
    const int bb = p.tiles_b < 8 ? p.tiles_b : 8, ba = 32 / bb;
    const int nbj = p.tiles_b / bb, nb = (p.tiles_a / ba) * nbj;  // blocks per expert
    const int xcd = (int)(v & 7);
    const int64_t j = v >> 3, seq = j >> 5;
    const int in = (int)(j & 31);
    const int64_t B = seq * 8 + ((xcd + 8 - (int)(seq & 7)) & 7);
    if (B >= (int64_t)nb * p.E) return false;
    e = (int)(B / nb);
    const int blk = (int)(B - (int64_t)e * nb);
    ta = (blk / nbj) * ba + in / bb;
    tb = (blk % nbj) * bb + in % bb;
    return true;
  }
  const int64_t lin = p.xcd_chunked ? xcd_linear_tile_of(v, per_e * p.E) : (v < per_e * p.E ? v : -1);
  if (lin < 0) return false;
  e = (int)(lin / per_e);
  const int within = (int)(lin - (int64_t)e * per_e);
  ta = within / p.tiles_b;
  tb = within % p.tiles_b;
  return true;
}


template <class C>
__global__ __launch_bounds__(C::NT) void varlen_k_kernel(const VarlenKParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  using Mma = typename C::Mma;
  using AL = AccLayout<Mma>;
  constexpr int FA = C::FA, FB = C::FB, BK = C::BK, NSTAGE = C::NSTAGE, FR = C::FR, QPF = AL::QPF;
  const uint32_t smem_base = lds_address(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave % C::WA, wb = wave / C::WA;

  int e, ta, tb;
  if (!decode_tile(p, (int64_t)blockIdx.x, e, ta, tb)) return;
  if (p.order != nullptr) e = p.order[e];
  const int a0 = ta * C::BA, b0 = tb * C::BB;
  int row_begin, row_end;
  if (p.off != nullptr) {
    row_begin = p.off[e];
    row_end = p.off[e + 1];
  } else {
    row_begin = e * p.uniform_rows;
    const int64_t end = (int64_t)(e + 1) * p.uniform_rows;
    row_end = (int)(end < p.total_rows ? end : p.total_rows);
  }
  const int cnt = row_end - row_begin;
  const int S = (cnt + BK - 1) / BK;

  // per-instruction token row inside a stage and column offset (elements) of this lane's 16-byte piece
  int r_col[C::R_INSTR], s_col[C::S_INSTR];
#pragma unroll
  for (int i = 0; i < C::R_INSTR; i++) {
    const int kl = (wave * C::R_INSTR + i) * C::R_RPI + lane / C::R_LPR;
    const int phys16 = lane % C::R_LPR;
    const int log32 = (phys16 >> 1) ^ mnswz(kl);
    int a = a0 + ((log32 << 1) | (phys16 & 1)) * 8;
    a = a <= p.NA - 8 ? a : p.NA - 8;
    r_col[i] = a;
  }
#pragma unroll
  for (int i = 0; i < C::S_INSTR; i++) {
    const int kl = (wave * C::S_INSTR + i) * C::S_RPI + lane / C::S_LPR;
    const int phys16 = lane % C::S_LPR;
    const int log32 = (phys16 >> 1) ^ mnswz(kl);
    int b = b0 + ((log32 << 1) | (phys16 & 1)) * 8;
    b = b <= p.NB - 8 ? b : p.NB - 8;
    s_col[i] = b;
  }

  // transpose-load fragment offsets (bytes inside a stage)
  int r_off[2 * FA], s_off[2 * FB];
  {
    // a fragment lane supplies column l % FR and the contraction elements 8 * (l / FR) + 0..7 of the k-slice; the
    // transpose load hands lane i of a 16-lane group column i of the 4 (k) x 16 block its lanes' addresses name
    const int grp = lane >> 4, i16 = lane & 15;
    const int kk = (C::FR == 32 ? 8 * (grp >> 1) : 8 * grp) + (i16 >> 2);
#pragma unroll
    for (int f = 0; f < FA; f++) {
      const int c16 = (wa * C::TA) / 16 + (C::FR == 32 ? f * 2 + (grp & 1) : f);
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = kk + 4 * h;
        r_off[f * 2 + h] = k * C::R_ROWB + ((c16 ^ mnswz(k)) << 5) + ((i16 & 3) << 3);
      }
    }
#pragma unroll
    for (int f = 0; f < FB; f++) {
      const int c16 = (wb * C::TB) / 16 + (C::FR == 32 ? f * 2 + (grp & 1) : f);
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = kk + 4 * h;
        s_off[f * 2 + h] = C::R_STAGE + k * C::S_ROWB + ((c16 ^ mnswz(k)) << 5) + ((i16 & 3) << 3);
      }
    }
  }

  typename Mma::Acc acc[FB][FA];
  clear_accumulators<Mma>(acc);

  // Token rows of a stage: wave w feeds rows [w*RPW, (w+1)*RPW) of each operand's stage, R_RPI resp. S_RPI rows per
  // load instruction.  The gather indices of those rows are wave-uniform, so they are fetched with SCALAR loads:
  // vector loads would share the in-order vmcnt counter with the direct-to-LDS loads and serialise the ring.
  static_assert(C::R_INSTR * C::R_RPI == C::S_INSTR * C::S_RPI, "both operands cover the same token rows per wave");
  constexpr int RPW = C::R_INSTR * C::R_RPI;  // token rows per wave and stage
  uint64_t zero = (uint64_t)smoe_zero_page;
  asm volatile("" : "+s"(zero));  // held in a scalar register pair instead of being re-derived from the pc per load
  // constant address space: a uniform address then becomes a scalar load (the indices are read-only here)
  typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
  const const_i32_ptr gidx = (const_i32_ptr)p.gidx;
  int tok[RPW];  // source row of token (stage base + wave*RPW + j); -1 past the expert's end
  // A wave's rows of a stage are consecutive, so their indices come with ONE wide scalar load whenever the whole run
  // lies inside the expert; element-wise loads (each one waited for before the next is issued, as the compiler
  // arranges them) are left to the expert's last, ragged stage.
  typedef int32_t __attribute__((ext_vector_type(RPW), aligned(4))) idx_run;
  typedef const __attribute__((address_space(4))) idx_run* const_run_ptr;
  // The run for the following stage is requested when a stage's FIRST load is issued and taken over after its last:
  // scalar loads return out of order, so the first wait on LDS data behind the request waits for it as well.
  int tok_next[RPW];
  auto fetch = [&](int s, int(&dst)[RPW]) {
    const int m0 = row_begin + s * BK + wave * RPW;
    if (m0 + RPW <= row_end) {
      if constexpr (C::R_GATHER || C::S_GATHER) {
        const idx_run run = *(const_run_ptr)(gidx + m0);
#pragma unroll
        for (int j = 0; j < RPW; j++) dst[j] = run[j];
      } else {
#pragma unroll
        for (int j = 0; j < RPW; j++) dst[j] = m0 + j;
      }
      return;
    }
    // the expert's last, ragged stage: rows past its end read the zero page.  The index array goes on behind the
    // expert (the next expert's rows) up to total_rows, so the run is still ONE wide load wherever it stays inside
    // the array; entries past the expert's end are discarded.
    if constexpr (C::R_GATHER || C::S_GATHER) {
      if ((int64_t)m0 + RPW <= p.total_rows) {
        const idx_run run = *(const_run_ptr)(gidx + m0);
#pragma unroll
        for (int j = 0; j < RPW; j++) dst[j] = m0 + j < row_end ? run[j] : -1;
        return;
      }
    }
#pragma unroll
    for (int j = 0; j < RPW; j++) {
      const int m = m0 + j;
      const int mc = m < row_end ? m : row_end - 1;
      const int g = (C::R_GATHER || C::S_GATHER) ? gidx[mc] : mc;
      dst[j] = m < row_end ? g : -1;
    }
  };
  // Address of this lane's 16-byte piece of load instruction i: ONE 32x32+64-bit multiply-add onto a per-lane pointer.
  // A gathered operand multiplies the lane's token row (picked among the instruction's RPI rows) onto its column
  // pointer; an operand read in place has the lane's row inside the expert folded into the pointer and multiplies
  // the stage's first row.  Rows past the expert's end read the zero page: a select, not a branch.
  const char* r_ptr[C::R_INSTR];
  const char* s_ptr[C::S_INSTR];
  const uint32_t r_row_bytes = (uint32_t)p.r_stride * 2u, s_row_bytes = (uint32_t)p.s_stride * 2u;
#pragma unroll
  for (int i = 0; i < C::R_INSTR; i++) {
    const int64_t row = C::R_GATHER ? 0 : row_begin + wave * RPW + i * C::R_RPI + lane / C::R_LPR;
    r_ptr[i] = (const char*)(p.R + row * p.r_stride + r_col[i]);
  }
#pragma unroll
  for (int i = 0; i < C::S_INSTR; i++) {
    const int64_t row = C::S_GATHER ? 0 : row_begin + wave * RPW + i * C::S_RPI + lane / C::S_LPR;
    s_ptr[i] = (const char*)(p.S + row * p.s_stride + s_col[i]);
  }
  auto piece = [&](const char* lane_ptr, uint32_t row_bytes, bool gather, int rpi, int lpr, int s, int i) {
    const int sel = lane / lpr;
    int t = tok[i * rpi];
#pragma unroll
    for (int j = 1; j < rpi; j++) t = sel == j ? tok[i * rpi + j] : t;
    const uint32_t row = gather ? (uint32_t)t : (uint32_t)(s * BK);
    const uint64_t src = (uint64_t)row * row_bytes + (uint64_t)lane_ptr;
    return (const uint16_t*)(t < 0 ? zero : src);
  };
  auto issue = [&](int buf, int s, auto i_c) {
    constexpr int i = decltype(i_c)::value;
    const uint32_t base = smem_base + buf * C::STAGE;
    if constexpr (i == 0)
      if (s + 1 < S) fetch(s + 1, tok_next);  // stages are issued in order
    if constexpr (i < C::R_INSTR) {
      load16_to_lds(piece(r_ptr[i], r_row_bytes, C::R_GATHER, C::R_RPI, C::R_LPR, s, i),
                    base + (wave * C::R_INSTR + i) * 1024);
    } else {
      constexpr int j = i - C::R_INSTR;
      load16_to_lds(piece(s_ptr[j], s_row_bytes, C::S_GATHER, C::S_RPI, C::S_LPR, s, j),
                    base + C::R_STAGE + (wave * C::S_INSTR + j) * 1024);
    }
    if constexpr (i == C::R_INSTR + C::S_INSTR - 1) {
#pragma unroll
      for (int j = 0; j < RPW; j++) tok[j] = tok_next[j];
    }
  };
  auto load = [&](int buf, int /*s*/, auto step_c, elemx8(&sf)[FB], elemx8(&rf)[C::NP]) {
    constexpr int step = decltype(step_c)::value;
    constexpr int kofs = Mma::kslice(step) * Mma::KSTEP, ph = Mma::phalf(step);
    const char* st = smem + buf * C::STAGE;
#pragma unroll
    for (int pp = 0; pp < C::NP; pp++) {
      const int f = ph * C::NP + pp;
      rf[pp] = lds_read_tr2(st + r_off[f * 2] + kofs * C::R_ROWB, st + r_off[f * 2 + 1] + kofs * C::R_ROWB);
    }
    if constexpr (Mma::reads_q(step)) {
#pragma unroll
      for (int f = 0; f < FB; f++)
        sf[f] = lds_read_tr2(st + s_off[f * 2] + kofs * C::S_ROWB, st + s_off[f * 2 + 1] + kofs * C::S_ROWB);
    }
  };
  if (S > 0) fetch(0, tok);
  // MFMA as D[b][a] += S[b][k] R[k][a]: lane owns output row a = l%32, register quads hold 4 consecutive columns b
  // two transpose loads per fragment: 12 reads for the 8 MFMAs of a slice, issued two per MFMA
  gemm_mainloop<FB, C::NP, 2 * (C::NP + FB), C::R_INSTR + C::S_INSTR, C::STEPS, NSTAGE, Mma, 2>(S, acc, issue, load);
  // epilogue through LDS (also writes the zeros of experts without tokens)
  using L = EpiLayout<C::TB>;
  char* region = smem + wave * (C::TA * L::ROW_BYTES);
  wait_vmem_all();
  lds_barrier();
  static_for<FA>([&](auto fa_c) {
    constexpr int fa = decltype(fa_c)::value;
    static_for<FB * QPF>([&](auto q_c) {
      constexpr int fb = decltype(q_c)::value / QPF, rg = decltype(q_c)::value % QPF;
      u32x2 v = {pack_elem2(acc[fb][fa][4 * rg + 0], acc[fb][fa][4 * rg + 1]),
                 pack_elem2(acc[fb][fa][4 * rg + 2], acc[fb][fa][4 * rg + 3])};
      *(u32x2*)(region + (fa * FR + AL::row(lane)) * L::ROW_BYTES + (fb * FR + AL::col(rg, lane)) * 2) = v;
    });
  });
  epilogue_flush<C::TA, C::TB>(region, lane, p.out + (int64_t)e * p.out_stride_e, p.out_stride_row, a0 + wa * C::TA,
                               p.NA, b0 + wb * C::TB, p.NB);
}


// ---- the same GEMM on the hand-scheduled loop, as a stream of tiles ---------------------------------------------------
// Schedule.  The 32 tiles an XCD's 32 workgroups run side by side are one block (BA_T x BB_T tiles) of ONE expert's
// output, as in the blocked order above - so all of them have the same length (the expert's token count) and a
// persistent workgroup that takes tile i of every block of its XCD is balanced against its 31 neighbours by
// construction.  Across the XCDs the blocks are dealt by cost: experts sorted by token count, largest first (or in the
// caller's expert_schedule_order), their blocks laid out in that order and dealt to the XCDs in snake order
// 0..7, 7..0, so every XCD gets one of the larger and one of the smaller blocks of each run of 16.  No queue, no
// atomics: the table is built by one small kernel per launch and every workgroup knows its next tiles in advance,
// which is what lets the load streams of the loop run across tile boundaries.
//   table: int32 count[8] (rounds per XCD), then block[8][max_rounds] (block id = expert * blocks_per_expert + block)
constexpr int SCHED_MAX_E = 4096;

static inline size_t block_schedule_bytes(int64_t blocks_total) {
  return (size_t)(8 + 8 * ((blocks_total + 7) / 8 + 1)) * sizeof(int32_t);
}

__global__ __launch_bounds__(1024) void build_block_schedule_kernel(const int32_t* __restrict__ off,
                                                                    const int32_t* __restrict__ order, int E, int nb,
                                                                    int max_rounds, int32_t* __restrict__ table) {
  __shared__ int32_t cost[SCHED_MAX_E];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) cost[e] = off[e + 1] - off[e];
  __syncthreads();
  const int64_t total = (int64_t)E * nb;
  for (int e = tid; e < E; e += 1024) {
    int pos = 0;  // position of expert e in the schedule order
    if (order != nullptr) {
      for (int i = 0; i < E; i++) pos = order[i] == e ? i : pos;
    } else {
      const int c = cost[e];
      for (int o = 0; o < E; o++) pos += (cost[o] > c || (cost[o] == c && o < e)) ? 1 : 0;
    }
    for (int j = 0; j < nb; j++) {
      const int64_t seq = (int64_t)pos * nb + j;
      const int r = (int)(seq & 15);
      const int x = r < 8 ? r : 15 - r;
      const int64_t round = 2 * (seq >> 4) + (r >= 8 ? 1 : 0);
      table[8 + (int64_t)x * max_rounds + round] = e * nb + j;
    }
  }
  if (tid < 8) {
    const int rem = (int)(total & 15);
    int n = (int)(2 * (total >> 4));
    if (tid < (rem < 8 ? rem : 8)) n += 1;
    if (rem > 8 && tid > 15 - rem) n += 1;
    table[tid] = n;
  }
}

// Four wavefronts as 2 x 2 wave tiles of 128 x 128; the contraction of a tile is the weight-gradient statement of
// tile_loop_gen.h, which fetches the gather indices, forms the gathered operand's addresses, keeps both load streams
// running into the next tile and leaves the tile in a[0:255].  Rows past the expert's end cost no code: the operand
// read in place has a buffer resource that ends at the expert's last row, the gathered one gets index -1, and either
// way the range check of the direct-to-LDS load writes zeros.  Experts with fewer than three stages of rows run three
// (the extra ones read nothing), so one pipeline shape serves every expert, the empty ones included.
typedef int32_t ki32x8 __attribute__((ext_vector_type(8)));
typedef int32_t ki32x16 __attribute__((ext_vector_type(16)));

struct BlockShape {
  int nb, nbj, ba, bb;  // blocks per expert, blocks along b, tiles per block along a / b
};

template <bool RG, bool SG>
__global__ __launch_bounds__(256) void varlen_k_stream_kernel(const VarlenKParams p, const BlockShape bs,
                                                              const int32_t* table, int max_rounds) {
  static_assert(RG != SG, "exactly one operand is gathered");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  typedef ElemMma Mma;
  constexpr int BA = 256, BB = 256, TA = 128, TB = 128, BK = 64, ROWB = 512, NINSTR = SMOE_TL_P_INSTR;
  static_assert(TA / 16 == SMOE_TL_FM && TB / 16 == SMOE_TL_FN && Mma::FR == 16, "the generated loop is written for this tile shape");
  const uint32_t smem_base = lds_address(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave % 2, wb = wave / 2;

  typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;  // workgroup b runs on XCD b % 8
  const const_i32_ptr tab = (const_i32_ptr)table, off = (const_i32_ptr)p.off;
  const int rounds = tab[xcd];
  if (rounds == 0) return;
  const const_i32_ptr blocks = tab + 8 + (int64_t)xcd * max_rounds;
  struct Tile {
    int e, row_begin, row_end, a0, b0;
  };
  // past the XCD's last round: an empty expert - every load out of range
  auto tile_at = [&](int r) {
    Tile t = {0, 0, 0, 0, 0};
    if (r < rounds) {
      const int B = blocks[r];
      t.e = B / bs.nb;
      const int blk = B - t.e * bs.nb;
      t.a0 = ((blk / bs.nbj) * bs.ba + slot / bs.bb) * BA;
      t.b0 = ((blk % bs.nbj) * bs.bb + slot % bs.bb) * BB;
      t.row_begin = off[t.e];
      t.row_end = off[t.e + 1];
    }
    return t;
  };
  auto stages_of = [&](const Tile& t) {
    const int S = (t.row_end - t.row_begin + BK - 1) / BK;
    return S < 3 ? 3 : S;
  };

  const uint32_t r_row_bytes = (uint32_t)p.r_stride * 2u, s_row_bytes = (uint32_t)p.s_stride * 2u;
  auto opaque_lane = [&]() {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  // per-lane source offsets of the 8 loads of a stage: load i of this wave covers the token rows 2 i, 2 i + 1 of the
  // wave's 16 (lanes 0-31 / 32-63) and 16 bytes per lane of the 512 the tile takes of a row
  auto lane_offsets = [&](const Tile& t, ki32x8& pvv, ki32x8& qvv) {
    const int ln = opaque_lane();
#pragma unroll
    for (int i = 0; i < NINSTR; i++) {
      const int kl = (wave * NINSTR + i) * 2 + ln / 32;
      const int phys16 = ln % 32;
      const int log32 = (phys16 >> 1) ^ mnswz(kl);
      const int c = ((log32 << 1) | (phys16 & 1)) * 8;
      int a = t.a0 + c, b = t.b0 + c;
      a = a <= p.NA - 8 ? a : p.NA - 8;
      b = b <= p.NB - 8 ? b : p.NB - 8;
      pvv[i] = (int32_t)((RG ? 0u : (uint32_t)kl * r_row_bytes) + (uint32_t)a * 2u);
      qvv[i] = (int32_t)((SG ? 0u : (uint32_t)kl * s_row_bytes) + (uint32_t)b * 2u);
    }
  };
  auto first_offsets = [&](const Tile& t, int32_t& ps, int32_t& qs) {
    const uint32_t run = (uint32_t)(t.row_begin + wave * 16) * 4u;
    ps = (int32_t)(RG ? run : (uint32_t)t.row_begin * r_row_bytes);
    qs = (int32_t)(SG ? run : (uint32_t)t.row_begin * s_row_bytes);
  };

  auto uniform = [](auto& v) {
#pragma unroll
    for (int k = 0; k < (int)(sizeof(v) / 4); k++) v[k] = __builtin_amdgcn_readfirstlane(v[k]);
  };
  Tile cur = tile_at(0), nxt = tile_at(1);
  ki32x8 pv, qv, pvn, qvn;
  lane_offsets(cur, pv, qv);
  lane_offsets(nxt, pvn, qvn);
  // transpose-read addresses inside a slot: fragment f, half h -> 2 f + h
  ki32x16 pra, qra;
  {
    const int grp = lane >> 4, i16 = lane & 15;
    const int kk = 8 * grp + (i16 >> 2);
#pragma unroll
    for (int f = 0; f < 8; f++) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = kk + 4 * h;
        pra[f * 2 + h] = k * ROWB + ((((wa * TA) / 16 + f) ^ mnswz(k)) << 5) + ((i16 & 3) << 3);
        qra[f * 2 + h] = k * ROWB + ((((wb * TB) / 16 + f) ^ mnswz(k)) << 5) + ((i16 & 3) << 3);
      }
    }
  }
  const int32_t half = lane >> 5;
  // extents: the operand read in place ends at the expert's last row, the gathered one at its tensor's end
  i32x4 p_rsrc = make_buffer_resource(p.R, RG ? (uint32_t)(p.gather_rows * p.r_stride * 2) : (uint32_t)cur.row_end * r_row_bytes);
  i32x4 q_rsrc = make_buffer_resource(p.S, SG ? (uint32_t)(p.gather_rows * p.s_stride * 2) : (uint32_t)cur.row_end * s_row_bytes);
  const i32x4 g_rsrc = make_buffer_resource(p.gidx, (uint32_t)(p.total_rows * 4));
  const uint32_t lds_p = smem_base, lds_q = smem_base + 2 * 32768;
  ki32x8 state = {}, next = {}, geo = {};
  {
    int32_t ps, qs;
    first_offsets(cur, ps, qs);
    state[SMOE_MM_PSOFF] = ps;
    state[SMOE_MM_QSOFF] = qs;
  }
  state[SMOE_MM_RLEFT] = cur.row_end - (cur.row_begin + wave * 16);
  state[SMOE_MM_PFILL] = (int32_t)lds_p;
  state[SMOE_MM_QFILL] = (int32_t)lds_q;
  geo[SMOE_MM_PSTEP] = (int32_t)(RG ? r_row_bytes : (uint32_t)BK * r_row_bytes);
  geo[SMOE_MM_QSTEP] = (int32_t)(SG ? s_row_bytes : (uint32_t)BK * s_row_bytes);
  geo[SMOE_MM_LDSP] = (int32_t)lds_p;
  geo[SMOE_MM_LDSQ] = (int32_t)lds_q;
  geo[SMOE_MM_WLDS] = wave * (NINSTR * 1024);
  if constexpr (SG) {
    SMOE_TILE_PROLOGUE_MM_QG(pra, qra, pv, qv, p_rsrc, q_rsrc, state, pvn, qvn, half, g_rsrc, next, geo);
  } else {
    SMOE_TILE_PROLOGUE_MM_PG(pra, qra, pv, qv, p_rsrc, q_rsrc, state, pvn, qvn, half, g_rsrc, next, geo);
  }
  uniform(state);
  uniform(p_rsrc);
  uniform(q_rsrc);
  // the prologue has requested one token-side stage and two weight-side stages of the first tile
  state[SMOE_MM_PLEFT] = stages_of(cur) - 1;
  state[SMOE_MM_QLEFT] = stages_of(cur) - 2;

  constexpr int PARK = 32 * EpiLayout<TB>::ROW_BYTES;
  static_assert(2 * PARK <= 32768, "parking must fit into a ring slot");
  for (int r = 0;; r++) {
    geo[SMOE_MM_NMID] = stages_of(cur) - 2;
    {
      int32_t ps, qs;
      first_offsets(nxt, ps, qs);
      next[SMOE_MM_PSOFFN] = ps;
      next[SMOE_MM_QSOFFN] = qs;
    }
    next[SMOE_MM_PEXTN] = (int32_t)((uint32_t)nxt.row_end * r_row_bytes);
    next[SMOE_MM_QEXTN] = (int32_t)((uint32_t)nxt.row_end * s_row_bytes);
    next[SMOE_MM_RLEFTN] = nxt.row_end - (nxt.row_begin + wave * 16);
    next[SMOE_MM_SNEXT] = stages_of(nxt);
    if constexpr (SG) {
      SMOE_TILE_LOOP_MM_QG(pra, qra, pv, qv, p_rsrc, q_rsrc, state, pvn, qvn, half, g_rsrc, next, geo);
    } else {
      SMOE_TILE_LOOP_MM_PG(pra, qra, pv, qv, p_rsrc, q_rsrc, state, pvn, qvn, half, g_rsrc, next, geo);
    }
    // (the compiler takes the scalar results of an assembly statement for per-lane values; say that they are uniform)
    uniform(state);
    uniform(p_rsrc);
    uniform(q_rsrc);
    // both streams are on nxt now; their next tile is the one after it
    const Tile nn = tile_at(r + 2);
    lane_offsets(nn, pvn, qvn);
    // epilogue out of the accumulation registers, 32 rows at a time through the two slots the last stage vacated
    char* region = smem + ((uint32_t)(wave < 2 ? state[SMOE_MM_PFILL] : state[SMOE_MM_QFILL]) - smem_base) + (wave & 1) * PARK;
    FwdEpilogueArgs ea;
    ea.bias = nullptr;
    ea.out0 = p.out + (int64_t)cur.e * p.out_stride_e;
    ea.out0_stride = p.out_stride_row;
    ea.out1 = nullptr;
    ea.out1_stride = 0;
    ea.m_base = cur.a0 + wa * TA;
    ea.row_end = p.NA;
    ea.n_base = cur.b0 + wb * TB;
    ea.N = p.NB;
    forward_epilogue_rows_agpr<Mma, TA, TB, false, SMOE_ACT_SWIGLU>(region, opaque_lane(), ea);
    if (r + 1 >= rounds) break;
    cur = nxt;
    nxt = nn;
    wait_lds_all();  // this wave has read its parked rows back; the loop's entry barrier then frees the two slots
  }
  wait_vmem_all();  // the streams ran on into ring slots nobody reads: let those (empty) loads land before the end
}

template <class C>
static int launch_varlen_k(const VarlenKParams& pin, hipStream_t st, void* workspace = nullptr, size_t workspace_bytes = 0) {
  static LdsLimitOnce lds_limit;
  auto kern = varlen_k_kernel<C>;
  {
    const int rc_attr = lds_limit.ensure((const void*)kern, C::SMEM);
    if (rc_attr) return rc_attr;
  }
  VarlenKParams p = pin;
  p.tiles_a = (int)ceil_div(p.NA, C::BA);
  p.tiles_b = (int)ceil_div(p.NB, C::BB);
  p.xcd_chunked = tuning().varlen_k_tile_order;
  const int64_t total = (int64_t)p.tiles_a * p.tiles_b * p.E;
  int64_t grid = ((total + 7) / 8) * 8;
  if (p.xcd_chunked == 2) {
    const int bb = p.tiles_b < 8 ? p.tiles_b : 8, ba = 32 / bb;
    if (32 % bb == 0 && p.tiles_b % bb == 0 && p.tiles_a % ba == 0) {
      const int64_t blocks = total / 32;
      grid = ((blocks + 7) / 8) * 256;
    } else {
      p.xcd_chunked = 0;  // the output does not split into whole blocks
    }
  }
  SMOE_REQUIRE(grid < (1ll << 31), SMOE_ERR_UNSUPPORTED, "weight-grad gemm: too many tiles");
  // the kernel forms source addresses as row * (row stride in bytes, 32 bits) + column pointer
  SMOE_REQUIRE(p.r_stride > 0 && p.r_stride < (1ll << 31) && p.s_stride > 0 && p.s_stride < (1ll << 31),
               SMOE_ERR_UNSUPPORTED, "weight-grad gemm: operand row stride out of range");
  if constexpr (C::R_GATHER != C::S_GATHER && C::BA == 256 && C::BB == 256) {
    // The tile streams on the hand-scheduled loop: whole blocks of 32 tiles per expert, a schedule table in the
    // workspace, and 32-bit byte offsets for both operands (the streams run a few stages past an expert's end before
    // they stop; rows past the end are told by a wrapped offset).
    const int64_t lim = (1ll << 32) - (1ll << 16);
    const int64_t r_rows = C::R_GATHER ? p.gather_rows : p.total_rows + 8 * C::BK;
    const int64_t s_rows = C::S_GATHER ? p.gather_rows : p.total_rows + 8 * C::BK;
    const bool fits = p.off != nullptr && p.gidx != nullptr && p.gather_rows > 0 && (r_rows + 1) * p.r_stride * 2 < lim &&
                      (s_rows + 1) * p.s_stride * 2 < lim && (p.total_rows + 8 * C::BK) * 4 < lim;
    // a block is ba x bb tiles with ba * bb = 32, as square as the tile counts allow (fewest operand panels per block)
    BlockShape bs = {0, 0, 0, 0};
    bool whole_blocks = false;
    for (int bb : {8, 4, 16, 2, 32, 1}) {
      if (p.tiles_b % bb == 0 && p.tiles_a % (32 / bb) == 0) {
        bs.bb = bb;
        bs.ba = 32 / bb;
        whole_blocks = true;
        break;
      }
    }
    if (tuning().gemm_asm && fits && whole_blocks && p.E <= SCHED_MAX_E && workspace != nullptr) {
      bs.nbj = p.tiles_b / bs.bb;
      bs.nb = (p.tiles_a / bs.ba) * bs.nbj;
      const int64_t blocks_total = (int64_t)bs.nb * p.E;
      if (block_schedule_bytes(blocks_total) <= workspace_bytes && blocks_total < (1ll << 30)) {
        const int max_rounds = (int)((blocks_total + 7) / 8 + 1);
        static LdsLimitOnce lds_limit_asm;
        auto akern = varlen_k_stream_kernel<C::R_GATHER, C::S_GATHER>;
        const int rc_a = lds_limit_asm.ensure((const void*)akern, 160 * 1024);
        if (rc_a) return rc_a;
        hipLaunchKernelGGL(build_block_schedule_kernel, dim3(1), dim3(1024), 0, st, p.off, p.order, p.E, bs.nb, max_rounds,
                           (int32_t*)workspace);
        SMOE_LAUNCH_CHECK();
        hipLaunchKernelGGL(akern, dim3(256), dim3(256), 160 * 1024, st, p, bs, (const int32_t*)workspace, max_rounds);
        SMOE_LAUNCH_CHECK();
        return SMOE_OK;
      }
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(C::NT), C::SMEM, st, p);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

// 256 x 256 output tile, 8 wavefronts as 2 x 4, 64 token rows per stage, double buffer
template <bool RG, bool SG>
static int launch_varlen_k_variant(const VarlenKParams& p, hipStream_t st, void* workspace = nullptr,
                                   size_t workspace_bytes = 0) {
  return launch_varlen_k<KCfg<256, 256, 2, 4, RG, SG, 64, 2>>(p, st, workspace, workspace_bytes);
}

int launch_dz(const void* dout, const void* z, const void* w2, int64_t w2_stride_e, int64_t w2_stride_row, void* dz,
              void* y1s, float* ds_partial, const float* scores, const int32_t* off, const int32_t* order,
              const int32_t* gidx, const int32_t* sidx, int64_t T, int64_t TK, int H, int I, int E,
              int activation, void* workspace, hipStream_t st);
int launch_dx(const void* dz, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row, void* dx_expanded,
              const int32_t* off, const int32_t* order, int64_t TK, int H, int N1, int E, void* workspace,
              hipStream_t st);

}  // namespace smoe

using namespace smoe;

static int check_bwd(int64_t TK, int H, int I, int E, const void* ws, size_t ws_bytes, const char* who) {
  SMOE_REQUIRE(TK >= 0 && TK < (1ll << 31), SMOE_ERR_INVALID, "%s: TK out of range", who);
  SMOE_REQUIRE(E >= 1, SMOE_ERR_INVALID, "%s: E must be >= 1", who);
  SMOE_REQUIRE(H >= 64 && H % 64 == 0, SMOE_ERR_UNSUPPORTED, "%s: H=%d must be a multiple of 64", who, H);
  SMOE_REQUIRE(I >= 64 && I % 64 == 0, SMOE_ERR_UNSUPPORTED, "%s: I=%d must be a multiple of 64", who, I);
  SMOE_REQUIRE(ws != nullptr && ws_bytes >= smoe_gemm_workspace_bytes(TK, E), SMOE_ERR_WORKSPACE,
               "%s: workspace too small", who);
  return SMOE_OK;
}

extern "C" int smoe_down_projection_backward(const void* dout, const void* z, const void* w2, int64_t w2_stride_e,
                                             int64_t w2_stride_row, const void* b2, void* dw2, int64_t dw2_stride_e,
                                             int64_t dw2_stride_row, void* db2, void* dz, void* y1s, float* ds,
                                             float* ds_partial, const float* scores, const int32_t* off,
                                             const int32_t* expert_schedule_order, const int32_t* x_gather_idx,
                                             const int32_t* s_scatter_idx, int64_t T, int64_t TK, int H, int I, int E,
                                             int activation, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_bwd(TK, H, I, E, workspace, workspace_bytes, "down_projection_backward");
  if (rc) return rc;
  SMOE_REQUIRE(activation >= SMOE_ACT_SWIGLU && activation <= SMOE_ACT_SILU, SMOE_ERR_INVALID,
               "down_projection_backward: unknown activation code %d", activation);
  SMOE_REQUIRE(off, SMOE_ERR_INVALID, "down_projection_backward: null pointer");
  SMOE_REQUIRE(dz || dw2 || db2, SMOE_ERR_INVALID,
               "down_projection_backward: nothing to compute (dz, dw2 and db2 are all null)");
  SMOE_REQUIRE(TK == 0 || (dout && x_gather_idx && (!dw2 || y1s)), SMOE_ERR_INVALID,
               "down_projection_backward: null pointer");
  SMOE_REQUIRE(TK == 0 || !dz || (z && w2 && y1s && ds && ds_partial && scores && s_scatter_idx), SMOE_ERR_INVALID,
               "down_projection_backward: null pointer");
  SMOE_REQUIRE(TK == 0 || !db2 || (scores && s_scatter_idx), SMOE_ERR_INVALID,
               "down_projection_backward: db2 needs scores and s_scatter_idx");
  SMOE_REQUIRE_ALIGNED("down_projection_backward", dout, z, w2, b2, dw2, db2, dz, y1s);
  SMOE_REQUIRE(stride8(w2_stride_e) && stride8(w2_stride_row) && stride8(dw2_stride_e) && stride8(dw2_stride_row),
               SMOE_ERR_UNSUPPORTED, "down_projection_backward: weight strides must be multiples of 8 elements");
  hipStream_t st = (hipStream_t)stream;
  if (TK > 0 && dz) {
    rc = launch_dz(dout, z, w2, w2_stride_e, w2_stride_row, dz, y1s, ds_partial, scores, off, expert_schedule_order,
                   x_gather_idx, s_scatter_idx, T, TK, H, I, E, activation, workspace, st);
    if (rc) return rc;
    rc = launch_ds_finalize(ds_partial, smoe_dz_partial_cols(I), s_scatter_idx, ds, TK, st);
    if (rc) return rc;
    if (b2) {  // y2 = y1 W2^T + b2 puts <dout, b2> into the score gradient
      rc = launch_ds_bias_term((const uint16_t*)dout, (const uint16_t*)b2, x_gather_idx, s_scatter_idx, off, E, H, ds,
                               TK, st);
      if (rc) return rc;
    }
  }
  if (db2) {
    rc = launch_expert_colsum((const uint16_t*)dout, H, H, x_gather_idx, scores, s_scatter_idx, off, E,
                              (uint16_t*)db2, st);
    if (rc) return rc;
  }
  if (!dw2) return SMOE_OK;
  VarlenKParams p = {};
  p.R = (const uint16_t*)dout;
  p.r_stride = H;
  p.S = (const uint16_t*)y1s;
  p.s_stride = I;
  p.gidx = x_gather_idx;
  p.off = off;
  p.out = (uint16_t*)dw2;
  p.out_stride_e = dw2_stride_e;
  p.out_stride_row = dw2_stride_row;
  p.NA = H;
  p.NB = I;
  p.E = E;
  p.order = expert_schedule_order;
  p.total_rows = TK;
  p.gather_rows = T;
  // the schedule table may take the place of the tile map: the activation-gradient GEMM that used it ran before
  return launch_varlen_k_variant<true, false>(p, st, workspace, workspace_bytes);
}

extern "C" int smoe_up_projection_backward(const void* x, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row,
                                           const void* dz, void* dw1, int64_t dw1_stride_e, int64_t dw1_stride_row,
                                           void* db1, void* dx_expanded, const int32_t* off,
                                           const int32_t* expert_schedule_order, const int32_t* x_gather_idx,
                                           int64_t T, int64_t TK, int H, int I, int E, int activation, void* workspace,
                                           size_t workspace_bytes, void* stream) {
  int rc = check_bwd(TK, H, I, E, workspace, workspace_bytes, "up_projection_backward");
  if (rc) return rc;
  SMOE_REQUIRE(activation >= SMOE_ACT_SWIGLU && activation <= SMOE_ACT_SILU, SMOE_ERR_INVALID,
               "up_projection_backward: unknown activation code %d", activation);
  SMOE_REQUIRE(off, SMOE_ERR_INVALID, "up_projection_backward: null pointer");
  SMOE_REQUIRE(dw1 || dx_expanded || db1, SMOE_ERR_INVALID,
               "up_projection_backward: nothing to compute (dw1, db1 and dx_expanded are all null)");
  SMOE_REQUIRE(TK == 0 || (dz && x_gather_idx && (!dw1 || x) && (!dx_expanded || w1)), SMOE_ERR_INVALID,
               "up_projection_backward: null pointer");
  SMOE_REQUIRE(TK == 0 || !dw1 || T > 0, SMOE_ERR_INVALID, "up_projection_backward: T must be positive");
  SMOE_REQUIRE_ALIGNED("up_projection_backward", x, w1, dz, dw1, db1, dx_expanded);
  SMOE_REQUIRE(stride8(w1_stride_e) && stride8(w1_stride_row) && stride8(dw1_stride_e) && stride8(dw1_stride_row),
               SMOE_ERR_UNSUPPORTED, "up_projection_backward: weight strides must be multiples of 8 elements");
  hipStream_t st = (hipStream_t)stream;
  const int N1 = activation <= SMOE_ACT_REGLU ? 2 * I : I;  // columns of z and dz: (gate, up) pairs when gated
  if (db1) {
    rc = launch_expert_colsum((const uint16_t*)dz, N1, N1, nullptr, nullptr, nullptr, off, E, (uint16_t*)db1, st);
    if (rc) return rc;
  }
  if (dw1) {
    VarlenKParams p = {};
    p.R = (const uint16_t*)dz;
    p.r_stride = N1;
    p.S = (const uint16_t*)x;
    p.s_stride = H;
    p.gidx = x_gather_idx;
    p.off = off;
    p.out = (uint16_t*)dw1;
    p.out_stride_e = dw1_stride_e;
    p.out_stride_row = dw1_stride_row;
    p.NA = N1;
    p.NB = H;
    p.E = E;
    p.order = expert_schedule_order;
    p.total_rows = TK;
    p.gather_rows = T;
    // the schedule table shares the workspace with the tile map the dx GEMM builds afterwards, in stream order
    rc = launch_varlen_k_variant<false, true>(p, st, workspace, workspace_bytes);
    if (rc) return rc;
  }
  if (TK > 0 && dx_expanded) {
    rc = launch_dx(dz, w1, w1_stride_e, w1_stride_row, dx_expanded, off, expert_schedule_order, TK, H, N1, E, workspace,
                   st);
    if (rc) return rc;
  }
  return SMOE_OK;
}

extern "C" int smoe_router_weight_grad(const void* dlogits, const void* x, void* partial, int64_t T, int E, int H,
                                       int chunks, void* stream) {
  SMOE_REQUIRE(T > 0 && T < (1ll << 31), SMOE_ERR_INVALID, "router_weight_grad: T out of range");
  SMOE_REQUIRE(E >= 8 && E % 8 == 0, SMOE_ERR_UNSUPPORTED, "router_weight_grad: E=%d must be a multiple of 8", E);
  SMOE_REQUIRE(H >= 8 && H % 8 == 0, SMOE_ERR_UNSUPPORTED, "router_weight_grad: H=%d must be a multiple of 8", H);
  SMOE_REQUIRE(chunks >= 1, SMOE_ERR_INVALID, "router_weight_grad: chunks must be positive");
  SMOE_REQUIRE(dlogits && x && partial, SMOE_ERR_INVALID, "router_weight_grad: null pointer");
  SMOE_REQUIRE_ALIGNED("router_weight_grad", dlogits, x, partial);
  VarlenKParams p = {};
  p.R = (const uint16_t*)dlogits;
  p.r_stride = E;
  p.S = (const uint16_t*)x;
  p.s_stride = H;
  p.gidx = nullptr;
  p.off = nullptr;
  p.uniform_rows = (int)((T + chunks - 1) / chunks);
  p.total_rows = T;
  p.out = (uint16_t*)partial;
  p.out_stride_e = (int64_t)E * H;
  p.out_stride_row = H;
  p.NA = E;
  p.NB = H;
  p.E = chunks;
  return launch_varlen_k_variant<false, false>(p, (hipStream_t)stream);
}

