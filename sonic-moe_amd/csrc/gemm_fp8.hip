// fp8 (OCP e4m3) forward grouped GEMMs with per-block scales, and the quantiser that produces their operands.
//
// Operand format ("MX" block scaling): along the contraction dimension every 32 consecutive elements share one
// power-of-two scale, stored as its biased exponent (e8m0, value 2^(byte - 127)); elements are e4m3 bytes.  This is the
// format v_mfma_scale_f32_32x32x64_f8f6f4 multiplies natively: the scale is applied inside the matrix instruction, so
// the main loop has no per-block floating-point work.
//   data   q (R, C) bytes, row-major
//   scales s (C / 128, R) 32-bit words: byte b of word [g][r] scales elements [128 g + 32 b, 128 g + 32 b + 32) of row r
// (one word per row and 128-element group = one pipeline stage, so that a stage's scales of 64 rows are one
// direct-to-LDS load of a wavefront).
//
// The GEMM is the K-major / K-major kernel of the bf16 path with 128 BYTES of contraction per row and stage:
//   up-projection    P = x rows gathered (fp8), Q = W1[e] (fp8)  -> z (bf16), y1 = act(z) (bf16)
//   down-projection  P = y1 rows (fp8),        Q = W2[e] (fp8)  -> y2 (bf16)
//   dz               P = dout rows gathered,   Q = W2[e]^T       -> dz, y1s (bf16), ds partial sums, dz again in fp8
//   dx               P = dz rows (fp8),        Q = W1[e]^T       -> dx_expanded (bf16)   (the down-projection kernel)
// Accumulation is fp32; outputs, biases and epilogues are those of the bf16 kernels.  The two activation-gradient
// GEMMs contract over the other index of the weights, so they read transposed quantised copies (the transposing
// quantiser below); the weight-gradient GEMMs, which contract over the tokens, stay in bf16.
#include "gemm_common.h"

namespace smoe {

typedef int i32x8 __attribute__((ext_vector_type(8)));

// ---- quantiser ---------------------------------------------------------------------------------------------------
// one lane = one 32-element block: 64 bytes in, 32 bytes + 1 scale byte out
__global__ __launch_bounds__(256) void mx_quantize_kernel(const uint16_t* __restrict__ src, int64_t src_stride,
                                                          int64_t R, int C, uint8_t* __restrict__ q,
                                                          uint32_t* __restrict__ scales) {
  const int blocks_per_row = C >> 5;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = R * blocks_per_row;
  const bool live = gid < total;
  const int64_t r = live ? gid / blocks_per_row : 0;
  const int b = live ? (int)(gid - r * blocks_per_row) : 0;
  float v[32];
  float amax = 0.f;
  if (live) {
    const u32x4* p = (const u32x4*)(src + r * src_stride + (int64_t)b * 32);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const u32x4 w = p[i];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        v[i * 8 + 2 * j] = elem_lo(w[j]);
        v[i * 8 + 2 * j + 1] = elem_hi(w[j]);
      }
    }
#pragma unroll
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
  }
  const int ex = mx_scale_exponent(amax);
  const float inv = __uint_as_float((uint32_t)(254 - ex) << 23);  // 2^-(ex-127); ex <= 254 keeps it finite, ex = 0 only for amax = 0
  if (live) {
    uint32_t out[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      int w = 0;
      w = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * i] * inv, v[4 * i + 1] * inv, w, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * i + 2] * inv, v[4 * i + 3] * inv, w, true);
      out[i] = (uint32_t)w;
    }
    u32x4* dst = (u32x4*)(q + r * C + (int64_t)b * 32);
    dst[0] = u32x4{out[0], out[1], out[2], out[3]};
    dst[1] = u32x4{out[4], out[5], out[6], out[7]};
  }
  // blocks 4g..4g+3 of a row sit in 4 consecutive lanes (C % 128 == 0): gather their bytes into one word
  uint32_t word = (uint32_t)ex << (8 * (b & 3));
  word |= __shfl_xor(word, 1, 64);
  word |= __shfl_xor(word, 2, 64);
  if (live && (b & 3) == 0) scales[(int64_t)(b >> 2) * R + r] = word;
}

// ---- GEMM --------------------------------------------------------------------------------------------------------
struct Fp8Params {
  const uint8_t* P;
  int64_t p_stride;  // bytes
  const uint32_t* p_scales;
  int64_t p_rows;    // rows of the P scale table (T or TK)
  int64_t data_rows; // rows of the P data operand = the range of gidx (0: the same as p_rows)
  const int32_t* gidx;
  int scales_grouped;  // the P scale table is in grouped row order although the data rows are gathered
  const uint8_t* Q;
  int64_t q_stride_e, q_stride_row;  // bytes
  const uint32_t* q_scales;
  int64_t q_rows;    // rows of the Q scale table (E * N)
  const int32_t* off;
  TileMap tm;
  int N, Kdim, n_tiles;
  const uint16_t* bias;
  uint16_t* out0;
  int64_t out0_stride;
  uint16_t* out1;
  int64_t out1_stride;
  uint8_t* yq;         // nullable: the activation output quantised in the epilogue, (TK, I) e4m3 bytes
  uint32_t* yq_scales; // its scale table (I / 128, TK)
  int64_t yq_rows;     // TK
  int I;
  // dz role: out0 = dz, out1 = y1s, yq / yq_scales / yq_rows = dz in fp8; N = I
  const uint16_t* zin;
  int64_t zin_stride;
  const float* scores;
  const int32_t* sidx;
  float* ds_partial;
  int ds_cols;
};

struct Fp8Cfg {
  // 8 wavefronts (two per SIMD), 128 x 64 each.  The fragments of an fp8 slice are twice as large as bf16 ones: a step
  // works on half of the wave's token rows, so two register sets of 2 + 2 fragments are all that is live beside the
  // 128 accumulator registers
  static constexpr int BM = 256, BN = 256, WM = 2, WN = 4, BKB = 128, NSTAGE = 2;  // BKB: contraction bytes per stage
  static constexpr int NW = WM * WN, NT = NW * 64;
  static constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32, NP = 1;
  static constexpr int P_STAGE = BM * BKB, Q_STAGE = BN * BKB, S_STAGE = (BM + BN) * 4;
  static constexpr int STAGE = P_STAGE + Q_STAGE + S_STAGE;
  static constexpr int P_INSTR = P_STAGE / 1024 / NW, Q_INSTR = Q_STAGE / 1024 / NW;
  static constexpr int KPR = BKB / 16, KRPI = 64 / KPR;  // 16-byte pieces per row, rows per load instruction
  static constexpr int EPI = NW * TM * (TN * 2 + 16);
  static constexpr int SMEM = NSTAGE * STAGE > EPI ? NSTAGE * STAGE : EPI;
  static constexpr int S_INSTR = (BM + BN) / 64 / NW;  // scale loads (64 rows each) per wave and stage
  // tile-stream kernel: two slots per operand, a slot = the operand's stage + its scale words.  Every wave fetches the
  // scale words of 32 rows of each operand (its upper 32 lanes repeat the lower ones), 256 bytes per wave and slot
  static constexpr int SC_BYTES = NW * 256, P_SLOT = P_STAGE + SC_BYTES, Q_SLOT = Q_STAGE + SC_BYTES;
  static constexpr int STREAM_SMEM = 2 * (P_SLOT + Q_SLOT);
  static constexpr int PS_INSTR = P_STAGE / 1024 / NW, QS_INSTR = Q_STAGE / 1024 / NW;  // data loads per wave and stage
  static_assert(BM == NW * 32 && BN == NW * 32, "32 scale rows of each operand per wave");
  static_assert(STREAM_SMEM <= 160 * 1024, "LDS budget of a CU");
  static_assert(S_INSTR * NW * 64 == BM + BN, "the scale rows must split evenly over the wavefronts");
  static_assert(SMEM <= 160 * 1024, "LDS budget of a CU");
  // smoe_dz_partial_cols() sizes the score-gradient partial sums for both the bf16 and the fp8 dz kernel
  static_assert(BN == 256 && WN == 4, "the partial sums' pitch is four columns per 256-column tile");
};

// direct-to-LDS load of one 32-bit word per lane through a buffer resource: the wavefront's 64 words land at
// lds_wave_base + 4 * lane
SMOE_DEV void buffer_load4_to_lds(i32x4 rsrc, uint32_t voff, uint32_t soff, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dword %0, %1, %2 offen lds"
               :
               : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_wave_base)
               : "memory");
}

// Operand fragment of v_mfma_scale_f32_32x32x64_f8f6f4: lane l holds row l%32 and, of the 64 contraction bytes of the
// slice, bytes [16h, 16h+16) and [32+16h, 48+16h) with h = l/32; its scale byte (bits 0-7) belongs to the 32-element
// block h of the slice.
struct Fp8Frag {
  i32x8 data;
  int scale;
};
struct Fp8Mma {
  typedef Fp8Frag Frag;
  typedef f32x16 Acc;
  // a step is ONE of the wave's four token fragments on one k-slice of 64 contraction bytes; the feature fragments
  // are read on the first of a slice's four steps (see ElemMma16).  Two sets of 1 + 2 fragments are live.
  static constexpr int FR = 32, KSTEP = 64, PH = 4, ACC_REGS = 16, FRAG_REGS = 9;
  static constexpr int qset(int step) { return (step >> 2) & 1; }
  static constexpr int phalf(int step) { return step & 3; }
  static constexpr bool reads_q(int step) { return (step & 3) == 0; }
  static constexpr int kslice(int step) { return step >> 2; }
  static __device__ __forceinline__ f32x16 run(const Frag& q, const Frag& p, f32x16 c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(q.data, p.data, c, 0, 0, 0, q.scale, 0, p.scale);
  }
};

// Activation output of the wave's TM x TN accumulator tile (bias already added) quantised straight from the fp32
// values: per 32-row fragment row, every 32 output columns get their power-of-two scale (lane-local maximum over the
// lane's columns of the block, one shuffle for the other half-wave), the e4m3 bytes are parked in LDS and written back
// 16 bytes per lane; the scale bytes go to the (I / 128, rows) table the down-projection reads.
template <int TM, int TN, int FM, int FN, int ACT>
SMOE_DEV void fp8_activation_epilogue(f32x16 (&acc)[FN][FM], char* region, int lane, uint8_t* yq, int I,
                                      uint32_t* yq_scales, int64_t yq_rows, int m_base, int row_end, int n_base) {
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int PW = act_pointwise(ACT);
  constexpr int YC = GLU ? TN / 2 : TN;      // output columns of the wave tile
  constexpr int NB = YC / 32, FPB = FN / NB;  // 32-column blocks, accumulator fragments per block
  constexpr int ROWB = YC + 16;               // parked row, padded against bank conflicts
  constexpr int LPR = YC / 16, RPP = 64 / LPR;
  // region: the wave's own parking region of the forward epilogue (32 padded rows are used)
  const int half = lane >> 5, mrow = lane & 31;
  const int y_base = GLU ? n_base / 2 : n_base;
  static_for<FM>([&](auto fm_c) {
    constexpr int fm = decltype(fm_c)::value;
    const int m = m_base + fm * 32 + mrow;
    static_for<NB>([&](auto b_c) {
      constexpr int b = decltype(b_c)::value;
      float y[FPB * 4 * (GLU ? 2 : 4)];
      float amax = 0.f;
      static_for<FPB * 4>([&](auto q_c) {
        constexpr int f = decltype(q_c)::value / 4, rg = decltype(q_c)::value % 4, fn = b * FPB + f;
        if constexpr (GLU) {
          const float y0 = pointwise<PW>(acc[fn][fm][4 * rg + 0]) * acc[fn][fm][4 * rg + 1];
          const float y1 = pointwise<PW>(acc[fn][fm][4 * rg + 2]) * acc[fn][fm][4 * rg + 3];
          y[(f * 4 + rg) * 2 + 0] = y0;
          y[(f * 4 + rg) * 2 + 1] = y1;
          amax = fmaxf(amax, fmaxf(fabsf(y0), fabsf(y1)));
        } else {
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float v = pointwise<PW>(acc[fn][fm][4 * rg + q]);
            y[rg * 4 + q] = v;
            amax = fmaxf(amax, fabsf(v));
          }
        }
      });
      amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
      const int ex = mx_scale_exponent(amax);
      const float inv = __uint_as_float((uint32_t)(254 - ex) << 23);
      static_for<FPB * 4>([&](auto q_c) {
        constexpr int f = decltype(q_c)::value / 4, rg = decltype(q_c)::value % 4;
        if constexpr (GLU) {
          const int w = __builtin_amdgcn_cvt_pk_fp8_f32(y[(f * 4 + rg) * 2] * inv, y[(f * 4 + rg) * 2 + 1] * inv, 0, false);
          *(uint16_t*)(region + mrow * ROWB + b * 32 + f * 16 + 4 * rg + 2 * half) = (uint16_t)w;
        } else {
          int w = __builtin_amdgcn_cvt_pk_fp8_f32(y[rg * 4] * inv, y[rg * 4 + 1] * inv, 0, false);
          w = __builtin_amdgcn_cvt_pk_fp8_f32(y[rg * 4 + 2] * inv, y[rg * 4 + 3] * inv, w, true);
          *(uint32_t*)(region + mrow * ROWB + b * 32 + 8 * rg + 4 * half) = (uint32_t)w;
        }
      });
      const int col = y_base + b * 32;  // first output column of the block
      if (half == 0 && m < row_end && col < I)
        ((uint8_t*)yq_scales)[((int64_t)(col >> 7) * yq_rows + m) * 4 + ((col >> 5) & 3)] = (uint8_t)ex;
    });
    // the wavefront's own LDS accesses execute in order: the rows parked above are complete here
#pragma unroll
    for (int it = 0; it < 32 / RPP; it++) {
      const int r = it * RPP + lane / LPR, c16 = lane % LPR;
      const u32x4 v = *(const u32x4*)(region + r * ROWB + c16 * 16);
      const int mm = m_base + fm * 32 + r, col = y_base + c16 * 16;
      if (mm < row_end && col < I) *(u32x4*)(yq + (int64_t)mm * I + col) = v;
    }
  });
}

// WITH_ACT: up-projection epilogue (activation ACT); DZ: epilogue of the down projection's activation gradient
template <bool WITH_ACT, int ACT, bool DZ = false>
__global__ __launch_bounds__(Fp8Cfg::NT) void fp8_varlen_m_kernel(const Fp8Params p) {
  using C = Fp8Cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int FM = C::FM, FN = C::FN, SLICES = C::BKB / 64;
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
  const int n0 = nt * C::BN;

  // Operands are fetched through buffer resources: a lane keeps one 32-bit byte offset per load, the position along
  // the contraction is a wave-uniform offset.  The token operand's resource starts at the tensor (gathered rows: row *
  // stride fits 32 bits, checked on the host) or at the tile's first row; the weight operand's at the tile's expert.
  const i32x4 p_rsrc = make_buffer_resource(p.gidx ? p.P : p.P + (int64_t)row0 * p.p_stride);
  const i32x4 q_rsrc = make_buffer_resource(p.Q + (int64_t)e * p.q_stride_e);
  uint32_t p_voff[C::P_INSTR], q_voff[C::Q_INSTR];
#pragma unroll
  for (int i = 0; i < C::P_INSTR; i++) {
    const int r = (wave * C::P_INSTR + i) * C::KRPI + lane / C::KPR;
    int m = row0 + r;
    m = m < row_end ? m : row_end - 1;
    const uint32_t src_row = p.gidx ? (uint32_t)p.gidx[m] : (uint32_t)(m - row0);
    p_voff[i] = src_row * (uint32_t)p.p_stride + (((lane % C::KPR) ^ kswz<64>(r)) << 4);
  }
#pragma unroll
  for (int i = 0; i < C::Q_INSTR; i++) {
    const int r = (wave * C::Q_INSTR + i) * C::KRPI + lane / C::KPR;
    int n = n0 + r;
    n = n < p.N ? n : p.N - 1;
    q_voff[i] = (uint32_t)n * (uint32_t)p.q_stride_row + (((lane % C::KPR) ^ kswz<64>(r)) << 4);
  }
  // this lane's scale words: load j of wave w covers rows (w * S_INSTR + j) * 64 .. + 63 of the tile's 256 token rows
  // followed by its 256 feature rows; a table row holds one 128-element block of the contraction for all rows
  i32x4 s_rsrc[C::S_INSTR];
  uint32_t s_voff[C::S_INSTR], s_step[C::S_INSTR];
#pragma unroll
  for (int j = 0; j < C::S_INSTR; j++) {
    const int r0 = (wave * C::S_INSTR + j) * 64;  // wave-uniform
    if (r0 < C::BM) {
      int m = row0 + r0 + lane;
      m = m < row_end ? m : row_end - 1;
      const bool by_index = p.gidx != nullptr && !p.scales_grouped;
      s_rsrc[j] = make_buffer_resource(by_index ? p.p_scales : p.p_scales + row0);
      s_voff[j] = (by_index ? (uint32_t)p.gidx[m] : (uint32_t)(m - row0)) * 4u;
      s_step[j] = (uint32_t)p.p_rows * 4u;
    } else {
      int n = n0 + r0 - C::BM + lane;
      n = n < p.N ? n : p.N - 1;
      s_rsrc[j] = make_buffer_resource(p.q_scales + (int64_t)e * p.N);
      s_voff[j] = (uint32_t)n * 4u;
      s_step[j] = (uint32_t)p.q_rows * 4u;
    }
  }

  const int S_total = p.Kdim / C::BKB;

  // per-lane LDS fragment offsets (bytes inside a stage): two 16-byte pieces per slice, one scale word per stage
  const int half = lane >> 5;
  int p_off[SLICES][2], q_off[SLICES][2];
  {
    const int prow = wm * C::TM + (lane & 31), qrow = wn * C::TN + (lane & 31);
    const int psw = kswz<64>(prow), qsw = kswz<64>(qrow);
#pragma unroll
    for (int ks = 0; ks < SLICES; ks++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int piece = 4 * ks + 2 * j + half;
        p_off[ks][j] = prow * C::BKB + ((piece ^ psw) << 4);
        q_off[ks][j] = C::P_STAGE + qrow * C::BKB + ((piece ^ qsw) << 4);
      }
  }
  const int ps_off = C::P_STAGE + C::Q_STAGE + (wm * C::TM + (lane & 31)) * 4;
  const int qs_off = C::P_STAGE + C::Q_STAGE + (C::BM + wn * C::TN + (lane & 31)) * 4;

  f32x16 acc[FN][FM];
#pragma unroll
  for (int fn = 0; fn < FN; fn++)
#pragma unroll
    for (int fm = 0; fm < FM; fm++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[fn][fm][r] = 0.f;

  auto issue = [&](int buf, int s, auto i_c) {
    constexpr int i = decltype(i_c)::value;
    const uint32_t base = smem_base + buf * C::STAGE;
    if constexpr (i < C::P_INSTR) {
      buffer_load16_to_lds(p_rsrc, p_voff[i], (uint32_t)s * C::BKB, base + (wave * C::P_INSTR + i) * 1024);
    } else if constexpr (i < C::P_INSTR + C::Q_INSTR) {
      constexpr int j = i - C::P_INSTR;
      buffer_load16_to_lds(q_rsrc, q_voff[j], (uint32_t)s * C::BKB, base + C::P_STAGE + (wave * C::Q_INSTR + j) * 1024);
    } else {
      constexpr int j = i - C::P_INSTR - C::Q_INSTR;
      buffer_load4_to_lds(s_rsrc[j], s_voff[j], (uint32_t)s * s_step[j],
                          base + C::P_STAGE + C::Q_STAGE + (wave * C::S_INSTR + j) * 256);
    }
  };
  auto load = [&](int buf, int /*s*/, auto step_c, Fp8Frag(&qf)[FN], Fp8Frag(&pf)[C::NP]) {
    constexpr int step = decltype(step_c)::value, ks = Fp8Mma::kslice(step), ph = Fp8Mma::phalf(step);
    const char* st = smem + buf * C::STAGE;
    const int shift = 8 * (2 * ks + half);
#pragma unroll
    for (int pp = 0; pp < C::NP; pp++) {
      const int fm = ph * C::NP + pp;
      const i32x4 lo = *(const i32x4*)(st + p_off[ks][0] + fm * 32 * C::BKB);
      const i32x4 hi = *(const i32x4*)(st + p_off[ks][1] + fm * 32 * C::BKB);
      pf[pp].data = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      pf[pp].scale = (int)(*(const uint32_t*)(st + ps_off + fm * 32 * 4) >> shift);
    }
    if constexpr (Fp8Mma::reads_q(step)) {
#pragma unroll
      for (int fn = 0; fn < FN; fn++) {
        const i32x4 lo = *(const i32x4*)(st + q_off[ks][0] + fn * 32 * C::BKB);
        const i32x4 hi = *(const i32x4*)(st + q_off[ks][1] + fn * 32 * C::BKB);
        qf[fn].data = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        qf[fn].scale = (int)(*(const uint32_t*)(st + qs_off + fn * 32 * 4) >> shift);
      }
    }
  };
  // 3 LDS reads per fragment (two 16-byte pieces and the scale word), dealt out three per matrix instruction
  gemm_mainloop<FN, C::NP, 3 * (FN + C::NP), C::P_INSTR + C::Q_INSTR + C::S_INSTR, Fp8Mma::PH * SLICES, C::NSTAGE, Fp8Mma, 4>(
      S_total, acc, issue, load);

  if constexpr (DZ) {
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
    da.m_base = row0 + wm * C::TM;
    da.row_end = row_end;
    da.n_base = n0 + wn * C::TN;
    da.N = p.N;
    da.dzq = p.yq;
    da.dzq_scales = p.yq_scales;
    da.dzq_rows = p.yq_rows;
    static_assert(C::NW * DzStaging<C::TN, ACT>::BYTES <= C::SMEM, "dz staging must fit into the idle stages");
    dz_epilogue<Fp8Mma, C::TM, C::TN, ACT, 1, true>(acc, smem + wave * DzStaging<C::TN, ACT>::BYTES, lane, da, [&]() {
      wait_vmem_all();
      wait_lds_all();
      lds_barrier();  // every wave has finished reading the last stage
    });
    return;
  }
  FwdEpilogueArgs ea;
  ea.bias = p.bias ? p.bias + (int64_t)e * p.N : nullptr;
  ea.out0 = p.out0;
  ea.out0_stride = p.out0_stride;
  ea.out1 = p.out1;
  ea.out1_stride = p.out1_stride;
  ea.m_base = row0 + wm * C::TM;
  ea.row_end = row_end;
  ea.n_base = n0 + wn * C::TN;
  ea.N = p.N;
  wait_vmem_all();
  lds_barrier();  // all waves are done reading the last stage
  forward_epilogue<Fp8Mma, C::TM, C::TN, WITH_ACT, ACT>(acc, smem, wave, lane, ea);
  if constexpr (WITH_ACT) {
    if (p.yq != nullptr)  // the parking area of forward_epilogue is read back by the same wave that wrote it: no barrier
      fp8_activation_epilogue<C::TM, C::TN, FM, FN, ACT>(acc, smem + wave * (C::TM * (C::TN * 2 + 16)), lane, p.yq, p.I,
                                                          p.yq_scales, p.yq_rows, ea.m_base, row_end, ea.n_base);
  }
}

// The same GEMM as a tile stream: one workgroup per compute unit walks through the tiles b, b + gridDim.x, ... and keeps
// its double buffer running across tile boundaries (gemm_stream_loop with two slots per operand): the first stage of
// the next tile is on its way while the finished tile's epilogue runs, and the epilogue's stores drain under the next
// tile's first stages.  Needs Kdim >= 2 stages.  The forward roles only: the dz epilogue stages 32 rows of z and y1s
// per wave (32-row fragments), which the two vacated slots cannot hold for eight waves.
template <bool WITH_ACT, int ACT>
__global__ __launch_bounds__(Fp8Cfg::NT) void fp8_stream_kernel(const Fp8Params p) {
  using C = Fp8Cfg;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int FM = C::FM, FN = C::FN, SLICES = C::BKB / 64, PI = C::PS_INSTR, QI = C::QS_INSTR;
  const uint32_t smem_base = lds_address(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % C::WM, wn = wave / C::WM;

  const StreamTiles tiles(p.tm, p.off, p.n_tiles, C::BN);
  int64_t vb = blockIdx.x;
  StreamTile cur = tiles.at(vb);
  if (!cur.valid) return;
  StreamTile nxt = tiles.at(vb += gridDim.x);
  bool more = nxt.valid;  // a tile follows the current one
  if (!more) nxt = cur;   // the streams always run on: past the last tile they re-read it into slots nobody reads
  StreamTile nn = tiles.at(vb += gridDim.x);

  // Everything a tile switch computes from the lane number starts from a copy of it the compiler cannot see through:
  // otherwise the per-lane parts are hoisted out of the tile loop and occupy registers the main loop needs.
  auto opaque_lane = [&]() {
    int l = lane;
    asm volatile("" : "+v"(l));
    return l;
  };
  // source rows of a tile's token operand: one per data load and the row whose scale word the lane fetches
  auto token_rows = [&](const StreamTile& t, int(&rows)[PI + 1]) {
    const int ln = opaque_lane();
#pragma unroll
    for (int i = 0; i <= PI; i++) {
      int m = t.row0 + (i < PI ? (wave * PI + i) * C::KRPI + ln / C::KPR : wave * 32 + (ln & 31));
      m = m < t.row_end ? m : t.row_end - 1;
      rows[i] = p.gidx && (i < PI || !p.scales_grouped) ? p.gidx[m] : m - t.row0;
    }
  };
  // Operands and scale tables are fetched through buffer resources: a lane keeps one 32-bit byte offset per load
  // (fixed for a tile), the position along the contraction is a wave-uniform offset.  The token operand's resources
  // start at the tensors (gathered rows) or at the tile's first row; the weight operand's at the tile's expert.
  uint32_t p_voff[PI + 1], q_voff[QI + 1];
  i32x4 p_rsrc = make_buffer_resource(p.P), ps_rsrc = make_buffer_resource(p.p_scales);
  i32x4 q_rsrc = make_buffer_resource(p.Q), qs_rsrc = make_buffer_resource(p.q_scales);
  const uint32_t p_row_bytes = (uint32_t)p.p_stride, q_row_bytes = (uint32_t)p.q_stride_row;
  const uint32_t ps_step = (uint32_t)p.p_rows * 4u, qs_step = (uint32_t)p.q_rows * 4u;
  auto point_p = [&](const int(&rows)[PI + 1], const StreamTile& t) {
    const int ln = opaque_lane();
    if (!p.gidx) p_rsrc = make_buffer_resource(p.P + (int64_t)t.row0 * p.p_stride);
    if (!p.gidx || p.scales_grouped) ps_rsrc = make_buffer_resource(p.p_scales + t.row0);
#pragma unroll
    for (int i = 0; i < PI; i++) {
      const int r = (wave * PI + i) * C::KRPI + ln / C::KPR;
      // rows and row sizes are below 2^24 (checked on the host): one 32-bit multiply-add per offset
      p_voff[i] = __umul24((uint32_t)rows[i], p_row_bytes) + ((((uint32_t)ln % C::KPR) ^ kswz<64>(r)) << 4);
    }
    p_voff[PI] = (uint32_t)rows[PI] * 4u;
  };
  auto point_q = [&](const StreamTile& t) {
    const int ln = opaque_lane();
    q_rsrc = make_buffer_resource(p.Q + (int64_t)t.e * p.q_stride_e);
    qs_rsrc = make_buffer_resource(p.q_scales + (int64_t)t.e * p.N);
#pragma unroll
    for (int i = 0; i <= QI; i++) {
      const int r = i < QI ? (wave * QI + i) * C::KRPI + ln / C::KPR : wave * 32 + (ln & 31);
      int n = t.n0 + r;
      n = n < p.N ? n : p.N - 1;
      q_voff[i] = i < QI ? __umul24((uint32_t)n, q_row_bytes) + ((((uint32_t)ln % C::KPR) ^ kswz<64>(r)) << 4) : (uint32_t)n * 4u;
    }
  };
  int rows_next[PI + 1];  // token rows of nxt: loaded at the start of a tile, picked up behind its first stage
  {
    int rows_cur[PI + 1];
    token_rows(cur, rows_cur);
    point_p(rows_cur, cur);
    point_q(cur);
    token_rows(nxt, rows_next);
  }

  const int S_total = p.Kdim / C::BKB;

  // per-lane LDS fragment offsets (bytes inside a slot): two 16-byte pieces per slice, one scale word per stage
  const int half = lane >> 5;
  int p_off[SLICES][2], q_off[SLICES][2];
  {
    const int prow = wm * C::TM + (lane & 31), qrow = wn * C::TN + (lane & 31);
    const int psw = kswz<64>(prow), qsw = kswz<64>(qrow);
#pragma unroll
    for (int ks = 0; ks < SLICES; ks++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int piece = 4 * ks + 2 * j + half;
        p_off[ks][j] = prow * C::BKB + ((piece ^ psw) << 4);
        q_off[ks][j] = qrow * C::BKB + ((piece ^ qsw) << 4);
      }
  }
  // the scale word of tile row r lies at (r / 32) * 256 + (r % 32) * 4 of the slot's scale area
  const int ps_off = C::P_STAGE + wm * (C::TM / 32) * 256 + (lane & 31) * 4;
  const int qs_off = C::Q_STAGE + wn * (C::TN / 32) * 256 + (lane & 31) * 4;

  f32x16 acc[FN][FM];  // started from zero by the first k-slice of every tile

  constexpr int Q_RING = 2 * C::P_SLOT;
  int p_stage = 0, q_stage = 0;  // stages issued to each stream for the tile it is on
  auto issue_p = [&](int slot, auto i_c) {
    constexpr int i = decltype(i_c)::value;
    const uint32_t base = smem_base + slot * C::P_SLOT;
    if constexpr (i < PI)
      buffer_load16_to_lds(p_rsrc, p_voff[i], (uint32_t)p_stage * C::BKB, base + (wave * PI + i) * 1024);
    else
      buffer_load4_to_lds(ps_rsrc, p_voff[PI], (uint32_t)p_stage * ps_step, base + C::P_STAGE + wave * 256);
  };
  auto issue_q = [&](int slot, auto j_c) {
    constexpr int j = decltype(j_c)::value;
    const uint32_t base = smem_base + Q_RING + slot * C::Q_SLOT;
    if constexpr (j < QI)
      buffer_load16_to_lds(q_rsrc, q_voff[j], (uint32_t)q_stage * C::BKB, base + (wave * QI + j) * 1024);
    else
      buffer_load4_to_lds(qs_rsrc, q_voff[QI], (uint32_t)q_stage * qs_step, base + C::Q_STAGE + wave * 256);
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
  auto load = [&](int p_slot, int q_slot, auto step_c, Fp8Frag(&qf)[FN], Fp8Frag(&pf)[C::NP]) {
    constexpr int step = decltype(step_c)::value, ks = Fp8Mma::kslice(step), ph = Fp8Mma::phalf(step);
    const char* ps = smem + p_slot * C::P_SLOT;
    const char* qs = smem + Q_RING + q_slot * C::Q_SLOT;
    const int shift = 8 * (2 * ks + half);
#pragma unroll
    for (int pp = 0; pp < C::NP; pp++) {
      const int fm = ph * C::NP + pp;
      const i32x4 lo = *(const i32x4*)(ps + p_off[ks][0] + fm * 32 * C::BKB);
      const i32x4 hi = *(const i32x4*)(ps + p_off[ks][1] + fm * 32 * C::BKB);
      pf[pp].data = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      pf[pp].scale = (int)(*(const uint32_t*)(ps + ps_off + fm * 256) >> shift);
    }
    if constexpr (Fp8Mma::reads_q(step)) {
#pragma unroll
      for (int fn = 0; fn < FN; fn++) {
        const i32x4 lo = *(const i32x4*)(qs + q_off[ks][0] + fn * 32 * C::BKB);
        const i32x4 hi = *(const i32x4*)(qs + q_off[ks][1] + fn * 32 * C::BKB);
        qf[fn].data = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        qf[fn].scale = (int)(*(const uint32_t*)(qs + qs_off + fn * 256) >> shift);
      }
    }
  };
  // the rows loaded in tile_end are complete here; naming them in an asm statement makes this the place where the
  // compiler waits for them
  auto first_boundary = [&]() {
#pragma unroll
    for (int i = 0; i <= PI; i++) asm volatile("" : "+v"(rows_next[i]));
  };
  // what a wave parks in the two slots the tile's last stage vacates: 32 rows of its output
  constexpr int PARK = 32 * EpiLayout<C::TN>::ROW_BYTES;
  static_assert((C::NW / 2) * PARK <= C::P_STAGE && (C::NW / 2) * PARK <= C::Q_STAGE, "parking must fit into a slot");
  auto tile_end = [&](int p_slot, int q_slot) {
    // waves 0..NW/2-1 park in the vacated token slot, the others in the vacated weight slot
    char* region = wave < C::NW / 2 ? smem + p_slot * C::P_SLOT + wave * PARK
                                    : smem + Q_RING + q_slot * C::Q_SLOT + (wave - C::NW / 2) * PARK;
    const int m_base = cur.row0 + wm * C::TM, n_base = cur.n0 + wn * C::TN;
    FwdEpilogueArgs ea;
    ea.bias = p.bias ? p.bias + (int64_t)cur.e * p.N : nullptr;
    ea.out0 = p.out0;
    ea.out0_stride = p.out0_stride;
    ea.out1 = p.out1;
    ea.out1_stride = p.out1_stride;
    ea.m_base = m_base;
    ea.row_end = cur.row_end;
    ea.n_base = n_base;
    ea.N = p.N;
    forward_epilogue_rows<Fp8Mma, C::TM, C::TN, WITH_ACT, ACT>(acc, region, opaque_lane(), ea);
    if constexpr (WITH_ACT) {
      if (p.yq != nullptr)  // the region is read back by the same wave that wrote it: no barrier
        fp8_activation_epilogue<C::TM, C::TN, FM, FN, ACT>(acc, region, opaque_lane(), p.yq, p.I, p.yq_scales,
                                                            p.yq_rows, m_base, cur.row_end, n_base);
    }
    if (!more) return false;
    cur = nxt;
    nxt = nn;
    more = nxt.valid;
    if (!more) nxt = cur;
    nn = tiles.at(vb += gridDim.x);
    token_rows(nxt, rows_next);
    return true;
  };
  // 3 LDS reads per fragment (two 16-byte pieces and the scale word), dealt out three per matrix instruction
  gemm_stream_loop<FN, C::NP, 3 * (FN + C::NP), PI + 1, QI + 1, Fp8Mma::PH * SLICES, Fp8Mma, 4, 2>(
      S_total, acc, issue_p, issue_q, load, issued_p, issued_q, first_boundary, tile_end);
}

template <bool WITH_ACT, int ACT, bool DZ = false>
static int launch_fp8(Fp8Params& p, const int32_t* off, void* workspace, int64_t TK, int E, hipStream_t st) {
  using C = Fp8Cfg;
  static LdsLimitOnce lds_limit;
  auto kern = fp8_varlen_m_kernel<WITH_ACT, ACT, DZ>;
  {
    const int rc_attr = lds_limit.ensure((const void*)kern, C::SMEM);
    if (rc_attr) return rc_attr;
  }
  p.tm = carve_tile_map(workspace, TK, E, C::BM);
  int rc = launch_build_tile_map(off, nullptr, E, C::BM, p.tm, st);
  if (rc) return rc;
  p.n_tiles = (int)ceil_div(p.N, C::BN);
  if (DZ) p.ds_cols = p.n_tiles * C::WN;
  // the kernel addresses its operands with 32-bit byte offsets from a buffer base
  const int64_t lim = 1ll << 32;
  const int64_t data_rows = p.data_rows ? p.data_rows : p.p_rows;
  SMOE_REQUIRE((p.gidx ? data_rows : (int64_t)C::BM) * p.p_stride < lim && (int64_t)p.N * p.q_stride_row < lim &&
                   (int64_t)(p.Kdim / C::BKB) * (p.p_rows > p.q_rows ? p.p_rows : p.q_rows) * 4 < lim,
               SMOE_ERR_UNSUPPORTED, "fp8 grouped gemm: operand too large for 32-bit offsets");
  const int64_t max_tiles = max_token_tiles(TK, E, C::BM) * p.n_tiles;
  const int64_t grid = ((max_tiles + 7) / 8) * 8;
  SMOE_REQUIRE(grid < (1ll << 31) && tile_map_fits(TK, E, C::BM), SMOE_ERR_UNSUPPORTED, "fp8 grouped gemm: too many tiles");
  const Tuning& tune = tuning();
  const int64_t lim24 = 1ll << 24;  // the tile-stream kernel forms its offsets with 24-bit multiplies
  const bool fits24 = data_rows < lim24 && p.p_rows < lim24 && p.p_stride < lim24 && p.N < lim24 && p.q_stride_row < lim24;
  if constexpr (!DZ) if (tune.gemm_stream && p.Kdim >= 2 * C::BKB && fits24) {
    static LdsLimitOnce lds_limit_stream;
    auto skern = fp8_stream_kernel<WITH_ACT, ACT>;
    const int rc_s = lds_limit_stream.ensure((const void*)skern, C::STREAM_SMEM);
    if (rc_s) return rc_s;
    int cus = 0;
    const int rc_cu = device_compute_units(&cus);
    if (rc_cu) return rc_cu;
    int64_t sgrid = ((int64_t)cus / 8) * 8;  // one resident workgroup per compute unit, the same number on every XCD
    // a smaller grid makes small problems run several tiles per workgroup (used by the tests)
    if (tune.gemm_stream_grid > 0) sgrid = ((int64_t)tune.gemm_stream_grid + 7) / 8 * 8;
    if (sgrid < 8) sgrid = 8;
    if (sgrid > grid) sgrid = grid;
    hipLaunchKernelGGL(skern, dim3((unsigned)sgrid), dim3(C::NT), C::STREAM_SMEM, st, p);
    SMOE_LAUNCH_CHECK();
    return SMOE_OK;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(C::NT), C::SMEM, st, p);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

static int launch_fp8_up(int act, Fp8Params& p, const int32_t* off, void* ws, int64_t TK, int E, hipStream_t st) {
  switch (act) {
    case SMOE_ACT_SWIGLU: return launch_fp8<true, SMOE_ACT_SWIGLU>(p, off, ws, TK, E, st);
    case SMOE_ACT_GEGLU: return launch_fp8<true, SMOE_ACT_GEGLU>(p, off, ws, TK, E, st);
    case SMOE_ACT_REGLU: return launch_fp8<true, SMOE_ACT_REGLU>(p, off, ws, TK, E, st);
    case SMOE_ACT_RELU_SQ: return launch_fp8<true, SMOE_ACT_RELU_SQ>(p, off, ws, TK, E, st);
    case SMOE_ACT_RELU: return launch_fp8<true, SMOE_ACT_RELU>(p, off, ws, TK, E, st);
    case SMOE_ACT_GELU: return launch_fp8<true, SMOE_ACT_GELU>(p, off, ws, TK, E, st);
    case SMOE_ACT_SILU: return launch_fp8<true, SMOE_ACT_SILU>(p, off, ws, TK, E, st);
  }
  set_error("unknown activation code %d", act);
  return SMOE_ERR_INVALID;
}

static int launch_fp8_dz(int act, Fp8Params& p, const int32_t* off, void* ws, int64_t TK, int E, hipStream_t st) {
  switch (act) {
    case SMOE_ACT_SWIGLU: return launch_fp8<false, SMOE_ACT_SWIGLU, true>(p, off, ws, TK, E, st);
    case SMOE_ACT_GEGLU: return launch_fp8<false, SMOE_ACT_GEGLU, true>(p, off, ws, TK, E, st);
    case SMOE_ACT_REGLU: return launch_fp8<false, SMOE_ACT_REGLU, true>(p, off, ws, TK, E, st);
    case SMOE_ACT_RELU_SQ: return launch_fp8<false, SMOE_ACT_RELU_SQ, true>(p, off, ws, TK, E, st);
    case SMOE_ACT_RELU: return launch_fp8<false, SMOE_ACT_RELU, true>(p, off, ws, TK, E, st);
    case SMOE_ACT_GELU: return launch_fp8<false, SMOE_ACT_GELU, true>(p, off, ws, TK, E, st);
    case SMOE_ACT_SILU: return launch_fp8<false, SMOE_ACT_SILU, true>(p, off, ws, TK, E, st);
  }
  set_error("unknown activation code %d", act);
  return SMOE_ERR_INVALID;
}

// ---- transposing quantiser -----------------------------------------------------------------------------------------
// src: E matrices (R, C) bf16, row stride src_stride_r, matrix stride src_stride_e.  q: E matrices (C, R) e4m3, the
// transposes, quantised along R (32 consecutive r share a scale); scales (R / 128, E * C) words as in mx_quantize.
// One workgroup transposes a 128 (r) x TC (c) tile through LDS: row-contiguous loads, column reads (one lane = one
// column and one 32-row block), bytes parked transposed, row-contiguous stores of 128 bytes per output row.
// BOTH: the same tile is also quantised along its rows (the forward GEMMs' operand, exactly what mx_quantize_kernel
// computes from the matrix in memory), so a weight is read from HBM once for both copies; the tile is 128 columns wide
// then, so that the row-quantised copy is written in whole 128-byte lines and whole scale words as well.
template <bool BOTH>
__global__ __launch_bounds__(256) void mx_quantize_transposed_kernel(const uint16_t* __restrict__ src,
                                                                     int64_t src_stride_e, int64_t src_stride_r, int R,
                                                                     int C, int E, uint8_t* __restrict__ q,
                                                                     uint32_t* __restrict__ scales,
                                                                     uint8_t* __restrict__ q_rows,
                                                                     uint32_t* __restrict__ scales_rows) {
  constexpr int TR = 128, TC = BOTH ? 128 : 64, IN_PITCH = TC * 2 + 4, OUT_PITCH = TR + 8;
  constexpr int LPR = TC / 8, RPP = 256 / LPR;  // lanes per input row (16 bytes each), input rows per pass
  __shared__ __attribute__((aligned(16))) char tile_in[TR * IN_PITCH];
  __shared__ __attribute__((aligned(16))) char tile_out[TC * OUT_PITCH];
  __shared__ uint8_t exps[TC][4];
  const int tid = threadIdx.x;
  const int c0 = blockIdx.x * TC, r0 = blockIdx.y * TR, e = blockIdx.z;
  const uint16_t* base = src + (int64_t)e * src_stride_e + (int64_t)r0 * src_stride_r + c0;
#pragma unroll
  for (int pass = 0; pass < TR / RPP; pass++) {
    const int r = pass * RPP + tid / LPR, piece = tid % LPR;
    const u32x4 v = *(const u32x4*)(base + (int64_t)r * src_stride_r + piece * 8);
    uint32_t* dst = (uint32_t*)(tile_in + r * IN_PITCH + piece * 16);
    dst[0] = v[0];
    dst[1] = v[1];
    dst[2] = v[2];
    dst[3] = v[3];
  }
  __syncthreads();
  if constexpr (BOTH) {
    // lane = (row, half of its 128 columns): two 32-column blocks, 64 contiguous output bytes
    const int r = tid / 2, hb = tid % 2;
    u32x4 o[4];
    uint32_t ex2 = 0;
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      float w[32];
      float am = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const uint32_t two = *(const uint32_t*)(tile_in + r * IN_PITCH + hb * 128 + blk * 64 + i * 4);
        w[2 * i] = elem_lo(two);
        w[2 * i + 1] = elem_hi(two);
        am = fmaxf(am, fmaxf(fabsf(w[2 * i]), fabsf(w[2 * i + 1])));
      }
      const int exr = mx_scale_exponent(am);
      const float invr = __uint_as_float((uint32_t)(254 - exr) << 23);
      ex2 |= (uint32_t)exr << (8 * blk);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        int ww = 0;
        ww = __builtin_amdgcn_cvt_pk_fp8_f32(w[4 * i] * invr, w[4 * i + 1] * invr, ww, false);
        ww = __builtin_amdgcn_cvt_pk_fp8_f32(w[4 * i + 2] * invr, w[4 * i + 3] * invr, ww, true);
        o[2 * blk + i / 4][i % 4] = (uint32_t)ww;
      }
    }
    const int64_t grow = (int64_t)e * R + r0 + r;  // row of the (E * R, C) code matrix
    u32x4* dst = (u32x4*)(q_rows + grow * C + c0 + hb * 64);
#pragma unroll
    for (int i = 0; i < 4; i++) dst[i] = o[i];
    // scale table (C / 128, E * R) words: the row's four blocks of this 128-column tile are one word
    const uint32_t other = __shfl_xor(ex2, 1, 64);
    if (hb == 0) scales_rows[(int64_t)(c0 >> 7) * ((int64_t)E * R) + grow] = ex2 | (other << 16);
  }
  // lane = (column, 32-row block)
#pragma unroll
  for (int rb = tid / TC; rb < TR / 32; rb += 256 / TC) {
    const int c = tid % TC;
    float v[32];
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const uint16_t h = *(const uint16_t*)(tile_in + (rb * 32 + i) * IN_PITCH + c * 2);
      v[i] = elem_bits_to_f32(h);
      amax = fmaxf(amax, fabsf(v[i]));
    }
    const int ex = mx_scale_exponent(amax);
    const float inv = __uint_as_float((uint32_t)(254 - ex) << 23);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[8 * i] * inv, v[8 * i + 1] * inv, 0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[8 * i + 2] * inv, v[8 * i + 3] * inv, w0, true);
      int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[8 * i + 4] * inv, v[8 * i + 5] * inv, 0, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[8 * i + 6] * inv, v[8 * i + 7] * inv, w1, true);
      *(u32x2*)(tile_out + c * OUT_PITCH + rb * 32 + i * 8) = u32x2{(uint32_t)w0, (uint32_t)w1};
    }
    exps[c][rb] = (uint8_t)ex;
  }
  __syncthreads();
  // 16 lanes x 8 bytes per output row, 16 rows per pass
  uint8_t* qbase = q + ((int64_t)e * C + c0) * R + r0;
#pragma unroll
  for (int pass = 0; pass < TC / 16; pass++) {
    const int cc = pass * 16 + tid / 16, piece = tid % 16;
    const u32x2 w = *(const u32x2*)(tile_out + cc * OUT_PITCH + piece * 8);
    *(u32x2*)(qbase + (int64_t)cc * R + piece * 8) = w;
  }
  if (tid < TC) scales[(int64_t)(r0 / 128) * ((int64_t)E * C) + (int64_t)e * C + c0 + tid] = *(const uint32_t*)exps[tid];
}

}  // namespace smoe

using namespace smoe;

extern "C" int smoe_mx_quantize_transposed(const void* src, int64_t src_stride_e, int64_t src_stride_r, int E, int R,
                                           int C, void* q, void* scales, void* stream) {
  SMOE_REQUIRE(E >= 1 && R > 0 && C > 0, SMOE_ERR_INVALID, "mx_quantize_transposed: bad shape");
  SMOE_REQUIRE(R % 128 == 0 && C % 64 == 0, SMOE_ERR_UNSUPPORTED,
               "mx_quantize_transposed: (%d, %d) matrices: rows must be a multiple of 128, columns of 64", R, C);
  SMOE_REQUIRE(src_stride_e % 8 == 0 && src_stride_r % 8 == 0, SMOE_ERR_UNSUPPORTED,
               "mx_quantize_transposed: strides must be multiples of 8 elements");
  SMOE_REQUIRE(src && q && scales, SMOE_ERR_INVALID, "mx_quantize_transposed: null pointer");
  SMOE_REQUIRE_ALIGNED("mx_quantize_transposed", src, q, scales);
  SMOE_REQUIRE(E < 65536 && R / 128 < 65536, SMOE_ERR_UNSUPPORTED, "mx_quantize_transposed: tensor too large");
  hipLaunchKernelGGL(mx_quantize_transposed_kernel<false>, dim3((unsigned)(C / 64), (unsigned)(R / 128), (unsigned)E),
                     dim3(256), 0, (hipStream_t)stream, (const uint16_t*)src, src_stride_e, src_stride_r, R, C, E,
                     (uint8_t*)q, (uint32_t*)scales, (uint8_t*)nullptr, (uint32_t*)nullptr);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_mx_quantize_both(const void* src, int64_t src_stride_e, int64_t src_stride_r, int E, int R, int C,
                                     void* q_rows, void* scales_rows, void* q_t, void* scales_t, void* stream) {
  SMOE_REQUIRE(E >= 1 && R > 0 && C > 0, SMOE_ERR_INVALID, "mx_quantize_both: bad shape");
  SMOE_REQUIRE(R % 128 == 0 && C % 128 == 0, SMOE_ERR_UNSUPPORTED,
               "mx_quantize_both: (%d, %d) matrices: rows and columns must be multiples of 128", R, C);
  SMOE_REQUIRE(src_stride_e % 8 == 0 && src_stride_r % 8 == 0, SMOE_ERR_UNSUPPORTED,
               "mx_quantize_both: strides must be multiples of 8 elements");
  SMOE_REQUIRE(src && q_rows && scales_rows && q_t && scales_t, SMOE_ERR_INVALID, "mx_quantize_both: null pointer");
  SMOE_REQUIRE_ALIGNED("mx_quantize_both", src, q_rows, scales_rows, q_t, scales_t);
  SMOE_REQUIRE(E < 65536 && R / 128 < 65536, SMOE_ERR_UNSUPPORTED, "mx_quantize_both: tensor too large");
  hipLaunchKernelGGL(mx_quantize_transposed_kernel<true>, dim3((unsigned)(C / 128), (unsigned)(R / 128), (unsigned)E),
                     dim3(256), 0, (hipStream_t)stream, (const uint16_t*)src, src_stride_e, src_stride_r, R, C, E,
                     (uint8_t*)q_t, (uint32_t*)scales_t, (uint8_t*)q_rows, (uint32_t*)scales_rows);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_mx_quantize(const void* src, int64_t src_stride, int64_t R, int C, void* q, void* scales,
                                void* stream) {
  SMOE_REQUIRE(R >= 0 && C > 0, SMOE_ERR_INVALID, "mx_quantize: bad shape");
  SMOE_REQUIRE(C % 128 == 0, SMOE_ERR_UNSUPPORTED, "mx_quantize: %d columns are not a multiple of 128", C);
  SMOE_REQUIRE(src_stride % 8 == 0, SMOE_ERR_UNSUPPORTED, "mx_quantize: row stride must be a multiple of 8 elements");
  if (R == 0) return SMOE_OK;
  SMOE_REQUIRE(src && q && scales, SMOE_ERR_INVALID, "mx_quantize: null pointer");
  const int64_t blocks = R * (C / 32);
  SMOE_REQUIRE(ceil_div(blocks, 256) < (1ll << 31), SMOE_ERR_UNSUPPORTED, "mx_quantize: tensor too large");
  hipLaunchKernelGGL(mx_quantize_kernel, dim3((unsigned)ceil_div(blocks, 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)src, src_stride, R, C, (uint8_t*)q, (uint32_t*)scales);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

// ---- scale words of a gathered token operand in grouped row order ---------------------------------------------------
// The GEMM kernels fetch one scale word per tile row and stage.  Through the gather index that is one cache line per
// row (64 scattered 4-byte reads per load instruction); from a table in grouped order it is two lines per 64 rows.
// dst[g][m] = src[g][gidx[m]] for the KB 128-element blocks of the contraction.
__global__ __launch_bounds__(256) void gather_scale_rows_kernel(const uint32_t* __restrict__ src, int64_t src_rows,
                                                                const int32_t* __restrict__ gidx,
                                                                uint32_t* __restrict__ dst, int64_t TK, int KB) {
  const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (m >= TK) return;
  const int64_t r = gidx[m];
  for (int g = 0; g < KB; g++) dst[(int64_t)g * TK + m] = src[(int64_t)g * src_rows + r];
}

static size_t grouped_scales_offset(int64_t TK, int E) { return (tile_map_bytes(TK, E) + 255) / 256 * 256; }

// Points p at a grouped copy of its token operand's scale table in the workspace behind the tile map, if the workspace
// is large enough for it (smoe_fp8_gemm_workspace_bytes); otherwise the kernels go through the gather index.
static int group_token_scales(Fp8Params& p, void* workspace, size_t workspace_bytes, int64_t TK, int E,
                              hipStream_t st) {
  const int KB = p.Kdim / 128;
  const size_t at = grouped_scales_offset(TK, E);
  if (p.gidx == nullptr || workspace_bytes < at + (size_t)KB * TK * sizeof(uint32_t)) return SMOE_OK;
  uint32_t* dst = (uint32_t*)((char*)workspace + at);
  hipLaunchKernelGGL(gather_scale_rows_kernel, dim3((unsigned)ceil_div(TK, 256)), dim3(256), 0, st, p.p_scales,
                     p.p_rows, p.gidx, dst, TK, KB);
  SMOE_LAUNCH_CHECK();
  p.p_scales = dst;
  if (p.data_rows == 0) p.data_rows = p.p_rows;  // the data operand keeps its T rows; only the scale table is regrouped
  p.p_rows = TK;
  p.scales_grouped = 1;
  return SMOE_OK;
}

extern "C" size_t smoe_fp8_gemm_workspace_bytes(int64_t TK, int E, int K) {
  if (TK < 0 || E < 1 || K < 128) return 0;
  return grouped_scales_offset(TK, E) + (size_t)(K / 128) * TK * sizeof(uint32_t);
}

static int check_fp8(int64_t TK, int Kdim, int N, int E, const void* ws, size_t ws_bytes, const char* who) {
  SMOE_REQUIRE(TK >= 0 && TK < (1ll << 31), SMOE_ERR_INVALID, "%s: TK out of range", who);
  SMOE_REQUIRE(E >= 1, SMOE_ERR_INVALID, "%s: E must be >= 1", who);
  SMOE_REQUIRE(Kdim >= 128 && Kdim % 128 == 0, SMOE_ERR_UNSUPPORTED,
               "%s: the contraction size %d must be a multiple of 128", who, Kdim);
  SMOE_REQUIRE(N >= 64 && N % 64 == 0, SMOE_ERR_UNSUPPORTED, "%s: the output width %d must be a multiple of 64", who, N);
  SMOE_REQUIRE(ws != nullptr && ws_bytes >= smoe_gemm_workspace_bytes(TK, E), SMOE_ERR_WORKSPACE,
               "%s: workspace too small", who);
  return SMOE_OK;
}

extern "C" int smoe_up_projection_forward_fp8(const void* xq, const void* x_scales, const void* w1q,
                                              const void* w1_scales, const void* b1, void* z, void* y1, void* y1q,
                                              void* y1q_scales, const int32_t* off, const int32_t* x_gather_idx,
                                              int64_t T, int64_t TK, int H, int I, int E, int activation,
                                              void* workspace, size_t workspace_bytes, void* stream) {
  SMOE_REQUIRE(activation >= SMOE_ACT_SWIGLU && activation <= SMOE_ACT_SILU, SMOE_ERR_INVALID,
               "up_projection_forward_fp8: unknown activation code %d", activation);
  const int N1 = act_is_glu(activation) ? 2 * I : I;
  int rc = check_fp8(TK, H, N1, E, workspace, workspace_bytes, "up_projection_forward_fp8");
  if (rc) return rc;
  SMOE_REQUIRE(I % 64 == 0, SMOE_ERR_UNSUPPORTED, "up_projection_forward_fp8: I=%d must be a multiple of 64", I);
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(xq && x_scales && w1q && w1_scales && off && x_gather_idx && T > 0, SMOE_ERR_INVALID,
               "up_projection_forward_fp8: null pointer");
  SMOE_REQUIRE(y1 || y1q, SMOE_ERR_INVALID, "up_projection_forward_fp8: neither y1 nor y1q is given");
  SMOE_REQUIRE((y1q == nullptr) == (y1q_scales == nullptr), SMOE_ERR_INVALID,
               "up_projection_forward_fp8: y1q and y1q_scales come together");
  SMOE_REQUIRE(!y1q || I % 128 == 0, SMOE_ERR_UNSUPPORTED,
               "up_projection_forward_fp8: a quantised y1 needs I=%d to be a multiple of 128", I);
  Fp8Params p = {};
  p.P = (const uint8_t*)xq;
  p.p_stride = H;
  p.p_scales = (const uint32_t*)x_scales;
  p.p_rows = T;
  p.gidx = x_gather_idx;
  p.Q = (const uint8_t*)w1q;
  p.q_stride_e = (int64_t)N1 * H;
  p.q_stride_row = H;
  p.q_scales = (const uint32_t*)w1_scales;
  p.q_rows = (int64_t)E * N1;
  p.off = off;
  p.N = N1;
  p.Kdim = H;
  p.bias = (const uint16_t*)b1;
  p.out0 = (uint16_t*)z;
  p.out0_stride = N1;
  p.out1 = (uint16_t*)y1;
  p.out1_stride = I;
  p.yq = (uint8_t*)y1q;
  p.yq_scales = (uint32_t*)y1q_scales;
  p.yq_rows = TK;
  p.I = I;
  rc = group_token_scales(p, workspace, workspace_bytes, TK, E, (hipStream_t)stream);
  if (rc) return rc;
  return launch_fp8_up(activation, p, off, workspace, TK, E, (hipStream_t)stream);
}

extern "C" int smoe_down_projection_forward_fp8(const void* y1q, const void* y1_scales, const void* w2q,
                                                const void* w2_scales, const void* b2, void* y2, const int32_t* off,
                                                int64_t TK, int H, int I, int E, void* workspace,
                                                size_t workspace_bytes, void* stream) {
  int rc = check_fp8(TK, I, H, E, workspace, workspace_bytes, "down_projection_forward_fp8");
  if (rc) return rc;
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(y1q && y1_scales && w2q && w2_scales && y2 && off, SMOE_ERR_INVALID,
               "down_projection_forward_fp8: null pointer");
  Fp8Params p = {};
  p.P = (const uint8_t*)y1q;
  p.p_stride = I;
  p.p_scales = (const uint32_t*)y1_scales;
  p.p_rows = TK;
  p.Q = (const uint8_t*)w2q;
  p.q_stride_e = (int64_t)H * I;
  p.q_stride_row = I;
  p.q_scales = (const uint32_t*)w2_scales;
  p.q_rows = (int64_t)E * H;
  p.off = off;
  p.N = H;
  p.Kdim = I;
  p.bias = (const uint16_t*)b2;
  p.out0 = (uint16_t*)y2;
  p.out0_stride = H;
  return launch_fp8<false, SMOE_ACT_SWIGLU>(p, off, workspace, TK, E, (hipStream_t)stream);
}

extern "C" int smoe_down_projection_backward_fp8(const void* doutq, const void* dout_scales, const void* w2tq,
                                                 const void* w2t_scales, const void* z, void* dz, void* dzq,
                                                 void* dzq_scales, void* y1s, float* ds, float* ds_partial,
                                                 const float* scores, const int32_t* off,
                                                 const int32_t* x_gather_idx, const int32_t* s_scatter_idx, int64_t T,
                                                 int64_t TK, int H, int I, int E, int activation, void* workspace,
                                                 size_t workspace_bytes, void* stream) {
  SMOE_REQUIRE(activation >= SMOE_ACT_SWIGLU && activation <= SMOE_ACT_SILU, SMOE_ERR_INVALID,
               "down_projection_backward_fp8: unknown activation code %d", activation);
  int rc = check_fp8(TK, H, I, E, workspace, workspace_bytes, "down_projection_backward_fp8");
  if (rc) return rc;
  const int zw = act_is_glu(activation) ? 2 : 1;
  SMOE_REQUIRE((zw * I) % 128 == 0, SMOE_ERR_UNSUPPORTED,
               "down_projection_backward_fp8: the width %d of dz must be a multiple of 128", zw * I);
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(doutq && dout_scales && w2tq && w2t_scales && z && dz && dzq && dzq_scales && y1s && ds && ds_partial &&
                   scores && off && x_gather_idx && s_scatter_idx && T > 0,
               SMOE_ERR_INVALID, "down_projection_backward_fp8: null pointer");
  SMOE_REQUIRE_ALIGNED("down_projection_backward_fp8", doutq, w2tq, z, dz, dzq, y1s);
  Fp8Params p = {};
  p.P = (const uint8_t*)doutq;
  p.p_stride = H;
  p.p_scales = (const uint32_t*)dout_scales;
  p.p_rows = T;
  p.gidx = x_gather_idx;
  p.Q = (const uint8_t*)w2tq;  // (E, I, H): W2[e]^T, contraction (h) contiguous
  p.q_stride_e = (int64_t)I * H;
  p.q_stride_row = H;
  p.q_scales = (const uint32_t*)w2t_scales;
  p.q_rows = (int64_t)E * I;
  p.off = off;
  p.N = I;
  p.Kdim = H;
  p.out0 = (uint16_t*)dz;
  p.out0_stride = (int64_t)zw * I;
  p.out1 = (uint16_t*)y1s;
  p.out1_stride = I;
  p.yq = (uint8_t*)dzq;
  p.yq_scales = (uint32_t*)dzq_scales;
  p.yq_rows = TK;
  p.I = I;
  p.zin = (const uint16_t*)z;
  p.zin_stride = (int64_t)zw * I;
  p.scores = scores;
  p.sidx = s_scatter_idx;
  p.ds_partial = ds_partial;
  hipStream_t st = (hipStream_t)stream;
  rc = group_token_scales(p, workspace, workspace_bytes, TK, E, st);
  if (rc) return rc;
  rc = launch_fp8_dz(activation, p, off, workspace, TK, E, st);
  if (rc) return rc;
  return launch_ds_finalize(ds_partial, p.ds_cols, s_scatter_idx, ds, TK, st);
}
