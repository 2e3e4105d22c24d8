// Weight-gradient grouped GEMMs ("varlen-K"): for every expert e
//     dW[e][a][b] = sum_{m in [off[e], off[e+1])} R[rowR(m)][a] * S[rowS(m)][b]
// The contraction runs over the expert's ragged token range; both operands are token-major in memory (a token row
// is contiguous along a resp. b), so both LDS stages are MN-major and both MFMA operands come from transpose loads.
// Either operand may be gathered through x_gather_idx, which re-reads the original activation rows instead of a
// materialised gathered copy.  Experts without tokens still get their zeros written.
//   dW1[e] (2I, H): R = dz rows,              S = x rows gathered
//   dW2[e] (H, I) : R = dout rows gathered,   S = y1s rows
#include "gemm_common.h"

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
};

template <int BA_, int BB_, int WA_, int WB_, bool R_GATHER_, bool S_GATHER_>
struct KCfg {
  static constexpr int BA = BA_, BB = BB_, WA = WA_, WB = WB_;
  static constexpr bool R_GATHER = R_GATHER_, S_GATHER = S_GATHER_;
  static constexpr int NW = WA * WB, NT = NW * 64;
  static constexpr int TA = BA / WA, TB = BB / WB;
  static constexpr int FA = TA / 32, FB = TB / 32;
  static constexpr int R_STAGE = BA * BK * 2, S_STAGE = BB * BK * 2;
  static constexpr int STAGE = R_STAGE + S_STAGE;
  static constexpr int SMEM = 2 * STAGE;
  static constexpr int R_ROWB = BA * 2, S_ROWB = BB * 2;
  static constexpr int R_LPR = R_ROWB / 16, S_LPR = S_ROWB / 16;
  static constexpr int R_RPI = 64 / R_LPR, S_RPI = 64 / S_LPR;
  static constexpr int R_INSTR = R_STAGE / 1024 / NW, S_INSTR = S_STAGE / 1024 / NW;
  static constexpr int R_SWM = (R_ROWB / 32 < 16 ? R_ROWB / 32 : 16) - 1;
  static constexpr int S_SWM = (S_ROWB / 32 < 16 ? S_ROWB / 32 : 16) - 1;
};

template <class C>
__global__ __launch_bounds__(C::NT) void varlen_k_kernel(const VarlenKParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int FA = C::FA, FB = C::FB;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave % C::WA, wb = wave / C::WA;

  const int64_t per_e = (int64_t)p.tiles_a * p.tiles_b;
  const int64_t lin = xcd_linear_tile(per_e * p.E);
  if (lin < 0) return;
  const int e = (int)(lin / per_e);
  const int within = (int)(lin - (int64_t)e * per_e);
  const int ta = within / p.tiles_b, tb = within % p.tiles_b;
  const int a0 = ta * C::BA, b0 = tb * C::BB;
  const int row_begin = p.off[e], row_end = p.off[e + 1];
  const int cnt = row_end - row_begin;
  const int KT = (cnt + BK - 1) / BK;

  // per-instruction k-row inside a stage and column offset (elements) of this lane's 16-byte piece
  int r_kl[C::R_INSTR], r_col[C::R_INSTR], s_kl[C::S_INSTR], s_col[C::S_INSTR];
#pragma unroll
  for (int i = 0; i < C::R_INSTR; i++) {
    const int kl = (wave * C::R_INSTR + i) * C::R_RPI + lane / C::R_LPR;
    const int phys16 = lane % C::R_LPR;
    const int log32 = (phys16 >> 1) ^ (kl & C::R_SWM);
    int a = a0 + ((log32 << 1) | (phys16 & 1)) * 8;
    a = a <= p.NA - 8 ? a : p.NA - 8;
    r_kl[i] = kl;
    r_col[i] = a;
  }
#pragma unroll
  for (int i = 0; i < C::S_INSTR; i++) {
    const int kl = (wave * C::S_INSTR + i) * C::S_RPI + lane / C::S_LPR;
    const int phys16 = lane % C::S_LPR;
    const int log32 = (phys16 >> 1) ^ (kl & C::S_SWM);
    int b = b0 + ((log32 << 1) | (phys16 & 1)) * 8;
    b = b <= p.NB - 8 ? b : p.NB - 8;
    s_kl[i] = kl;
    s_col[i] = b;
  }

  // transpose-load fragment offsets (bytes inside a stage)
  int r_off[2 * FA], s_off[2 * FB];
  {
    const int grp = lane >> 4, i16 = lane & 15;
    const int kk = 8 * (grp >> 1) + (i16 >> 2);
#pragma unroll
    for (int f = 0; f < FA; f++) {
      const int c32 = (wa * C::TA) / 16 + f * 2 + (grp & 1);
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = kk + 4 * h;
        r_off[f * 2 + h] = k * C::R_ROWB + ((c32 ^ (k & C::R_SWM)) << 5) + ((i16 & 3) << 3);
      }
    }
#pragma unroll
    for (int f = 0; f < FB; f++) {
      const int c32 = (wb * C::TB) / 16 + f * 2 + (grp & 1);
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = kk + 4 * h;
        s_off[f * 2 + h] = C::R_STAGE + k * C::S_ROWB + ((c32 ^ (k & C::S_SWM)) << 5) + ((i16 & 3) << 3);
      }
    }
  }

  f32x16 acc[FB][FA];
#pragma unroll
  for (int fb = 0; fb < FB; fb++)
#pragma unroll
    for (int fa = 0; fa < FA; fa++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[fb][fa][r] = 0.f;

  // source row of token (row_begin + kt*64 + kl), clamped to the expert's last token
  auto token_row = [&](int kt, int kl, bool gather) -> int64_t {
    int m = row_begin + kt * BK + kl;
    m = m < row_end ? m : row_end - 1;
    return gather ? (int64_t)p.gidx[m] : (int64_t)m;
  };

  int64_t r_row[C::R_INSTR], s_row[C::S_INSTR];
  auto fetch_rows = [&](int kt) {
#pragma unroll
    for (int i = 0; i < C::R_INSTR; i++) r_row[i] = token_row(kt, r_kl[i], C::R_GATHER);
#pragma unroll
    for (int i = 0; i < C::S_INSTR; i++) s_row[i] = token_row(kt, s_kl[i], C::S_GATHER);
  };
  auto issue = [&](int stage) {
    char* base = smem + stage * C::STAGE;
#pragma unroll
    for (int i = 0; i < C::R_INSTR; i++)
      load16_to_lds(p.R + r_row[i] * p.r_stride + r_col[i], base + (wave * C::R_INSTR + i) * 1024);
#pragma unroll
    for (int i = 0; i < C::S_INSTR; i++)
      load16_to_lds(p.S + s_row[i] * p.s_stride + s_col[i], base + C::R_STAGE + (wave * C::S_INSTR + i) * 1024);
  };

  if (KT > 0) {
    fetch_rows(0);
    issue(0);
    if (KT > 1) fetch_rows(1);
  }
  for (int kt = 0; kt < KT; kt++) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (kt + 1 < KT) {
      issue((kt + 1) & 1);
      if (kt + 2 < KT) fetch_rows(kt + 2);
    }
    const char* st = smem + (kt & 1) * C::STAGE;
    const int kvalid = cnt - kt * BK;  // tokens of this stage that exist (>= 64: all)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      bf16x8 rf[FA], sf[FB];
#pragma unroll
      for (int f = 0; f < FA; f++)
        rf[f] = lds_read_tr2(st + r_off[f * 2] + ks * 16 * C::R_ROWB, st + r_off[f * 2 + 1] + ks * 16 * C::R_ROWB);
#pragma unroll
      for (int f = 0; f < FB; f++)
        sf[f] = lds_read_tr2(st + s_off[f * 2] + ks * 16 * C::S_ROWB, st + s_off[f * 2 + 1] + ks * 16 * C::S_ROWB);
      if (kvalid < BK) {  // ragged end of the expert: rows past it were clamped copies, remove them from one side
        const int kbase = ks * 16 + 8 * (lane >> 5);
#pragma unroll
        for (int f = 0; f < FB; f++) {
          u32x4 w = __builtin_bit_cast(u32x4, sf[f]);
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const uint32_t keep = (kbase + 2 * q < kvalid ? 0x0000ffffu : 0u) | (kbase + 2 * q + 1 < kvalid ? 0xffff0000u : 0u);
            w[q] &= keep;
          }
          sf[f] = __builtin_bit_cast(bf16x8, w);
        }
      }
#pragma unroll
      for (int fb = 0; fb < FB; fb++)
#pragma unroll
        for (int fa = 0; fa < FA; fa++) acc[fb][fa] = mfma32(sf[fb], rf[fa], acc[fb][fa]);
    }
  }

  // epilogue: lane owns output row a = l%32, four consecutive columns b per register quad
  uint16_t* oe = p.out + (int64_t)e * p.out_stride_e;
#pragma unroll
  for (int fa = 0; fa < FA; fa++) {
    const int a = a0 + wa * C::TA + fa * 32 + (lane & 31);
    if (a >= p.NA) continue;
#pragma unroll
    for (int fb = 0; fb < FB; fb++) {
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const int b = b0 + wb * C::TB + fb * 32 + 8 * rg + 4 * (lane >> 5);
        if (b < p.NB) {
          u32x2 v = {pack_bf16x2(acc[fb][fa][4 * rg + 0], acc[fb][fa][4 * rg + 1]),
                     pack_bf16x2(acc[fb][fa][4 * rg + 2], acc[fb][fa][4 * rg + 3])};
          *(u32x2*)(oe + (int64_t)a * p.out_stride_row + b) = v;
        }
      }
    }
  }
}

template <class C>
static int launch_varlen_k(const VarlenKParams& p, hipStream_t st) {
  static bool attr_set = false;
  auto kern = varlen_k_kernel<C>;
  if (!attr_set) {
    SMOE_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM));
    attr_set = true;
  }
  const int64_t total = (int64_t)p.tiles_a * p.tiles_b * p.E;
  const int64_t grid = ((total + 7) / 8) * 8;
  SMOE_REQUIRE(grid < (1ll << 31), SMOE_ERR_UNSUPPORTED, "weight-grad gemm: too many tiles");
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(C::NT), C::SMEM, st, p);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

using KCfgDW1 = KCfg<256, 256, 2, 2, false, true>;
using KCfgDW2 = KCfg<256, 256, 2, 2, true, false>;

int launch_dz(const void* dout, const void* z, const void* w2, int64_t w2_stride_e, int64_t w2_stride_row, void* dz,
              void* y1s, float* ds_partial, const float* scores, const int32_t* off, const int32_t* gidx,
              const int32_t* sidx, int64_t TK, int H, int I, int E, void* workspace, hipStream_t st);
int launch_dx(const void* dz, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row, void* dx_expanded,
              const int32_t* off, int64_t TK, int H, int I, int E, void* workspace, hipStream_t st);

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
                                             int64_t w2_stride_row, void* dw2, int64_t dw2_stride_e,
                                             int64_t dw2_stride_row, void* dz, void* y1s, float* ds, float* ds_partial,
                                             const float* scores, const int32_t* off, const int32_t* x_gather_idx,
                                             const int32_t* s_scatter_idx, int64_t T, int64_t TK, int H, int I, int E,
                                             int activation, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_bwd(TK, H, I, E, workspace, workspace_bytes, "down_projection_backward");
  if (rc) return rc;
  SMOE_REQUIRE(activation == SMOE_ACT_SWIGLU, SMOE_ERR_UNSUPPORTED,
               "down_projection_backward: only SwiGLU is implemented (activation=%d)", activation);
  SMOE_REQUIRE(dw2 && off, SMOE_ERR_INVALID, "down_projection_backward: null pointer");
  SMOE_REQUIRE(TK == 0 || (dout && z && w2 && dz && y1s && ds && ds_partial && scores && x_gather_idx && s_scatter_idx),
               SMOE_ERR_INVALID, "down_projection_backward: null pointer");
  (void)T;
  hipStream_t st = (hipStream_t)stream;
  if (TK > 0) {
    rc = launch_dz(dout, z, w2, w2_stride_e, w2_stride_row, dz, y1s, ds_partial, scores, off, x_gather_idx,
                   s_scatter_idx, TK, H, I, E, workspace, st);
    if (rc) return rc;
    rc = launch_ds_finalize(ds_partial, smoe_dz_partial_cols(I), s_scatter_idx, ds, TK, st);
    if (rc) return rc;
  }
  using C = KCfgDW2;
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
  p.tiles_a = (int)ceil_div(H, C::BA);
  p.tiles_b = (int)ceil_div(I, C::BB);
  p.E = E;
  return launch_varlen_k<C>(p, st);
}

extern "C" int smoe_up_projection_backward(const void* x, const void* w1, int64_t w1_stride_e, int64_t w1_stride_row,
                                           const void* dz, void* dw1, int64_t dw1_stride_e, int64_t dw1_stride_row,
                                           void* dx_expanded, const int32_t* off, const int32_t* x_gather_idx,
                                           int64_t T, int64_t TK, int H, int I, int E, int activation, void* workspace,
                                           size_t workspace_bytes, void* stream) {
  int rc = check_bwd(TK, H, I, E, workspace, workspace_bytes, "up_projection_backward");
  if (rc) return rc;
  SMOE_REQUIRE(activation == SMOE_ACT_SWIGLU, SMOE_ERR_UNSUPPORTED,
               "up_projection_backward: only SwiGLU is implemented (activation=%d)", activation);
  SMOE_REQUIRE(dw1 && off, SMOE_ERR_INVALID, "up_projection_backward: null pointer");
  SMOE_REQUIRE(TK == 0 || (x && w1 && dz && dx_expanded && x_gather_idx), SMOE_ERR_INVALID,
               "up_projection_backward: null pointer");
  (void)T;
  hipStream_t st = (hipStream_t)stream;
  {
    using C = KCfgDW1;
    VarlenKParams p = {};
    p.R = (const uint16_t*)dz;
    p.r_stride = 2 * I;
    p.S = (const uint16_t*)x;
    p.s_stride = H;
    p.gidx = x_gather_idx;
    p.off = off;
    p.out = (uint16_t*)dw1;
    p.out_stride_e = dw1_stride_e;
    p.out_stride_row = dw1_stride_row;
    p.NA = 2 * I;
    p.NB = H;
    p.tiles_a = (int)ceil_div(2 * I, C::BA);
    p.tiles_b = (int)ceil_div(H, C::BB);
    p.E = E;
    rc = launch_varlen_k<C>(p, st);
    if (rc) return rc;
  }
  if (TK > 0) {
    rc = launch_dx(dz, w1, w1_stride_e, w1_stride_row, dx_expanded, off, TK, H, I, E, workspace, st);
    if (rc) return rc;
  }
  return SMOE_OK;
}
