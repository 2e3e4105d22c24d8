// Router in one pass over x: logits = x Wr^T on the matrix cores, and from the accumulators, without a second kernel
// or a trip through memory, the bf16 logits, the top-K winners with their softmax scores, and (optionally) the column
// sums of the full row softmax that the load-balancing loss needs.
//
// Replaces, for bf16 inputs, the chain router_logits = F.linear(x, router_w) -> sonicmoe::_softmax_topk_fwd
// (sonicmoe/functional/__init__.py:438-439, forward.py:224-237) and the F.softmax(router_logits, dtype=fp32).sum(0)
// of MoE._compute_switch_loss (sonicmoe/moe.py:247-274).
//
// A wavefront owns 16 tokens and all E columns.  The operand fragments of v_mfma_f32_16x16x32_bf16 are 16 contiguous
// bytes per lane of a row of x resp. Wr (row l % 16, contraction elements 8 * (l / 16) + 0..7): the x fragments are
// loaded straight from global memory into registers, 8 k-steps ahead (x is read exactly once, from HBM); Wr (E x H,
// 1 MiB at E = 128, L2-resident) is staged through a double-buffered LDS batch of 64 contraction elements that the
// workgroup's four wavefronts share (every wave reading all of Wr from L2 by itself made the kernel L2-bound: 277 us
// at T = 32768, H = 4096, E = 128).  After the contraction a
// token's E logits sit in the four lanes l % 16 = token, 4 * E / 16 values each: top-K is K rounds of "maximum key of
// the lane, then of the 4 lanes" on the 64-bit keys of topk_softmax_kernel (same tie rule: lower column wins), the
// softmax over the winners is its sequential fp32 sum, and both work on the logits ROUNDED to bf16, i.e. on exactly
// the values that are stored: the scores and indices equal smoe_topk_softmax_fwd applied to the stored logits bit for
// bit.
#include "gemm_common.h"

namespace smoe {

// This kernel is bf16 whatever the library's element type: the winner search orders the logits by the 16 bits of their
// bf16 form.  The fp16 build of the library refuses the entry point and callers take the unfused chain.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
SMOE_DEV uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

SMOE_DEV uint32_t rf_orderable(uint32_t bits) { return bits ^ ((bits >> 31) ? 0xffffffffu : 0x80000000u); }
SMOE_DEV uint32_t rf_unorderable(uint32_t o) { return o ^ ((o >> 31) ? 0x80000000u : 0xffffffffu); }
SMOE_DEV uint64_t rf_shfl_xor_u64(uint64_t v, int mask) {
  uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  lo = __shfl_xor(lo, mask, 64);
  hi = __shfl_xor(hi, mask, 64);
  return ((uint64_t)hi << 32) | lo;
}

// waves per workgroup (16 tokens each): 8 up to E = 128 (69 us against 87 with 4 at T = 32768, H = 4096, E = 128: half
// the Wr traffic from L2 per token), 4 above (more registers per wave: 82 us against 86 at T = 16384, E = 256)
constexpr int rf_waves(int EF) { return EF <= 8 ? 8 : 4; }
constexpr int RF_XB = 8;                           // k-steps of x a wave keeps in flight (its prefetch distance)
constexpr int RF_WB = 2;                           // k-steps of Wr per LDS batch, even (two k-steps = 64 contraction elements = one block of 128-byte rows)

// EF = E / 16 column fragments (E is a multiple of 16, EF <= 16)
template <int EF>
__global__ __launch_bounds__(rf_waves(EF) * 64) void router_fused_kernel(const uint16_t* __restrict__ x,
                                                                     const uint16_t* __restrict__ wr, int64_t T, int H,
                                                                     int K, uint16_t* __restrict__ logits,
                                                                     float* __restrict__ scores,
                                                                     int32_t* __restrict__ indices,
                                                                     float* __restrict__ colsum_partial) {
  constexpr int E = EF * 16, VPL = EF * 4, RF_WAVES = rf_waves(EF), RF_TOKENS = 16 * RF_WAVES;
  constexpr int SUBS = RF_WB / 2;                              // a batch is SUBS blocks of [E rows][64 k = 128 bytes]
  constexpr int WR_BATCH = SUBS * E * 128;                     // bytes of one Wr batch in LDS
  constexpr int PIECES = SUBS * E * 8, PPT = (PIECES + RF_WAVES * 64 - 1) / (RF_WAVES * 64);  // 16-byte pieces per batch, per thread
  __shared__ __attribute__((aligned(16))) char wr_lds[2][WR_BATCH];
  __shared__ float wave_cols[RF_WAVES][E];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, r16 = lane & 15;
  const int64_t tok = (int64_t)blockIdx.x * RF_TOKENS + wave * 16 + r16;
  const bool tok_ok = tok < T;
  const uint16_t* xrow = x + (tok_ok ? tok : T - 1) * (int64_t)H + 8 * g;

  // Wr goes through LDS, shared by the workgroup's wavefronts: a batch is [E rows][64 k], the K-major layout of the
  // grouped GEMMs (16-byte piece c of row r sits at c ^ kswz(r): conflict-free fragment reads).  Thread t stages the
  // pieces t, t + (number of threads), ... of a batch: piece p = block p / (8 E), row (p / 8) % E, 16-byte column p % 8.
  const uint16_t* wsrc[PPT];
  int wdst[PPT];
#pragma unroll
  for (int i = 0; i < PPT; i++) {
    int p = threadIdx.x + i * RF_WAVES * 64;
    p = p < PIECES ? p : PIECES - 1;
    const int sub = p / (E * 8), row = (p >> 3) % E, c = p & 7;
    wsrc[i] = wr + (int64_t)row * H + sub * 64 + c * 8;
    wdst[i] = sub * (E * 128) + row * 128 + ((c ^ kswz<64, 16>(row)) << 4);
  }
  // fragment f of k-step s (0 or 1) of a batch: row f * 16 + r16, piece 4 s + g
  int wfrag[RF_WB];
#pragma unroll
  for (int s = 0; s < RF_WB; s++)  // + f * 2048: kswz(row) = kswz(row % 16)
    wfrag[s] = (s / 2) * (E * 128) + r16 * 128 + (((4 * (s % 2) + g) ^ kswz<64, 16>(r16)) << 4);

  f32x4 acc[EF];
#pragma unroll
  for (int f = 0; f < EF; f++) acc[f] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Vector-memory loads complete in order.  The x fragments come from HBM and are requested RF_XB k-steps before their
  // use; the Wr batches come from L2 but have to be requested just as early: a wait for a YOUNGER Wr load would also be
  // a wait for every x load issued before it, and the x prefetch would shrink to one batch (measured: 100 us instead of
  // the 60 the stream of x alone needs).  So DW batches of Wr are in flight in registers, each written to the LDS
  // double buffer one batch before its use.
  const int steps = H / 32;  // a multiple of RF_XB
  constexpr int NB = RF_XB / RF_WB;        // batches per trip of the outer loop
  constexpr int DW = EF > 8 ? 2 : NB;      // Wr batches in flight in registers (divides NB)
  static_assert(NB % DW == 0 && NB >= 2, "the register ring of Wr batches is indexed statically");
  const int batches = steps / RF_WB;
  u32x4 wst[DW][PPT];
  auto load_w = [&](int batch, auto slot_c) {
    constexpr int slot = decltype(slot_c)::value;
#pragma unroll
    for (int i = 0; i < PPT; i++) wst[slot][i] = *(const u32x4*)(wsrc[i] + batch * (RF_WB * 32));
  };
  auto store_w = [&](int buf, auto slot_c) {
    constexpr int slot = decltype(slot_c)::value;
#pragma unroll
    for (int i = 0; i < PPT; i++)
      if (PIECES % (RF_WAVES * 64) == 0 || (int)threadIdx.x + i * RF_WAVES * 64 < PIECES)
        *(u32x4*)(wr_lds[buf] + wdst[i]) = wst[slot][i];
  };
  bf16x8 xf[RF_XB];
  // (loads past the end re-read the last batch / step instead of being branched around: with the loads in straight-line
  // code the compiler's wait counts are exact, behind branches it waits for nearly everything)
  const int last_batch = batches - 1, last_step = steps - 1;
  static_for<DW>([&](auto d_c) {
    constexpr int d = decltype(d_c)::value;
    load_w(d < last_batch ? d : last_batch, d_c);
  });
#pragma unroll
  for (int s = 0; s < RF_XB; s++) xf[s] = *(const bf16x8*)(xrow + s * 32);
  store_w(0, std::integral_constant<int, 0>{});
  load_w(DW < last_batch ? DW : last_batch, std::integral_constant<int, 0>{});
  __syncthreads();
  for (int s0 = 0; s0 < steps; s0 += RF_XB) {
    static_for<NB>([&](auto jb_c) {
      constexpr int jb = decltype(jb_c)::value, j = jb * RF_WB;
      const int batch = s0 / RF_WB + jb, nxt = batch + 1;
      constexpr std::integral_constant<int, (jb + 1) % DW> slot{};  // batch n lives in slot n % DW
      store_w(nxt & 1, slot);  // past the end: a copy of the last batch that nobody reads
      load_w(nxt + DW < last_batch ? nxt + DW : last_batch, slot);
      const char* wl = wr_lds[batch & 1];
#pragma unroll
      for (int s = 0; s < RF_WB; s++) {
        bf16x8 w[EF];
#pragma unroll
        for (int f = 0; f < EF; f++) w[f] = *(const bf16x8*)(wl + wfrag[s] + f * 2048);
#pragma unroll
        for (int f = 0; f < EF; f++) acc[f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[f], xf[j + s], acc[f], 0, 0, 0);
        // this step's x register is free: fetch the step RF_XB further on into it
        const int ahead = s0 + RF_XB + j + s;
        xf[j + s] = *(const bf16x8*)(xrow + (ahead < last_step ? ahead : last_step) * 32);
      }
      __syncthreads();  // the next batch is complete in LDS; everyone is done reading this one
    });
  }

  // ---- logits, rounded to bf16: lane (token r16, group g) holds columns f * 16 + 4 g + 0..3 of fragment f ----
  uint32_t bits[VPL];  // the stored value of every logit as fp32 bits
#pragma unroll
  for (int f = 0; f < EF; f++) {
    const uint32_t p0 = pack_bf16x2(acc[f][0], acc[f][1]), p1 = pack_bf16x2(acc[f][2], acc[f][3]);
    if (tok_ok) *(u32x2*)(logits + tok * E + f * 16 + 4 * g) = u32x2{p0, p1};
    bits[4 * f + 0] = p0 << 16;
    bits[4 * f + 1] = p0 & 0xffff0000u;
    bits[4 * f + 2] = p1 << 16;
    bits[4 * f + 3] = p1 & 0xffff0000u;
  }

  // ---- top-K over the token's E logits (4 lanes x VPL keys), softmax over the winners ----
  // key = (order-preserving image of the 16 value bits) << 16 | (0xffff - column): the ordering of topk_softmax_kernel's
  // 64-bit keys (larger value first, then lower column) in 32 bits, which bf16 values and E <= 256 allow
  uint32_t key[VPL];
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const uint32_t col = (uint32_t)((i >> 2) * 16 + 4 * g + (i & 3));
    key[i] = (rf_orderable(bits[i]) & 0xffff0000u) | (0xffffu - col);
  }
  float vmax = 0.f, esum = 0.f;
  for (int r = 0; r < K; r++) {
    uint32_t best = key[0];
#pragma unroll
    for (int i = 1; i < VPL; i++) best = key[i] > best ? key[i] : best;
    uint32_t o = (uint32_t)__shfl_xor((int)best, 16, 64);
    best = o > best ? o : best;
    o = (uint32_t)__shfl_xor((int)best, 32, 64);
    best = o > best ? o : best;
#pragma unroll
    for (int i = 0; i < VPL; i++) key[i] = (key[i] == best) ? 0 : key[i];
    // the low 16 bits of an orderable image are all ones for a negative value and all zeros otherwise
    const uint32_t hi = best & 0xffff0000u;
    const float v = __uint_as_float(rf_unorderable(hi | ((hi >> 31) ? 0u : 0xffffu)) & 0xffff0000u);
    if (r == 0) vmax = v;
    if (g == 0 && tok_ok) {
      const float ev = expf(v - vmax);
      esum += ev;
      scores[tok * K + r] = ev;
      indices[tok * K + r] = (int)(0xffffu - (best & 0xffffu));
    }
  }
  if (g == 0 && tok_ok) {
    for (int r = 0; r < K; r++) scores[tok * K + r] = scores[tok * K + r] / esum;
  }

  // ---- column sums of the full row softmax (fp32, from the stored logits): the load-balancing loss's first factor ----
  if (colsum_partial != nullptr) {
    float p[VPL];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
      p[i] = __expf(__uint_as_float(bits[i]) - vmax);  // vmax (the first winner) is the row maximum, known to all 4 lanes
      s += p[i];
    }
    s += __shfl_xor(s, 16, 64);
    s += __shfl_xor(s, 32, 64);
    const float inv = tok_ok ? 1.0f / s : 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
      float c = p[i] * inv;  // add the 16 tokens of the wave: lanes with equal g
      c += __shfl_xor(c, 1, 64);
      c += __shfl_xor(c, 2, 64);
      c += __shfl_xor(c, 4, 64);
      c += __shfl_xor(c, 8, 64);
      if (r16 == 0) wave_cols[wave][(i >> 2) * 16 + 4 * g + (i & 3)] = c;
    }
    __syncthreads();
    for (int c = threadIdx.x; c < E; c += RF_WAVES * 64) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < RF_WAVES; w++) t += wave_cols[w][c];
      colsum_partial[(int64_t)blockIdx.x * E + c] = t;
    }
  }
}

template <int EF>
static void launch_router_fused(const void* x, const void* wr, int64_t T, int H, int K, void* logits, float* scores,
                                int32_t* indices, float* colsum_partial, hipStream_t st) {
  const unsigned grid = (unsigned)ceil_div(T, (int64_t)(16 * rf_waves(EF)));
  hipLaunchKernelGGL(router_fused_kernel<EF>, dim3(grid), dim3(rf_waves(EF) * 64), 0, st, (const uint16_t*)x,
                     (const uint16_t*)wr, T, H, K, (uint16_t*)logits, scores, indices, colsum_partial);
}

}  // namespace smoe

using namespace smoe;

extern "C" int64_t smoe_router_fused_partials(int64_t T, int E) {
  return T <= 0 || E < 16 ? 0 : ceil_div(T, (int64_t)(16 * rf_waves(E / 16)));
}

extern "C" int smoe_router_forward_fused(const void* x, const void* wr, int64_t T, int H, int E, int K, void* logits,
                                         float* scores, int32_t* indices, float* colsum_partial, void* stream) {
  SMOE_REQUIRE(T >= 0 && T < (1ll << 31), SMOE_ERR_INVALID, "router_forward_fused: T out of range");
  SMOE_REQUIRE(E >= 16 && E <= 256 && E % 16 == 0, SMOE_ERR_UNSUPPORTED,
               "router_forward_fused: E=%d must be a multiple of 16 in [16, 256]", E);
  SMOE_REQUIRE(H >= 32 * RF_XB && H % (32 * RF_XB) == 0, SMOE_ERR_UNSUPPORTED,
               "router_forward_fused: H=%d must be a multiple of %d", H, 32 * RF_XB);
  SMOE_REQUIRE(K >= 1 && K <= E, SMOE_ERR_INVALID, "router_forward_fused: K=%d out of range [1, E]", K);
#ifdef SMOE_ELEM_F16
  SMOE_REQUIRE(false, SMOE_ERR_UNSUPPORTED, "router_forward_fused: bf16 only (this is the fp16 build of the library)");
#endif
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(x && wr && logits && scores && indices, SMOE_ERR_INVALID, "router_forward_fused: null pointer");
  SMOE_REQUIRE_ALIGNED("router_forward_fused", x, wr, logits);
  hipStream_t st = (hipStream_t)stream;
  switch (E / 16) {
#define SMOE_RF_CASE(EF) \
  case EF: launch_router_fused<EF>(x, wr, T, H, K, logits, scores, indices, colsum_partial, st); break;
    SMOE_RF_CASE(1) SMOE_RF_CASE(2) SMOE_RF_CASE(3) SMOE_RF_CASE(4) SMOE_RF_CASE(5) SMOE_RF_CASE(6) SMOE_RF_CASE(7)
    SMOE_RF_CASE(8) SMOE_RF_CASE(9) SMOE_RF_CASE(10) SMOE_RF_CASE(11) SMOE_RF_CASE(12) SMOE_RF_CASE(13)
    SMOE_RF_CASE(14) SMOE_RF_CASE(15) SMOE_RF_CASE(16)
#undef SMOE_RF_CASE
  }
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}
