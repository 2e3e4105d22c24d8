// Weighted gather-sum over a token's routed rows (forward combine, backward dx reduction), the ds finalise and the
// bias-gradient reductions.  HBM-bound: each row is read exactly once in 16-byte pieces, each output row written once.
#include "gemm_common.h"

namespace smoe {

// One workgroup per token; thread c owns the 8-column chunks c, c+blockDim, ...  UNROLL slots are in flight.
template <int UNROLL>
__global__ __launch_bounds__(512) void gather_sum_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ out,
                                                         const float* __restrict__ w, const int32_t* __restrict__ ridx,
                                                         const int32_t* __restrict__ tok_off, int K, int H) {
  const int64_t t = blockIdx.x;
  int64_t lo, hi;
  if (tok_off) {
    lo = tok_off[t];
    hi = tok_off[t + 1];
  } else {
    lo = t * K;
    hi = lo + K;
  }
  const int chunks = H >> 3;
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;
    for (int64_t j0 = lo; j0 < hi; j0 += UNROLL) {
      u32x4 v[UNROLL];
      float ws[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; u++) {
        const int64_t j = j0 + u;
        if (j < hi) {
          const int64_t r = ridx[j];
          ws[u] = w ? w[j] : 1.0f;
          v[u] = __builtin_nontemporal_load((const u32x4*)(src + r * H + (int64_t)c * 8));
        } else {
          ws[u] = 0.f;
          v[u] = u32x4{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; u++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
          acc[2 * q] += ws[u] * elem_lo(v[u][q]);
          acc[2 * q + 1] += ws[u] * elem_hi(v[u][q]);
        }
      }
    }
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; q++) o[q] = pack_elem2(acc[2 * q], acc[2 * q + 1]);
    __builtin_nontemporal_store(o, (u32x4*)(out + t * H + (int64_t)c * 8));
  }
}

// ds[sidx[m]] = sum_n ds_partial[m][n]
__global__ __launch_bounds__(256) void ds_finalize_kernel(const float* __restrict__ ds_partial, int ncols,
                                                          const int32_t* __restrict__ sidx, float* __restrict__ ds,
                                                          int64_t TK) {
  const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (m >= TK) return;
  float s = 0.f;
  for (int n = 0; n < ncols; n++) s += ds_partial[m * ncols + n];
  ds[sidx[m]] = s;
}

int launch_ds_finalize(const float* ds_partial, int ncols, const int32_t* sidx, float* ds, int64_t TK,
                       hipStream_t st) {
  if (TK == 0) return SMOE_OK;
  hipLaunchKernelGGL(ds_finalize_kernel, dim3((unsigned)ceil_div(TK, 256)), dim3(256), 0, st, ds_partial, ncols, sidx,
                     ds, TK);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

// Per-expert weighted column sums.  Workgroup (e, column block of 512): its four wavefronts walk the expert's rows
// four apart, every lane keeps 8 columns in fp32; the four partial sums meet in LDS and are rounded once.
__global__ __launch_bounds__(256) void expert_colsum_kernel(const uint16_t* __restrict__ src, int64_t src_stride,
                                                            int ncols, const int32_t* __restrict__ gidx,
                                                            const float* __restrict__ scores,
                                                            const int32_t* __restrict__ sidx,
                                                            const int32_t* __restrict__ off,
                                                            uint16_t* __restrict__ out) {
  __shared__ float part[4][64][8];
  const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = (blockIdx.y * 64 + lane) * 8;
  const bool active = col < ncols;
  const int begin = off[e], end = off[e + 1];
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = 0.f;
  constexpr int UNROLL = 4;
  for (int m0 = begin + wave; m0 < end; m0 += 4 * UNROLL) {
    u32x4 v[UNROLL];
    float w[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const int m = m0 + 4 * u;
      v[u] = u32x4{0, 0, 0, 0};
      w[u] = 0.f;
      if (m < end && active) {
        const int64_t row = gidx ? (int64_t)gidx[m] : (int64_t)m;
        w[u] = scores ? scores[sidx[m]] : 1.f;
        v[u] = *(const u32x4*)(src + row * src_stride + col);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        acc[2 * q] += w[u] * elem_lo(v[u][q]);
        acc[2 * q + 1] += w[u] * elem_hi(v[u][q]);
      }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) part[wave][lane][i] = acc[i];
  __syncthreads();
  if (wave == 0 && active) {
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const float a = part[0][lane][2 * q] + part[1][lane][2 * q] + part[2][lane][2 * q] + part[3][lane][2 * q];
      const float b = part[0][lane][2 * q + 1] + part[1][lane][2 * q + 1] + part[2][lane][2 * q + 1] +
                      part[3][lane][2 * q + 1];
      o[q] = pack_elem2(a, b);
    }
    *(u32x4*)(out + (int64_t)e * ncols + col) = o;
  }
}

int launch_expert_colsum(const uint16_t* src, int64_t src_stride, int ncols, const int32_t* gidx, const float* scores,
                         const int32_t* sidx, const int32_t* off, int E, uint16_t* out, hipStream_t st) {
  SMOE_REQUIRE(ncols % 8 == 0, SMOE_ERR_UNSUPPORTED, "bias gradient: %d columns are not a multiple of 8", ncols);
  hipLaunchKernelGGL(expert_colsum_kernel, dim3((unsigned)E, (unsigned)ceil_div(ncols, 512)), dim3(256), 0, st, src,
                     src_stride, ncols, gidx, scores, sidx, off, out);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

// One wavefront per grouped row m: its expert by bisection of the offsets, then a dot product over H.
__global__ __launch_bounds__(256) void ds_bias_term_kernel(const uint16_t* __restrict__ dout,
                                                           const uint16_t* __restrict__ b2,
                                                           const int32_t* __restrict__ gidx,
                                                           const int32_t* __restrict__ sidx,
                                                           const int32_t* __restrict__ off, int E, int H,
                                                           float* __restrict__ ds, int64_t TK) {
  const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= TK) return;
  const int lane = threadIdx.x & 63;
  int lo = 0, hi = E;  // largest e with off[e] <= m
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (off[mid] <= m) lo = mid; else hi = mid;
  }
  const uint16_t* row = dout + (int64_t)gidx[m] * H;
  const uint16_t* bias = b2 + (int64_t)lo * H;
  float s = 0.f;
  for (int c = lane * 8; c < H; c += 512) {
    const u32x4 a = *(const u32x4*)(row + c), b = *(const u32x4*)(bias + c);
#pragma unroll
    for (int q = 0; q < 4; q++) s += elem_lo(a[q]) * elem_lo(b[q]) + elem_hi(a[q]) * elem_hi(b[q]);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
  if (lane == 0) ds[sidx[m]] += s;
}

int launch_ds_bias_term(const uint16_t* dout, const uint16_t* b2, const int32_t* gidx, const int32_t* sidx,
                        const int32_t* off, int E, int H, float* ds, int64_t TK, hipStream_t st) {
  if (TK == 0) return SMOE_OK;
  hipLaunchKernelGGL(ds_bias_term_kernel, dim3((unsigned)ceil_div(TK, 4)), dim3(256), 0, st, dout, b2, gidx, sidx, off,
                     E, H, ds, TK);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

}  // namespace smoe

using namespace smoe;

extern "C" int smoe_gather_sum(const void* src, void* out, const float* w, const int32_t* ridx, const int32_t* tok_off,
                               int64_t T, int K, int H, void* stream) {
  SMOE_REQUIRE(T >= 0, SMOE_ERR_INVALID, "gather_sum: negative T");
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(out && ridx && src, SMOE_ERR_INVALID, "gather_sum: null pointer");
  SMOE_REQUIRE(H > 0 && H % 8 == 0, SMOE_ERR_UNSUPPORTED, "gather_sum: H=%d must be a positive multiple of 8", H);
  SMOE_REQUIRE(tok_off != nullptr || K >= 1, SMOE_ERR_INVALID, "gather_sum: K must be >= 1 without tok_off");
  SMOE_REQUIRE(T < (1ll << 31), SMOE_ERR_UNSUPPORTED, "gather_sum: T too large");
  hipStream_t st = (hipStream_t)stream;
  int threads = H / 8;  // 512 threads (one 16-byte chunk each at H = 4096) measured 4-7 % faster than 256 or 1024 at C2
  if (threads > 512) threads = 512;
  if (threads < 64) threads = 64;
  hipLaunchKernelGGL(gather_sum_kernel<8>, dim3((unsigned)T), dim3(threads), 0, st, (const uint16_t*)src,
                     (uint16_t*)out, w, ridx, tok_off, K, H);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_score_grad_bias_term(const void* dout, const void* b2, const int32_t* off,
                                         const int32_t* x_gather_idx, const int32_t* s_scatter_idx, float* ds,
                                         int64_t TK, int H, int E, void* stream) {
  SMOE_REQUIRE(TK >= 0 && E >= 1, SMOE_ERR_INVALID, "score_grad_bias_term: TK=%lld, E=%d", (long long)TK, E);
  if (TK == 0) return SMOE_OK;
  SMOE_REQUIRE(dout && b2 && off && x_gather_idx && s_scatter_idx && ds, SMOE_ERR_INVALID,
               "score_grad_bias_term: null pointer");
  SMOE_REQUIRE(H > 0 && H % 8 == 0, SMOE_ERR_UNSUPPORTED, "score_grad_bias_term: H=%d must be a positive multiple of 8",
               H);
  SMOE_REQUIRE_ALIGNED("score_grad_bias_term", dout, b2);
  return launch_ds_bias_term((const uint16_t*)dout, (const uint16_t*)b2, x_gather_idx, s_scatter_idx, off, E, H, ds, TK,
                             (hipStream_t)stream);
}
