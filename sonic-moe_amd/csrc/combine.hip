// Weighted gather-sum over a token's routed rows (forward combine, backward dx reduction) and the ds finalise.
// HBM-bound: each grouped row is read exactly once in 16-byte pieces, each output row written once.
#include "common.h"

namespace smoe {

// One workgroup per token; thread c owns the 8-column chunks c, c+blockDim, ...  UNROLL slots are in flight.
template <int UNROLL>
__global__ __launch_bounds__(256) void gather_sum_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ out,
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
          v[u] = *(const u32x4*)(src + r * H + (int64_t)c * 8);
        } else {
          ws[u] = 0.f;
          v[u] = u32x4{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; u++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
          acc[2 * q] += ws[u] * bf16_lo(v[u][q]);
          acc[2 * q + 1] += ws[u] * bf16_hi(v[u][q]);
        }
      }
    }
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; q++) o[q] = pack_bf16x2(acc[2 * q], acc[2 * q + 1]);
    *(u32x4*)(out + t * H + (int64_t)c * 8) = o;
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
  int threads = H / 8;
  if (threads > 256) threads = 256;
  if (threads < 64) threads = 64;
  hipLaunchKernelGGL(gather_sum_kernel<8>, dim3((unsigned)T), dim3(threads), 0, st, (const uint16_t*)src,
                     (uint16_t*)out, w, ridx, tok_off, K, H);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}
