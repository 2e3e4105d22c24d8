// Load-balancing ("switch") auxiliary loss of the MoE layer for gfx950, forward and backward, without the (T, E) fp32
// probability tensor the reference materialises (sonicmoe/moe.py:247-274):
//     acc[e] = sum_t softmax(logits[t, :])[e]           (fp32)
//     aux    = E * < acc / max(|acc|_1, eps), freq / max(|freq|_1, eps) >,   eps = 1e-12 (F.normalize's default)
// Forward: one pass over the logits (a wavefront owns a row at a time, lane l holds columns l, l+64, ...; column sums
// stay in registers over all rows of the wavefront), per-workgroup partial sums, then one small workgroup adds the
// partials in a fixed order and forms the scalar: no atomics, results do not depend on the launch.  Backward: the row
// softmax is recomputed and d aux / d logits[t, j] = g * p[t,j] * (dacc[j] - sum_e dacc[e] p[t,e]) is written in the
// logits' dtype, with dacc[j] = E / (S F) * (freq[j] - D / S), S = |acc|_1, F = |freq|_1, D = <acc, freq>.
#include <hip/hip_fp16.h>

#include "common.h"

namespace smoe {

template <typename T>
SMOE_DEV float sl_load(const T* p);
template <>
__device__ __forceinline__ float sl_load<uint16_t>(const uint16_t* p) {  // bf16
  return __uint_as_float((uint32_t)(*p) << 16);
}
template <>
__device__ __forceinline__ float sl_load<__half>(const __half* p) {
  return __half2float(*p);
}
template <>
__device__ __forceinline__ float sl_load<float>(const float* p) {
  return *p;
}
template <typename T>
SMOE_DEV void sl_store(T* p, float v);
template <>
__device__ __forceinline__ void sl_store<uint16_t>(uint16_t* p, float v) {
  *p = f32_to_bf16_bits(v);
}
template <>
__device__ __forceinline__ void sl_store<__half>(__half* p, float v) {
  *p = __float2half(v);
}
template <>
__device__ __forceinline__ void sl_store<float>(float* p, float v) {
  *p = v;
}

SMOE_DEV float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}
SMOE_DEV float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

constexpr int SL_WAVES = 4;            // wavefronts per workgroup of the backward pass
constexpr int SL_MAX_PARTIALS = 256;  // workgroups of the forward pass

// softmax of one row held as VPL values per lane (columns lane + 64 i); columns >= E hold -inf and come out as 0
template <int VPL>
SMOE_DEV void row_softmax(float (&v)[VPL]) {
  float m = v[0];
#pragma unroll
  for (int i = 1; i < VPL; i++) m = fmaxf(m, v[i]);
  m = wave_max(m);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    v[i] = __expf(v[i] - m);
    s += v[i];
  }
  s = wave_sum(s);
  const float inv = 1.0f / s;
#pragma unroll
  for (int i = 0; i < VPL; i++) v[i] *= inv;
}

// R rows at once: the R wave reductions are independent chains the hardware overlaps (one row at a time leaves a
// wavefront waiting on 12 dependent cross-lane moves per row)
template <int VPL, int R>
SMOE_DEV void rows_softmax(float (&v)[R][VPL]) {
  float m[R], s[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    m[r] = v[r][0];
#pragma unroll
    for (int i = 1; i < VPL; i++) m[r] = fmaxf(m[r], v[r][i]);
  }
#pragma unroll
  for (int k = 32; k >= 1; k >>= 1)
#pragma unroll
    for (int r = 0; r < R; r++) m[r] = fmaxf(m[r], __shfl_xor(m[r], k, 64));
#pragma unroll
  for (int r = 0; r < R; r++) {
    s[r] = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
      v[r][i] = __expf(v[r][i] - m[r]);
      s[r] += v[r][i];
    }
  }
#pragma unroll
  for (int k = 32; k >= 1; k >>= 1)
#pragma unroll
    for (int r = 0; r < R; r++) s[r] += __shfl_xor(s[r], k, 64);
#pragma unroll
  for (int r = 0; r < R; r++) {
    const float inv = 1.0f / s[r];
#pragma unroll
    for (int i = 0; i < VPL; i++) v[r][i] *= inv;
  }
}

// rows a wavefront works on at once
template <int VPL>
struct RowsAtOnce {
  static constexpr int value = VPL <= 4 ? 4 : (VPL <= 16 ? 2 : 1);
};

template <typename T, int VPL>
SMOE_DEV void load_row(const T* row, int E, int lane, float (&v)[VPL]) {
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const int c = lane + 64 * i;
    v[i] = c < E ? sl_load<T>(row + c) : -INFINITY;
  }
}

template <typename T, int VPL>
__global__ __launch_bounds__(VPL <= 16 ? 1024 : 256) void softmax_colsum_kernel(const T* __restrict__ logits,
                                                                       int64_t row_stride, int64_t Trows, int E,
                                                                       float* __restrict__ partial) {
  extern __shared__ float sl_lds[];  // waves x E
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  float acc[VPL];
#pragma unroll
  for (int i = 0; i < VPL; i++) acc[i] = 0.f;
  constexpr int R = RowsAtOnce<VPL>::value;
  const int64_t step = (int64_t)gridDim.x * nw;
  int64_t r = (int64_t)blockIdx.x * nw + wave;
  for (; r + (R - 1) * step < Trows; r += R * step) {
    float v[R][VPL];
#pragma unroll
    for (int k = 0; k < R; k++) load_row<T, VPL>(logits + (r + k * step) * row_stride, E, lane, v[k]);
    rows_softmax<VPL, R>(v);
#pragma unroll
    for (int k = 0; k < R; k++)
#pragma unroll
      for (int i = 0; i < VPL; i++) acc[i] += v[k][i];
  }
  for (; r < Trows; r += step) {
    float v[VPL];
    load_row<T, VPL>(logits + r * row_stride, E, lane, v);
    row_softmax<VPL>(v);
#pragma unroll
    for (int i = 0; i < VPL; i++) acc[i] += v[i];
  }
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const int c = lane + 64 * i;
    if (c < E) sl_lds[wave * E + c] = acc[i];
  }
  __syncthreads();
  for (int c = threadIdx.x; c < E; c += blockDim.x) {
    float s = 0.f;
    for (int w = 0; w < nw; w++) s += sl_lds[w * E + c];
    partial[(int64_t)blockIdx.x * E + c] = s;
  }
}

// block-wide sum of three values; every thread gets the totals
SMOE_DEV void block_sum3(float& a, float& b, float& c, float* scratch /* 3 * 16 floats */) {
  a = wave_sum(a);
  b = wave_sum(b);
  c = wave_sum(c);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if (lane == 0) {
    scratch[wave] = a;
    scratch[16 + wave] = b;
    scratch[32 + wave] = c;
  }
  __syncthreads();
  a = b = c = 0.f;
  for (int w = 0; w < nw; w++) {
    a += scratch[w];
    b += scratch[16 + w];
    c += scratch[32 + w];
  }
  __syncthreads();
}

// one workgroup of 1024 threads: acc = sum of the partials, then the scalar.  The threads form 1024 / CW slices of CW
// columns (CW = E rounded up to a power of two, at most 1024); slice s adds partials s, s + NS, ... of its column and
// the slices are added in order: the summation order is fixed by (n_partial, E) alone.
__global__ __launch_bounds__(1024) void switch_loss_finalize_kernel(const float* __restrict__ partial, int n_partial,
                                                                    const int32_t* __restrict__ freq, int E, int CW,
                                                                    float* __restrict__ acc, float* __restrict__ aux) {
  __shared__ float scratch[48];
  __shared__ float slices[1024];
  const int col = threadIdx.x % CW, slice = threadIdx.x / CW, NS = 1024 / CW;
  float s = 0.f, f = 0.f, d = 0.f;
  for (int c0 = 0; c0 < E; c0 += CW) {
    const int c = c0 + col;
    float a = 0.f;
    if (c < E)
      for (int g = slice; g < n_partial; g += NS) a += partial[(int64_t)g * E + c];
    slices[slice * CW + col] = a;
    __syncthreads();
    if (slice == 0 && c < E) {
      for (int k = 1; k < NS; k++) a += slices[k * CW + col];
      acc[c] = a;
      const float fc = (float)freq[c];
      s += a;
      f += fabsf(fc);
      d += a * fc;
    }
    __syncthreads();
  }
  block_sum3(s, f, d, scratch);
  if (threadIdx.x == 0) aux[0] = (float)E * d / (fmaxf(s, 1e-12f) * fmaxf(f, 1e-12f));
}

template <typename T, int VPL>
__global__ __launch_bounds__(SL_WAVES * 64) void switch_loss_bwd_kernel(const T* __restrict__ logits,
                                                                        int64_t row_stride, int64_t Trows, int E,
                                                                        const int32_t* __restrict__ freq,
                                                                        const float* __restrict__ acc,
                                                                        const float* __restrict__ grad_aux,
                                                                        T* __restrict__ dlogits,
                                                                        int64_t d_row_stride) {
  __shared__ float scratch[48];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // S, F, D again (E values: cheaper than a round trip through memory and one more argument)
  float s = 0.f, f = 0.f, d = 0.f;
  for (int c = threadIdx.x; c < E; c += SL_WAVES * 64) {
    const float a = acc[c], fc = (float)freq[c];
    s += a;
    f += fabsf(fc);
    d += a * fc;
  }
  block_sum3(s, f, d, scratch);
  const float g = grad_aux[0];
  // below eps the norm is clamped and the loss is linear in acc
  const bool clamped = s < 1e-12f;
  const float sn = fmaxf(s, 1e-12f), fn = fmaxf(f, 1e-12f);
  const float coef = g * (float)E / (sn * fn), shift = clamped ? 0.f : d / sn;
  float dacc[VPL];
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const int c = lane + 64 * i;
    dacc[i] = c < E ? coef * ((float)freq[c] - shift) : 0.f;
  }
  constexpr int R = RowsAtOnce<VPL>::value;
  const int64_t step = (int64_t)gridDim.x * SL_WAVES;
  int64_t r = (int64_t)blockIdx.x * SL_WAVES + wave;
  for (; r + (R - 1) * step < Trows; r += R * step) {
    float v[R][VPL], dot[R];
#pragma unroll
    for (int k = 0; k < R; k++) load_row<T, VPL>(logits + (r + k * step) * row_stride, E, lane, v[k]);
    rows_softmax<VPL, R>(v);
#pragma unroll
    for (int k = 0; k < R; k++) {
      dot[k] = 0.f;
#pragma unroll
      for (int i = 0; i < VPL; i++) dot[k] += v[k][i] * dacc[i];
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
#pragma unroll
      for (int k = 0; k < R; k++) dot[k] += __shfl_xor(dot[k], m, 64);
#pragma unroll
    for (int k = 0; k < R; k++) {
      T* out = dlogits + (r + k * step) * d_row_stride;
#pragma unroll
      for (int i = 0; i < VPL; i++) {
        const int c = lane + 64 * i;
        if (c < E) sl_store<T>(out + c, v[k][i] * (dacc[i] - dot[k]));
      }
    }
  }
  for (; r < Trows; r += step) {
    float v[VPL];
    load_row<T, VPL>(logits + r * row_stride, E, lane, v);
    row_softmax<VPL>(v);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++) dot += v[i] * dacc[i];
    dot = wave_sum(dot);
    T* out = dlogits + r * d_row_stride;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
      const int c = lane + 64 * i;
      if (c < E) sl_store<T>(out + c, v[i] * (dacc[i] - dot));
    }
  }
}

static int sl_grid(int64_t T) {
  int64_t g = ceil_div(T, (int64_t)64);  // a workgroup (16 or 4 wavefronts) gets at least 64 rows
  if (g < 1) g = 1;
  return (int)(g < SL_MAX_PARTIALS ? g : SL_MAX_PARTIALS);
}

template <typename T, int VPL>
static void launch_colsum(const void* logits, int64_t row_stride, int64_t Trows, int E, float* partial, int grid,
                          hipStream_t st) {
  const int waves = E <= 1024 ? 16 : 4;  // 16 x E floats of LDS at most 64 KiB
  hipLaunchKernelGGL((softmax_colsum_kernel<T, VPL>), dim3(grid), dim3(waves * 64), (size_t)waves * E * sizeof(float),
                     st, (const T*)logits, row_stride, Trows, E, partial);
}
template <typename T, int VPL>
static void launch_sl_bwd(const void* logits, int64_t row_stride, int64_t Trows, int E, const int32_t* freq,
                          const float* acc, const float* grad_aux, void* dlogits, int64_t d_row_stride, int grid,
                          hipStream_t st) {
  hipLaunchKernelGGL((switch_loss_bwd_kernel<T, VPL>), dim3(grid), dim3(SL_WAVES * 64), 0, st, (const T*)logits,
                     row_stride, Trows, E, freq, acc, grad_aux, (T*)dlogits, d_row_stride);
}

// dispatch on the values per lane (E <= 64 * VPL)
#define SL_DISPATCH_VPL(FN, TYPE, ...)             \
  do {                                             \
    if (E <= 64) FN<TYPE, 1>(__VA_ARGS__);         \
    else if (E <= 128) FN<TYPE, 2>(__VA_ARGS__);   \
    else if (E <= 256) FN<TYPE, 4>(__VA_ARGS__);   \
    else if (E <= 512) FN<TYPE, 8>(__VA_ARGS__);   \
    else if (E <= 1024) FN<TYPE, 16>(__VA_ARGS__); \
    else if (E <= 2048) FN<TYPE, 32>(__VA_ARGS__); \
    else FN<TYPE, 64>(__VA_ARGS__);                \
  } while (0)

}  // namespace smoe

using namespace smoe;

extern "C" size_t smoe_switch_loss_workspace_bytes(int64_t T, int E) {
  if (T < 0 || E < 1) return 0;
  return (size_t)sl_grid(T) * (size_t)E * sizeof(float);
}

extern "C" int smoe_switch_loss_fwd(const void* logits, int dtype, int64_t row_stride, int64_t T, int E,
                                    const int32_t* freq, float* acc, float* aux, void* ws, size_t ws_bytes,
                                    void* stream) {
  SMOE_REQUIRE(T >= 1, SMOE_ERR_INVALID, "switch_loss_fwd: T must be positive");
  SMOE_REQUIRE(E >= 1 && E <= 4096, SMOE_ERR_UNSUPPORTED, "switch_loss_fwd: E=%d out of range [1, 4096]", E);
  SMOE_REQUIRE(logits && freq && acc && aux, SMOE_ERR_INVALID, "switch_loss_fwd: null pointer");
  SMOE_REQUIRE(row_stride >= E, SMOE_ERR_INVALID, "switch_loss_fwd: row stride below E");
  SMOE_REQUIRE(ws && ws_bytes >= smoe_switch_loss_workspace_bytes(T, E), SMOE_ERR_WORKSPACE,
               "switch_loss_fwd: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  const int grid = sl_grid(T);
  float* partial = (float*)ws;
  switch (dtype) {
    case SMOE_DT_BF16:
      SL_DISPATCH_VPL(launch_colsum, uint16_t, logits, row_stride, T, E, partial, grid, st);
      break;
    case SMOE_DT_F16:
      SL_DISPATCH_VPL(launch_colsum, __half, logits, row_stride, T, E, partial, grid, st);
      break;
    case SMOE_DT_F32:
      SL_DISPATCH_VPL(launch_colsum, float, logits, row_stride, T, E, partial, grid, st);
      break;
    default:
      set_error("switch_loss_fwd: unknown dtype %d", dtype);
      return SMOE_ERR_INVALID;
  }
  SMOE_LAUNCH_CHECK();
  int cw = 64;
  while (cw < E && cw < 1024) cw *= 2;
  hipLaunchKernelGGL(switch_loss_finalize_kernel, dim3(1), dim3(1024), 0, st, partial, grid, freq, E, cw, acc, aux);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_switch_loss_from_partials(const float* partial, int64_t n_partial, int E, const int32_t* freq,
                                              float* acc, float* aux, void* stream) {
  SMOE_REQUIRE(n_partial >= 1 && n_partial < (1ll << 31), SMOE_ERR_INVALID, "switch_loss_from_partials: bad count");
  SMOE_REQUIRE(E >= 1 && E <= 4096, SMOE_ERR_UNSUPPORTED, "switch_loss_from_partials: E=%d out of range [1, 4096]", E);
  SMOE_REQUIRE(partial && freq && acc && aux, SMOE_ERR_INVALID, "switch_loss_from_partials: null pointer");
  int cw = 64;
  while (cw < E && cw < 1024) cw *= 2;
  hipLaunchKernelGGL(switch_loss_finalize_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, partial, (int)n_partial,
                     freq, E, cw, acc, aux);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_switch_loss_bwd(const void* logits, int dtype, int64_t row_stride, int64_t T, int E,
                                    const int32_t* freq, const float* acc, const float* grad_aux, void* dlogits,
                                    int64_t d_row_stride, void* stream) {
  SMOE_REQUIRE(T >= 1, SMOE_ERR_INVALID, "switch_loss_bwd: T must be positive");
  SMOE_REQUIRE(E >= 1 && E <= 4096, SMOE_ERR_UNSUPPORTED, "switch_loss_bwd: E=%d out of range [1, 4096]", E);
  SMOE_REQUIRE(logits && freq && acc && grad_aux && dlogits, SMOE_ERR_INVALID, "switch_loss_bwd: null pointer");
  SMOE_REQUIRE(row_stride >= E && d_row_stride >= E, SMOE_ERR_INVALID, "switch_loss_bwd: row stride below E");
  hipStream_t st = (hipStream_t)stream;
  int64_t g = ceil_div(T, (int64_t)SL_WAVES * 4);
  const int grid = (int)(g < 1 ? 1 : (g < 2048 ? g : 2048));
  switch (dtype) {
    case SMOE_DT_BF16:
      SL_DISPATCH_VPL(launch_sl_bwd, uint16_t, logits, row_stride, T, E, freq, acc, grad_aux, dlogits, d_row_stride,
                      grid, st);
      break;
    case SMOE_DT_F16:
      SL_DISPATCH_VPL(launch_sl_bwd, __half, logits, row_stride, T, E, freq, acc, grad_aux, dlogits, d_row_stride,
                      grid, st);
      break;
    case SMOE_DT_F32:
      SL_DISPATCH_VPL(launch_sl_bwd, float, logits, row_stride, T, E, freq, acc, grad_aux, dlogits, d_row_stride, grid,
                      st);
      break;
    default:
      set_error("switch_loss_bwd: unknown dtype %d", dtype);
      return SMOE_ERR_INVALID;
  }
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}
