// Routing kernels for gfx950: fused top-K + softmax, expert histogram / prefix sum, stable counting-sort routing
// metadata, router backward.  All integer outputs are deterministic (no order-dependent atomics reach an output).
#include <hip/hip_fp16.h>

#include <mutex>

#include "common.h"

namespace smoe {

// ============================================================================================================
// top-K + softmax
// ============================================================================================================
// One row is owned by a group of G consecutive lanes (G a power of two <= 64); lane g of the group holds the
// VPL consecutive columns [g*VPL, (g+1)*VPL) as 64-bit keys
//     key = (order-preserving image of the fp32 value) << 32 | (0xffffffff - column)
// so that the maximum key is the largest value and, among equal values, the lowest column.  K rounds of
// "group arg-max, then retire the winner" give the winners in descending order.

SMOE_DEV uint32_t orderable(uint32_t bits) { return bits ^ ((bits >> 31) ? 0xffffffffu : 0x80000000u); }
SMOE_DEV uint32_t unorderable(uint32_t o) { return o ^ ((o >> 31) ? 0x80000000u : 0xffffffffu); }

SMOE_DEV uint64_t shfl_xor_u64(uint64_t v, int mask) {
  uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  lo = __shfl_xor(lo, mask, 64);
  hi = __shfl_xor(hi, mask, 64);
  return ((uint64_t)hi << 32) | lo;
}

template <typename T>
SMOE_DEV uint32_t load_as_f32_bits(const T* p);
template <>
__device__ __forceinline__ uint32_t load_as_f32_bits<uint16_t>(const uint16_t* p) {  // bf16
  return (uint32_t)(*p) << 16;
}
template <>
__device__ __forceinline__ uint32_t load_as_f32_bits<__half>(const __half* p) {
  return __float_as_uint(__half2float(*p));
}
template <>
__device__ __forceinline__ uint32_t load_as_f32_bits<float>(const float* p) {
  return __float_as_uint(*p);
}

template <typename T, int VPL>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T* __restrict__ logits, int64_t row_stride,
                                                           int64_t Trows, int E, int K, int G, uint32_t clear_mask,
                                                           float* __restrict__ scores, int32_t* __restrict__ indices,
                                                           int do_softmax) {
  const int lane_in_block = threadIdx.x;
  const int rows_per_block = 256 / G;
  const int g = lane_in_block % G;
  const int64_t row = (int64_t)blockIdx.x * rows_per_block + lane_in_block / G;
  const bool row_ok = row < Trows;
  const int64_t rrow = row_ok ? row : 0;

  uint64_t key[VPL];
  const T* src = logits + rrow * row_stride;
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const int col = g * VPL + i;
    uint64_t k = 0;  // 0 = retired / out of range: below every real key (real keys have a non-zero column part)
    if (col < E) {
      uint32_t bits = load_as_f32_bits<T>(src + col) & clear_mask;
      k = ((uint64_t)orderable(bits) << 32) | (uint64_t)(0xffffffffu - (uint32_t)col);
    }
    key[i] = k;
  }

  float vmax = 0.f, esum = 0.f;
  for (int r = 0; r < K; r++) {
    uint64_t best = key[0];
#pragma unroll
    for (int i = 1; i < VPL; i++) best = key[i] > best ? key[i] : best;
    for (int m = 1; m < G; m <<= 1) {
      uint64_t o = shfl_xor_u64(best, m);
      best = o > best ? o : best;
    }
#pragma unroll
    for (int i = 0; i < VPL; i++) key[i] = (key[i] == best) ? 0 : key[i];
    if (g == 0 && row_ok) {
      const float v = __uint_as_float(unorderable((uint32_t)(best >> 32)));
      const int col = (int)(0xffffffffu - (uint32_t)best);
      float outv = v;
      if (do_softmax) {
        if (r == 0) vmax = v;
        outv = expf(v - vmax);
        esum += outv;
      }
      scores[row * K + r] = outv;
      indices[row * K + r] = col;
    }
  }
  if (do_softmax && g == 0 && row_ok) {
    for (int r = 0; r < K; r++) scores[row * K + r] = scores[row * K + r] / esum;
  }
}

template <typename T>
static int launch_topk(const void* logits, int64_t T_, int E, int K, int64_t row_stride, float* scores,
                       int32_t* indices, int softmax, uint32_t clear_mask, hipStream_t st) {
  int G = 1;
  while (G < 64 && G * 16 < E) G <<= 1;
  int vpl = 1;
  while (vpl * G < E) vpl <<= 1;
  const int rows_per_block = 256 / G;
  const dim3 grid((unsigned)ceil_div(T_, rows_per_block)), block(256);
  const T* p = (const T*)logits;
#define SMOE_TOPK_CASE(V)                                                                                          \
  case V:                                                                                                          \
    hipLaunchKernelGGL((topk_softmax_kernel<T, V>), grid, block, 0, st, p, row_stride, T_, E, K, G, clear_mask,    \
                       scores, indices, softmax);                                                                  \
    break;
  switch (vpl) {
    SMOE_TOPK_CASE(1)
    SMOE_TOPK_CASE(2)
    SMOE_TOPK_CASE(4)
    SMOE_TOPK_CASE(8)
    SMOE_TOPK_CASE(16)
    SMOE_TOPK_CASE(32)
    SMOE_TOPK_CASE(64)
    default:
      set_error("topk: unsupported E=%d", E);
      return SMOE_ERR_UNSUPPORTED;
  }
#undef SMOE_TOPK_CASE
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

// ============================================================================================================
// router backward
// ============================================================================================================
template <typename T>
SMOE_DEV void store_from_f32(T* p, float v);
template <>
__device__ __forceinline__ void store_from_f32<uint16_t>(uint16_t* p, float v) {
  *p = (uint16_t)f32_to_bf16_bits(v);
}
template <>
__device__ __forceinline__ void store_from_f32<__half>(__half* p, float v) {
  *p = __float2half(v);
}
template <>
__device__ __forceinline__ void store_from_f32<float>(float* p, float v) {
  *p = v;
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_topk_bwd_kernel(T* __restrict__ dlogits, int64_t row_stride,
                                                               const T* dlogits_add, const float* __restrict__ dscores,
                                                               const float* __restrict__ scores,
                                                               const int32_t* __restrict__ indices, int64_t Trows,
                                                               int K) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= Trows) return;
  const float* g = dscores + row * K;
  const float* s = scores + row * K;
  const int32_t* ix = indices + row * K;
  float dot = 0.f;
  for (int k = 0; k < K; k++) dot += g[k] * s[k];
  T* out = dlogits + row * row_stride;
  // dlogits_add (may be dlogits itself): a gradient that reached the selected logits some other way is added in
  const T* add = dlogits_add ? dlogits_add + row * row_stride : nullptr;
  for (int k = 0; k < K; k++) {
    float v = s[k] * (g[k] - dot);
    if (add) v += __uint_as_float(load_as_f32_bits<T>(add + ix[k]));
    store_from_f32<T>(out + ix[k], v);
  }
}

// Backward of the un-fused top-K (values without softmax): the gradient of a selected logit is the gradient of its
// value.  One thread per token; the caller has zero-filled dlogits.
template <typename T>
__global__ __launch_bounds__(256) void topk_bwd_kernel(T* __restrict__ dlogits, int64_t row_stride,
                                                       const float* __restrict__ dvalues,
                                                       const int32_t* __restrict__ indices, int64_t Trows, int K) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= Trows) return;
  T* out = dlogits + row * row_stride;
  for (int k = 0; k < K; k++) store_from_f32<T>(out + indices[row * K + k], dvalues[row * K + k]);
}

// ============================================================================================================
// count + inclusive cumsum (standalone operator)
// ============================================================================================================
__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

template <typename IdxT, bool USE_LDS>
__global__ __launch_bounds__(1024) void count_kernel(const IdxT* __restrict__ x, int64_t n, int E,
                                                     int32_t* __restrict__ count) {
  extern __shared__ int32_t hist[];
  if (USE_LDS) {
    for (int e = threadIdx.x; e < E; e += blockDim.x) hist[e] = 0;
    __syncthreads();
  }
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t v = (int64_t)x[i];
    if (v >= 0 && v < E) {
      if (USE_LDS)
        atomicAdd(&hist[v], 1);
      else
        atomicAdd(&count[v], 1);
    }
  }
  if (USE_LDS) {
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
      const int32_t c = hist[e];
      if (c) atomicAdd(&count[e], c);
    }
  }
}

// single block, 1024 threads: inclusive scan of count[0..E)
__global__ __launch_bounds__(1024) void inclusive_scan_kernel(const int32_t* __restrict__ count, int E,
                                                              int32_t* __restrict__ cumsum) {
  __shared__ int32_t wave_tot[16];
  const int per = (E + 1023) / 1024;
  const int lo = threadIdx.x * per;
  int32_t local = 0;
  for (int i = 0; i < per; i++)
    if (lo + i < E) local += count[lo + i];
  // inclusive scan of `local` across the block
  int32_t v = local;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int d = 1; d < 64; d <<= 1) {
    int32_t o = __shfl_up(v, d, 64);
    if (lane >= d) v += o;
  }
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  int32_t base = 0;
  for (int w = 0; w < wave; w++) base += wave_tot[w];
  int32_t run = base + v - local;  // exclusive prefix of this thread's chunk
  for (int i = 0; i < per; i++)
    if (lo + i < E) {
      run += count[lo + i];
      cumsum[lo + i] = run;
    }
}

// ============================================================================================================
// routing metadata: stable counting sort of TK expert ids
// ============================================================================================================
// A "segment" is SEG consecutive flat slots, owned by ONE wavefront so that the order inside a segment is the
// lane / iteration order.  Pass A: per-segment histogram -> hist_t[e][s].  Pass B: one wavefront per expert scans
// its row of hist_t -> base_t[e][s] (slots of expert e that precede segment s) and freq[e].  Pass C: every
// segment rebuilds off[] from freq, seeds a cursor per expert and assigns positions with ballot-based ranking.
constexpr int SEG = 1024;
constexpr int META_WAVES = 4;

__global__ __launch_bounds__(64 * META_WAVES) void meta_hist_kernel(const int32_t* __restrict__ expert_idx,
                                                                    int64_t TK, int E, int NS,
                                                                    int32_t* __restrict__ hist_t) {
  extern __shared__ int32_t lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int32_t* hist = lds + (size_t)wave * E;
  const int s = blockIdx.x * META_WAVES + wave;
  if (s >= NS) return;
  for (int e = lane; e < E; e += 64) hist[e] = 0;
  __builtin_amdgcn_wave_barrier();
  const int64_t lo = (int64_t)s * SEG;
  const int64_t hi = lo + SEG < TK ? lo + SEG : TK;
  for (int64_t j = lo + lane; j < hi; j += 64) {
    const int e = expert_idx[j];
    if (e >= 0 && e < E) atomicAdd(&hist[e], 1);
  }
  __builtin_amdgcn_wave_barrier();
  for (int e = lane; e < E; e += 64) hist_t[(size_t)e * NS + s] = hist[e];
}

__global__ __launch_bounds__(256) void meta_scan_kernel(const int32_t* __restrict__ hist_t, int E, int NS,
                                                        int32_t* __restrict__ base_t, int32_t* __restrict__ freq) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + wave;
  if (e >= E) return;
  int32_t carry = 0;
  for (int s0 = 0; s0 < NS; s0 += 64) {
    const int s = s0 + lane;
    const int32_t h = s < NS ? hist_t[(size_t)e * NS + s] : 0;
    int32_t v = h;
    for (int d = 1; d < 64; d <<= 1) {
      int32_t o = __shfl_up(v, d, 64);
      if (lane >= d) v += o;
    }
    if (s < NS) base_t[(size_t)e * NS + s] = carry + v - h;
    carry += __shfl(v, 63, 64);
  }
  if (lane == 0) freq[e] = carry;
}

__global__ __launch_bounds__(64 * META_WAVES) void meta_scatter_kernel(
    const int32_t* __restrict__ expert_idx, const int32_t* __restrict__ token_idx, int64_t TK, int64_t T, int E,
    int K, int NS, int ebits, const int32_t* __restrict__ freq, const int32_t* __restrict__ base_t,
    int32_t* __restrict__ off, int32_t* __restrict__ gidx, int32_t* __restrict__ sidx, int32_t* __restrict__ ridx,
    int32_t* __restrict__ tok_off) {
  extern __shared__ int32_t lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int32_t* cursor = lds + (size_t)wave * E;
  const int s = blockIdx.x * META_WAVES + wave;
  if (s >= NS) return;

  // exclusive scan of freq -> off (every segment needs it; segment 0 also publishes it)
  int32_t carry = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int32_t f = e < E ? freq[e] : 0;
    int32_t v = f;
    for (int d = 1; d < 64; d <<= 1) {
      int32_t o = __shfl_up(v, d, 64);
      if (lane >= d) v += o;
    }
    if (e < E) {
      const int32_t excl = carry + v - f;
      cursor[e] = excl + base_t[(size_t)e * NS + s];
      if (s == 0) off[e] = excl;
    }
    carry += __shfl(v, 63, 64);
  }
  if (s == 0 && lane == 0) off[E] = carry;
  __builtin_amdgcn_wave_barrier();

  const int64_t lo = (int64_t)s * SEG;
  const int64_t hi = lo + SEG < TK ? lo + SEG : TK;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int64_t j0 = lo; j0 < hi; j0 += 64) {
    const int64_t j = j0 + lane;
    const bool valid = j < hi;
    int e = valid ? expert_idx[j] : 0;
    const bool in_range = valid && e >= 0 && e < E;
    if (!in_range) e = 0;
    uint64_t peers = __ballot(in_range);
    for (int b = 0; b < ebits; b++) {
      const uint64_t bal = __ballot((e >> b) & 1);
      peers &= ((e >> b) & 1) ? bal : ~bal;
    }
    int32_t pos = 0;
    if (in_range) {
      pos = cursor[e] + __popcll(peers & lt_mask);
    }
    __builtin_amdgcn_wave_barrier();
    if (in_range && (peers >> lane) >> 1 == 0) cursor[e] = pos + 1;  // highest peer lane advances the cursor
    __builtin_amdgcn_wave_barrier();
    if (in_range) {
      sidx[pos] = (int32_t)j;
      ridx[j] = pos;
      gidx[pos] = token_idx ? token_idx[j] : (int32_t)(j / K);
    }
    if (tok_off && valid) {
      if (token_idx) {
        const int32_t t = token_idx[j];
        const int32_t tprev = j == 0 ? -1 : token_idx[j - 1];
        for (int32_t u = tprev + 1; u <= t; u++) tok_off[u] = (int32_t)j;
        if (j == TK - 1)
          for (int64_t u = (int64_t)t + 1; u <= T; u++) tok_off[u] = (int32_t)TK;
      } else {
        if (j % K == 0) tok_off[j / K] = (int32_t)j;
        if (j == TK - 1) tok_off[T] = (int32_t)TK;
      }
    }
  }
  if (tok_off && TK == 0 && s == 0)
    for (int64_t u = lane; u <= T; u += 64) tok_off[u] = 0;
}

}  // namespace smoe

using namespace smoe;

extern "C" int smoe_count_cumsum(const void* x, int x_is_int64, int64_t n, int E, int32_t* count, int32_t* cumsum,
                                 void* stream) {
  SMOE_REQUIRE(count != nullptr && (x != nullptr || n == 0), SMOE_ERR_INVALID, "count_cumsum: null pointer");
  SMOE_REQUIRE(n >= 0, SMOE_ERR_INVALID, "count_cumsum: negative length");
  SMOE_REQUIRE(E >= 1 && E <= 65536, SMOE_ERR_UNSUPPORTED, "count_cumsum: E=%d outside [1, 65536]", E);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)ceil_div(E, 256)), dim3(256), 0, st, count, (int64_t)E, 0);
  SMOE_LAUNCH_CHECK();
  if (n > 0) {
    const bool use_lds = E <= 8192;
    int blocks = (int)(ceil_div(n, 1024 * 8) < 256 ? ceil_div(n, 1024 * 8) : 256);
    if (blocks < 1) blocks = 1;
    const size_t smem = use_lds ? (size_t)E * 4 : 0;
    if (x_is_int64) {
      if (use_lds)
        hipLaunchKernelGGL((count_kernel<int64_t, true>), dim3(blocks), dim3(1024), smem, st, (const int64_t*)x, n,
                           E, count);
      else
        hipLaunchKernelGGL((count_kernel<int64_t, false>), dim3(blocks), dim3(1024), 0, st, (const int64_t*)x, n, E,
                           count);
    } else {
      if (use_lds)
        hipLaunchKernelGGL((count_kernel<int32_t, true>), dim3(blocks), dim3(1024), smem, st, (const int32_t*)x, n,
                           E, count);
      else
        hipLaunchKernelGGL((count_kernel<int32_t, false>), dim3(blocks), dim3(1024), 0, st, (const int32_t*)x, n, E,
                           count);
    }
    SMOE_LAUNCH_CHECK();
  }
  if (cumsum) {
    hipLaunchKernelGGL(inclusive_scan_kernel, dim3(1), dim3(1024), 0, st, count, E, cumsum);
    SMOE_LAUNCH_CHECK();
  }
  return SMOE_OK;
}

extern "C" int smoe_topk_softmax_fwd(const void* logits, int dtype, int64_t T, int E, int K, int64_t row_stride,
                                     float* scores, int32_t* indices, int softmax, void* stream) {
  SMOE_REQUIRE(T >= 0, SMOE_ERR_INVALID, "topk: negative T");
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(logits && scores && indices, SMOE_ERR_INVALID, "topk: null pointer");
  SMOE_REQUIRE(E >= 1 && E <= 4096, SMOE_ERR_UNSUPPORTED, "topk: E=%d outside [1, 4096]", E);
  SMOE_REQUIRE(K >= 1 && K <= E && K <= 64, SMOE_ERR_UNSUPPORTED, "topk: K=%d outside [1, min(E, 64)]", K);
  SMOE_REQUIRE(row_stride >= E, SMOE_ERR_INVALID, "topk: row stride %lld < E", (long long)row_stride);
  hipStream_t st = (hipStream_t)stream;
  uint32_t p2 = 1;
  while ((int)p2 < E) p2 <<= 1;
  switch (dtype) {
    case SMOE_DT_BF16:
      return launch_topk<uint16_t>(logits, T, E, K, row_stride, scores, indices, softmax, 0xffffffffu, st);
    case SMOE_DT_F16:
      return launch_topk<__half>(logits, T, E, K, row_stride, scores, indices, softmax, ~(p2 - 1), st);
    case SMOE_DT_F32:
      return launch_topk<float>(logits, T, E, K, row_stride, scores, indices, softmax, ~(p2 - 1), st);
  }
  set_error("topk: unknown dtype %d", dtype);
  return SMOE_ERR_INVALID;
}

extern "C" int smoe_softmax_topk_bwd(void* dlogits, int dtype, int64_t row_stride, const void* dlogits_add,
                                     const float* dscores, const float* scores, const int32_t* indices, int64_t T, int K,
                                     void* stream) {
  SMOE_REQUIRE(T >= 0 && K >= 1, SMOE_ERR_INVALID, "softmax_topk_bwd: bad sizes");
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(dlogits && dscores && scores && indices, SMOE_ERR_INVALID, "softmax_topk_bwd: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)ceil_div(T, 256)), block(256);
  switch (dtype) {
    case SMOE_DT_BF16:
      hipLaunchKernelGGL(softmax_topk_bwd_kernel<uint16_t>, grid, block, 0, st, (uint16_t*)dlogits, row_stride,
                         (const uint16_t*)dlogits_add, dscores, scores, indices, T, K);
      break;
    case SMOE_DT_F16:
      hipLaunchKernelGGL(softmax_topk_bwd_kernel<__half>, grid, block, 0, st, (__half*)dlogits, row_stride,
                         (const __half*)dlogits_add, dscores, scores, indices, T, K);
      break;
    case SMOE_DT_F32:
      hipLaunchKernelGGL(softmax_topk_bwd_kernel<float>, grid, block, 0, st, (float*)dlogits, row_stride,
                         (const float*)dlogits_add, dscores, scores, indices, T, K);
      break;
    default:
      set_error("softmax_topk_bwd: unknown dtype %d", dtype);
      return SMOE_ERR_INVALID;
  }
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_topk_bwd(void* dlogits, int dtype, int64_t row_stride, const float* dvalues, const int32_t* indices,
                             int64_t T, int K, void* stream) {
  SMOE_REQUIRE(T >= 0 && K >= 1, SMOE_ERR_INVALID, "topk_bwd: bad sizes");
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(dlogits && dvalues && indices, SMOE_ERR_INVALID, "topk_bwd: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)ceil_div(T, 256)), block(256);
  switch (dtype) {
    case SMOE_DT_BF16:
      hipLaunchKernelGGL(topk_bwd_kernel<uint16_t>, grid, block, 0, st, (uint16_t*)dlogits, row_stride, dvalues, indices,
                         T, K);
      break;
    case SMOE_DT_F16:
      hipLaunchKernelGGL(topk_bwd_kernel<__half>, grid, block, 0, st, (__half*)dlogits, row_stride, dvalues, indices, T,
                         K);
      break;
    case SMOE_DT_F32:
      hipLaunchKernelGGL(topk_bwd_kernel<float>, grid, block, 0, st, (float*)dlogits, row_stride, dvalues, indices, T, K);
      break;
    default:
      set_error("topk_bwd: unknown dtype %d", dtype);
      return SMOE_ERR_INVALID;
  }
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

static inline int meta_segments(int64_t TK) {
  int64_t ns = ceil_div(TK, smoe::SEG);
  return (int)(ns < 1 ? 1 : ns);
}

extern "C" size_t smoe_routing_metadata_workspace_bytes(int64_t TK, int E) {
  if (TK < 0 || E < 1) return 0;
  return (size_t)2 * (size_t)E * (size_t)meta_segments(TK) * sizeof(int32_t);
}

// argument checks shared by the two metadata entry points (everything but the scratch memory)
static int check_routing_metadata_args(const int32_t* expert_idx, const int32_t* token_idx, int64_t TK, int64_t T, int E,
                                       int K, const int32_t* freq, const int32_t* off, const int32_t* x_gather_idx,
                                       const int32_t* s_scatter_idx, const int32_t* s_reverse_scatter_idx) {
  SMOE_REQUIRE(TK >= 0 && T >= 0, SMOE_ERR_INVALID, "routing_metadata: negative size");
  SMOE_REQUIRE(TK < (1ll << 31), SMOE_ERR_UNSUPPORTED, "routing_metadata: TK does not fit int32");
  SMOE_REQUIRE(E >= 1 && E <= 4096, SMOE_ERR_UNSUPPORTED, "routing_metadata: E=%d outside [1, 4096]", E);
  SMOE_REQUIRE(freq && off, SMOE_ERR_INVALID, "routing_metadata: null pointer");
  SMOE_REQUIRE(TK == 0 || (expert_idx && x_gather_idx && s_scatter_idx && s_reverse_scatter_idx), SMOE_ERR_INVALID,
               "routing_metadata: null pointer");
  SMOE_REQUIRE(token_idx != nullptr || K >= 1, SMOE_ERR_INVALID, "routing_metadata: K must be >= 1 without token_idx");
  return SMOE_OK;
}

// the three passes of the counting sort; `workspace` holds the two (E, NS) int32 tables, both written in full by
// the first two passes before they are read (nothing in it has to start at zero)
static int launch_routing_metadata(const int32_t* expert_idx, const int32_t* token_idx, int64_t TK, int64_t T, int E,
                                   int K, int32_t* freq, int32_t* off, int32_t* x_gather_idx, int32_t* s_scatter_idx,
                                   int32_t* s_reverse_scatter_idx, int32_t* tok_off, void* workspace, hipStream_t st) {
  const int NS = meta_segments(TK);
  int32_t* hist_t = (int32_t*)workspace;
  int32_t* base_t = hist_t + (size_t)E * NS;
  int ebits = 0;
  while ((1 << ebits) < E) ebits++;
  const dim3 grid_seg((unsigned)ceil_div(NS, META_WAVES)), block_seg(64 * META_WAVES);
  const size_t smem = (size_t)META_WAVES * E * sizeof(int32_t);
  hipLaunchKernelGGL(meta_hist_kernel, grid_seg, block_seg, smem, st, expert_idx, TK, E, NS, hist_t);
  SMOE_LAUNCH_CHECK();
  hipLaunchKernelGGL(meta_scan_kernel, dim3((unsigned)ceil_div(E, 4)), dim3(256), 0, st, hist_t, E, NS, base_t, freq);
  SMOE_LAUNCH_CHECK();
  hipLaunchKernelGGL(meta_scatter_kernel, grid_seg, block_seg, smem, st, expert_idx, token_idx, TK, T, E, K, NS, ebits,
                     freq, base_t, off, x_gather_idx, s_scatter_idx, s_reverse_scatter_idx, tok_off);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_routing_metadata(const int32_t* expert_idx, const int32_t* token_idx, int64_t TK, int64_t T,
                                     int E, int K, int32_t* freq, int32_t* off, int32_t* x_gather_idx,
                                     int32_t* s_scatter_idx, int32_t* s_reverse_scatter_idx, int32_t* tok_off,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = check_routing_metadata_args(expert_idx, token_idx, TK, T, E, K, freq, off, x_gather_idx, s_scatter_idx,
                                             s_reverse_scatter_idx);
  if (rc) return rc;
  SMOE_REQUIRE(workspace != nullptr, SMOE_ERR_INVALID, "routing_metadata: null pointer");
  SMOE_REQUIRE(workspace_bytes >= smoe_routing_metadata_workspace_bytes(TK, E), SMOE_ERR_WORKSPACE,
               "routing_metadata: workspace too small");
  return launch_routing_metadata(expert_idx, token_idx, TK, T, E, K, freq, off, x_gather_idx, s_scatter_idx,
                                 s_reverse_scatter_idx, tok_off, workspace, (hipStream_t)stream);
}

// ---- the same operator for callers that cannot allocate ------------------------------------------------------
// The two tables live in a device array that is part of the library image: one copy per GPU, at an address of its
// own on each, looked up once per device.  In host code the array's NAME is only a handle for that look-up; the
// kernels get the looked-up pointer.
static __device__ __align__(256) unsigned char scratch[SMOE_ROUTING_METADATA_STATIC_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES] = {};  // device address of `scratch` on each GPU, null = not looked up yet
}  // namespace

// device address of this GPU's copy of `scratch`
static int static_scratch(void** out) {
  int dev = 0;
  SMOE_HIP_CHECK(hipGetDevice(&dev));
  SMOE_REQUIRE(dev >= 0 && dev < MAX_DEVICES, SMOE_ERR_UNSUPPORTED, "routing_metadata_static: device %d out of range",
               dev);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    SMOE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SMOE_REQUIRE(p != nullptr, SMOE_ERR_HIP, "routing_metadata_static: no device address for the scratch array");
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return SMOE_OK;
}

extern "C" size_t smoe_routing_metadata_static_capacity(void) { return SMOE_ROUTING_METADATA_STATIC_BYTES; }

extern "C" int smoe_routing_metadata_static(const int32_t* expert_idx, const int32_t* token_idx, int64_t TK, int64_t T,
                                            int E, int K, int32_t* freq, int32_t* off, int32_t* x_gather_idx,
                                            int32_t* s_scatter_idx, int32_t* s_reverse_scatter_idx, int32_t* tok_off,
                                            void* stream) {
  int rc = check_routing_metadata_args(expert_idx, token_idx, TK, T, E, K, freq, off, x_gather_idx, s_scatter_idx,
                                       s_reverse_scatter_idx);
  if (rc) return rc;
  const size_t need = smoe_routing_metadata_workspace_bytes(TK, E);
  SMOE_REQUIRE(need <= (size_t)SMOE_ROUTING_METADATA_STATIC_BYTES, SMOE_ERR_WORKSPACE,
               "routing_metadata_static: TK=%lld, E=%d need %zu bytes of scratch, the built-in array holds %zu; use "
               "smoe_routing_metadata with a workspace of your own",
               (long long)TK, E, need, (size_t)SMOE_ROUTING_METADATA_STATIC_BYTES);
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc) return rc;
  return launch_routing_metadata(expert_idx, token_idx, TK, T, E, K, freq, off, x_gather_idx, s_scatter_idx,
                                 s_reverse_scatter_idx, tok_off, ws, (hipStream_t)stream);
}
