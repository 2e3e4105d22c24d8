// Token-rounding router on the device: token-choice top-K first, then every expert's token count is rounded to a
// multiple of the GEMM token tile by dropping its lowest-ranked picks or adding its best non-picked tokens
// (benchmarks/moe-token-rounding.py:139-191 of the reference, where it is a chain of dense torch ops with a (T, E)
// argsort along the token axis).  Here the per-expert argsort is a two-pass radix SELECT of the k-th largest 16-bit
// ranking value plus an ordered pass that resolves ties towards the lower token index; nothing is sorted.
//
//   tr_softmax   probs = softmax(logits, fp32) rounded to the logits' 16-bit dtype                       (:149)
//   (top-K of probs and the expert histogram come from smoe_topk_softmax_fwd / smoe_count_cumsum)        (:152-154)
//   tr_rank      renormalise the K picks, write them back into probs, rank = pick ? value : probs - 1    (:158-164)
//   tr_select    per expert: keep the target[e] highest-ranked tokens                                    (:167-184)
//   tr_row_counts / tr_compact  the kept (token, expert) pairs in token order with their scores          (:187-191)
#include <hip/hip_fp16.h>

#include "common.h"

namespace smoe {

template <typename T>
SMOE_DEV float h2f(T v);
template <>
__device__ __forceinline__ float h2f<uint16_t>(uint16_t v) { return bf16_bits_to_f32(v); }
template <>
__device__ __forceinline__ float h2f<__half>(__half v) { return __half2float(v); }
template <typename T>
SMOE_DEV T f2h(float v);
template <>
__device__ __forceinline__ uint16_t f2h<uint16_t>(float v) { return (uint16_t)f32_to_bf16_bits(v); }
template <>
__device__ __forceinline__ __half f2h<__half>(float v) { return __float2half_rn(v); }
template <typename T>
SMOE_DEV uint16_t raw16(T v);
template <>
__device__ __forceinline__ uint16_t raw16<uint16_t>(uint16_t v) { return v; }
template <>
__device__ __forceinline__ uint16_t raw16<__half>(__half v) { return __half_as_ushort(v); }

// order-preserving image of a 16-bit float: larger value <=> larger key
SMOE_DEV uint32_t orderable16(uint16_t bits) { return (bits & 0x8000u) ? (uint16_t)~bits : (uint16_t)(bits | 0x8000u); }

SMOE_DEV float wave_max(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
  return v;
}
SMOE_DEV float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
  return v;
}

// one wavefront per token
template <typename T>
__global__ __launch_bounds__(256) void tr_softmax_kernel(const T* __restrict__ logits, int64_t row_stride,
                                                         int64_t Trows, int E, T* __restrict__ probs) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= Trows) return;
  const T* src = logits + t * row_stride;
  float m = -INFINITY;
  for (int e = lane; e < E; e += 64) m = fmaxf(m, h2f<T>(src[e]));
  m = wave_max(m);
  float s = 0.f;
  for (int e = lane; e < E; e += 64) s += expf(h2f<T>(src[e]) - m);
  s = wave_sum(s);
  for (int e = lane; e < E; e += 64) probs[t * E + e] = f2h<T>(expf(h2f<T>(src[e]) - m) / s);
}

// one wavefront per token: picks are renormalised (their sum and the quotients rounded to the 16-bit dtype, as the
// reference's tensor arithmetic does), written back into probs, and the ranking matrix is filled.  The picks' columns
// are marked in a per-wavefront LDS row first, so that every output element is written exactly once.
template <typename T>
__global__ __launch_bounds__(256) void tr_rank_kernel(T* __restrict__ probs, T* __restrict__ rank,
                                                      const float* __restrict__ top_v,
                                                      const int32_t* __restrict__ top_i, int64_t Trows, int E, int K) {
  extern __shared__ uint32_t pick_row[];  // [4 wavefronts][E]: 0 = not a pick, else 0x10000 | renormalised value bits
  const int lane = threadIdx.x & 63;
  uint32_t* mine = pick_row + (threadIdx.x >> 6) * E;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= Trows) return;
  for (int e = lane; e < E; e += 64) mine[e] = 0;
  const float v = lane < K ? top_v[t * K + lane] : 0.f;  // K <= 64; the values are already 16-bit representable
  const float sum = h2f<T>(f2h<T>(wave_sum(v)));
  if (lane < K) mine[top_i[t * K + lane]] = 0x10000u | raw16<T>(f2h<T>(v / sum));
  for (int e = lane; e < E; e += 64) {
    const uint32_t m = mine[e];
    if (m) {
      const uint16_t q = (uint16_t)m;
      probs[t * E + e] = *(const T*)&q;
      rank[t * E + e] = *(const T*)&q;
    } else {
      rank[t * E + e] = f2h<T>(h2f<T>(probs[t * E + e]) - 1.0f);
    }
  }
}

// One workgroup per expert.  Pass 1 / 2: histograms of the high / low byte of the 16-bit ranking keys give the key of
// the target-th largest value; pass 3 walks the tokens in order and keeps the larger keys plus the first `need`
// tokens that tie with it.
template <typename T>
__global__ __launch_bounds__(1024) void tr_select_kernel(const T* __restrict__ rank, const int32_t* __restrict__ target,
                                                         uint8_t* __restrict__ keep, int Trows, int E) {
  __shared__ int hist[256];
  __shared__ int sh_bin, sh_need;
  __shared__ int wave_cnt[16];
  __shared__ int running;
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int tgt = target[e];
  tgt = tgt < 0 ? 0 : (tgt > Trows ? Trows : tgt);
  if (tgt == 0 || tgt == Trows) {
    for (int t = tid; t < Trows; t += 1024) keep[(int64_t)t * E + e] = tgt ? 1 : 0;
    return;
  }
  auto key_of = [&](int t) { return orderable16(raw16<T>(rank[(int64_t)t * E + e])); };
  // descending scan of a 256-bin histogram: the bin where the running count reaches `need`
  auto find_bin = [&](int need) {
    __syncthreads();
    if (tid == 0) {
      int acc = 0, b = 255;
      for (; b > 0; b--) {
        if (acc + hist[b] >= need) break;
        acc += hist[b];
      }
      sh_bin = b;
      sh_need = need - acc;  // how many are still to be taken inside bin b
    }
    __syncthreads();
  };
  if (tid < 256) hist[tid] = 0;
  __syncthreads();
  for (int t = tid; t < Trows; t += 1024) atomicAdd(&hist[key_of(t) >> 8], 1);
  find_bin(tgt);
  const int hi = sh_bin, need_hi = sh_need;
  __syncthreads();
  if (tid < 256) hist[tid] = 0;
  __syncthreads();
  for (int t = tid; t < Trows; t += 1024) {
    const uint32_t k = key_of(t);
    if ((int)(k >> 8) == hi) atomicAdd(&hist[k & 255], 1);
  }
  find_bin(need_hi);
  const uint32_t kstar = ((uint32_t)hi << 8) | (uint32_t)sh_bin;
  const int need = sh_need;  // tokens equal to kstar to keep, lowest token index first
  if (tid == 0) running = 0;
  __syncthreads();
  for (int base = 0; base < Trows; base += 1024) {
    const int t = base + tid;
    const uint32_t k = t < Trows ? key_of(t) : 0;
    const bool tie = t < Trows && k == kstar;
    const uint64_t bal = __ballot(tie);
    const int before_in_wave = __popcll(bal & ((1ull << lane) - 1));
    if (lane == 0) wave_cnt[wave] = __popcll(bal);
    __syncthreads();
    int before = running;
    for (int w = 0; w < wave; w++) before += wave_cnt[w];
    before += before_in_wave;
    if (t < Trows) keep[(int64_t)t * E + e] = (k > kstar || (tie && before < need)) ? 1 : 0;
    __syncthreads();
    if (tid == 0) {
      int tot = 0;
      for (int w = 0; w < 16; w++) tot += wave_cnt[w];
      running += tot;
    }
    __syncthreads();
  }
}

// one wavefront per token: number of kept experts
__global__ __launch_bounds__(256) void tr_row_counts_kernel(const uint8_t* __restrict__ keep, int64_t Trows, int E,
                                                            int32_t* __restrict__ counts) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= Trows) return;
  int c = 0;
  for (int e = lane; e < E; e += 64) c += keep[t * E + e];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) c += __shfl_xor(c, d, 64);
  if (lane == 0) counts[t] = c;
}

// one wavefront per token: its kept pairs, experts ascending, at [tok_off[t], tok_off[t+1])
template <typename T>
__global__ __launch_bounds__(256) void tr_compact_kernel(const uint8_t* __restrict__ keep, const T* __restrict__ probs,
                                                         const int32_t* __restrict__ tok_off, int64_t Trows, int E,
                                                         T* __restrict__ scores, int32_t* __restrict__ tok,
                                                         int32_t* __restrict__ exp) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= Trows) return;
  int pos = tok_off[t];
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const bool k = e < E && keep[t * E + e];
    const uint64_t bal = __ballot(k);
    if (k) {
      const int p = pos + __popcll(bal & ((1ull << lane) - 1));
      scores[p] = probs[t * E + e];
      tok[p] = (int32_t)t;
      exp[p] = e;
    }
    pos += __popcll(bal);
  }
}

}  // namespace smoe

using namespace smoe;

static int check_tr(int64_t T, int E, int dtype, const char* who) {
  SMOE_REQUIRE(T >= 0 && T < (1ll << 31), SMOE_ERR_INVALID, "%s: T out of range", who);
  SMOE_REQUIRE(E >= 1 && E <= 4096, SMOE_ERR_UNSUPPORTED, "%s: E=%d outside [1, 4096]", who, E);
  SMOE_REQUIRE(dtype == SMOE_DT_BF16 || dtype == SMOE_DT_F16, SMOE_ERR_UNSUPPORTED,
               "%s: the ranking values are 16-bit keys, fp32 router probabilities are not supported", who);
  return SMOE_OK;
}

extern "C" int smoe_tr_softmax(const void* logits, int dtype, int64_t T, int E, int64_t row_stride, void* probs,
                               void* stream) {
  int rc = check_tr(T, E, dtype, "tr_softmax");
  if (rc) return rc;
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(logits && probs && row_stride >= E, SMOE_ERR_INVALID, "tr_softmax: bad argument");
  const dim3 grid((unsigned)ceil_div(T, 4)), block(256);
  if (dtype == SMOE_DT_BF16)
    hipLaunchKernelGGL(tr_softmax_kernel<uint16_t>, grid, block, 0, (hipStream_t)stream, (const uint16_t*)logits,
                       row_stride, T, E, (uint16_t*)probs);
  else
    hipLaunchKernelGGL(tr_softmax_kernel<__half>, grid, block, 0, (hipStream_t)stream, (const __half*)logits,
                       row_stride, T, E, (__half*)probs);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_tr_rank(void* probs, void* rank, int dtype, const float* top_v, const int32_t* top_i, int64_t T,
                            int E, int K, void* stream) {
  int rc = check_tr(T, E, dtype, "tr_rank");
  if (rc) return rc;
  SMOE_REQUIRE(K >= 1 && K <= 64 && K <= E, SMOE_ERR_UNSUPPORTED, "tr_rank: K=%d outside [1, min(E, 64)]", K);
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(probs && rank && top_v && top_i, SMOE_ERR_INVALID, "tr_rank: null pointer");
  const dim3 grid((unsigned)ceil_div(T, 4)), block(256);
  if (dtype == SMOE_DT_BF16)
    hipLaunchKernelGGL(tr_rank_kernel<uint16_t>, grid, block, (size_t)4 * E * 4, (hipStream_t)stream, (uint16_t*)probs,
                       (uint16_t*)rank, top_v, top_i, T, E, K);
  else
    hipLaunchKernelGGL(tr_rank_kernel<__half>, grid, block, (size_t)4 * E * 4, (hipStream_t)stream, (__half*)probs, (__half*)rank,
                       top_v, top_i, T, E, K);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_tr_select(const void* rank, int dtype, const int32_t* target, uint8_t* keep, int64_t T, int E,
                              void* stream) {
  int rc = check_tr(T, E, dtype, "tr_select");
  if (rc) return rc;
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(rank && target && keep, SMOE_ERR_INVALID, "tr_select: null pointer");
  if (dtype == SMOE_DT_BF16)
    hipLaunchKernelGGL(tr_select_kernel<uint16_t>, dim3((unsigned)E), dim3(1024), 0, (hipStream_t)stream,
                       (const uint16_t*)rank, target, keep, (int)T, E);
  else
    hipLaunchKernelGGL(tr_select_kernel<__half>, dim3((unsigned)E), dim3(1024), 0, (hipStream_t)stream,
                       (const __half*)rank, target, keep, (int)T, E);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_tr_row_counts(const uint8_t* keep, int64_t T, int E, int32_t* counts, void* stream) {
  SMOE_REQUIRE(T >= 0 && E >= 1, SMOE_ERR_INVALID, "tr_row_counts: bad shape");
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(keep && counts, SMOE_ERR_INVALID, "tr_row_counts: null pointer");
  hipLaunchKernelGGL(tr_row_counts_kernel, dim3((unsigned)ceil_div(T, 4)), dim3(256), 0, (hipStream_t)stream, keep, T,
                     E, counts);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

extern "C" int smoe_tr_compact(const uint8_t* keep, const void* probs, int dtype, const int32_t* tok_off, int64_t T,
                               int E, void* scores, int32_t* token_idx, int32_t* expert_idx, void* stream) {
  int rc = check_tr(T, E, dtype, "tr_compact");
  if (rc) return rc;
  if (T == 0) return SMOE_OK;
  SMOE_REQUIRE(keep && probs && tok_off, SMOE_ERR_INVALID, "tr_compact: null pointer");
  const dim3 grid((unsigned)ceil_div(T, 4)), block(256);
  if (dtype == SMOE_DT_BF16)
    hipLaunchKernelGGL(tr_compact_kernel<uint16_t>, grid, block, 0, (hipStream_t)stream, keep, (const uint16_t*)probs,
                       tok_off, T, E, (uint16_t*)scores, token_idx, expert_idx);
  else
    hipLaunchKernelGGL(tr_compact_kernel<__half>, grid, block, 0, (hipStream_t)stream, keep, (const __half*)probs,
                       tok_off, T, E, (__half*)scores, token_idx, expert_idx);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}
