// Sustained MFMA rate under the power limit with random operand data: 32x32x16 against 16x16x32 (bf16) and the scaled
// fp8 32x32x64 form, same wave tile
// (128 x 64 outputs per wave, 8 waves per CU), operands rotating through several random fragment sets in registers.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ inline uint32_t hash(uint32_t x) { x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }
// a random bf16 pair: random sign and mantissa, exponent near 1.0 (scale: exponent offset)
__device__ inline uint32_t rnd_pair(uint32_t seed, int zero, int small) {
  if (zero) return 0;
  uint32_t h = hash(seed);
  uint32_t lo = (h & 0x80ffu) | ((uint32_t)(120 + ((h >> 24) & 7) - (small ? 6 : 0)) << 7);
  uint32_t hi = ((h >> 8) & 0x80ffu) | ((uint32_t)(120 + ((h >> 28) & 7) - (small ? 6 : 0)) << 7);
  return lo | (hi << 16);
}
__device__ inline bf16x8 rnd_frag(uint32_t seed, int zero, int small) {
  u32x4 v = {rnd_pair(seed, zero, small), rnd_pair(seed + 1, zero, small), rnd_pair(seed + 2, zero, small), rnd_pair(seed + 3, zero, small)};
  return __builtin_bit_cast(bf16x8, v);
}
template <int SETS>
__global__ __launch_bounds__(512) void k32(float* out, int iters, int zero) {
  bf16x8 p[SETS][4], q[SETS][2];
  const uint32_t s0 = (blockIdx.x * 512 + threadIdx.x) * 64;
  for (int s = 0; s < SETS; s++) { for (int i = 0; i < 4; i++) p[s][i] = rnd_frag(s0 + s * 24 + i * 4, zero, 0); for (int i = 0; i < 2; i++) q[s][i] = rnd_frag(s0 + s * 24 + 16 + i * 4, zero, 1); }
  f32x16 acc[2][4];
  for (int a = 0; a < 2; a++) for (int b = 0; b < 4; b++) for (int i = 0; i < 16; i++) acc[a][b][i] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int s = 0; s < SETS; s++)
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(q[s][a], p[s][b], acc[a][b], 0, 0, 0);
  }
  float sum = 0; for (int a = 0; a < 2; a++) for (int b = 0; b < 4; b++) for (int i = 0; i < 16; i++) sum += acc[a][b][i];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}
template <int SETS>
__global__ __launch_bounds__(512) void k16(float* out, int iters, int zero) {
  bf16x8 p[SETS][8], q[SETS][4];   // one set covers k = 32: 8 token fragments of 16 rows, 4 feature fragments of 16
  const uint32_t s0 = (blockIdx.x * 512 + threadIdx.x) * 64;
  for (int s = 0; s < SETS; s++) { for (int i = 0; i < 8; i++) p[s][i] = rnd_frag(s0 + s * 48 + i * 4, zero, 0); for (int i = 0; i < 4; i++) q[s][i] = rnd_frag(s0 + s * 48 + 32 + i * 4, zero, 1); }
  f32x4 acc[4][8];
  for (int a = 0; a < 4; a++) for (int b = 0; b < 8; b++) for (int i = 0; i < 4; i++) acc[a][b][i] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int s = 0; s < SETS; s++)
#pragma unroll
      for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 8; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(q[s][a], p[s][b], acc[a][b], 0, 0, 0);
  }
  float sum = 0; for (int a = 0; a < 4; a++) for (int b = 0; b < 8; b++) for (int i = 0; i < 4; i++) sum += acc[a][b][i];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}
// e4m3 operands of v_mfma_scale_f32_32x32x64_f8f6f4 (unit scales): random bytes with the top exponent bit cleared (no NaN)
typedef int i32x8 __attribute__((ext_vector_type(8)));
__device__ inline i32x8 rnd_frag8(uint32_t seed, int zero) {
  i32x8 v;
  for (int i = 0; i < 8; i++) v[i] = zero ? 0 : (int)(hash(seed + i) & 0xbfbfbfbfu);
  return v;
}
template <int SETS>
__global__ __launch_bounds__(512) void kf8(float* out, int iters, int zero) {
  i32x8 p[SETS][4], q[SETS][2];  // one set covers k = 64: 4 token fragments of 32 rows, 2 feature fragments
  const uint32_t s0 = (blockIdx.x * 512 + threadIdx.x) * 128;
  for (int s = 0; s < SETS; s++) { for (int i = 0; i < 4; i++) p[s][i] = rnd_frag8(s0 + s * 48 + i * 8, zero); for (int i = 0; i < 2; i++) q[s][i] = rnd_frag8(s0 + s * 48 + 32 + i * 8, zero); }
  f32x16 acc[2][4];
  for (int a = 0; a < 2; a++) for (int b = 0; b < 4; b++) for (int i = 0; i < 16; i++) acc[a][b][i] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int s = 0; s < SETS; s++)
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 4; b++)
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(q[s][a], p[s][b], acc[a][b], 0, 0, 0, 127, 0, 127);
  }
  float sum = 0; for (int a = 0; a < 2; a++) for (int b = 0; b < 4; b++) for (int i = 0; i < 16; i++) sum += acc[a][b][i];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}
int main() {
  float* out; hipMalloc(&out, 1024 * 512 * 4);
  hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
  // per iteration and wave: k32<4>: 4 sets x 8 MFMA x 32768 flop; k16<2>: 2 sets x 32 MFMA x 16384 flop = the same 1 MiFLOP
  const int iters = 60000;
  for (int rep = 0; rep < 3; rep++) {
    for (int zero = 0; zero < 2; zero++) {
      float ms;
      hipEventRecord(e0); k32<4><<<256, 512>>>(out, iters, zero); hipEventRecord(e1); hipEventSynchronize(e1); hipEventElapsedTime(&ms, e0, e1);
      double fl = 256.0 * 8 * iters * 4 * 8 * 32768.0;
      printf("mfma 32x32x16 %s: %8.2f ms %7.1f TFLOP/s\n", zero ? "zeros " : "random", ms, fl / ms / 1e9);
      hipEventRecord(e0); k16<2><<<256, 512>>>(out, iters, zero); hipEventRecord(e1); hipEventSynchronize(e1); hipEventElapsedTime(&ms, e0, e1);
      fl = 256.0 * 8 * iters * 2 * 32 * 16384.0;
      printf("mfma 16x16x32 %s: %8.2f ms %7.1f TFLOP/s\n", zero ? "zeros " : "random", ms, fl / ms / 1e9);
      hipEventRecord(e0); kf8<2><<<256, 512>>>(out, iters, zero); hipEventRecord(e1); hipEventSynchronize(e1); hipEventElapsedTime(&ms, e0, e1);
      fl = 256.0 * 8 * iters * 2 * 8 * 131072.0;
      printf("mfma fp8 32x32x64 (scaled) %s: %8.2f ms %7.1f TFLOP/s\n", zero ? "zeros " : "random", ms, fl / ms / 1e9);
    }
  }
  return 0;
}
