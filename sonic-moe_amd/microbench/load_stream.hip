// Continuous direct-to-LDS streaming per wave with N loads kept in flight (s_waitcnt vmcnt(N-1) before every issue),
// L2-resident data, 256 workgroups of NW waves.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); return 1;} }while(0)
typedef int i32x4 __attribute__((ext_vector_type(4)));
template <int N> __device__ inline void wait_upto() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
template <int N, int NW>
__global__ __launch_bounds__(NW * 64) void k(const char* buf, size_t region, int iters, unsigned long long* clk, float* out) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const char* base = buf + (size_t)xcd * region;
  const uint32_t lbase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)smem;
  i32x4 srd;
  const uint64_t b = (uint64_t)base;
  srd[0] = __builtin_amdgcn_readfirstlane((uint32_t)b);
  srd[1] = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32) & 0xffff);
  srd[2] = __builtin_amdgcn_readfirstlane((int)region);
  srd[3] = 0x00020000;
  const uint32_t lane_off = (uint32_t)(lane >> 3) * 8192 + (lane & 7) * 16;   // 8 rows x 128 B, rows 8 KiB apart
  uint32_t pos = (uint32_t)(((size_t)slot * 65536 + (size_t)wave * 65536) % (region - 131072));
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long t0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const uint32_t vo = pos + lane_off + u * 128;
      const uint32_t l = lbase + ((wave * 16 + u) % 32) * 1024;
      wait_upto<N - 1>();
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, 0 offen lds" ::"v"(vo), "s"(srd), "s"(l) : "memory");
    }
    pos += 2048;
    if (pos >= region - 131072) pos = 0;
  }
  wait_upto<0>();
  const unsigned long long c1 = __builtin_readcyclecounter();
  const unsigned long long t1 = wall_clock64();
  if (threadIdx.x == 0 && blockIdx.x == 0) { clk[0] = c1 - c0; clk[1] = t1 - t0; }
  out[blockIdx.x * blockDim.x + threadIdx.x] = ((float*)smem)[threadIdx.x];
}
template <int N, int NW>
int run(const char* buf, size_t region, unsigned long long* clk, float* out) {
  const int iters = 1000;
  CK(hipFuncSetAttribute((const void*)k<N, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, 32 * 1024));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  k<N, NW><<<256, NW * 64, 32 * 1024>>>(buf, region, 50, clk, out);
  CK(hipEventRecord(e0));
  k<N, NW><<<256, NW * 64, 32 * 1024>>>(buf, region, iters, clk, out);
  CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  unsigned long long h[2]; CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
  const double bytes_per_cu = (double)iters * 16 * 1024 * NW;
  const double ghz = (double)h[0] / ((double)h[1] * 10.0);
  printf("buffer -> LDS continuous, %2d in flight per wave, %d waves: %7.3f ms  %6.2f TB/s chip  clock %.2f GHz  %5.1f B/clk/CU\n", N, NW, ms,
         bytes_per_cu * 256 / ms / 1e9, ghz, bytes_per_cu / (ms * 1e6 * ghz));
  return 0;
}
int main() {
  const size_t region = (size_t)2 << 20;
  char* buf; CK(hipMalloc(&buf, 8 * region + (1 << 20))); CK(hipMemset(buf, 1, 8 * region + (1 << 20)));
  float* out; CK(hipMalloc(&out, 4 << 20));
  unsigned long long* clk; CK(hipMalloc(&clk, 64));
  if (run<8, 4>(buf, region, clk, out)) return 1;
  if (run<16, 4>(buf, region, clk, out)) return 1;
  if (run<32, 4>(buf, region, clk, out)) return 1;
  if (run<48, 4>(buf, region, clk, out)) return 1;
  if (run<8, 8>(buf, region, clk, out)) return 1;
  if (run<16, 8>(buf, region, clk, out)) return 1;
  if (run<32, 8>(buf, region, clk, out)) return 1;
  return 0;
}
