// What would a combine fused into the down-projection epilogue cost?  The epilogue would add s * y2[m][:] into
// o[token(m)][:] with atomics (a token's K rows come from K different expert tiles on different XCDs).  This times the
// atomic traffic alone, in the pattern the epilogue would produce (256-byte contiguous pieces of scattered rows).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); return 1;} }while(0)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// one wave per grouped row m: MODE 0 fp32 atomics into (T,H) fp32, MODE 1 packed-bf16 atomics into (T,H) bf16,
// MODE 2 plain bf16 stores into (TK,H) (the y2 the unfused path writes)
template <int MODE>
__global__ __launch_bounds__(256) void k(float* of, uint32_t* ob, uint16_t* y2, const int* gidx, int64_t TK, int H) {
  const int lane = threadIdx.x & 63;
  const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= TK) return;
  const int t = gidx[m];
  if (MODE == 0) {
    float* row = of + (int64_t)t * H;
    for (int c = lane; c < H; c += 64) unsafeAtomicAdd(row + c, 1.0f + c);
  } else if (MODE == 1) {
    uint32_t* row = ob + (int64_t)t * (H / 2);
    for (int c = lane; c < H / 2; c += 64) {
      bf16x2_t v = {(__bf16)1.0f, (__bf16)2.0f};
      __builtin_amdgcn_global_atomic_fadd_v2bf16((__attribute__((address_space(1))) bf16x2_t*)(row + c), v);
    }
  } else {
    uint4* row = (uint4*)(y2 + m * H);
    for (int c = lane; c < H / 8; c += 64) row[c] = uint4{1, 2, 3, 4};
  }
}
int main() {
  const int64_t T = 32768, K = 8, TK = T * K; const int H = 4096;
  float* of; uint32_t* ob; uint16_t* y2; int* gidx;
  CK(hipMalloc(&of, T * H * 4)); CK(hipMalloc(&ob, T * H * 2)); CK(hipMalloc(&y2, TK * H * 2)); CK(hipMalloc(&gidx, TK * 4));
  int* h = (int*)malloc(TK * 4);
  // expert-sorted order: row m of expert e; a token's K rows lie in K different experts => scattered
  for (int64_t m = 0; m < TK; m++) h[m] = (int)((m * 2654435761ull) % T);
  CK(hipMemcpy(gidx, h, TK * 4, hipMemcpyHostToDevice));
  CK(hipMemset(of, 0, T * H * 4)); CK(hipMemset(ob, 0, T * H * 2));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const char* names[3] = {"fp32 atomics into (T,H) fp32 ", "pk-bf16 atomics into (T,H) bf16", "plain bf16 stores of (TK,H) y2 "};
  for (int mode = 0; mode < 3; mode++) {
    for (int rep = 0; rep < 3; rep++) {
      CK(hipEventRecord(e0));
      if (mode == 0) k<0><<<TK / 4, 256>>>(of, ob, y2, gidx, TK, H);
      if (mode == 1) k<1><<<TK / 4, 256>>>(of, ob, y2, gidx, TK, H);
      if (mode == 2) k<2><<<TK / 4, 256>>>(of, ob, y2, gidx, TK, H);
      CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1));
      printf("%s: %.3f ms\n", names[mode], ms);
    }
  }
  float chk; CK(hipMemcpy(&chk, of, 4, hipMemcpyDeviceToHost));
  printf("check o[0][0] = %.1f (3 launches x multiplicity of token 0)\n", chk);
  return 0;
}
