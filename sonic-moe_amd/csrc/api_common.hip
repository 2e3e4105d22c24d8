// Library-wide pieces of the C ABI: version, thread-local error text, and the tile-map builder that turns the
// expert offsets into a list of token tiles on the device (no host synchronisation anywhere on the hot path).
#include <stdarg.h>

#include "gemm_common.h"

namespace smoe {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

__global__ __launch_bounds__(1024) void build_tile_map_kernel(const int32_t* __restrict__ off, int E, int BM,
                                                              TileMap tm) {
  __shared__ int32_t wave_tot[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int32_t base = 0;
  for (int e0 = 0; e0 < E; e0 += 1024) {
    const int e = e0 + tid;
    int32_t lo = 0, cnt = 0;
    if (e < E) {
      lo = off[e];
      cnt = off[e + 1] - lo;
    }
    const int32_t tiles = (cnt + BM - 1) / BM;
    int32_t v = tiles;
    for (int d = 1; d < 64; d <<= 1) {
      int32_t o = __shfl_up(v, d, 64);
      if (lane >= d) v += o;
    }
    __syncthreads();  // wave_tot reuse across iterations
    if (lane == 63) wave_tot[wave] = v;
    __syncthreads();
    int32_t wbase = 0, tot = 0;
    for (int w = 0; w < 16; w++) {
      if (w < wave) wbase += wave_tot[w];
      tot += wave_tot[w];
    }
    const int32_t start = base + wbase + v - tiles;
    for (int32_t i = 0; i < tiles; i++) {
      tm.expert[start + i] = e;
      tm.row0[start + i] = lo + i * BM;
    }
    base += tot;
  }
  if (tid == 0) tm.header[0] = base;
}

int launch_build_tile_map(const int32_t* off, int E, int BM, TileMap tm, hipStream_t st) {
  hipLaunchKernelGGL(build_tile_map_kernel, dim3(1), dim3(1024), 0, st, off, E, BM, tm);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

}  // namespace smoe

extern "C" int smoe_version(void) { return 220; }
extern "C" const char* smoe_last_error(void) { return smoe::g_error; }
