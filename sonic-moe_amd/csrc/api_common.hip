// Library-wide pieces of the C ABI: version, thread-local error text, and the tile-map builder that turns the
// expert offsets into a list of token tiles on the device (no host synchronisation anywhere on the hot path).
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "gemm_common.h"

namespace smoe {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

namespace {
std::once_flag g_tuning_once;
Tuning g_tuning = {1, 0, 2, 1, 1, 8, 1};

struct Knob {
  const char* name;
  const char* env;
  int Tuning::*field;
  int lo, hi, def;
};
const Knob g_knobs[] = {
    {"gemm_stream", "SMOE_GEMM_STREAM", &Tuning::gemm_stream, 0, 1, 1},
    {"gemm_stream_grid", "SMOE_GEMM_STREAM_GRID", &Tuning::gemm_stream_grid, 0, 1 << 30, 0},
    {"varlen_k_tile_order", "SMOE_VARLEN_K_TILE_ORDER", &Tuning::varlen_k_tile_order, 0, 2, 2},
    {"dz_stream", "SMOE_DZ_STREAM", &Tuning::dz_stream, 0, 1, 1},
    {"gemm_asm", "SMOE_GEMM_ASM", &Tuning::gemm_asm, 0, 1, 1},
    {"gemm_group_tiles", "SMOE_GEMM_GROUP_TILES", &Tuning::gemm_group_tiles, 1, TILE_GROUP_MAX, 8},
    {"gemm_group_snake", "SMOE_GEMM_GROUP_SNAKE", &Tuning::gemm_group_snake, 0, 1, 1},
};

void read_tuning_env() {
  for (const Knob& k : g_knobs) {
    const char* v = getenv(k.env);
    if (v == nullptr || *v == 0) continue;
    const long x = strtol(v, nullptr, 10);
    g_tuning.*(k.field) = x < k.lo || x > k.hi ? k.def : (int)x;
  }
}
}  // namespace

const Tuning& tuning() {
  std::call_once(g_tuning_once, read_tuning_env);
  return g_tuning;
}

int device_compute_units(int* out) {
  static int cus[64] = {};
  int dev = 0;
  SMOE_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64 || cus[dev] == 0) {
    int n = 0;
    SMOE_HIP_CHECK(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
    if (dev < 0 || dev >= 64) {
      *out = n;
      return SMOE_OK;
    }
    cus[dev] = n;
  }
  *out = cus[dev];
  return SMOE_OK;
}

// order == nullptr: experts are listed 0, 1, ...; otherwise position i of the list holds expert order[i]
__global__ __launch_bounds__(1024) void build_tile_map_kernel(const int32_t* __restrict__ off,
                                                              const int32_t* __restrict__ order, int E, int BM,
                                                              int gmax, int snake, TileMap tm) {
  __shared__ int32_t wave_tot[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int32_t base = 0;
  for (int e0 = 0; e0 < E; e0 += 1024) {
    int e = e0 + tid;
    int32_t lo = 0, cnt = 0;
    if (e < E) {
      if (order != nullptr) e = order[e];
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
    // groups of nearly equal height: the first `taller` of them have one token tile more
    const int32_t ngroups = (tiles + gmax - 1) / gmax;
    const int32_t hbase = ngroups ? tiles / ngroups : 0, taller = ngroups ? tiles % ngroups : 0;
    const int32_t split = taller * (hbase + 1);
    for (int32_t i = 0; i < tiles; i++) {
      tm.expert[start + i] = e;
      tm.row0[start + i] = lo + i * BM;
      int32_t g, first, h;
      if (i < split) {
        h = hbase + 1;
        g = i / h;
        first = g * h;
      } else {
        h = hbase;
        g = (i - split) / h;
        first = split + g * h;
        g += taller;
      }
      tm.group[start + i] = (int32_t)((uint32_t)(start + first) | (uint32_t)h << 24 | (uint32_t)(snake & g & 1) << 31);
    }
    base += tot;
  }
  if (tid == 0) tm.header[0] = base;
}

int launch_build_tile_map(const int32_t* off, const int32_t* order, int E, int BM, TileMap tm, hipStream_t st) {
  const Tuning& tune = tuning();
  hipLaunchKernelGGL(build_tile_map_kernel, dim3(1), dim3(1024), 0, st, off, order, E, BM, tune.gemm_group_tiles,
                     tune.gemm_group_snake, tm);
  SMOE_LAUNCH_CHECK();
  return SMOE_OK;
}

}  // namespace smoe

extern "C" int smoe_version(void) { return 310; }
extern "C" const char* smoe_last_error(void) { return smoe::g_error; }

extern "C" int smoe_set_tuning(const char* name, int value) {
  SMOE_REQUIRE(name != nullptr, SMOE_ERR_INVALID, "set_tuning: null name");
  smoe::tuning();  // the environment is read first, so that it cannot overwrite this call later
  for (const smoe::Knob& k : smoe::g_knobs) {
    if (strcmp(name, k.name) != 0) continue;
    if (value < 0) value = k.def;
    SMOE_REQUIRE(value >= k.lo && value <= k.hi, SMOE_ERR_INVALID, "set_tuning: %s = %d outside [%d, %d]", name, value,
                 k.lo, k.hi);
    smoe::g_tuning.*(k.field) = value;
    return SMOE_OK;
  }
  smoe::set_error("set_tuning: unknown knob '%s'", name);
  return SMOE_ERR_INVALID;
}
