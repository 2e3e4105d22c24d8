// Building blocks shared by the grouped GEMM kernels (gfx950, wave64, bf16 MFMA 32x32x16, fp32 accumulate).
//
// Vocabulary.  A GEMM tile multiplies a "P" operand (token side) with a "Q" operand (weight side) over a
// contraction index k.  Both live in LDS as BK = 64 deep stages, filled by direct-to-LDS loads
// (global_load_lds_dwordx4: every lane names its own 16 global bytes, the wavefront's 64 pieces land in 1024
// consecutive LDS bytes), so the LDS position of a piece is fixed by (wave, instruction, lane) and swizzling is
// done by choosing WHICH global piece a lane fetches.
//
//   K-major stage : [rows][64 k]   row = 128 B = 8 pieces; piece c of row r sits at c ^ kswz(r).
//                   MFMA operand fragment = one ds_read_b128 per lane (row l%32, pieces 2*ks + l/32).
//   MN-major stage: [64 k][cols]   row = cols*2 B; 32-byte group g of k-row k sits at g ^ (k & 15) (mod groups).
//                   MFMA operand fragment = two ds_read_b64_tr_b16 per lane (the transpose load hands lane i of a
//                   16-lane group column i of a 4 x 16 block whose rows are named by the lanes' addresses).
//
// The MFMA is issued as D[n][m] += Q[n][k] P[k][m]: lane l of the accumulator owns token column m = l % 32 and,
// in register r, feature n = 8*(r/4) + 4*(l/32) + r%4, so four consecutive features (two gate/up pairs) sit in
// one lane and per-token scalars are per-lane.
#pragma once
#include <type_traits>

#include "common.h"

namespace smoe {

constexpr int BK = 64;  // contraction depth of one LDS stage

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

SMOE_DEV void load16_to_lds(const void* g, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)g, (lds_ptr_t)lds_wave_base, 16, 0, 0);
}

SMOE_DEV int kswz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

SMOE_DEV bf16x8 lds_read_b128(const char* p) { return *(const bf16x8*)p; }

SMOE_DEV bf16x8 lds_read_tr2(const char* p0, const char* p1) {
  typedef __attribute__((address_space(3))) s16x4* tr_ptr_t;
  s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)p0);
  s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)p1);
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
  s16x8 r = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, r);
}

// compile-time loop: f(std::integral_constant<int, i>) for i in [0, N); keeps register-array indices static
template <int I, int N, class F>
SMOE_DEV void static_for_impl(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for_impl<I + 1, N>(f);
  }
}
template <int N, class F>
SMOE_DEV void static_for(F&& f) {
  static_for_impl<0, N>(f);
}

SMOE_DEV f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

// ---- tile map ------------------------------------------------------------------------------------------------
// Built on the device from the expert offsets; header[0] = number of token tiles.  Entry i = (expert, first row).
struct TileMap {
  int32_t* header;  // [4]
  int32_t* expert;  // [max_tiles]
  int32_t* row0;    // [max_tiles]
};

static inline int64_t max_token_tiles(int64_t TK, int E, int BM) { return TK / BM + E; }

static inline size_t tile_map_bytes(int64_t TK, int E) {
  // sized for the smallest token tile any kernel uses (64 rows)
  return (size_t)(4 + 2 * max_token_tiles(TK, E, 64)) * sizeof(int32_t);
}

static inline TileMap carve_tile_map(void* ws, int64_t TK, int E, int BM) {
  TileMap t;
  t.header = (int32_t*)ws;
  t.expert = t.header + 4;
  t.row0 = t.expert + max_token_tiles(TK, E, BM);
  return t;
}

// single workgroup of 1024 threads
__global__ void build_tile_map_kernel(const int32_t* __restrict__ off, int E, int BM, TileMap tm);

int launch_build_tile_map(const int32_t* off, int E, int BM, TileMap tm, hipStream_t st);

// XCD-aware linear tile id: workgroups are dealt round-robin to the 8 XCDs, so workgroup b runs on XCD b % 8;
// give every XCD one contiguous range of the tile space so that tiles sharing operands share an L2.
SMOE_DEV int64_t xcd_linear_tile(int64_t total) {
  const int64_t b = blockIdx.x;
  const int64_t per = (total + 7) >> 3;
  const int64_t slot = b >> 3;
  if (slot >= per) return -1;
  const int64_t lin = (b & 7) * per + slot;
  return lin < total ? lin : -1;
}

int launch_ds_finalize(const float* ds_partial, int ncols, const int32_t* sidx, float* ds, int64_t TK, hipStream_t st);

}  // namespace smoe
