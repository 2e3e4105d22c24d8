// Shared host/device helpers for the gfx950 kernels of the MoE-layer hot path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/sonicmoe_hip.h"

namespace smoe {

// ---- error reporting -------------------------------------------------------------------------------------
void set_error(const char* fmt, ...);  // thread-local message behind smoe_last_error()

#define SMOE_REQUIRE(cond, code, ...)    \
  do {                                   \
    if (!(cond)) {                       \
      ::smoe::set_error(__VA_ARGS__);    \
      return (code);                     \
    }                                    \
  } while (0)

#define SMOE_HIP_CHECK(expr)                                                                  \
  do {                                                                                        \
    hipError_t _e = (expr);                                                                   \
    if (_e != hipSuccess) {                                                                   \
      ::smoe::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
      return SMOE_ERR_HIP;                                                                    \
    }                                                                                         \
  } while (0)

#define SMOE_LAUNCH_CHECK() SMOE_HIP_CHECK(hipGetLastError())

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// The GEMM kernels move operands in 16-byte pieces (8 bf16): base pointers must be 16-byte aligned and row / expert
// strides multiples of 8 elements.  Null pointers (optional arguments) pass.
static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
static inline bool stride8(int64_t s) { return s % 8 == 0; }
#define SMOE_REQUIRE_ALIGNED(who, ...)                                                                       \
  do {                                                                                                       \
    const void* _ptrs[] = {__VA_ARGS__};                                                                     \
    for (const void* _p : _ptrs)                                                                             \
      SMOE_REQUIRE(::smoe::aligned16(_p), SMOE_ERR_UNSUPPORTED, "%s: tensor pointers must be 16-byte aligned", who); \
  } while (0)

// ---- device-side types -----------------------------------------------------------------------------------
// The 16-bit element type of the tensors the GEMM-side kernels read and write (x, the weights, z, y1, y2, dout, dz,
// ...).  The library is built twice from the same sources: with bf16 elements (libsonicmoe_hip.so) and, with
// SMOE_ELEM_F16 defined, with fp16 elements (libsonicmoe_hip_f16.so); both export the same entry points.  Comments that
// say "bf16" about such a tensor mean this element type.  Kernels that take a smoe_dtype code (top-k, switch loss,
// token rounding) do not depend on it.
#ifdef SMOE_ELEM_F16
typedef _Float16 elem_t;
#define SMOE_ELEM_ASM "f16"  // suffix of the matrix instructions' mnemonics
#else
typedef __bf16 elem_t;
#define SMOE_ELEM_ASM "bf16"
#endif
typedef __attribute__((__vector_size__(8 * sizeof(elem_t)))) elem_t elemx8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

#define SMOE_DEV static __device__ __forceinline__

// bf16 <-> fp32.  fp32 -> bf16 is the hardware conversion (v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN);
// written out in integer arithmetic it costs ten instructions and a divergent branch per value, which made the GEMM
// epilogues instruction-bound.
SMOE_DEV float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
SMOE_DEV uint32_t f32_to_bf16_bits(float f) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{f, 0.f}, bf16x2_t)) & 0xffffu;
}

// element type <-> fp32, two elements per 32-bit word (lo = the lower address); fp32 -> element rounds to nearest even
SMOE_DEV uint32_t pack_elem2(float lo, float hi) {
  typedef elem_t elemx2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, elemx2_t));
}
#ifdef SMOE_ELEM_F16
SMOE_DEV float elem_lo(uint32_t w) {
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  return (float)__builtin_bit_cast(f16x2_t, w)[0];
}
SMOE_DEV float elem_hi(uint32_t w) {
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  return (float)__builtin_bit_cast(f16x2_t, w)[1];
}
#else
SMOE_DEV float elem_lo(uint32_t w) { return __uint_as_float(w << 16); }
SMOE_DEV float elem_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
#endif
SMOE_DEV float elem_bits_to_f32(uint32_t h) { return elem_lo(h); }

// 1 / (1 + e^-x) with the hardware reciprocal (1 ulp): a correctly rounded division is a dozen instructions per value
SMOE_DEV float fast_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

}  // namespace smoe
