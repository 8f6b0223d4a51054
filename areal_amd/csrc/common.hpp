// Shared device helpers for the gfx950 kernels of the RL training hot path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define DEVI __device__ __forceinline__

typedef unsigned short u16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Error codes returned by every extern "C" entry point (0 = success).
enum ArealStatus : int {
  AREAL_OK = 0,
  AREAL_ERR_BAD_ARG = -1,        // null pointer, negative size, unsupported flag
  AREAL_ERR_ALIGNMENT = -2,      // pointer or leading dimension not 16-byte aligned
  AREAL_ERR_WORKSPACE = -3,      // workspace smaller than *_workspace_bytes()
  AREAL_ERR_LAUNCH = -4,         // hipGetLastError() != hipSuccess after a launch
  AREAL_ERR_UNSUPPORTED = -5,    // shape outside what the kernels implement
};

#define AREAL_CHECK_LAUNCH()                                   \
  do {                                                         \
    if (hipGetLastError() != hipSuccess) return AREAL_ERR_LAUNCH; \
  } while (0)

static inline int64_t round_up_i64(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
static inline int64_t ceil_div_i64(int64_t x, int64_t m) { return (x + m - 1) / m; }

// Hardware base-2 exponential (v_exp_f32). About 1 ulp; flushes denormal results.
DEVI float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
DEVI float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

DEVI float neg_inf() { return -__builtin_inff(); }
DEVI float pos_inf() { return __builtin_inff(); }

// Round-to-nearest-even float -> bf16 bit pattern.
DEVI u16 f32_to_bf16_bits(float f) {
  __bf16 h = (__bf16)f;
  return __builtin_bit_cast(u16, h);
}
// Two floats to a pair of bf16 in one register (lo in bits 0-15): one v_cvt_pk_bf16_f32, the same
// round-to-nearest-even as the scalar conversion.
typedef float f32x2_cvt __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_cvt __attribute__((ext_vector_type(2)));
DEVI uint32_t pack_bf16x2(float lo, float hi) {
  const bf16x2_cvt h = __builtin_convertvector(f32x2_cvt{lo, hi}, bf16x2_cvt);
  return __builtin_bit_cast(uint32_t, h);
}
DEVI float bf16_bits_to_f32(u16 b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// Wave-wide (64 lanes) reductions through cross-lane shuffles.
template <typename T>
DEVI T wave_sum(T v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
DEVI float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
DEVI float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}
