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

// ---------------------------------------------------------------------------------------
// Streaming per-token kernels (losses, statistics)
// ---------------------------------------------------------------------------------------
// Per-token arrays are moved VEC elements per thread and access: VEC = 4 takes 16-byte loads and
// stores for the fp32 arrays and 4-byte ones for the byte masks (every array 16-byte, resp.
// 4-byte, aligned; the host checks), VEC = 1 is the element-wise form for anything else and for
// the last n % 4 tokens. Plain loads and stores: a micro-batch's per-token arrays (a few hundred MB
// at most) come from and go to kernels next to this one through the 256 MB memory-side cache,
// which accesses with the non-temporal hint bypass (measured on 4 Mi tokens: 5.0 TB/s with the
// hint, 6.5 to 7.5 without).
template <int VEC>
DEVI void load_f32(const float* p, int64_t t, float (&v)[VEC]) {
  if (p == nullptr) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = 0.f;
  } else if (VEC == 4) {
    const f32x4 x = *(const f32x4*)(p + t);
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = x[i];
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = p[t + i];
  }
}
template <int VEC>
DEVI void load_mask(const uint8_t* p, int64_t t, bool (&v)[VEC]) {
  if (VEC == 4) {
    const uint32_t x = *(const uint32_t*)(p + t);
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = ((x >> (8 * i)) & 0xffu) != 0;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = p[t + i] != 0;
  }
}
template <int VEC>
DEVI void store_f32(float* p, int64_t t, const float (&v)[VEC]) {
  if (p == nullptr) return;
  if (VEC == 4) {
    const f32x4 x = {v[0], v[1], v[2], v[3]};
    *(f32x4*)(p + t) = x;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[t + i] = v[i];
  }
}
template <int VEC>
DEVI void store_mask(uint8_t* p, int64_t t, const bool (&v)[VEC]) {
  if (p == nullptr) return;
  if (VEC == 4) {
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) x |= (v[i] ? 1u : 0u) << (8 * i);
    *(uint32_t*)(p + t) = x;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[t + i] = v[i];
  }
}


// Running extremes of logged statistics with torch.min / torch.max's NaN propagation (the sign of a
// zero does not matter there): IEEE 754-2019 minimum / maximum, one instruction each.
DEVI float stat_min(float a, float b) { return __builtin_elementwise_minimum(a, b); }
DEVI float stat_max(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// VEC = 4 needs every per-token fp32 array 16-byte aligned and every byte array 4-byte aligned
// (null pointers pass); it pays once the batch gives every CU a block of four-token threads.
static inline bool aligned_to(const void* p, uintptr_t a) { return p == nullptr || ((uintptr_t)p & (a - 1)) == 0; }
constexpr int64_t VEC4_MIN_TOKENS = (int64_t)4 * 256 * 256;
