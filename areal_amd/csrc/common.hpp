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

// ---------------------------------------------------------------------------------------
// Cross-lane movement inside a 64-lane wave without the LDS crossbar. A ds_bpermute shuffle goes
// through the CU's one LDS unit, which every wave of the CU shares: a block-end reduction of a few
// values by sixteen resident waves queues there for microseconds. DPP operands (data-parallel
// primitives: a VALU instruction reads its source from another lane of the same row of 16) and
// v_readlane stay inside the SIMD.
// ---------------------------------------------------------------------------------------
constexpr int DPP_ROW_SHL = 0x100;  // + n (1..15): lane i reads lane i + n of its row
constexpr int DPP_ROW_SHR = 0x110;  // + n: lane i reads lane i - n of its row
constexpr int DPP_ROW_ROR = 0x120;  // + n: lane i reads lane (i - n) mod 16 of its row
constexpr int DPP_WAVE_SHR1 = 0x138;  // lane i reads lane i - 1 of the wave (lane 0 has no source)

// x of the lane CTRL names; a lane whose source falls outside its row keeps `old`.
template <int CTRL>
DEVI int dpp_move(int old, int x) { return __builtin_amdgcn_update_dpp(old, x, CTRL, 0xf, 0xf, false); }
template <int CTRL>
DEVI unsigned dpp_move(unsigned old, unsigned x) { return (unsigned)dpp_move<CTRL>((int)old, (int)x); }
template <int CTRL>
DEVI float dpp_move(float old, float x) {
  return __builtin_bit_cast(float, dpp_move<CTRL>(__builtin_bit_cast(int, old), __builtin_bit_cast(int, x)));
}
template <int CTRL>
DEVI double dpp_move(double old, double x) {
  const int2 o = __builtin_bit_cast(int2, old), v = __builtin_bit_cast(int2, x);
  int2 r;
  r.x = dpp_move<CTRL>(o.x, v.x);
  r.y = dpp_move<CTRL>(o.y, v.y);
  return __builtin_bit_cast(double, r);
}
template <int CTRL>
DEVI long long dpp_move(long long old, long long x) {
  return __builtin_bit_cast(long long, dpp_move<CTRL>(__builtin_bit_cast(double, old), __builtin_bit_cast(double, x)));
}

template <int CTRL>
DEVI unsigned long long dpp_move(unsigned long long old, unsigned long long x) {
  return (unsigned long long)dpp_move<CTRL>((long long)old, (long long)x);
}
template <int CTRL>
DEVI long dpp_move(long old, long x) { return (long)dpp_move<CTRL>((long long)old, (long long)x); }

// x of lane `lane` (a constant) in every lane.
DEVI int lane_value(int x, int lane) { return __builtin_amdgcn_readlane(x, lane); }
DEVI unsigned lane_value(unsigned x, int lane) { return (unsigned)__builtin_amdgcn_readlane((int)x, lane); }
DEVI float lane_value(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}
DEVI double lane_value(double x, int lane) {
  const int2 v = __builtin_bit_cast(int2, x);
  int2 r;
  r.x = __builtin_amdgcn_readlane(v.x, lane);
  r.y = __builtin_amdgcn_readlane(v.y, lane);
  return __builtin_bit_cast(double, r);
}
DEVI long long lane_value(long long x, int lane) {
  return __builtin_bit_cast(long long, lane_value(__builtin_bit_cast(double, x), lane));
}
DEVI unsigned long long lane_value(unsigned long long x, int lane) {
  return (unsigned long long)lane_value((long long)x, lane);
}
DEVI long lane_value(long x, int lane) { return (long)lane_value((long long)x, lane); }

// Wave-wide (64 lanes) reduction with a commutative, associative op; the result in every lane.
// Four rotations leave each row's result in all of its lanes; the four rows are then combined
// from lanes 0, 16, 32 and 48 in that order, so the result does not depend on the calling lane.
template <typename T, typename Op>
DEVI T wave_reduce(T v, Op op) {
  v = op(v, dpp_move<DPP_ROW_ROR + 8>(v, v));
  v = op(v, dpp_move<DPP_ROW_ROR + 4>(v, v));
  v = op(v, dpp_move<DPP_ROW_ROR + 2>(v, v));
  v = op(v, dpp_move<DPP_ROW_ROR + 1>(v, v));
  return op(op(lane_value(v, 0), lane_value(v, 16)), op(lane_value(v, 32), lane_value(v, 48)));
}
// The first half of wave_reduce alone: each row's result in all 16 lanes of the row (lanes 0, 16,
// 32 and 48 then hold the wave's four partial results).
template <typename T, typename Op>
DEVI T row_reduce(T v, Op op) {
  v = op(v, dpp_move<DPP_ROW_ROR + 8>(v, v));
  v = op(v, dpp_move<DPP_ROW_ROR + 4>(v, v));
  v = op(v, dpp_move<DPP_ROW_ROR + 2>(v, v));
  v = op(v, dpp_move<DPP_ROW_ROR + 1>(v, v));
  return v;
}
// Inclusive prefix scan over the wave's 64 lanes with an associative, commutative op: inside each
// row of 16 through DPP shifts (a lane without a source takes the identity), then the results of
// the rows to the left (lanes 15, 31, 47) are folded in.
template <typename T, typename Op>
DEVI T wave_inclusive_scan(T v, T identity, Op op) {
  v = op(v, dpp_move<DPP_ROW_SHR + 1>(identity, v));
  v = op(v, dpp_move<DPP_ROW_SHR + 2>(identity, v));
  v = op(v, dpp_move<DPP_ROW_SHR + 4>(identity, v));
  v = op(v, dpp_move<DPP_ROW_SHR + 8>(identity, v));
  const T t0 = lane_value(v, 15), t1 = lane_value(v, 31), t2 = lane_value(v, 47);
  const int row = (threadIdx.x & 63) >> 4;
  T left = identity;
  if (row >= 1) left = t0;
  if (row >= 2) left = op(left, t1);
  if (row >= 3) left = op(left, t2);
  return op(left, v);
}
// The value of the lane before (lane 0: the identity).
template <typename T>
DEVI T wave_shift_up(T v, T identity) { return dpp_move<DPP_WAVE_SHR1>(identity, v); }

template <typename T>
DEVI T wave_sum(T v) { return wave_reduce(v, [](T a, T b) { return a + b; }); }
DEVI float wave_max(float v) { return wave_reduce(v, [](float a, float b) { return fmaxf(a, b); }); }
DEVI float wave_min(float v) { return wave_reduce(v, [](float a, float b) { return fminf(a, b); }); }

// #{i in [0, n) : ends[i] <= x} for a non-decreasing array, by one wave: every round probes 64
// positions and keeps the gap after the last probe that is <= x.
template <class I>
DEVI int wave_count_le(const I* ends, int n, int64_t x, int lane) {
  int base = 0, len = n;
  while (len > 0) {
    const int step = (len + 63) >> 6;
    const int idx = base + lane * step;
    const bool le = (idx < base + len) && ((int64_t)ends[idx] <= x);
    const int cnt = __popcll(__builtin_amdgcn_ballot_w64(le));
    if (cnt == 0) break;  // ends[base] > x
    const int hit = base + (cnt - 1) * step;  // last probe <= x
    const int lim = base + len;
    base = hit + 1;
    len = step - 1;
    if (base + len > lim) len = lim - base;
  }
  return base;
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
DEVI float wave_stat_min(float v) { return wave_reduce(v, [](float a, float b) { return stat_min(a, b); }); }
DEVI float wave_stat_max(float v) { return wave_reduce(v, [](float a, float b) { return stat_max(a, b); }); }

// VEC = 4 needs every per-token fp32 array 16-byte aligned and every byte array 4-byte aligned
// (null pointers pass); it pays once the batch gives every CU a block of four-token threads.
static inline bool aligned_to(const void* p, uintptr_t a) { return p == nullptr || ((uintptr_t)p & (a - 1)) == 0; }
constexpr int64_t VEC4_MIN_TOKENS = (int64_t)4 * 256 * 256;
