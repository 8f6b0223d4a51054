// Logits-in label log-probabilities and entropy (forward and backward), one workgroup per row.
//
// Follows areal/utils/functional/vocab_parallel.py:16-30: log_softmax(logits.float() / T),
// gather at the label, entropy = -sum p log p; row chunking (:42-82) does not change values.
// The forward reads each logit once (online max / sum-exp); the backward reads it once more
// and writes d loss / d logits in the dtype of the logits:
//     d lp_label / d x_j = (1[j == label] - p_j) / T
//     d entropy  / d x_j = -p_j (log p_j + entropy) / T
#include "common.hpp"

namespace {

constexpr int ROW_THREADS = 256;
constexpr float LOG2E_F = 1.4426950408889634f;
constexpr float LN2_F = 0.6931471805599453f;

// Vector loads and stores carry the non-temporal hint: every logit is read once per kernel (and every
// dlogit written once), and a plain read of a [4096, 151936] bf16 array in this access pattern
// measures 6.15 TB/s without the hint, 7.04 TB/s with it.
template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int VEC = 4;
  static DEVI float load(const float* p) { return *p; }
  static DEVI void loadv(const float* p, float (&o)[4]) {
    const f32x4 v = __builtin_nontemporal_load((const f32x4*)p);
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
  }
  static DEVI void store(float* p, float v) { *p = v; }
  static DEVI void storev(float* p, const float (&o)[4]) {
    f32x4 v = {o[0], o[1], o[2], o[3]};
    __builtin_nontemporal_store(v, (f32x4*)p);
  }
};
template <> struct Elem<u16> {  // bf16 bit patterns
  static constexpr int VEC = 8;
  static DEVI float load(const u16* p) { return bf16_bits_to_f32(*p); }
  static DEVI void loadv(const u16* p, float (&o)[8]) {
    const u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __builtin_bit_cast(float, v[i] << 16);
      o[2 * i + 1] = __builtin_bit_cast(float, v[i] & 0xffff0000u);
    }
  }
  static DEVI void store(u16* p, float v) { *p = f32_to_bf16_bits(v); }
  static DEVI void storev(u16* p, const float (&o)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v[i] = (uint32_t)f32_to_bf16_bits(o[2 * i]) | ((uint32_t)f32_to_bf16_bits(o[2 * i + 1]) << 16);
    __builtin_nontemporal_store(v, (u32x4*)p);
  }
};

struct Online {
  float m, s, q;  // max of z2 = x*c2, sum 2^(z2-m), sum (z2-m) 2^(z2-m)
};
DEVI void online_merge(Online& a, const Online& b) {
  const float m = fmaxf(a.m, b.m);
  if (!(m > neg_inf())) return;
  float s = 0.f, q = 0.f;
  if (a.m > neg_inf()) { const float d = a.m - m, al = fast_exp2(d); s += al * a.s; q += al * fmaf(d, a.s, a.q); }
  if (b.m > neg_inf()) { const float d = b.m - m, al = fast_exp2(d); s += al * b.s; q += al * fmaf(d, b.s, b.q); }
  a.m = m; a.s = s; a.q = q;
}
// x: raw logits; the exponents are z2 = x * c2 (c2 > 0). The running maximum is kept as the
// rounded product of the largest logit and every exponent is taken relative to it with one fused
// multiply-subtract, as the backward evaluates them against lse2.
template <int N>
DEVI void online_add(Online& st, const float (&x)[N], float c2) {
  float xm = x[0];
#pragma unroll
  for (int i = 1; i < N; ++i) xm = fmaxf(xm, x[i]);
  const float vm = xm * c2;
  if (vm > st.m) {
    if (st.m > neg_inf()) {
      const float d = st.m - vm, al = fast_exp2(d);
      st.q = al * fmaf(d, st.s, st.q);
      st.s = al * st.s;
    }
    st.m = vm;
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float t = fmaf(x[i], c2, -st.m);
    const float e = fast_exp2(t);
    st.s += e;
    st.q = fmaf(t, e, st.q);
  }
}

DEVI Online block_merge(Online st, Online* smem) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Online other;
    other.m = __shfl_xor(st.m, o, 64); other.s = __shfl_xor(st.s, o, 64);
    other.q = __shfl_xor(st.q, o, 64);
    online_merge(st, other);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) smem[w] = st;
  __syncthreads();
  Online r = smem[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) online_merge(r, smem[i]);
  return r;
}

// lse2[t] = max + log2(sum) in base-2 units of z2 = x * inv_temp * log2(e).
template <typename T, bool VECTOR>
__global__ __launch_bounds__(ROW_THREADS) void rows_fwd_kernel(const T* __restrict__ logits,
                                                               int64_t ld,
                                                               const int64_t* __restrict__ labels,
                                                               int V, float inv_temp,
                                                               float* __restrict__ logprobs,
                                                               float* __restrict__ entropy,
                                                               float* __restrict__ lse2_out) {
  __shared__ Online smem[ROW_THREADS / 64];
  const int64_t row = blockIdx.x;
  const T* x = logits + row * ld;
  const float c2 = inv_temp * LOG2E_F;
  Online st{neg_inf(), 0.f, 0.f};
  constexpr int VEC = Elem<T>::VEC;
  if (VECTOR) {
    for (int v0 = threadIdx.x * VEC; v0 < V; v0 += ROW_THREADS * VEC) {
      float z[VEC];
      Elem<T>::loadv(x + v0, z);
      online_add(st, z, c2);
    }
  } else {
    for (int v = threadIdx.x; v < V; v += ROW_THREADS) {
      float z[1] = {Elem<T>::load(x + v)};
      online_add(st, z, c2);
    }
  }
  const Online r = block_merge(st, smem);
  if (threadIdx.x == 0) {
    const float log2s = fast_log2(r.s);
    const float lse2 = r.m + log2s;
    const int64_t lab = labels[row];
    float lp = 0.f;
    if (lab >= 0 && lab < V) {
      // the label's exponent as the sums saw it: relative to the running maximum, by one fused
      // multiply-subtract
      const float tl = fmaf(Elem<T>::load(x + lab), c2, -r.m);
      lp = fminf((tl - log2s) * LN2_F, 0.f);
    }
    if (logprobs) logprobs[row] = lp;
    if (entropy) entropy[row] = (log2s - r.q / r.s) * LN2_F;
    if (lse2_out) lse2_out[row] = lse2;
  }
}

template <typename T, bool VECTOR>
__global__ __launch_bounds__(ROW_THREADS) void rows_bwd_kernel(
    const T* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels, int V,
    float inv_temp, const float* __restrict__ lse2, const float* __restrict__ entropy,
    const float* __restrict__ grad_lp, const float* __restrict__ grad_ent, T* __restrict__ dlogits,
    int64_t ldd) {
  const int64_t row = blockIdx.x;
  const T* x = logits + row * ld;
  T* d = dlogits + row * ldd;
  const float c2 = inv_temp * LOG2E_F;
  const float l2 = lse2[row];
  const float glp = (grad_lp ? grad_lp[row] : 0.f) * inv_temp;
  const float gen = (grad_ent ? grad_ent[row] : 0.f) * inv_temp;
  const float ent = (grad_ent ? entropy[row] : 0.f);
  const int64_t lab64 = labels[row];
  const int lab = (lab64 >= 0 && lab64 < V) ? (int)lab64 : -1;
  constexpr int VEC = Elem<T>::VEC;
  if (VECTOR) {
    for (int v0 = threadIdx.x * VEC; v0 < V; v0 += ROW_THREADS * VEC) {
      float z[VEC];
      Elem<T>::loadv(x + v0, z);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float t = fmaf(z[i], c2, -l2);
        const float p = fast_exp2(t);
        float g = -p * glp;
        if (v0 + i == lab) g += glp;
        if (grad_ent) g -= gen * p * (t * LN2_F + ent);
        z[i] = g;
      }
      Elem<T>::storev(d + v0, z);
    }
  } else {
    for (int v = threadIdx.x; v < V; v += ROW_THREADS) {
      const float t = fmaf(Elem<T>::load(x + v), c2, -l2);
      const float p = fast_exp2(t);
      float g = -p * glp;
      if (v == lab) g += glp;
      if (grad_ent) g -= gen * p * (t * LN2_F + ent);
      Elem<T>::store(d + v, g);
    }
  }
}

template <typename T>
int launch_rows_fwd(const void* logits, int64_t ld, const int64_t* labels, int64_t T_, int64_t V,
                    float inv_temp, float* lp, float* ent, float* lse2, hipStream_t stream) {
  constexpr int VEC = Elem<T>::VEC;
  const bool vec = (V % VEC == 0) && (ld % VEC == 0) && (((uintptr_t)logits & 15) == 0);
  if (vec)
    hipLaunchKernelGGL((rows_fwd_kernel<T, true>), dim3((unsigned)T_), dim3(ROW_THREADS), 0, stream,
                       (const T*)logits, ld, labels, (int)V, inv_temp, lp, ent, lse2);
  else
    hipLaunchKernelGGL((rows_fwd_kernel<T, false>), dim3((unsigned)T_), dim3(ROW_THREADS), 0,
                       stream, (const T*)logits, ld, labels, (int)V, inv_temp, lp, ent, lse2);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

template <typename T>
int launch_rows_bwd(const void* logits, int64_t ld, const int64_t* labels, int64_t T_, int64_t V,
                    float inv_temp, const float* lse2, const float* ent, const float* glp,
                    const float* gent, void* dlogits, int64_t ldd, hipStream_t stream) {
  constexpr int VEC = Elem<T>::VEC;
  const bool vec = (V % VEC == 0) && (ld % VEC == 0) && (ldd % VEC == 0) &&
                   (((uintptr_t)logits & 15) == 0) && (((uintptr_t)dlogits & 15) == 0);
  if (vec)
    hipLaunchKernelGGL((rows_bwd_kernel<T, true>), dim3((unsigned)T_), dim3(ROW_THREADS), 0, stream,
                       (const T*)logits, ld, labels, (int)V, inv_temp, lse2, ent, glp, gent,
                       (T*)dlogits, ldd);
  else
    hipLaunchKernelGGL((rows_bwd_kernel<T, false>), dim3((unsigned)T_), dim3(ROW_THREADS), 0,
                       stream, (const T*)logits, ld, labels, (int)V, inv_temp, lse2, ent, glp, gent,
                       (T*)dlogits, ldd);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // namespace

extern "C" {

// dtype: 0 = fp32 logits, 1 = bf16 logits. logits [T, V] with row pitch ld (elements).
// Outputs fp32 [T]: logprobs, entropy (nullable), lse2 (nullable; log-sum-exp in base-2 units,
// the only state the backward needs besides entropy).
int areal_logits_logprobs_entropy_fwd(const void* logits, int dtype, int64_t ld,
                                      const int64_t* labels, int64_t T, int64_t V,
                                      float inv_temperature, float* logprobs, float* entropy,
                                      float* lse2, hipStream_t stream) {
  if (T < 0 || V <= 0 || ld < V || !(inv_temperature > 0.f)) return AREAL_ERR_BAD_ARG;
  if (T == 0) return AREAL_OK;
  if (!logits || !labels) return AREAL_ERR_BAD_ARG;
  if (V > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  if (dtype == 0)
    return launch_rows_fwd<float>(logits, ld, labels, T, V, inv_temperature, logprobs, entropy, lse2,
                                  stream);
  if (dtype == 1)
    return launch_rows_fwd<u16>(logits, ld, labels, T, V, inv_temperature, logprobs, entropy, lse2,
                                stream);
  return AREAL_ERR_BAD_ARG;
}

// dlogits [T, V] (same dtype as logits, row pitch ldd) = grad_logprobs * d lp / d logits
// + grad_entropy * d entropy / d logits; either upstream gradient may be null.
int areal_logits_logprobs_entropy_bwd(const void* logits, int dtype, int64_t ld,
                                      const int64_t* labels, int64_t T, int64_t V,
                                      float inv_temperature, const float* lse2,
                                      const float* entropy, const float* grad_logprobs,
                                      const float* grad_entropy, void* dlogits, int64_t ldd,
                                      hipStream_t stream) {
  if (T < 0 || V <= 0 || ld < V || ldd < V || !(inv_temperature > 0.f)) return AREAL_ERR_BAD_ARG;
  if (T == 0) return AREAL_OK;
  if (!logits || !labels || !lse2 || !dlogits) return AREAL_ERR_BAD_ARG;
  if (grad_entropy != nullptr && entropy == nullptr) return AREAL_ERR_BAD_ARG;
  if (V > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  if (dtype == 0)
    return launch_rows_bwd<float>(logits, ld, labels, T, V, inv_temperature, lse2, entropy,
                                  grad_logprobs, grad_entropy, dlogits, ldd, stream);
  if (dtype == 1)
    return launch_rows_bwd<u16>(logits, ld, labels, T, V, inv_temperature, lse2, entropy,
                                grad_logprobs, grad_entropy, dlogits, ldd, stream);
  return AREAL_ERR_BAD_ARG;
}

}  // extern "C"
