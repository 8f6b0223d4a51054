// PPO / GRPO / CISPO actor loss with rejection sampling (IcePop ratio bounds, KPop binary KL,
// k1/k2/k3 estimators), token and sequence level, forward and closed-form backward.
//
// Follows areal/utils/functional/functional.py: apply_rejection_sampling (:185-437),
// compute_binary_kl_divergence (:440-449), ppo_actor_loss_fn (:452-596), cispo_loss_fn
// (:678-793), _compute_sequence_level_ratio_and_advantages (:56-149) and
// KLEstimator._compute_approx_kl (areal/utils/data.py:1662-1698).
//
// All per-token arithmetic is fp32 and is written operation by operation in the order of the
// reference's tensor expressions (this file is compiled with -ffp-contract=off), so that the
// boolean outputs agree with a CPU evaluation except where exp/log differ in their last bit.
// Sums use fp64 block partials reduced in a fixed order: results are run-to-run identical.
#include "common.hpp"

#include <mutex>

namespace {

constexpr int LOSS_THREADS = 256;
constexpr int MAX_LOSS_BLOCKS = 2048;
constexpr int FINAL_THREADS = 512;  // loss_finalize_kernel: 4 block partials per thread

enum { METRIC_RATIO = 0, METRIC_K1 = 1, METRIC_K2 = 2, METRIC_K3 = 3, METRIC_BINARY_KL = 4 };
enum { AGG_SUM = 0, AGG_MEAN = 1, AGG_MAX = 2 };
enum { LOSS_NONE = -1, LOSS_PPO = 0, LOSS_CISPO = 1 };

struct LossCfg {
  int loss_kind;       // LOSS_*
  float clip_lo;       // 1 - eps_clip (rounded from double on the host)
  float clip_hi;       // 1 + eps_clip_higher
  int has_c_clip;
  float c_clip;
  int seq_is;          // importance_sampling_level == "sequence"
  int rs_enabled;
  int rs_seq_level;    // rejection_sampling.level == "sequence"
  int rs_clamp;        // action == "clamp"
  int rs_metric;       // METRIC_*
  int rs_agg;          // AGG_*
  float rs_upper;
  int rs_has_lower;
  float rs_lower;
};

struct LossIO {
  const float* lp;      // current policy log-probs (null when loss_kind == LOSS_NONE)
  const float* prox;
  const float* old;     // may be null when !rs_enabled
  const float* adv;
  const uint8_t* mask;  // bool loss mask (pre rejection)
  const int32_t* cu;    // [n_seqs + 1] or null
  int64_t n;
  int n_seqs;
  int64_t uniform_len;  // > 0: sequence s covers [s*uniform_len, (s+1)*uniform_len)
  // per-sequence inputs produced by the segmented kernels
  const float* seq_rs;    // [n_seqs][2]: {in_bounds (0/1), uniform weight}
  const float* seq_is;    // [n_seqs][4]: {ratio_s, adv_mean_s, sum_w_s, 1/count_s}
  // outputs (any may be null)
  float* dlp;             // d(loss_sum)/dlp, not yet divided by the token count
  float* stat_loss;
  float* stat_ratio;
  float* stat_kl;
  uint8_t* clip_mask;
  uint8_t* dual_mask;
  uint8_t* new_mask;
  float* behave_w;
  float* behave_kl;
  uint8_t* behave_mask;
  // fused logging statistics (loss_token_kernel<true> only)
  const float* entropy;   // optional per-token input
  const float* extra0;    // optional per-token inputs reduced over all tokens
  const float* extra1;
};

// Logged statistics reduced inside the token pass (the tensors grpo_loss_fn hands to the stats
// tracker, areal/trainer/ppo/actor.py:662-733, each under its denominator mask).
enum {
  ST_IMPORTANCE_WEIGHT = 0, ST_APPROX_KL, ST_NEW_LOGP, ST_OLD_LOGP, ST_ENTROPY, ST_ACTOR_LOSS,
  ST_CLIP_RATIO, ST_DUAL_CLIP_RATIO, ST_LOGP_DIFF, ST_LOGP_ABS_DIFF, ST_BEHAVE_FILTERED_RATIO,
  ST_BEHAVE_IMP_WEIGHT, ST_BEHAVE_APPROX_KL, ST_CLIPPED_NEW_LOGP, ST_CLIPPED_OLD_LOGP,
  ST_EXTRA0, ST_EXTRA1, N_LOSS_STATS
};
// denominators: 0 loss mask (before rejection), 1 clip mask, 2 behave mask, 3 every token
__device__ const int STAT_DENOM[N_LOSS_STATS] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 2, 2, 1, 1, 3, 3};

struct StatPartial {
  double sum;
  float mn, mx;
};

struct Partial {
  double loss_sum;
  long long n_valid, n_kept, n_filtered, n_clip, n_dual, n_behave;
};

DEVI int seq_of(const LossIO& io, int64_t t) {
  if (io.uniform_len > 0) return (int)(t / io.uniform_len);
  int lo = 0, hi = io.n_seqs;  // find last s with cu[s] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)io.cu[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// torch.clamp keeps NaN (fminf/fmaxf would drop it).
DEVI float torch_clamp(float x, float lo, float hi) {
  if (x != x) return x;
  return x < lo ? lo : (x > hi ? hi : x);
}
DEVI float torch_max(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : (a > b ? a : b); }
DEVI float torch_min(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : (a < b ? a : b); }
// Bernoulli KL(P||Q) with p = clamp(exp(log_p), 1e-8, 1 - 1e-8): in fp32 the upper bound
// rounds to 1.0f, which is what the reference's fp32 tensors see.
DEVI float binary_kl(float log_p, float log_q) {
  const float lo = 1e-8f, hi = (float)(1.0 - 1e-8);
  const float p = torch_clamp(expf(log_p), lo, hi);
  const float q = torch_clamp(expf(log_q), lo, hi);
  const float a = p * logf(p / q);
  const float b = (1.0f - p) * logf((1.0f - p) / (1.0f - q));
  return a + b;
}

DEVI bool in_bounds(float metric, const LossCfg& c) {
  bool ok = metric <= c.rs_upper;
  if (c.rs_has_lower) ok = ok && (metric >= c.rs_lower);
  return ok;
}

// Per-token divergence metric between proximal and behaviour policy. exp_lr = expf(lr_sane), which
// the caller has already (the behaviour weight).
DEVI float rs_metric(float prox, float old, float exp_lr, int metric) {
  switch (metric) {
    case METRIC_RATIO: return exp_lr;
    case METRIC_K1: return prox - old;
    case METRIC_K2: { const float d = prox - old; return (d * d) / 2.0f; }
    case METRIC_K3: { const float d = -(prox - old); return (expf(d) - 1.0f) - d; }
    default: return torch_max(binary_kl(prox, old), binary_kl(old, prox));
  }
}

DEVI float sane_log_ratio(float prox, float old) {
  const float lr = prox - old;
  return __builtin_isfinite(lr) ? lr : 0.0f;
}

template <typename T>
DEVI T block_sum(T v, T* smem) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) smem[w] = v;
  __syncthreads();
  T r = 0;
  const int nw = (blockDim.x + 63) >> 6;
  for (int i = 0; i < nw; ++i) r += smem[i];
  return r;
}

// ---------------------------------------------------------------------------------------
// Segmented pass 1: per-sequence aggregate of the rejection metric (one block per sequence).
// Writes seq_rs[s] = {in_bounds, uniform weight exp(mean log ratio)}.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(LOSS_THREADS) void seq_rs_kernel(LossIO io, LossCfg c, float* seq_rs) {
  __shared__ double sm_d[8];
  __shared__ float sm_f[8];
  const int s = blockIdx.x;
  int64_t t0, t1;
  if (io.uniform_len > 0) { t0 = (int64_t)s * io.uniform_len; t1 = t0 + io.uniform_len; }
  else { t0 = io.cu[s]; t1 = io.cu[s + 1]; }
  if (t1 > io.n) t1 = io.n;
  double sum_lr = 0.0, sum_m = 0.0;
  float mx = neg_inf();
  long long cnt = 0;
  const bool log_agg = (c.rs_metric == METRIC_RATIO);
  for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x) {
    if (!io.mask[t]) continue;
    const float prox = io.prox[t], old = io.old[t];
    const float lr = sane_log_ratio(prox, old);
    const float v = log_agg ? lr : rs_metric(prox, old, 0.0f, c.rs_metric);  // (the ratio metric aggregates lr)
    cnt += 1;
    sum_lr += (double)lr;
    sum_m += (double)v;
    mx = (v != v || mx != mx) ? __builtin_nanf("") : fmaxf(mx, v);
  }
  sum_lr = block_sum(sum_lr, sm_d);
  sum_m = block_sum(sum_m, sm_d);
  // max with NaN propagation: reduce a NaN flag and the max separately
  float nanflag = (mx != mx) ? 1.f : 0.f;
  float mxc = (mx != mx) ? neg_inf() : mx;
  mxc = wave_max(mxc);
  nanflag = wave_max(nanflag);
  {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) { sm_f[w] = mxc; sm_f[4 + w] = nanflag; }
    __syncthreads();
    mxc = fmaxf(fmaxf(sm_f[0], sm_f[1]), fmaxf(sm_f[2], sm_f[3]));
    nanflag = fmaxf(fmaxf(sm_f[4], sm_f[5]), fmaxf(sm_f[6], sm_f[7]));
  }
  __shared__ long long sm_l[8];
  const long long total = block_sum(cnt, sm_l);
  if (threadIdx.x == 0) {
    const float denom = (float)(total > 0 ? total : 1);
    float agg;
    if (c.rs_agg == AGG_SUM) agg = (float)sum_m;
    else if (c.rs_agg == AGG_MEAN) agg = (float)sum_m / denom;
    else agg = total == 0 ? 0.0f : (nanflag > 0.f ? __builtin_nanf("") : mxc);
    const float seq_metric = log_agg ? expf(agg) : agg;
    seq_rs[2 * s + 0] = in_bounds(seq_metric, c) ? 1.0f : 0.0f;
    seq_rs[2 * s + 1] = log_agg ? expf((float)sum_lr / denom) : 0.0f;
  }
}

// Rejection sampling for one token. Returns the narrowed mask; sets w (not yet zeroed outside
// the mask) and whether the token counts as filtered / clamped.
DEVI bool rs_token(const LossIO& io, const LossCfg& c, int64_t t, bool m, float prox, float old, float& w,
                   bool& counted) {
  const float lr = sane_log_ratio(prox, old);
  w = expf(lr);
  bool keep = true;
  counted = false;
  if (c.rs_seq_level) {
    const int s = seq_of(io, t);
    const bool seq_ok = io.seq_rs[2 * s] != 0.0f;
    if (c.rs_metric == METRIC_RATIO) w = io.seq_rs[2 * s + 1];
    if (c.rs_clamp) {
      const float orig = w;
      if (!seq_ok) w = torch_clamp(w, c.rs_has_lower ? c.rs_lower : 0.0f, c.rs_upper);
      counted = m && (orig != w);
    } else {
      keep = seq_ok;
      counted = m && !keep;
    }
  } else if (c.rs_clamp) {
    const float orig = w;
    w = torch_clamp(w, c.rs_has_lower ? c.rs_lower : 0.0f, c.rs_upper);
    counted = m && (orig != w);
  } else {
    keep = in_bounds(rs_metric(prox, old, w, c.rs_metric), c);
    counted = m && !keep;
  }
  return c.rs_clamp ? m : (m && keep);
}

// ---------------------------------------------------------------------------------------
// Segmented pass 2 (GSPO): per-sequence geometric-mean ratio and mean advantage over the
// narrowed mask. Writes seq_is[s] = {ratio_s, adv_mean_s, sum of behave weights, 1/count}.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(LOSS_THREADS) void seq_is_kernel(LossIO io, LossCfg c, float* seq_is) {
  __shared__ double sm_d[8];
  const int s = blockIdx.x;
  int64_t t0, t1;
  if (io.uniform_len > 0) { t0 = (int64_t)s * io.uniform_len; t1 = t0 + io.uniform_len; }
  else { t0 = io.cu[s]; t1 = io.cu[s + 1]; }
  if (t1 > io.n) t1 = io.n;
  double sum_lr = 0.0, sum_adv = 0.0, sum_w = 0.0, cnt = 0.0;
  for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x) {
    const bool m2 = c.rs_enabled ? (io.new_mask[t] != 0) : (io.mask[t] != 0);
    if (!m2) continue;
    cnt += 1.0;
    sum_lr += (double)(io.lp[t] - io.prox[t]);
    sum_adv += (double)io.adv[t];
    sum_w += c.rs_enabled ? (double)io.behave_w[t] : 1.0;
  }
  sum_lr = block_sum(sum_lr, sm_d);
  sum_adv = block_sum(sum_adv, sm_d);
  sum_w = block_sum(sum_w, sm_d);
  cnt = block_sum(cnt, sm_d);
  if (threadIdx.x == 0) {
    const float denom = (float)(cnt > 0.0 ? cnt : 1.0);
    seq_is[4 * s + 0] = expf((float)sum_lr / denom);
    seq_is[4 * s + 1] = (float)sum_adv / denom;
    seq_is[4 * s + 2] = (float)sum_w;
    seq_is[4 * s + 3] = 1.0f / denom;
  }
}

// ---------------------------------------------------------------------------------------
// Token kernel
// ---------------------------------------------------------------------------------------
// Running sums of one thread. Counts fit 32 bits per thread (a thread sees n / gridsize tokens).
struct TokenAcc {
  double loss_sum;
  int n_valid, n_kept, n_filtered, n_clip, n_dual, n_behave;
};

// The logged statistics a thread reduces itself. The three 0/1-valued ones (clip_ratio,
// dual_clip_ratio, behave_filtered_ratio) are not among them: their sums are the integer counters
// and their extremes follow from those (loss_finalize_kernel). A thread sees at most a few
// thousand tokens (n / (grid * LOSS_THREADS), 16 of 4 Mi), which it sums in fp32, as the
// reference's tracker sums whole tensors; so are the 16 threads of a row, and from there on the
// sums are fp64.
template <bool STATS>
struct StatAcc {
  float sum[STATS ? N_LOSS_STATS : 1], mn[STATS ? N_LOSS_STATS : 1], mx[STATS ? N_LOSS_STATS : 1];
  DEVI void init() {
    if (STATS) {
#pragma unroll
      for (int k = 0; k < N_LOSS_STATS; ++k) { sum[k] = 0.f; mn[k] = pos_inf(); mx[k] = neg_inf(); }
    }
  }
  DEVI void add(int k, float v) {
    if (STATS) {
      sum[k] += v;
      mn[k] = stat_min(mn[k], v);
      mx[k] = stat_max(mx[k], v);
    }
  }
};

// One token: the loss term, its gradient and every per-token output, from values in registers.
struct TokenIn {
  float lp, prox, old, adv, entropy, extra0, extra1;
  bool m;
};
struct TokenOut {
  float dlp, loss, ratio, kl, behave_w, behave_kl;
  bool clip, dual, m2, bm;
};

template <bool STATS>
DEVI void token_body(const LossIO& io, const LossCfg& c, int64_t t, const TokenIn& in, TokenOut& out,
                     TokenAcc& acc, StatAcc<STATS>& st) {
  const bool m = in.m;
  bool m2 = m;
  float w = 1.0f;
  if (c.rs_enabled) {
    bool counted;
    m2 = rs_token(io, c, t, m, in.prox, in.old, w, counted);
    w = m2 ? w : 0.0f;
    acc.n_filtered += counted;
  }
  out.m2 = m2;
  out.behave_w = w;
  acc.n_valid += m;
  acc.n_kept += m2;
  if (STATS) {
    if (io.extra0) st.add(ST_EXTRA0, in.extra0);
    if (io.extra1) st.add(ST_EXTRA1, in.extra1);
  }
  out.dlp = 0.f; out.loss = 0.f; out.ratio = 0.f; out.kl = 0.f; out.behave_kl = 0.f;
  out.clip = false; out.dual = false; out.bm = false;
  if (c.loss_kind == LOSS_NONE) return;

  const float lp = in.lp, prox = in.prox, adv = in.adv;
  const float kl = lp - prox;
  float pg, dsel, ratio_out;
  bool clip = false, dual = false;
  if (c.loss_kind == LOSS_CISPO) {
    const float ratio = expf(kl);
    const float rc = torch_clamp(ratio, c.clip_lo, c.clip_hi);
    const float coef = (-rc) * adv;
    pg = coef * lp;
    dsel = coef;  // d pg / d lp
    clip = (rc != ratio) && m2;
    ratio_out = ratio;
  } else {
    float ratio, a = adv, dratio;  // dratio = d ratio / d lp[t] factor handled below
    if (c.seq_is) {
      const int s = seq_of(io, t);
      ratio = m2 ? io.seq_is[4 * s + 0] : 0.0f;
      a = m2 ? io.seq_is[4 * s + 1] : 0.0f;
      dratio = 0.f;  // gradient assembled per sequence below
    } else {
      ratio = m ? expf(kl) : 0.0f;
      dratio = ratio;
    }
    const float clipped = torch_clamp(ratio, c.clip_lo, c.clip_hi);
    const float pg1 = (-a) * ratio;
    const float pg2 = (-a) * clipped;
    clip = pg1 < pg2;
    pg = torch_max(pg1, pg2);
    // d pg / d ratio following torch.max (ties split evenly) and clamp (closed interval)
    const float in_band = (ratio >= c.clip_lo && ratio <= c.clip_hi) ? 1.0f : 0.0f;
    float g1 = pg1 > pg2 ? 1.0f : (pg1 == pg2 ? 0.5f : 0.0f);
    float g2 = pg2 > pg1 ? 1.0f : (pg1 == pg2 ? 0.5f : 0.0f);
    float dpg = (-a) * (g1 + g2 * in_band);
    if (c.has_c_clip) {
      const float sgn = a > 0.f ? 1.0f : (a < 0.f ? -1.0f : 0.0f);
      const float pg3 = (sgn * c.c_clip) * a;
      dual = pg3 < pg;
      const float keep = pg < pg3 ? 1.0f : (pg == pg3 ? 0.5f : 0.0f);
      pg = torch_min(pg, pg3);
      dpg *= keep;
    }
    if (c.seq_is) {
      // every kept token of the sequence receives ratio_s/count_s * sum_w_s * dpg_s
      const int s = seq_of(io, t);
      dsel = m2 ? dpg * ratio * io.seq_is[4 * s + 2] * io.seq_is[4 * s + 3] : 0.0f;
    } else {
      dsel = dpg * dratio;
    }
    clip = clip && m;
    dual = dual && m;
    ratio_out = ratio;
  }
  if (c.rs_enabled) {
    pg = pg * w;
    if (!(c.loss_kind == LOSS_PPO && c.seq_is)) dsel = dsel * w;
    const bool bm = (w > 0.0f) && m2;
    acc.n_behave += bm;
    out.bm = bm;
    out.behave_kl = bm ? (prox - in.old) : 0.0f;
    if (STATS && bm) {
      st.add(ST_BEHAVE_IMP_WEIGHT, w);
      st.add(ST_BEHAVE_APPROX_KL, prox - in.old);
    }
  }
  if (STATS) {
    if (m) {
      st.add(ST_IMPORTANCE_WEIGHT, ratio_out);
      st.add(ST_APPROX_KL, kl);
      st.add(ST_NEW_LOGP, lp);
      st.add(ST_ACTOR_LOSS, pg);
      if (io.entropy) st.add(ST_ENTROPY, in.entropy);
      if (io.old) {
        st.add(ST_OLD_LOGP, in.old);
        st.add(ST_LOGP_DIFF, in.old - lp);
        st.add(ST_LOGP_ABS_DIFF, fabsf(in.old - lp));
      }
    }
    if (clip) {
      st.add(ST_CLIPPED_NEW_LOGP, lp);
      if (io.old) st.add(ST_CLIPPED_OLD_LOGP, in.old);
    }
  }
  if (m2) acc.loss_sum += (double)pg;
  acc.n_clip += clip;
  acc.n_dual += dual;
  out.dlp = m2 ? dsel : 0.0f;
  out.loss = pg;
  out.ratio = ratio_out;
  out.kl = kl;
  out.clip = clip;
  out.dual = dual;
}

// The per-token inputs of VEC consecutive tokens, in registers.
template <int VEC>
struct TokenLoad {
  float lp[VEC], prox[VEC], old[VEC], adv[VEC], ent[VEC], x0[VEC], x1[VEC];
  bool m[VEC];
};
template <bool STATS, int VEC>
DEVI void token_group_load(const LossIO& io, const LossCfg& c, int64_t t, TokenLoad<VEC>& in) {
  load_mask<VEC>(io.mask, t, in.m);
  load_f32<VEC>(io.prox, t, in.prox);
  load_f32<VEC>(io.old, t, in.old);
  load_f32<VEC>(c.loss_kind == LOSS_NONE ? nullptr : io.lp, t, in.lp);
  load_f32<VEC>(c.loss_kind == LOSS_NONE ? nullptr : io.adv, t, in.adv);
  load_f32<VEC>(STATS ? io.entropy : nullptr, t, in.ent);
  load_f32<VEC>(STATS ? io.extra0 : nullptr, t, in.x0);
  load_f32<VEC>(STATS ? io.extra1 : nullptr, t, in.x1);
}
template <bool STATS, int VEC>
DEVI void token_group_compute(const LossIO& io, const LossCfg& c, int64_t t, const TokenLoad<VEC>& ld,
                              TokenAcc& acc, StatAcc<STATS>& st) {
  float dlp[VEC], loss[VEC], ratio[VEC], kl[VEC], bw[VEC], bkl[VEC];
  bool clip[VEC], dual[VEC], m2[VEC], bm[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    const TokenIn in{ld.lp[i], ld.prox[i], ld.old[i], ld.adv[i], ld.ent[i], ld.x0[i], ld.x1[i], ld.m[i]};
    TokenOut o;
    token_body<STATS>(io, c, t + i, in, o, acc, st);
    dlp[i] = o.dlp; loss[i] = o.loss; ratio[i] = o.ratio; kl[i] = o.kl; bw[i] = o.behave_w; bkl[i] = o.behave_kl;
    clip[i] = o.clip; dual[i] = o.dual; m2[i] = o.m2; bm[i] = o.bm;
  }
  if (c.rs_enabled) {
    store_mask<VEC>(io.new_mask, t, m2);
    store_f32<VEC>(io.behave_w, t, bw);
  }
  if (c.loss_kind == LOSS_NONE) return;
  if (c.rs_enabled) {
    store_mask<VEC>(io.behave_mask, t, bm);
    store_f32<VEC>(io.behave_kl, t, bkl);
  }
  store_f32<VEC>(io.dlp, t, dlp);
  store_f32<VEC>(io.stat_loss, t, loss);
  store_f32<VEC>(io.stat_ratio, t, ratio);
  store_f32<VEC>(io.stat_kl, t, kl);
  store_mask<VEC>(io.clip_mask, t, clip);
  store_mask<VEC>(io.dual_mask, t, dual);
}

// STATS: also reduce the logged statistics (sum, min, max per block) into stat_partials
// [gridDim.x][N_LOSS_STATS]; min / max propagate NaN as torch.min / torch.max do.
template <bool STATS, int VEC>
__global__ __launch_bounds__(LOSS_THREADS) void loss_token_kernel(LossIO io, LossCfg c,
                                                                   Partial* partials,
                                                                   StatPartial* stat_partials) {
  TokenAcc acc{0.0, 0, 0, 0, 0, 0, 0};
  StatAcc<STATS> st;
  st.init();
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const int64_t n_vec = io.n - io.n % VEC;
  TokenLoad<VEC> in;
  for (int64_t t = gid * VEC; t < n_vec; t += nthreads * VEC) {
    token_group_load<STATS, VEC>(io, c, t, in);
    token_group_compute<STATS, VEC>(io, c, t, in, acc, st);
  }
  if (VEC > 1 && n_vec + gid < io.n) {
    TokenLoad<1> tail;
    token_group_load<STATS, 1>(io, c, n_vec + gid, tail);
    token_group_compute<STATS, 1>(io, c, n_vec + gid, tail, acc, st);
  }

  // One barrier pair for everything the block hands on. A wave sums its counters as 32-bit integers
  // (a thread sees at most a few thousand tokens); statistics are reduced inside each row of 16
  // lanes only, and the 16 row results of the block are combined from LDS in a fixed order.
  constexpr int NW = LOSS_THREADS / 64, NROW = LOSS_THREADS / 16;
  __shared__ double sh_loss[NW];
  __shared__ int sh_cnt[NW][6];
  __shared__ double sh_sum[STATS ? NROW : 1][STATS ? N_LOSS_STATS : 1];
  __shared__ float sh_mn[STATS ? NROW : 1][STATS ? N_LOSS_STATS : 1], sh_mx[STATS ? NROW : 1][STATS ? N_LOSS_STATS : 1];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  {
    const double ls = wave_sum(acc.loss_sum);
    const int cnt[6] = {wave_sum(acc.n_valid), wave_sum(acc.n_kept), wave_sum(acc.n_filtered),
                        wave_sum(acc.n_clip), wave_sum(acc.n_dual), wave_sum(acc.n_behave)};
    if (lane == 0) {
      sh_loss[w] = ls;
#pragma unroll
      for (int k = 0; k < 6; ++k) sh_cnt[w][k] = cnt[k];
    }
  }
  if (STATS) {
    const int row = threadIdx.x >> 4;
#pragma unroll
    for (int k = 0; k < N_LOSS_STATS; ++k) {
      // (the 16 threads' fp32 sums are added in fp32 like the thread's own tokens; fp64 from here)
      const double sv = (double)row_reduce(st.sum[k], [](float a, float b) { return a + b; });
      const float mn = row_reduce(st.mn[k], [](float a, float b) { return stat_min(a, b); });
      const float mx = row_reduce(st.mx[k], [](float a, float b) { return stat_max(a, b); });
      if ((threadIdx.x & 15) == 0) { sh_sum[row][k] = sv; sh_mn[row][k] = mn; sh_mx[row][k] = mx; }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    Partial p{sh_loss[0], sh_cnt[0][0], sh_cnt[0][1], sh_cnt[0][2], sh_cnt[0][3], sh_cnt[0][4], sh_cnt[0][5]};
    for (int i = 1; i < NW; ++i) {
      p.loss_sum += sh_loss[i];
      p.n_valid += sh_cnt[i][0]; p.n_kept += sh_cnt[i][1]; p.n_filtered += sh_cnt[i][2];
      p.n_clip += sh_cnt[i][3]; p.n_dual += sh_cnt[i][4]; p.n_behave += sh_cnt[i][5];
    }
    partials[blockIdx.x] = p;
  }
  if (STATS) {
    if (threadIdx.x >= 64 && threadIdx.x < 64 + N_LOSS_STATS) {  // a wave other than thread 0's
      const int k = threadIdx.x - 64;
      StatPartial sp{sh_sum[0][k], sh_mn[0][k], sh_mx[0][k]};
      for (int i = 1; i < NROW; ++i) {
        sp.sum += sh_sum[i][k];
        sp.mn = stat_min(sp.mn, sh_mn[i][k]);
        sp.mx = stat_max(sp.mx, sh_mx[i][k]);
      }
      stat_partials[(size_t)blockIdx.x * N_LOSS_STATS + k] = sp;
    }
  }
}

// counters: [0] loss_sum [1] n_valid [2] n_kept [3] n_filtered [4] n_clip [5] n_dual
//           [6] n_behave [7] loss = loss_sum / max(n_valid, 1)
// Block 0 folds the token kernel's block partials into the counters and the loss, in a fixed order
// (thread partials -> wave shuffles -> 4 wave slots). With statistics, block 1 + k folds statistic
// k into stats [N_LOSS_STATS][4] = {sum, count, min, max}; the count is the statistic's denominator.
// The three 0/1-valued statistics are not reduced per token: their sums are token counts and
// their extremes follow from whether every / any counted token has the value 1. Each block sums
// the counts it needs itself, so one launch does everything.
__global__ __launch_bounds__(FINAL_THREADS) void loss_finalize_kernel(
    const Partial* __restrict__ partials, const StatPartial* __restrict__ stat_partials, int nparts,
    float* loss_out, double* __restrict__ counters, double n_tokens, double* __restrict__ stats,
    int loss_active, int rs_enabled) {
  constexpr int NW = FINAL_THREADS / 64;
  __shared__ double sh_d[NW][2];     // loss sum, statistic sum
  __shared__ long long sh_l[NW][6];
  __shared__ float sh_f[NW][2];      // statistic minimum, maximum
  const int k = (int)blockIdx.x - 1;  // the block's statistic; block 0: the counters and the loss
  const bool reduced = k >= 0 && !(k == ST_CLIP_RATIO || k == ST_DUAL_CLIP_RATIO || k == ST_BEHAVE_FILTERED_RATIO);
  // the thread's partials are fetched together (one memory latency, not one per partial) and
  // added in index order
  constexpr int PER_THREAD = MAX_LOSS_BLOCKS / FINAL_THREADS;
  Partial pp[PER_THREAD];
  StatPartial sp[PER_THREAD];
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const int i = threadIdx.x + j * FINAL_THREADS;
    pp[j] = i < nparts ? partials[i] : Partial{0.0, 0, 0, 0, 0, 0, 0};
    sp[j] = StatPartial{0.0, pos_inf(), neg_inf()};
    if (reduced && i < nparts) sp[j] = stat_partials[(size_t)i * N_LOSS_STATS + k];
  }
  double ls = 0.0, sum = 0.0;
  long long a[6] = {0, 0, 0, 0, 0, 0};
  float mn = pos_inf(), mx = neg_inf();
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    ls += pp[j].loss_sum;
    a[0] += pp[j].n_valid; a[1] += pp[j].n_kept; a[2] += pp[j].n_filtered;
    a[3] += pp[j].n_clip; a[4] += pp[j].n_dual; a[5] += pp[j].n_behave;
    sum += sp[j].sum;
    mn = stat_min(mn, sp[j].mn);
    mx = stat_max(mx, sp[j].mx);
  }
  // wave results into LDS, one barrier, then thread 0 adds the waves in order
  ls = wave_sum(ls);
#pragma unroll
  for (int q = 0; q < 6; ++q) a[q] = wave_sum(a[q]);
  if (reduced) {
    sum = wave_sum(sum);
    mn = wave_stat_min(mn);
    mx = wave_stat_max(mx);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) {
    sh_d[w][0] = ls; sh_d[w][1] = sum;
#pragma unroll
    for (int q = 0; q < 6; ++q) sh_l[w][q] = a[q];
    sh_f[w][0] = mn; sh_f[w][1] = mx;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  ls = sh_d[0][0]; sum = sh_d[0][1]; mn = sh_f[0][0]; mx = sh_f[0][1];
#pragma unroll
  for (int q = 0; q < 6; ++q) a[q] = sh_l[0][q];
  for (int i = 1; i < NW; ++i) {
    ls += sh_d[i][0]; sum += sh_d[i][1];
#pragma unroll
    for (int q = 0; q < 6; ++q) a[q] += sh_l[i][q];
    mn = stat_min(mn, sh_f[i][0]); mx = stat_max(mx, sh_f[i][1]);
  }
  if (k < 0) {
    counters[0] = ls;
    for (int q = 0; q < 6; ++q) counters[1 + q] = (double)a[q];
    const double denom = a[0] > 0 ? (double)a[0] : 1.0;
    const float loss = (float)ls / (float)denom;
    counters[7] = (double)loss;
    if (loss_out) *loss_out = loss;
    return;
  }
  const long long n_valid = a[0], n_clip = a[3], n_dual = a[4], n_behave = a[5];
  const int d = STAT_DENOM[k];
  const double count = d == 0 ? (double)n_valid : (d == 1 ? (double)n_clip : (d == 2 ? (double)n_behave : n_tokens));
  if (!reduced) {
    // ones among the n_valid tokens under the loss mask
    sum = 0.0; mn = pos_inf(); mx = neg_inf();
    const bool on = loss_active && (k != ST_BEHAVE_FILTERED_RATIO || rs_enabled);
    const long long ones = k == ST_CLIP_RATIO ? n_clip : (k == ST_DUAL_CLIP_RATIO ? n_dual : n_valid - n_behave);
    if (on && n_valid > 0) {
      sum = (double)ones;
      mn = ones == n_valid ? 1.0f : 0.0f;
      mx = ones > 0 ? 1.0f : 0.0f;
    }
  }
  stats[4 * k + 0] = sum;
  stats[4 * k + 1] = count;
  stats[4 * k + 2] = (double)mn;
  stats[4 * k + 3] = (double)mx;
}

// out[t] = dlp[t] * upstream[0] / max(n_valid, 1); VEC as in the token kernel
template <int VEC>
__global__ void loss_grad_scale_kernel(const float* __restrict__ dlp,
                                       const float* __restrict__ upstream,
                                       const double* __restrict__ counters,
                                       float* __restrict__ out, int64_t n) {
  const float nv = (float)(counters[1] > 0.0 ? counters[1] : 1.0);
  const float g = upstream[0];
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const int64_t n_vec = n - n % VEC;
  for (int64_t t = gid * VEC; t < n_vec; t += nthreads * VEC) {
    float v[VEC];
    load_f32<VEC>(dlp, t, v);
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = (v[i] * g) / nv;
    store_f32<VEC>(out, t, v);
  }
  if (VEC > 1 && n_vec + gid < n) out[n_vec + gid] = (dlp[n_vec + gid] * g) / nv;
}

int loss_grid(int64_t n, int vec = 1) {
  int64_t b = ceil_div_i64(n, (int64_t)LOSS_THREADS * vec);
  if (b > MAX_LOSS_BLOCKS) b = MAX_LOSS_BLOCKS;
  if (b < 1) b = 1;
  return (int)b;
}

}  // namespace

// Plain-C mirror of LossCfg (see include/areal_hip.h).
struct areal_loss_config {
  int loss_kind;
  float clip_lo, clip_hi;
  int has_c_clip;
  float c_clip;
  int seq_is;
  int rs_enabled, rs_seq_level, rs_clamp, rs_metric, rs_agg;
  float rs_upper;
  int rs_has_lower;
  float rs_lower;
};

namespace {

constexpr size_t STAT_PARTIAL_BYTES = (size_t)MAX_LOSS_BLOCKS * N_LOSS_STATS * sizeof(StatPartial);

size_t loss_workspace_bytes(int64_t n_seqs, bool with_stats) {
  if (n_seqs < 0) n_seqs = 0;
  return (size_t)MAX_LOSS_BLOCKS * sizeof(Partial) + (with_stats ? STAT_PARTIAL_BYTES : 0) +
         (size_t)n_seqs * 6 * sizeof(float) + 256;
}

// Optional inputs and the output of the fused logging statistics.
struct LossStatsArgs {
  const float* entropy;
  const float* extra0;
  const float* extra1;
  double* stats;  // [N_LOSS_STATS][4]
};

// Scratch of areal_actor_loss_static: the block partials and the per-sequence aggregates of
// one call, for up to STATIC_MAX_SEQS sequences. Every GPU the library runs on holds its own
// copy of this array for the life of the process (about 1.6 MB). Nothing in it has to start at
// zero: a call writes every partial and every per-sequence slot it later reads.
constexpr int64_t STATIC_MAX_SEQS = 65536;
constexpr size_t STATIC_SCRATCH_BYTES =
    (size_t)MAX_LOSS_BLOCKS * sizeof(Partial) + (size_t)STATIC_MAX_SEQS * 6 * sizeof(float) + 256;
static_assert(STATIC_SCRATCH_BYTES < (2u << 20), "the static scratch is meant to stay small");
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

// Device address of `scratch` on each GPU (the array's name is only a host-side handle).
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex scratch_lock;
void* scratch_ptr[STATIC_MAX_DEVICES];

int scratch_for_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) return AREAL_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return AREAL_ERR_LAUNCH;
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return AREAL_OK;
}

int actor_loss_impl(const float* logprobs, const float* proximal, const float* old_logprobs,
                    const float* advantages, const uint8_t* loss_mask, const int32_t* cu_seqlens,
                    int64_t n_tokens, int64_t n_seqs, int64_t uniform_len,
                    const areal_loss_config* cfg, float* loss, float* dlogprobs, float* stat_loss,
                    float* stat_ratio, float* stat_approx_kl, uint8_t* clip_mask,
                    uint8_t* dual_clip_mask, uint8_t* new_mask, float* behave_imp_weight,
                    float* behave_approx_kl, uint8_t* behave_mask, double* counters,
                    const LossStatsArgs* sa, void* workspace, size_t workspace_bytes,
                    hipStream_t stream);

}  // namespace

extern "C" {

size_t areal_actor_loss_workspace_bytes(int64_t n_tokens, int64_t n_seqs) {
  (void)n_tokens;
  return loss_workspace_bytes(n_seqs, false);
}

size_t areal_actor_loss_stats_workspace_bytes(int64_t n_tokens, int64_t n_seqs) {
  (void)n_tokens;
  return loss_workspace_bytes(n_seqs, true);
}

// Actor loss forward + backward in one pass over the tokens.
//   loss_kind -1: rejection sampling only (lp / adv / loss outputs ignored)
//              0: PPO clip (optionally dual clip, optionally sequence-level ratio)
//              1: CISPO
// Sequences are given by cu_seqlens [n_seqs+1] (packed) or by uniform_len (> 0, padded
// [n_seqs, uniform_len] layout); both are needed only for sequence-level options.
// counters is a device array of 8 doubles (layout above loss_finalize_kernel).
int areal_actor_loss(const float* logprobs, const float* proximal, const float* old_logprobs,
                     const float* advantages, const uint8_t* loss_mask,
                     const int32_t* cu_seqlens, int64_t n_tokens, int64_t n_seqs,
                     int64_t uniform_len, const areal_loss_config* cfg, float* loss,
                     float* dlogprobs, float* stat_loss, float* stat_ratio, float* stat_approx_kl,
                     uint8_t* clip_mask, uint8_t* dual_clip_mask, uint8_t* new_mask,
                     float* behave_imp_weight, float* behave_approx_kl, uint8_t* behave_mask,
                     double* counters, void* workspace, size_t workspace_bytes,
                     hipStream_t stream) {
  return actor_loss_impl(logprobs, proximal, old_logprobs, advantages, loss_mask, cu_seqlens, n_tokens,
                         n_seqs, uniform_len, cfg, loss, dlogprobs, stat_loss, stat_ratio,
                         stat_approx_kl, clip_mask, dual_clip_mask, new_mask, behave_imp_weight,
                         behave_approx_kl, behave_mask, counters, nullptr, workspace, workspace_bytes,
                         stream);
}

// areal_actor_loss that also reduces the logged statistics in the token pass: stats
// [17][4] double = {sum, count, min, max} of, in this order: importance_weight, approx_kl,
// new_logp, old_logp, entropy, actor_loss, clip_ratio, dual_clip_ratio, logp_diff,
// logp_abs_diff, behave_filtered_ratio (all under the loss mask before rejection),
// behave_imp_weight, behave_approx_kl (under the behave mask), clipped_new_logp,
// clipped_old_logp (under the clip mask), extra0, extra1 (every token). entropy / extra0 /
// extra1 / old_logprobs may be null: their statistics then come out as sum 0, min +inf, max -inf.
// Every per-token output may be null, so a caller that logs only reduced values moves
// 17 bytes per token in and 4 out (dlogprobs).
int areal_actor_loss_stats(const float* logprobs, const float* proximal, const float* old_logprobs,
                           const float* advantages, const uint8_t* loss_mask,
                           const int32_t* cu_seqlens, int64_t n_tokens, int64_t n_seqs,
                           int64_t uniform_len, const areal_loss_config* cfg,
                           const float* entropy, const float* extra0, const float* extra1,
                           float* loss, float* dlogprobs, float* stat_loss, float* stat_ratio,
                           float* stat_approx_kl, uint8_t* clip_mask, uint8_t* dual_clip_mask,
                           uint8_t* new_mask, float* behave_imp_weight, float* behave_approx_kl,
                           uint8_t* behave_mask, double* counters, double* stats, void* workspace,
                           size_t workspace_bytes, hipStream_t stream) {
  const LossStatsArgs sa{entropy, extra0, extra1, stats};
  return actor_loss_impl(logprobs, proximal, old_logprobs, advantages, loss_mask, cu_seqlens, n_tokens,
                         n_seqs, uniform_len, cfg, loss, dlogprobs, stat_loss, stat_ratio,
                         stat_approx_kl, clip_mask, dual_clip_mask, new_mask, behave_imp_weight,
                         behave_approx_kl, behave_mask, counters, &sa, workspace, workspace_bytes,
                         stream);
}

// The same computation with the scratch in a static device array instead of a caller's
// workspace: no allocation anywhere on the call path. Must be called with the stream's device
// current. Sequence-level options accept at most 65536 sequences (AREAL_ERR_UNSUPPORTED beyond).
// Calls on one GPU share that GPU's array: two calls that overlap in time (different streams)
// race; calls on one stream are ordered and safe.
int areal_actor_loss_static(const float* logprobs, const float* proximal,
                            const float* old_logprobs, const float* advantages,
                            const uint8_t* loss_mask, const int32_t* cu_seqlens,
                            int64_t n_tokens, int64_t n_seqs, int64_t uniform_len,
                            const areal_loss_config* cfg, float* loss, float* dlogprobs,
                            float* stat_loss, float* stat_ratio, float* stat_approx_kl,
                            uint8_t* clip_mask, uint8_t* dual_clip_mask, uint8_t* new_mask,
                            float* behave_imp_weight, float* behave_approx_kl,
                            uint8_t* behave_mask, double* counters, hipStream_t stream) {
  if (n_seqs > STATIC_MAX_SEQS) return AREAL_ERR_UNSUPPORTED;
  void* ws = nullptr;
  const int rc = scratch_for_current_device(&ws);
  if (rc != AREAL_OK) return rc;
  return actor_loss_impl(logprobs, proximal, old_logprobs, advantages, loss_mask, cu_seqlens, n_tokens,
                         n_seqs, uniform_len, cfg, loss, dlogprobs, stat_loss, stat_ratio,
                         stat_approx_kl, clip_mask, dual_clip_mask, new_mask, behave_imp_weight,
                         behave_approx_kl, behave_mask, counters, nullptr, ws, STATIC_SCRATCH_BYTES,
                         stream);
}

}  // extern "C"

namespace {

int actor_loss_impl(const float* logprobs, const float* proximal, const float* old_logprobs,
                    const float* advantages, const uint8_t* loss_mask, const int32_t* cu_seqlens,
                    int64_t n_tokens, int64_t n_seqs, int64_t uniform_len,
                    const areal_loss_config* cfg, float* loss, float* dlogprobs, float* stat_loss,
                    float* stat_ratio, float* stat_approx_kl, uint8_t* clip_mask,
                    uint8_t* dual_clip_mask, uint8_t* new_mask, float* behave_imp_weight,
                    float* behave_approx_kl, uint8_t* behave_mask, double* counters,
                    const LossStatsArgs* sa, void* workspace, size_t workspace_bytes,
                    hipStream_t stream) {
  if (cfg == nullptr || n_tokens < 0 || counters == nullptr) return AREAL_ERR_BAD_ARG;
  const bool with_stats = sa != nullptr;
  if (with_stats && sa->stats == nullptr) return AREAL_ERR_BAD_ARG;
  if (cfg->loss_kind < LOSS_NONE || cfg->loss_kind > LOSS_CISPO) return AREAL_ERR_BAD_ARG;
  if (n_tokens > 0 && (proximal == nullptr || loss_mask == nullptr)) return AREAL_ERR_BAD_ARG;
  if (cfg->loss_kind != LOSS_NONE && n_tokens > 0 && (logprobs == nullptr || advantages == nullptr))
    return AREAL_ERR_BAD_ARG;
  if (cfg->rs_enabled && n_tokens > 0 && old_logprobs == nullptr) return AREAL_ERR_BAD_ARG;
  const bool need_seq = (cfg->rs_enabled && cfg->rs_seq_level) || (cfg->loss_kind == LOSS_PPO && cfg->seq_is);
  if (need_seq && n_tokens > 0) {
    if (n_seqs <= 0) return AREAL_ERR_BAD_ARG;
    if (uniform_len <= 0 && cu_seqlens == nullptr) return AREAL_ERR_BAD_ARG;
    if (cfg->rs_enabled && (new_mask == nullptr || behave_imp_weight == nullptr) && cfg->seq_is)
      return AREAL_ERR_BAD_ARG;
  }
  if (workspace == nullptr || workspace_bytes < loss_workspace_bytes(n_seqs, with_stats))
    return AREAL_ERR_WORKSPACE;

  LossCfg c;
  c.loss_kind = cfg->loss_kind; c.clip_lo = cfg->clip_lo; c.clip_hi = cfg->clip_hi;
  c.has_c_clip = cfg->has_c_clip; c.c_clip = cfg->c_clip;
  c.seq_is = (cfg->loss_kind == LOSS_PPO) ? cfg->seq_is : 0;
  c.rs_enabled = cfg->rs_enabled; c.rs_seq_level = cfg->rs_seq_level; c.rs_clamp = cfg->rs_clamp;
  c.rs_metric = cfg->rs_metric; c.rs_agg = cfg->rs_agg; c.rs_upper = cfg->rs_upper;
  c.rs_has_lower = cfg->rs_has_lower; c.rs_lower = cfg->rs_lower;

  char* wp = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  Partial* partials = (Partial*)wp;
  wp += (size_t)MAX_LOSS_BLOCKS * sizeof(Partial);
  StatPartial* stat_partials = with_stats ? (StatPartial*)wp : nullptr;
  if (with_stats) wp += STAT_PARTIAL_BYTES;
  float* seq_rs = (float*)wp;
  float* seq_is = seq_rs + 2 * (n_seqs > 0 ? n_seqs : 0);

  LossIO io;
  io.lp = logprobs; io.prox = proximal; io.old = old_logprobs; io.adv = advantages;
  io.mask = loss_mask; io.cu = cu_seqlens; io.n = n_tokens; io.n_seqs = (int)n_seqs;
  io.uniform_len = uniform_len; io.seq_rs = seq_rs; io.seq_is = seq_is;
  io.dlp = dlogprobs; io.stat_loss = stat_loss; io.stat_ratio = stat_ratio;
  io.stat_kl = stat_approx_kl; io.clip_mask = clip_mask; io.dual_mask = dual_clip_mask;
  io.new_mask = new_mask; io.behave_w = behave_imp_weight; io.behave_kl = behave_approx_kl;
  io.behave_mask = behave_mask;
  io.entropy = with_stats ? sa->entropy : nullptr;
  io.extra0 = with_stats ? sa->extra0 : nullptr;
  io.extra1 = with_stats ? sa->extra1 : nullptr;

  // four tokens per thread once that still gives every CU a block; a smaller batch is bound by
  // latency, not by bandwidth, and runs faster spread over four times as many threads
  const bool vec4 = n_tokens >= (int64_t)4 * LOSS_THREADS * 256 && aligned_to(logprobs, 16) && aligned_to(proximal, 16) && aligned_to(old_logprobs, 16) &&
                    aligned_to(advantages, 16) && aligned_to(dlogprobs, 16) && aligned_to(stat_loss, 16) &&
                    aligned_to(stat_ratio, 16) && aligned_to(stat_approx_kl, 16) &&
                    aligned_to(behave_imp_weight, 16) && aligned_to(behave_approx_kl, 16) &&
                    aligned_to(io.entropy, 16) && aligned_to(io.extra0, 16) && aligned_to(io.extra1, 16) &&
                    aligned_to(loss_mask, 4) && aligned_to(clip_mask, 4) && aligned_to(dual_clip_mask, 4) &&
                    aligned_to(new_mask, 4) && aligned_to(behave_mask, 4);
  // with statistics a block's end costs a third of eight tokens' work per thread: half the blocks
  int grid = loss_grid(n_tokens, vec4 ? 4 : 1);
  if (with_stats && grid > MAX_LOSS_BLOCKS / 2) grid = MAX_LOSS_BLOCKS / 2;
  auto token_pass = [&](const LossIO& i, const LossCfg& cc, bool stats) {
    if (stats && vec4)
      hipLaunchKernelGGL((loss_token_kernel<true, 4>), dim3(grid), dim3(LOSS_THREADS), 0, stream, i, cc, partials, stat_partials);
    else if (stats)
      hipLaunchKernelGGL((loss_token_kernel<true, 1>), dim3(grid), dim3(LOSS_THREADS), 0, stream, i, cc, partials, stat_partials);
    else if (vec4)
      hipLaunchKernelGGL((loss_token_kernel<false, 4>), dim3(grid), dim3(LOSS_THREADS), 0, stream, i, cc, partials, (StatPartial*)nullptr);
    else
      hipLaunchKernelGGL((loss_token_kernel<false, 1>), dim3(grid), dim3(LOSS_THREADS), 0, stream, i, cc, partials, (StatPartial*)nullptr);
  };
  if (n_tokens > 0 && c.rs_enabled && c.rs_seq_level) {
    hipLaunchKernelGGL(seq_rs_kernel, dim3((unsigned)n_seqs), dim3(LOSS_THREADS), 0, stream, io, c,
                       seq_rs);
    AREAL_CHECK_LAUNCH();
  }
  if (n_tokens > 0 && c.seq_is) {
    if (c.rs_enabled) {
      // first materialise the narrowed mask and the behaviour weight, then aggregate on them
      LossCfg c0 = c;
      c0.loss_kind = LOSS_NONE;
      token_pass(io, c0, false);
      AREAL_CHECK_LAUNCH();
    }
    hipLaunchKernelGGL(seq_is_kernel, dim3((unsigned)n_seqs), dim3(LOSS_THREADS), 0, stream, io, c,
                       seq_is);
    AREAL_CHECK_LAUNCH();
  }
  token_pass(io, c, with_stats);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(loss_finalize_kernel, dim3(with_stats ? 1 + N_LOSS_STATS : 1), dim3(FINAL_THREADS), 0, stream,
                     partials, stat_partials, grid, loss, counters, (double)n_tokens,
                     with_stats ? sa->stats : nullptr, c.loss_kind != LOSS_NONE ? 1 : 0, c.rs_enabled);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // namespace

extern "C" {

// grad_logprobs[t] = dlogprobs[t] * upstream[0] / max(counters[1], 1)
int areal_actor_loss_grad(const float* dlogprobs, const float* upstream, const double* counters,
                          float* grad_logprobs, int64_t n_tokens, hipStream_t stream) {
  if (n_tokens < 0) return AREAL_ERR_BAD_ARG;
  if (n_tokens == 0) return AREAL_OK;
  if (!dlogprobs || !upstream || !counters || !grad_logprobs) return AREAL_ERR_BAD_ARG;
  if (n_tokens >= (int64_t)4 * LOSS_THREADS * 256 && aligned_to(dlogprobs, 16) && aligned_to(grad_logprobs, 16))
    hipLaunchKernelGGL(loss_grad_scale_kernel<4>, dim3(loss_grid(n_tokens, 4)), dim3(LOSS_THREADS), 0,
                       stream, dlogprobs, upstream, counters, grad_logprobs, n_tokens);
  else
    hipLaunchKernelGGL(loss_grad_scale_kernel<1>, dim3(loss_grid(n_tokens)), dim3(LOSS_THREADS), 0,
                       stream, dlogprobs, upstream, counters, grad_logprobs, n_tokens);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // extern "C"
