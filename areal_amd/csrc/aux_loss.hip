// Losses that share the actor loss's data layout: SAPO soft-gate policy loss, the clipped PPO
// critic loss, and the per-sequence log-probability sums of DPO.
//
// Follows areal/utils/functional/functional.py: sapo_loss_fn (:599-675) with
// _compute_sequence_level_ratio_and_advantages (:56-149), ppo_critic_loss_fn (:869-933) with
// _huber_loss / _mse_loss (:859-866), dpo_pair_logratios (:796-841).
//
// fp32 per-token arithmetic in the order of the reference's tensor expressions (compiled with
// -ffp-contract=off); sums are fp64 block partials reduced in a fixed order. Forward and the
// closed-form gradient come out of the same pass.
#include "common.hpp"

namespace {

constexpr int AUX_THREADS = 256;
constexpr int AUX_MAX_BLOCKS = 1024;

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

int aux_grid(int64_t n, int vec = 1) {
  int64_t b = ceil_div_i64(n, (int64_t)AUX_THREADS * vec);
  if (b > AUX_MAX_BLOCKS) b = AUX_MAX_BLOCKS;
  if (b < 1) b = 1;
  return (int)b;
}

struct SeqLayout {
  const int32_t* cu;    // [n_seqs + 1] or null
  int n_seqs;
  int64_t uniform_len;  // > 0: sequence s covers [s*uniform_len, (s+1)*uniform_len)
};
DEVI int seq_of(const SeqLayout& q, int64_t t) {
  if (q.uniform_len > 0) return (int)(t / q.uniform_len);
  int lo = 0, hi = q.n_seqs;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)q.cu[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}
DEVI void seq_range(const SeqLayout& q, int s, int64_t n, int64_t& t0, int64_t& t1) {
  if (q.uniform_len > 0) { t0 = (int64_t)s * q.uniform_len; t1 = t0 + q.uniform_len; }
  else { t0 = q.cu[s]; t1 = q.cu[s + 1]; }
  if (t1 > n) t1 = n;
}

struct SumCount {
  double sum;
  long long n_valid, n_clip;
};

// Block partial of one logged statistic.
struct StatPart {
  double sum;
  float mn, mx;
};

// counters: [0] loss sum [1] masked-token count [4] clipped count [7] loss; the layout of the
// actor loss, so that its gradient-scaling entry point serves these losses too.
// denom_mode 0: sum / max(count, 1); 1: sum / count (0/0 = NaN, as torch); 2: sum / n_total.
// With statistics (stat_parts [nparts][n_stats]), block 1 + k folds statistic k into
// stats[k] = {sum, count, min, max}; count = the masked-token count for k < n_masked_stats, every
// token for the rest. Each block sums the counts itself, so one launch does everything.
__global__ __launch_bounds__(AUX_THREADS) void aux_finalize_kernel(
    const SumCount* parts, int nparts, int denom_mode, double n_total, float* loss_out, double* counters,
    const StatPart* __restrict__ stat_parts, int n_stats, int n_masked_stats, double* __restrict__ stats) {
  __shared__ double sm_d[8];
  __shared__ long long sm_l[8];
  __shared__ float sm_f[8];
  double s = 0.0;
  long long nv = 0, nc = 0;
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) {
    s += parts[i].sum; nv += parts[i].n_valid; nc += parts[i].n_clip;
  }
  s = block_sum(s, sm_d);
  nv = block_sum(nv, sm_l);
  nc = block_sum(nc, sm_l);
  if (blockIdx.x > 0) {
    const int k = blockIdx.x - 1;
    double sum = 0.0;
    float mn = pos_inf(), mx = neg_inf();
    for (int i = threadIdx.x; i < nparts; i += blockDim.x) {
      const StatPart sp = stat_parts[(size_t)i * n_stats + k];
      sum += sp.sum;
      mn = stat_min(mn, sp.mn);
      mx = stat_max(mx, sp.mx);
    }
    sum = block_sum(sum, sm_d);
    mn = wave_stat_min(mn);
    mx = wave_stat_max(mx);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) { sm_f[w] = mn; sm_f[4 + w] = mx; }
    __syncthreads();
    if (threadIdx.x == 0) {
      mn = stat_min(stat_min(sm_f[0], sm_f[1]), stat_min(sm_f[2], sm_f[3]));
      mx = stat_max(stat_max(sm_f[4], sm_f[5]), stat_max(sm_f[6], sm_f[7]));
      stats[4 * k + 0] = sum;
      stats[4 * k + 1] = k < n_masked_stats ? (double)nv : n_total;
      stats[4 * k + 2] = (double)mn;
      stats[4 * k + 3] = (double)mx;
    }
    return;
  }
  if (threadIdx.x == 0) {
    for (int k = 0; k < 8; ++k) counters[k] = 0.0;
    counters[0] = s;
    float loss;
    if (denom_mode == 0) {
      counters[1] = (double)nv;
      loss = (float)s / (float)(nv > 0 ? nv : 1);
    } else if (denom_mode == 1) {
      // the gradient scaling divides by max(counters[1], 1): an empty mask gives NaN loss and
      // zero gradient times NaN upstream, as 0/0 does in the reference
      counters[1] = (double)nv;
      loss = (float)s / (float)nv;
    } else {
      counters[1] = n_total;
      loss = (float)s / (float)n_total;
    }
    counters[4] = (double)nc;
    counters[7] = (double)loss;
    if (loss_out) *loss_out = loss;
  }
}

// ---------------------------------------------------------------------------------------
// SAPO
// ---------------------------------------------------------------------------------------
struct SapoIO {
  const float* lp;
  const float* old;
  const float* adv;
  const uint8_t* mask;
  SeqLayout seq;
  int64_t n;
  float tau_pos, tau_neg;
  int seq_level;
  const float* seq_stat;  // [n_seqs][3]: ratio_s, mean advantage, count
  float* dlp;
  float* stat_loss;
  float* stat_ratio;
  float* stat_kl;
  float* soft_gate;
  float* gate_pos;
  float* gate_neg;
  // optional per-token inputs of the reduced statistics
  const float* entropy;
  const float* extra0;
  const float* extra1;
};
template <int N> struct IntTag { static constexpr int value = N; };

// Per-sequence geometric-mean ratio and mean advantage over the mask (one block per sequence).
__global__ __launch_bounds__(AUX_THREADS) void sapo_seq_kernel(SapoIO io, float* seq_stat) {
  __shared__ double sm_d[8];
  const int s = blockIdx.x;
  int64_t t0, t1;
  seq_range(io.seq, s, io.n, t0, t1);
  double sum_lr = 0.0, sum_adv = 0.0, cnt = 0.0;
  for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x) {
    if (io.mask[t] == 0) continue;
    cnt += 1.0;
    sum_lr += (double)(io.lp[t] - io.old[t]);
    sum_adv += (double)io.adv[t];
  }
  sum_lr = block_sum(sum_lr, sm_d);
  sum_adv = block_sum(sum_adv, sm_d);
  cnt = block_sum(cnt, sm_d);
  if (threadIdx.x == 0) {
    const float denom = (float)(cnt > 0.0 ? cnt : 1.0);
    seq_stat[3 * s + 0] = expf((float)sum_lr / denom);
    seq_stat[3 * s + 1] = (float)sum_adv / denom;
    seq_stat[3 * s + 2] = (float)cnt;
  }
}

DEVI float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

// Statistics the token pass can reduce itself (sum, min, max per block) instead of writing the
// per-token tensors: what grpo_loss_fn logs for a SAPO step (areal/trainer/ppo/actor.py:662-733,
// :735-741), the first SAPO_MASKED_STATS under the loss mask, the extras over every token.
enum {
  SS_IMPORTANCE_WEIGHT = 0, SS_APPROX_KL, SS_NEW_LOGP, SS_OLD_LOGP, SS_ENTROPY, SS_ACTOR_LOSS, SS_LOGP_DIFF,
  SS_LOGP_ABS_DIFF, SS_SOFT_GATE, SS_GATE_POS, SS_GATE_NEG, SS_EXTRA0, SS_EXTRA1, N_SAPO_STATS
};
constexpr int SAPO_MASKED_STATS = SS_EXTRA0;

// VEC tokens per thread and access (see load_f32); STATS: per-thread fp32 sums and extremes of the
// statistics above (a thread sees a few tokens; from the wave level on the sums are fp64).
template <bool STATS, int VEC>
__global__ __launch_bounds__(AUX_THREADS) void sapo_token_kernel(SapoIO io, SumCount* parts,
                                                                 StatPart* stat_parts) {
  __shared__ double sm_d[8];
  __shared__ long long sm_l[8];
  double loss_sum = 0.0;
  long long n_valid = 0;
  float st_sum[STATS ? N_SAPO_STATS : 1], st_mn[STATS ? N_SAPO_STATS : 1], st_mx[STATS ? N_SAPO_STATS : 1];
  if (STATS) {
#pragma unroll
    for (int k = 0; k < N_SAPO_STATS; ++k) { st_sum[k] = 0.f; st_mn[k] = pos_inf(); st_mx[k] = neg_inf(); }
  }
  auto stat = [&](int k, float v) {
    if (STATS) { st_sum[k] += v; st_mn[k] = stat_min(st_mn[k], v); st_mx[k] = stat_max(st_mx[k], v); }
  };
  const float scale_pos = 4.0f / io.tau_pos, scale_neg = 4.0f / io.tau_neg;
  auto group = [&](auto vec_tag, int64_t t) {
    constexpr int W = decltype(vec_tag)::value;
    bool m[W];
    float lp[W], old[W], adv[W], ent[W], x0[W], x1[W];
    load_mask<W>(io.mask, t, m);
    load_f32<W>(io.lp, t, lp);
    load_f32<W>(io.old, t, old);
    load_f32<W>(io.adv, t, adv);
    load_f32<W>(STATS ? io.entropy : nullptr, t, ent);
    load_f32<W>(STATS ? io.extra0 : nullptr, t, x0);
    load_f32<W>(STATS ? io.extra1 : nullptr, t, x1);
    float d[W], pg[W], ratio[W], kl[W], gate[W], sp[W], sn[W];
#pragma unroll
    for (int i = 0; i < W; ++i) {
      kl[i] = lp[i] - old[i];
      float a;
      if (io.seq_level) {
        // every masked token of the sequence carries the same term; the sum over them of
        // d ratio_s / d lp[t] = ratio_s / count is ratio_s
        const int s = seq_of(io.seq, t + i);
        ratio[i] = m[i] ? io.seq_stat[3 * s] : 0.0f;
        a = m[i] ? io.seq_stat[3 * s + 1] : 0.0f;
      } else {
        ratio[i] = expf(kl[i]);
        a = adv[i];
      }
      const float gp = sigmoidf(io.tau_pos * (ratio[i] - 1.0f));
      const float gn = sigmoidf(io.tau_neg * (ratio[i] - 1.0f));
      sp[i] = gp * scale_pos;
      sn[i] = gn * scale_neg;
      const bool pos = a > 0.0f;
      gate[i] = pos ? sp[i] : sn[i];
      pg[i] = (-gate[i]) * a;
      // d gate / d ratio = scale * tau * g (1 - g) = 4 g (1 - g)
      const float g = pos ? gp : gn;
      const float dgate = 4.0f * g * (1.0f - g);
      d[i] = m[i] ? ((-dgate) * a) * ratio[i] : 0.0f;
      if (m[i]) { loss_sum += (double)pg[i]; n_valid += 1; }
      if (STATS) {
        if (m[i]) {
          stat(SS_IMPORTANCE_WEIGHT, ratio[i]);
          stat(SS_APPROX_KL, kl[i]);
          stat(SS_NEW_LOGP, lp[i]);
          stat(SS_OLD_LOGP, old[i]);
          if (io.entropy) stat(SS_ENTROPY, ent[i]);
          stat(SS_ACTOR_LOSS, pg[i]);
          stat(SS_LOGP_DIFF, old[i] - lp[i]);
          stat(SS_LOGP_ABS_DIFF, fabsf(old[i] - lp[i]));
          stat(SS_SOFT_GATE, gate[i]);
          stat(SS_GATE_POS, sp[i]);
          stat(SS_GATE_NEG, sn[i]);
        }
        if (io.extra0) stat(SS_EXTRA0, x0[i]);
        if (io.extra1) stat(SS_EXTRA1, x1[i]);
      }
    }
    store_f32<W>(io.dlp, t, d);
    store_f32<W>(io.stat_loss, t, pg);
    store_f32<W>(io.stat_ratio, t, ratio);
    store_f32<W>(io.stat_kl, t, kl);
    store_f32<W>(io.soft_gate, t, gate);
    store_f32<W>(io.gate_pos, t, sp);
    store_f32<W>(io.gate_neg, t, sn);
  };
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const int64_t n_vec = io.n - io.n % VEC;
  for (int64_t t = gid * VEC; t < n_vec; t += nthreads * VEC) group(IntTag<VEC>{}, t);
  if (VEC > 1 && n_vec + gid < io.n) group(IntTag<1>{}, n_vec + gid);
  loss_sum = block_sum(loss_sum, sm_d);
  n_valid = block_sum(n_valid, sm_l);
  if (threadIdx.x == 0) parts[blockIdx.x] = SumCount{loss_sum, n_valid, 0};
  if (STATS) {
    // reduced inside each row of 16 lanes; the block's 16 row results meet in LDS and are combined
    // in a fixed order
    constexpr int NROW = AUX_THREADS / 16;
    __shared__ double sh_sum[NROW][N_SAPO_STATS];
    __shared__ float sh_mn[NROW][N_SAPO_STATS], sh_mx[NROW][N_SAPO_STATS];
    const int row = threadIdx.x >> 4;
#pragma unroll
    for (int k = 0; k < N_SAPO_STATS; ++k) {
      const double sv = row_reduce((double)st_sum[k], [](double a, double b) { return a + b; });
      const float mn = row_reduce(st_mn[k], [](float a, float b) { return stat_min(a, b); });
      const float mx = row_reduce(st_mx[k], [](float a, float b) { return stat_max(a, b); });
      if ((threadIdx.x & 15) == 0) { sh_sum[row][k] = sv; sh_mn[row][k] = mn; sh_mx[row][k] = mx; }
    }
    __syncthreads();
    if (threadIdx.x < N_SAPO_STATS) {
      const int k = threadIdx.x;
      StatPart sp{sh_sum[0][k], sh_mn[0][k], sh_mx[0][k]};
      for (int i = 1; i < NROW; ++i) {
        sp.sum += sh_sum[i][k];
        sp.mn = stat_min(sp.mn, sh_mn[i][k]);
        sp.mx = stat_max(sp.mx, sh_mx[i][k]);
      }
      stat_parts[(size_t)blockIdx.x * N_SAPO_STATS + k] = sp;
    }
  }
}

// ---------------------------------------------------------------------------------------
// Critic loss
// ---------------------------------------------------------------------------------------
DEVI float value_loss(float x, float y, int huber, float& dx) {
  if (huber) {
    const float delta = 10.0f;
    const float diff = fabsf(x - y);
    if (diff < delta) { dx = x - y; return (0.5f * diff) * diff; }
    dx = (x > y ? delta : (x < y ? -delta : 0.0f));
    return delta * (diff - 0.5f * delta);
  }
  const float e = x - y;
  dx = e;
  return (0.5f * e) * e;
}

template <int VEC>
__global__ __launch_bounds__(AUX_THREADS) void critic_token_kernel(
    const float* value, const float* old_value, const float* target, const uint8_t* mask, int64_t n,
    float eps, int huber, float* dvalue, float* stat_loss, uint8_t* clip_mask, SumCount* parts) {
  __shared__ double sm_d[8];
  __shared__ long long sm_l[8];
  double loss_sum = 0.0;
  long long n_valid = 0, n_clip = 0;
  auto group = [&](auto vec_tag, int64_t t) {
    constexpr int W = decltype(vec_tag)::value;
    bool m[W], clip[W];
    float v[W], ov[W], tg[W], dout[W], l[W];
    if (mask != nullptr) {
      load_mask<W>(mask, t, m);
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) m[i] = true;
    }
    load_f32<W>(value, t, v);
    load_f32<W>(old_value, t, ov);
    load_f32<W>(target, t, tg);
#pragma unroll
    for (int i = 0; i < W; ++i) {
      float d_orig, d_clip;
      const float l_orig = value_loss(v[i], tg[i], huber, d_orig);
      const float dv = v[i] - ov[i];
      const float dc = dv != dv ? dv : (dv < -eps ? -eps : (dv > eps ? eps : dv));
      const float vc = ov[i] + dc;
      const float l_clip = value_loss(vc, tg[i], huber, d_clip);
      // clamp passes the gradient inside the closed band; torch.max splits ties evenly
      const float pass = (dv >= -eps && dv <= eps) ? 1.0f : 0.0f;
      const float w_orig = l_orig > l_clip ? 1.0f : (l_orig == l_clip ? 0.5f : 0.0f);
      const float w_clip = l_clip > l_orig ? 1.0f : (l_orig == l_clip ? 0.5f : 0.0f);
      l[i] = (l_orig != l_orig || l_clip != l_clip) ? __builtin_nanf("") : (l_orig > l_clip ? l_orig : l_clip);
      clip[i] = (l_clip > l_orig) && m[i];
      if (m[i]) { loss_sum += (double)l[i]; n_valid += 1; }
      n_clip += clip[i];
      dout[i] = m[i] ? (w_orig * d_orig + w_clip * (d_clip * pass)) : 0.0f;
    }
    store_f32<W>(dvalue, t, dout);
    store_f32<W>(stat_loss, t, l);
    store_mask<W>(clip_mask, t, clip);
  };
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const int64_t n_vec = n - n % VEC;
  for (int64_t t = gid * VEC; t < n_vec; t += nthreads * VEC) group(IntTag<VEC>{}, t);
  if (VEC > 1 && n_vec + gid < n) group(IntTag<1>{}, n_vec + gid);
  loss_sum = block_sum(loss_sum, sm_d);
  n_valid = block_sum(n_valid, sm_l);
  n_clip = block_sum(n_clip, sm_l);
  if (threadIdx.x == 0) parts[blockIdx.x] = SumCount{loss_sum, n_valid, n_clip};
}

// ---------------------------------------------------------------------------------------
// DPO: per-sequence sums of the shifted-mask log-probabilities (fp64), one block per sequence.
// shifted_mask[t] = loss_mask[t + 1] (0 at the very end), and 0 at the last token of every
// non-empty sequence. out[s] = {sum policy, sum reference, count}.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(AUX_THREADS) void dpo_seq_kernel(const float* lp, const float* ref,
                                                              const uint8_t* mask, SeqLayout seq,
                                                              int64_t n, double* out,
                                                              uint8_t* shifted_mask) {
  __shared__ double sm_d[8];
  const int s = blockIdx.x;
  int64_t t0, t1;
  seq_range(seq, s, n, t0, t1);
  double sp = 0.0, sr = 0.0, cnt = 0.0;
  for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x) {
    const bool m = (t + 1 < t1) && (mask[t + 1] != 0);
    if (shifted_mask) shifted_mask[t] = m;
    if (!m) continue;
    // the reference multiplies in the log-probs' dtype and then widens
    sp += (double)(lp[t] * 1.0f);
    sr += (double)(ref[t] * 1.0f);
    cnt += 1.0;
  }
  sp = block_sum(sp, sm_d);
  sr = block_sum(sr, sm_d);
  cnt = block_sum(cnt, sm_d);
  if (threadIdx.x == 0) { out[3 * s] = sp; out[3 * s + 1] = sr; out[3 * s + 2] = cnt; }
}

// grad_lp[t] = shifted_mask[t] * grad_seq[seq(t)]  (fp64 upstream, fp32 out)
__global__ __launch_bounds__(AUX_THREADS) void dpo_seq_grad_kernel(const double* grad_seq,
                                                                   const uint8_t* shifted_mask,
                                                                   SeqLayout seq, int64_t n,
                                                                   float* grad_lp) {
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n;
       t += (int64_t)gridDim.x * blockDim.x)
    grad_lp[t] = shifted_mask[t] ? (float)grad_seq[seq_of(seq, t)] : 0.0f;
}


// ---------------------------------------------------------------------------------------
// M2PO second-moment mask (areal/trainer/ppo/actor.py:933-1014): among the tokens of the loss
// mask, drop the tokens with the largest m2 = (old - prox)^2 until the mean m2 of the rest is
// below the threshold (always keeping at least one). The reference sorts; here the cut is found
// by a 4 x 8-bit radix select over the bit patterns of m2 (non-negative floats order like
// unsigned integers): every pass builds a 256-bin (count, sum) histogram of the still undecided
// tokens and a single thread walks the bins upwards, keeping whole bins while the running mean
// stays below the threshold and descending into the first bin that would break it. The mean of
// the j smallest values is non-decreasing in j, so the kept set is a prefix of the ascending
// order. Ties at the cut value are kept in index order.
// ---------------------------------------------------------------------------------------
constexpr int M2_BLOCKS = 512;
constexpr int M2_FOLD = 32;  // partial histograms summed per block of m2_fold_kernel
struct M2State {
  unsigned int prefix;          // decided high bits of the cut value
  int all_kept;                 // every token kept: nothing to cut
  unsigned long long kept;      // tokens strictly below the undecided range
  double kept_sum;
  unsigned long long group;     // after the last pass: tokens equal to the cut value
  unsigned long long take;      // ... and how many of them are kept
};
DEVI unsigned int m2_key(const float* old, const float* prox, int64_t t) {
  const float d = old[t] - prox[t];
  return __float_as_uint(d * d) & 0x7fffffffu;
}
__global__ void m2_init_kernel(M2State* st) {
  st->prefix = 0; st->all_kept = 0; st->kept = 0; st->kept_sum = 0.0; st->group = 0; st->take = 0;
}
// pass with `shift` in {24, 16, 8, 0}: histogram of bits [shift, shift+8) over the tokens whose
// higher bits equal the prefix
__global__ __launch_bounds__(AUX_THREADS) void m2_hist_kernel(const float* old, const float* prox,
                                                              const uint8_t* mask, int64_t n, int shift,
                                                              const M2State* st, unsigned int* part_cnt,
                                                              double* part_sum) {
  __shared__ unsigned int h_cnt[256];
  __shared__ double h_sum[256];
  h_cnt[threadIdx.x] = 0; h_sum[threadIdx.x] = 0.0;
  __syncthreads();
  const unsigned int prefix = st->prefix;
  const bool skip = st->all_kept != 0;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n && !skip;
       t += (int64_t)gridDim.x * blockDim.x) {
    if (mask[t] == 0) continue;
    const unsigned int key = m2_key(old, prox, t);
    if (shift < 24 && (key >> (shift + 8)) != (prefix >> (shift + 8))) continue;
    const unsigned int b = (key >> shift) & 255u;
    atomicAdd(&h_cnt[b], 1u);
    atomicAdd(&h_sum[b], (double)__uint_as_float(key));
  }
  __syncthreads();
  part_cnt[(int64_t)blockIdx.x * 256 + threadIdx.x] = h_cnt[threadIdx.x];
  part_sum[(int64_t)blockIdx.x * 256 + threadIdx.x] = h_sum[threadIdx.x];
}
// Sums M2_FOLD consecutive partial histograms into one (fixed order), so that the single block of
// m2_select_kernel reads nparts / M2_FOLD of them: one CU cannot stream all the partials fast.
__global__ __launch_bounds__(256) void m2_fold_kernel(const unsigned int* part_cnt, const double* part_sum,
                                                       int nparts, unsigned long long* fold_cnt,
                                                       double* fold_sum) {
  const int i0 = blockIdx.x * M2_FOLD;
  const int i1 = i0 + M2_FOLD < nparts ? i0 + M2_FOLD : nparts;
  unsigned long long c = 0; double s = 0.0;
#pragma unroll 8
  for (int i = i0; i < i1; ++i) {
    c += part_cnt[(int64_t)i * 256 + threadIdx.x];
    s += part_sum[(int64_t)i * 256 + threadIdx.x];
  }
  fold_cnt[(int64_t)blockIdx.x * 256 + threadIdx.x] = c;
  fold_sum[(int64_t)blockIdx.x * 256 + threadIdx.x] = s;
}
// One block of M2_SELECT_THREADS: bin = thread % 256, and the partial histograms are split over
// the thread / 256 lanes of a bin, whose sums meet in LDS in a fixed order.
constexpr int M2_SELECT_THREADS = 1024;
__global__ __launch_bounds__(M2_SELECT_THREADS) void m2_select_kernel(const unsigned long long* part_cnt,
                                                                      const double* part_sum, int nparts,
                                                                      int shift, double thr, M2State* st) {
  constexpr int LANES = M2_SELECT_THREADS / 256;
  __shared__ unsigned long long cnt_l[LANES][256];
  __shared__ double sum_l[LANES][256];
  __shared__ unsigned long long cnt[256];
  __shared__ double sum[256];
  {
    const int bin = threadIdx.x & 255, q = threadIdx.x >> 8;
    unsigned long long c = 0; double s = 0.0;
#pragma unroll 8
    for (int i = q; i < nparts; i += LANES) {
      c += part_cnt[(int64_t)i * 256 + bin];
      s += part_sum[(int64_t)i * 256 + bin];
    }
    cnt_l[q][bin] = c; sum_l[q][bin] = s;
  }
  __syncthreads();
  if (threadIdx.x < 256) {
    unsigned long long c = 0; double s = 0.0;
#pragma unroll
    for (int q = 0; q < LANES; ++q) { c += cnt_l[q][threadIdx.x]; s += sum_l[q][threadIdx.x]; }
    cnt[threadIdx.x] = c; sum[threadIdx.x] = s;
  }
  __syncthreads();
  if (threadIdx.x != 0 || st->all_kept) return;
  unsigned long long C = st->kept; double S = st->kept_sum;
  int cut = -1;
  for (int b = 0; b < 256; ++b) {
    if (cnt[b] == 0) continue;
    const double mean = (S + sum[b]) / (double)(C + cnt[b]);
    if (mean < thr) { C += cnt[b]; S += sum[b]; }
    else { cut = b; break; }
  }
  if (cut < 0) { st->all_kept = 1; return; }
  st->kept = C; st->kept_sum = S;
  st->prefix |= (unsigned int)cut << shift;
  if (shift == 0) {
    // tokens equal to the cut value v: keep the largest r with (S + r v) / (C + r) < thr
    const unsigned long long g = cnt[cut];
    const double v = (double)__uint_as_float(st->prefix);
    unsigned long long r = 0;
    for (unsigned long long lo = 0, hi = g; lo < hi;) {  // bisection on r (the mean is monotone in r)
      const unsigned long long mid = lo + (hi - lo + 1) / 2;
      if ((S + (double)mid * v) / (double)(C + mid) < thr) { lo = mid; r = mid; } else { hi = mid - 1; }
    }
    if (C + r == 0) r = 1;  // the reference keeps one token when no suffix mean is below
    st->group = g; st->take = r;
  }
}
// rank of the tokens equal to the cut value, in index order: per-block counts, then offsets
__global__ __launch_bounds__(AUX_THREADS) void m2_tie_count_kernel(const float* old, const float* prox,
                                                                   const uint8_t* mask, int64_t n,
                                                                   int64_t per_block, const M2State* st,
                                                                   unsigned long long* block_eq) {
  __shared__ unsigned long long sm[8];
  const int64_t t0 = (int64_t)blockIdx.x * per_block;
  const int64_t t1 = t0 + per_block < n ? t0 + per_block : n;
  unsigned long long c = 0;
  if (!st->all_kept)
    for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x)
      c += (mask[t] != 0 && m2_key(old, prox, t) == st->prefix);
  c = block_sum(c, sm);
  if (threadIdx.x == 0) block_eq[blockIdx.x] = c;
}
__global__ __launch_bounds__(AUX_THREADS) void m2_apply_kernel(const float* old, const float* prox,
                                                               const uint8_t* mask, int64_t n,
                                                               int64_t per_block, int nblocks,
                                                               const M2State* st,
                                                               const unsigned long long* block_eq,
                                                               uint8_t* new_mask) {
  __shared__ unsigned long long sm_scan[AUX_THREADS];
  const int64_t t0 = (int64_t)blockIdx.x * per_block;
  const int64_t t1 = t0 + per_block < n ? t0 + per_block : n;
  if (st->all_kept) {
    for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x) new_mask[t] = mask[t] != 0;
    return;
  }
  const unsigned int vstar = st->prefix;
  const unsigned long long take = st->take;
  unsigned long long before = 0;  // equal tokens in earlier blocks
  for (int i = 0; i < (int)blockIdx.x; ++i) before += block_eq[i];
  // each thread owns a contiguous slice of the block's range, so ranks follow the index order
  const int64_t len = t1 - t0;
  const int64_t per_thread = (len + blockDim.x - 1) / blockDim.x;
  const int64_t a = t0 + (int64_t)threadIdx.x * per_thread;
  const int64_t b = a + per_thread < t1 ? a + per_thread : t1;
  unsigned long long mine = 0;
  for (int64_t t = a; t < b; ++t) mine += (mask[t] != 0 && m2_key(old, prox, t) == vstar);
  sm_scan[threadIdx.x] = mine;
  __syncthreads();
  for (int d = 1; d < AUX_THREADS; d <<= 1) {
    const unsigned long long v = (int)threadIdx.x >= d ? sm_scan[threadIdx.x - d] : 0;
    __syncthreads();
    sm_scan[threadIdx.x] += v;
    __syncthreads();
  }
  unsigned long long rank = before + sm_scan[threadIdx.x] - mine;
  for (int64_t t = a; t < b; ++t) {
    bool keep = false;
    if (mask[t] != 0) {
      const unsigned int key = m2_key(old, prox, t);
      if (key < vstar) keep = true;
      else if (key == vstar) { keep = rank < take; ++rank; }
    }
    new_mask[t] = keep;
  }
  (void)nblocks;
}


// ---------------------------------------------------------------------------------------
// Proximal log-prob approximations (compute_prox_logp_approximations,
// areal/trainer/ppo/actor.py:768-848): version-aware interpolation between the behaviour and
// the current policy. method 0: log-linear, 1: linear in probability space, 2: rollout.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(AUX_THREADS) void prox_approx_kernel(const float* old, const float* lp,
                                                                  const int64_t* versions, int64_t n,
                                                                  int current_version, int method,
                                                                  float* out) {
  const float v_theta = (float)current_version;
  const float v_prox = (float)(current_version - 1);
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t ver = versions[t];
    const float v_behave = (float)ver;
    const float diff = v_theta - v_behave, gap = v_prox - v_behave;
    float alpha = (diff > 0.0f && ver >= 0) ? gap / diff : 0.0f;
    alpha = alpha != alpha ? alpha : (alpha < 0.0f ? 0.0f : (alpha > 1.0f ? 1.0f : alpha));
    const float o = old[t], l = lp[t];
    float r;
    if (method == 0) r = o + alpha * (l - o);
    else if (method == 1) r = logf(((1.0f - alpha) * expf(o) + alpha * expf(l)) + 1e-10f);
    else r = o;
    out[t] = r;
  }
}

// ---------------------------------------------------------------------------------------
// Distillation terms of the actor loss (areal/trainer/ppo/actor.py:629-658), masked sums with
// the closed-form gradient w.r.t. the current log-probs.
//   mode 0 (joint KD + RL): term = (lp - teacher) * mask
//   mode 1 (pure KD, reverse KL with importance weight): term = exp(lp - old) * (teacher - lp)
//          * mask, the reward (teacher - lp) treated as a constant
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(AUX_THREADS) void distill_token_kernel(const float* lp, const float* old,
                                                                    const float* teacher,
                                                                    const uint8_t* mask, int64_t n,
                                                                    int mode, float* dlp, float* term_out,
                                                                    SumCount* parts) {
  __shared__ double sm_d[8];
  __shared__ long long sm_l[8];
  double sum = 0.0;
  long long cnt = 0;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n;
       t += (int64_t)gridDim.x * blockDim.x) {
    const float m = mask[t] != 0 ? 1.0f : 0.0f;
    float term, d;
    if (mode == 0) {
      term = (lp[t] - teacher[t]) * m;
      d = m;
    } else {
      const float reward = teacher[t] - lp[t];
      const float iw = expf(lp[t] - old[t]);
      term = (iw * reward) * m;
      d = term;  // d iw / d lp = iw
    }
    sum += (double)term;
    cnt += mask[t] != 0;
    if (dlp) dlp[t] = d;
    if (term_out) term_out[t] = term;
  }
  sum = block_sum(sum, sm_d);
  cnt = block_sum(cnt, sm_l);
  if (threadIdx.x == 0) parts[blockIdx.x] = SumCount{sum, cnt, 0};
}

}  // namespace

extern "C" {

size_t areal_aux_loss_workspace_bytes(int64_t n_tokens, int64_t n_seqs) {
  (void)n_tokens;
  if (n_seqs < 0) n_seqs = 0;
  return (size_t)AUX_MAX_BLOCKS * (sizeof(SumCount) + N_SAPO_STATS * sizeof(StatPart)) +
         (size_t)n_seqs * 3 * sizeof(float) + 256;
}

// SAPO policy loss: forward, closed-form d(loss sum)/d logprobs (to be scaled with
// areal_actor_loss_grad), per-token statistics. seq_level != 0 uses the geometric-mean ratio
// and the mean advantage of each sequence (cu_seqlens or uniform_len).
// stats (nullable) [13][4] double = {sum, count, min, max} of, in this order: importance_weight,
// approx_kl, new_logp, old_logp, entropy, actor_loss, logp_diff, logp_abs_diff, sapo_soft_gate,
// sapo_scaled_gate_pos, sapo_scaled_gate_neg (under the loss mask), extra0, extra1 (every token),
// reduced in the token pass itself; entropy / extra0 / extra1 are optional per-token inputs of it
// (a null one comes out as sum 0, min +inf, max -inf). With stats every per-token output may be
// null: a caller that logs reduced values only moves 13 bytes per token in and 4 out.
int areal_sapo_loss(const float* logprobs, const float* old_logprobs, const float* advantages,
                    const uint8_t* loss_mask, const int32_t* cu_seqlens, int64_t n_tokens,
                    int64_t n_seqs, int64_t uniform_len, float tau_pos, float tau_neg,
                    int seq_level, float* loss, float* dlogprobs, float* stat_loss,
                    float* stat_ratio, float* stat_approx_kl, float* soft_gate, float* gate_pos,
                    float* gate_neg, double* counters, const float* entropy, const float* extra0,
                    const float* extra1, double* stats, void* workspace, size_t workspace_bytes,
                    hipStream_t stream) {
  if (n_tokens < 0 || counters == nullptr) return AREAL_ERR_BAD_ARG;
  if (!(tau_pos > 0.f) || !(tau_neg > 0.f)) return AREAL_ERR_BAD_ARG;
  if (n_tokens > 0 && (!logprobs || !old_logprobs || !advantages || !loss_mask))
    return AREAL_ERR_BAD_ARG;
  if (seq_level && n_tokens > 0 && (n_seqs <= 0 || (uniform_len <= 0 && cu_seqlens == nullptr)))
    return AREAL_ERR_BAD_ARG;
  if (workspace == nullptr || workspace_bytes < areal_aux_loss_workspace_bytes(n_tokens, n_seqs))
    return AREAL_ERR_WORKSPACE;
  char* wp = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  SumCount* parts = (SumCount*)wp;
  StatPart* stat_parts = (StatPart*)(wp + (size_t)AUX_MAX_BLOCKS * sizeof(SumCount));
  float* seq_stat = (float*)(stat_parts + (size_t)AUX_MAX_BLOCKS * N_SAPO_STATS);
  const bool with_stats = stats != nullptr;
  SapoIO io{logprobs, old_logprobs, advantages, loss_mask,
            SeqLayout{cu_seqlens, (int)n_seqs, uniform_len}, n_tokens, tau_pos, tau_neg,
            seq_level, seq_stat, dlogprobs, stat_loss, stat_ratio, stat_approx_kl, soft_gate,
            gate_pos, gate_neg, with_stats ? entropy : nullptr, with_stats ? extra0 : nullptr,
            with_stats ? extra1 : nullptr};
  const bool vec4 = n_tokens >= VEC4_MIN_TOKENS && aligned_to(logprobs, 16) && aligned_to(old_logprobs, 16) &&
                    aligned_to(advantages, 16) && aligned_to(loss_mask, 4) && aligned_to(dlogprobs, 16) &&
                    aligned_to(stat_loss, 16) && aligned_to(stat_ratio, 16) && aligned_to(stat_approx_kl, 16) &&
                    aligned_to(soft_gate, 16) && aligned_to(gate_pos, 16) && aligned_to(gate_neg, 16) &&
                    aligned_to(io.entropy, 16) && aligned_to(io.extra0, 16) && aligned_to(io.extra1, 16);
  const int grid = aux_grid(n_tokens, vec4 ? 4 : 1);
  if (seq_level && n_tokens > 0) {
    hipLaunchKernelGGL(sapo_seq_kernel, dim3((unsigned)n_seqs), dim3(AUX_THREADS), 0, stream, io,
                       seq_stat);
    AREAL_CHECK_LAUNCH();
  }
  if (with_stats && vec4)
    hipLaunchKernelGGL((sapo_token_kernel<true, 4>), dim3(grid), dim3(AUX_THREADS), 0, stream, io, parts, stat_parts);
  else if (with_stats)
    hipLaunchKernelGGL((sapo_token_kernel<true, 1>), dim3(grid), dim3(AUX_THREADS), 0, stream, io, parts, stat_parts);
  else if (vec4)
    hipLaunchKernelGGL((sapo_token_kernel<false, 4>), dim3(grid), dim3(AUX_THREADS), 0, stream, io, parts, stat_parts);
  else
    hipLaunchKernelGGL((sapo_token_kernel<false, 1>), dim3(grid), dim3(AUX_THREADS), 0, stream, io, parts, stat_parts);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(aux_finalize_kernel, dim3(with_stats ? 1 + N_SAPO_STATS : 1), dim3(AUX_THREADS), 0, stream,
                     parts, grid, 0, (double)n_tokens, loss, counters, (const StatPart*)stat_parts, N_SAPO_STATS,
                     SAPO_MASKED_STATS, stats);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// Clipped PPO critic loss (mse or huber with delta 10). loss_mask may be null (plain mean).
int areal_critic_loss(const float* value, const float* old_value, const float* target_value,
                      const uint8_t* loss_mask, int64_t n, float value_eps_clip, int huber,
                      float* loss, float* dvalue, float* stat_loss, uint8_t* clip_mask,
                      double* counters, void* workspace, size_t workspace_bytes,
                      hipStream_t stream) {
  if (n < 0 || counters == nullptr) return AREAL_ERR_BAD_ARG;
  if (n > 0 && (!value || !old_value || !target_value)) return AREAL_ERR_BAD_ARG;
  if (workspace == nullptr || workspace_bytes < areal_aux_loss_workspace_bytes(n, 0))
    return AREAL_ERR_WORKSPACE;
  SumCount* parts = (SumCount*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  const bool vec4 = n >= VEC4_MIN_TOKENS && aligned_to(value, 16) && aligned_to(old_value, 16) &&
                    aligned_to(target_value, 16) && aligned_to(loss_mask, 4) && aligned_to(dvalue, 16) &&
                    aligned_to(stat_loss, 16) && aligned_to(clip_mask, 4);
  const int grid = aux_grid(n, vec4 ? 4 : 1);
  if (vec4)
    hipLaunchKernelGGL(critic_token_kernel<4>, dim3(grid), dim3(AUX_THREADS), 0, stream, value,
                       old_value, target_value, loss_mask, n, value_eps_clip, huber, dvalue,
                       stat_loss, clip_mask, parts);
  else
    hipLaunchKernelGGL(critic_token_kernel<1>, dim3(grid), dim3(AUX_THREADS), 0, stream, value,
                       old_value, target_value, loss_mask, n, value_eps_clip, huber, dvalue,
                       stat_loss, clip_mask, parts);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(aux_finalize_kernel, dim3(1), dim3(AUX_THREADS), 0, stream, parts, grid,
                     loss_mask ? 1 : 2, (double)n, loss, counters, (const StatPart*)nullptr, 0, 0,
                     (double*)nullptr);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// DPO: seq_sums [n_seqs][3] fp64 = {sum of policy log-probs, sum of reference log-probs,
// token count} over the shifted mask of each packed sequence; shifted_mask [n] is written for
// the backward.
int areal_dpo_seq_logps(const float* logprobs, const float* ref_logprobs, const uint8_t* loss_mask,
                        const int32_t* cu_seqlens, int64_t n_tokens, int64_t n_seqs,
                        double* seq_sums, uint8_t* shifted_mask, hipStream_t stream) {
  if (n_tokens < 0 || n_seqs < 0) return AREAL_ERR_BAD_ARG;
  if (n_seqs == 0) return AREAL_OK;
  if (!logprobs || !ref_logprobs || !loss_mask || !cu_seqlens || !seq_sums)
    return AREAL_ERR_BAD_ARG;
  hipLaunchKernelGGL(dpo_seq_kernel, dim3((unsigned)n_seqs), dim3(AUX_THREADS), 0, stream, logprobs,
                     ref_logprobs, loss_mask, SeqLayout{cu_seqlens, (int)n_seqs, 0}, n_tokens,
                     seq_sums, shifted_mask);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// grad_logprobs[t] = shifted_mask[t] * grad_seq[sequence of t]
int areal_dpo_seq_logps_grad(const double* grad_seq, const uint8_t* shifted_mask,
                             const int32_t* cu_seqlens, int64_t n_tokens, int64_t n_seqs,
                             float* grad_logprobs, hipStream_t stream) {
  if (n_tokens < 0 || n_seqs < 0) return AREAL_ERR_BAD_ARG;
  if (n_tokens == 0) return AREAL_OK;
  if (!grad_seq || !shifted_mask || !cu_seqlens || !grad_logprobs || n_seqs == 0)
    return AREAL_ERR_BAD_ARG;
  hipLaunchKernelGGL(dpo_seq_grad_kernel, dim3(aux_grid(n_tokens)), dim3(AUX_THREADS), 0, stream,
                     grad_seq, shifted_mask, SeqLayout{cu_seqlens, (int)n_seqs, 0}, n_tokens,
                     grad_logprobs);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

size_t areal_m2po_mask_workspace_bytes(int64_t n_tokens) {
  (void)n_tokens;
  return sizeof(M2State) + (size_t)M2_BLOCKS * 256 * (sizeof(unsigned int) + sizeof(double)) +
         (size_t)(M2_BLOCKS / M2_FOLD) * 256 * (sizeof(unsigned long long) + sizeof(double)) +
         (size_t)M2_BLOCKS * sizeof(unsigned long long) + 1024;
}

// new_mask[t] = loss_mask[t] and token t is not among the largest-m2 tokens that have to go for
// the mean of m2 = (old - prox)^2 over the rest to fall below m2_threshold (at least one token
// of a non-empty mask is kept).
int areal_m2po_mask(const float* old_logprobs, const float* proximal_logprobs,
                    const uint8_t* loss_mask, int64_t n_tokens, float m2_threshold,
                    uint8_t* new_mask, void* workspace, size_t workspace_bytes,
                    hipStream_t stream) {
  if (n_tokens < 0) return AREAL_ERR_BAD_ARG;
  if (n_tokens == 0) return AREAL_OK;
  if (!old_logprobs || !proximal_logprobs || !loss_mask || !new_mask) return AREAL_ERR_BAD_ARG;
  if (workspace == nullptr || workspace_bytes < areal_m2po_mask_workspace_bytes(n_tokens))
    return AREAL_ERR_WORKSPACE;
  char* wp = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  M2State* st = (M2State*)wp;
  double* part_sum = (double*)(wp + 256);
  unsigned int* part_cnt = (unsigned int*)(part_sum + (size_t)M2_BLOCKS * 256);
  unsigned long long* block_eq = (unsigned long long*)(part_cnt + (size_t)M2_BLOCKS * 256);
  double* fold_sum = (double*)(block_eq + M2_BLOCKS);
  unsigned long long* fold_cnt = (unsigned long long*)(fold_sum + (size_t)(M2_BLOCKS / M2_FOLD) * 256);
  int blocks = (int)ceil_div_i64(n_tokens, AUX_THREADS * 4);
  if (blocks > M2_BLOCKS) blocks = M2_BLOCKS;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(m2_init_kernel, dim3(1), dim3(1), 0, stream, st);
  AREAL_CHECK_LAUNCH();
  for (int shift = 24; shift >= 0; shift -= 8) {
    hipLaunchKernelGGL(m2_hist_kernel, dim3(blocks), dim3(AUX_THREADS), 0, stream, old_logprobs,
                       proximal_logprobs, loss_mask, n_tokens, shift, st, part_cnt, part_sum);
    AREAL_CHECK_LAUNCH();
    const int nfold = (blocks + M2_FOLD - 1) / M2_FOLD;
    hipLaunchKernelGGL(m2_fold_kernel, dim3(nfold), dim3(256), 0, stream, part_cnt, part_sum, blocks,
                       fold_cnt, fold_sum);
    AREAL_CHECK_LAUNCH();
    hipLaunchKernelGGL(m2_select_kernel, dim3(1), dim3(M2_SELECT_THREADS), 0, stream, fold_cnt, fold_sum,
                       nfold, shift, (double)m2_threshold, st);
    AREAL_CHECK_LAUNCH();
  }
  const int64_t per_block = ceil_div_i64(n_tokens, blocks);
  hipLaunchKernelGGL(m2_tie_count_kernel, dim3(blocks), dim3(AUX_THREADS), 0, stream, old_logprobs,
                     proximal_logprobs, loss_mask, n_tokens, per_block, st, block_eq);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(m2_apply_kernel, dim3(blocks), dim3(AUX_THREADS), 0, stream, old_logprobs,
                     proximal_logprobs, loss_mask, n_tokens, per_block, blocks, st, block_eq,
                     new_mask);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// out[t] = approximation of the proximal policy's log-prob from the behaviour policy's
// (old_logprobs, generated at versions[t], negative for prompt tokens) and the current one's.
// method 0 log-linear, 1 linear in probability space, 2 rollout (= old_logprobs).
int areal_prox_logp_approx(const float* old_logprobs, const float* logprobs, const int64_t* versions,
                           int64_t n_tokens, int current_version, int method, float* out,
                           hipStream_t stream) {
  if (n_tokens < 0 || method < 0 || method > 2) return AREAL_ERR_BAD_ARG;
  if (n_tokens == 0) return AREAL_OK;
  if (!old_logprobs || !logprobs || !versions || !out) return AREAL_ERR_BAD_ARG;
  hipLaunchKernelGGL(prox_approx_kernel, dim3(aux_grid(n_tokens)), dim3(AUX_THREADS), 0, stream,
                     old_logprobs, logprobs, versions, n_tokens, current_version, method, out);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// value = sum(term) / max(count(mask), 1), dlogprobs = d(sum)/d logprobs, term per token; mode 0:
// (logprobs - teacher) * mask; mode 1: exp(logprobs - old) * (teacher - logprobs) * mask with the
// second factor held constant. counters as in areal_sapo_loss.
int areal_distill_terms(const float* logprobs, const float* old_logprobs, const float* teacher_logprobs,
                        const uint8_t* loss_mask, int64_t n_tokens, int mode, float* value,
                        float* dlogprobs, float* term, double* counters, void* workspace,
                        size_t workspace_bytes, hipStream_t stream) {
  if (n_tokens < 0 || counters == nullptr || mode < 0 || mode > 1) return AREAL_ERR_BAD_ARG;
  if (n_tokens > 0 && (!logprobs || !teacher_logprobs || !loss_mask || (mode == 1 && !old_logprobs)))
    return AREAL_ERR_BAD_ARG;
  if (workspace == nullptr || workspace_bytes < areal_aux_loss_workspace_bytes(n_tokens, 0))
    return AREAL_ERR_WORKSPACE;
  SumCount* parts = (SumCount*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  const int grid = aux_grid(n_tokens);
  hipLaunchKernelGGL(distill_token_kernel, dim3(grid), dim3(AUX_THREADS), 0, stream, logprobs,
                     old_logprobs, teacher_logprobs, loss_mask, n_tokens, mode, dlogprobs, term, parts);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(aux_finalize_kernel, dim3(1), dim3(AUX_THREADS), 0, stream, parts, grid, 0, 0.0,
                     value, counters, (const StatPart*)nullptr, 0, 0, (double*)nullptr);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // extern "C"
