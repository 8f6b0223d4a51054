// Packed-sequence GAE (segmented reverse scan) and masked group/batch normalisation.
//
// GAE follows areal/trainer/ppo/gae.py:10-36 (token-level recurrence on padded [bs, L]
// tensors); here it runs on the packed layout (or on the padded layout seen as bs sequences of
// length L). Normalisation follows areal/utils/data.py:1382-1637 (class Normalization) and
// areal/utils/functional/functional.py:16-53 (masked_normalization).
//
// GAE as a scan.  Going right to left, the carried state is (A, nv) = (last advantage, next
// value) and token t applies the affine map
//     A'  = A*((1-m) + c*m) + nv*(gamma*m) + (r - v)*m        c = gamma*lambda_seq
//     nv' = nv*(1-m) + v*m
// while the last token of a sequence applies the constant map (A', nv') = (0, no_eos ? v : 0).
// Affine maps compose associatively and constant maps absorb whatever lies to their right, so
// one unsegmented suffix scan over the whole packed array gives every sequence its own
// recurrence. Maps are held in fp64 (five coefficients); outputs are rounded to fp32.
#include "common.hpp"

namespace {

constexpr int GAE_THREADS = 256;
constexpr int GAE_ITEMS = 8;
constexpr int GAE_TILE = GAE_THREADS * GAE_ITEMS;
constexpr int GAE_SEG_WAVES = GAE_THREADS / 64;  // entries per (tile, group) segment of GaeArgs::seg_stats

// R = double in the three-launch scan (maps composed over the whole array); R = float in the
// single-pass kernel, where a map spans at most one tile and the state carried from tile to
// tile stays in fp64 (each output then sees ~20 fp32 roundings, like the reference's fp32 loop
// over as many tokens).
template <class R>
struct MapT {
  R a11, a12, a22, b1, b2;
};
using Map = MapT<double>;
using MapF = MapT<float>;
template <class R>
DEVI MapT<R> map_identity_t() { return MapT<R>{R(1), R(0), R(1), R(0), R(0)}; }
DEVI Map map_identity() { return map_identity_t<double>(); }
// (f o g): apply g first, then f.
template <class R>
DEVI MapT<R> compose(const MapT<R>& f, const MapT<R>& g) {
  // explicit fma: this file is compiled without contraction (the normalisation kernels follow
  // the reference's fp32 rounding), but the maps are more exact with it and cost half
  MapT<R> r;
  r.a11 = f.a11 * g.a11;
  r.a12 = fma(f.a11, g.a12, f.a12 * g.a22);
  r.a22 = f.a22 * g.a22;
  r.b1 = fma(f.a11, g.b1, fma(f.a12, g.b2, f.b1));
  r.b2 = fma(f.a22, g.b2, f.b2);
  return r;
}
// The map of the lane that CTRL names (common.hpp); the identity where that lane lies outside
// the row of 16.
template <int CTRL, class R>
DEVI MapT<R> dpp_map(const MapT<R>& m) {
  MapT<R> r;
  r.a11 = dpp_move<CTRL>(R(1), m.a11); r.a12 = dpp_move<CTRL>(R(0), m.a12);
  r.a22 = dpp_move<CTRL>(R(1), m.a22); r.b1 = dpp_move<CTRL>(R(0), m.b1);
  r.b2 = dpp_move<CTRL>(R(0), m.b2);
  return r;
}
template <class R>
DEVI MapT<R> lane_map(const MapT<R>& m, int lane) {
  return MapT<R>{lane_value(m.a11, lane), lane_value(m.a12, lane), lane_value(m.a22, lane),
                 lane_value(m.b1, lane), lane_value(m.b2, lane)};
}
// Inclusive suffix scan inside each row of 16 lanes: lane i gets the composition of the maps of
// lanes i..15 of its row (lane i applied last). No LDS traffic: the sixteen waves of a CU would
// queue at its one LDS unit with ds_bpermute shuffles.
template <class R>
DEVI MapT<R> row_suffix_scan(MapT<R> acc) {
  acc = compose(acc, dpp_map<DPP_ROW_SHL + 1>(acc));
  acc = compose(acc, dpp_map<DPP_ROW_SHL + 2>(acc));
  acc = compose(acc, dpp_map<DPP_ROW_SHL + 4>(acc));
  acc = compose(acc, dpp_map<DPP_ROW_SHL + 8>(acc));
  return acc;
}
// Composition of the maps of all 64 lanes (lane 0 applied last), in every lane.
template <class R>
DEVI MapT<R> wave_total_map(const MapT<R>& mine) {
  const MapT<R> acc = row_suffix_scan(mine);
  return compose(lane_map(acc, 0), compose(lane_map(acc, 16), compose(lane_map(acc, 32), lane_map(acc, 48))));
}
// Inclusive suffix scan over the wave: lane i gets the composition of lanes i..63.
template <class R>
DEVI MapT<R> wave_suffix_scan(const MapT<R>& mine, MapT<R>& total) {
  const MapT<R> acc = row_suffix_scan(mine);
  const MapT<R> t0 = lane_map(acc, 0), t1 = lane_map(acc, 16), t2 = lane_map(acc, 32), t3 = lane_map(acc, 48);
  const MapT<R> r1 = compose(t2, t3);  // all that lies right of row 1
  const MapT<R> r0 = compose(t1, r1);  // right of row 0
  total = compose(t0, r0);
  const int row = (threadIdx.x & 63) >> 4;
  const MapT<R> id = map_identity_t<R>();
  MapT<R> right;
  right.a11 = row == 0 ? r0.a11 : row == 1 ? r1.a11 : row == 2 ? t3.a11 : id.a11;
  right.a12 = row == 0 ? r0.a12 : row == 1 ? r1.a12 : row == 2 ? t3.a12 : id.a12;
  right.a22 = row == 0 ? r0.a22 : row == 1 ? r1.a22 : row == 2 ? t3.a22 : id.a22;
  right.b1 = row == 0 ? r0.b1 : row == 1 ? r1.b1 : row == 2 ? t3.b1 : id.b1;
  right.b2 = row == 0 ? r0.b2 : row == 1 ? r1.b2 : row == 2 ? t3.b2 : id.b2;
  return compose(acc, right);
}

// N sums at once: one pair of barriers instead of N.
template <int N>
DEVI void block_sum_n(double (&v)[N], double* smem /* [4][N] */) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < N; ++k) v[k] = wave_sum(v[k]);
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) smem[w * N + k] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < N; ++k) {
    double r = 0.0;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) r += smem[i * N + k];
    v[k] = r;
  }
}

struct GaeArgs {
  const float* rewards;
  const float* values;
  const float* mask;         // float 0/1
  const int32_t* cu;         // [n_seqs+1] or null when uniform_len > 0
  const uint8_t* no_eos;     // [n_seqs] or null (all false)
  const float* lam_seq;      // [n_seqs] per-sequence lambda or null
  int64_t n;
  int n_seqs;
  int64_t uniform_len;
  float discount;
  float lam;
  float* adv;
  float* ret;
  int block_per_seq;         // single-pass kernel, padded rows of at least a tile: block = row
  double* row_stats;         // nullable, with block_per_seq only: [5][n_seqs] sums over each row of
                             // m, x m, m^2, m^2 x, m^2 x^2 (x = the advantage written, m = mask):
                             // the statistics pass of the normalisation that follows, for free
  // packed tile kernel with statistics: the same five sums per (tile, group) segment. goff [G+1]
  // are the groups' token offsets (a partition of [0, n)); segment (tile k, group j) lands in slot
  // k + j of seg_stats [5][seg_slots][4] (one entry per wave of the tile's block), seg_slots =
  // tiles + G. Slots no segment maps to are zeroed.
  const int64_t* goff;
  int n_groups;
  double* seg_stats;
  int64_t seg_slots;
};

DEVI int gae_seq_of(const GaeArgs& g, int64_t t) {
  if (g.uniform_len > 0) return (int)(t / g.uniform_len);
  int lo = 0, hi = g.n_seqs;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)g.cu[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}
DEVI int64_t gae_seq_end(const GaeArgs& g, int s) {
  return g.uniform_len > 0 ? (int64_t)(s + 1) * g.uniform_len : (int64_t)g.cu[s + 1];
}

// Maps of the thread's GAE_ITEMS consecutive tokens starting at t0 (identity beyond n).
DEVI void load_maps(const GaeArgs& g, int64_t t0, Map (&mp)[GAE_ITEMS], float (&v)[GAE_ITEMS]) {
  if (t0 >= g.n) {
#pragma unroll
    for (int i = 0; i < GAE_ITEMS; ++i) { mp[i] = map_identity(); v[i] = 0.f; }
    return;
  }
  float rw[GAE_ITEMS], ms[GAE_ITEMS];
  if (t0 + GAE_ITEMS <= g.n) {  // t0 is a multiple of GAE_ITEMS: 16-byte aligned vector loads
#pragma unroll
    for (int q = 0; q < GAE_ITEMS / 4; ++q) {
      const f32x4 a = *(const f32x4*)(g.rewards + t0 + 4 * q);
      const f32x4 b = *(const f32x4*)(g.values + t0 + 4 * q);
      const f32x4 c = *(const f32x4*)(g.mask + t0 + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) { rw[4 * q + e] = a[e]; v[4 * q + e] = b[e]; ms[4 * q + e] = c[e]; }
    }
  } else {
#pragma unroll
    for (int i = 0; i < GAE_ITEMS; ++i) {
      const bool in = t0 + i < g.n;
      rw[i] = in ? g.rewards[t0 + i] : 0.f;
      v[i] = in ? g.values[t0 + i] : 0.f;
      ms[i] = in ? g.mask[t0 + i] : 0.f;
    }
  }
  int s = gae_seq_of(g, t0);
  int64_t e = gae_seq_end(g, s);
#pragma unroll
  for (int i = 0; i < GAE_ITEMS; ++i) {
    const int64_t t = t0 + i;
    if (t >= g.n) { mp[i] = map_identity(); v[i] = 0.f; continue; }
    while (t >= e && s + 1 < g.n_seqs) { ++s; e = gae_seq_end(g, s); }
    const float val = v[i];
    if (t == e - 1) {
      const bool ne = g.no_eos != nullptr && g.no_eos[s] != 0;
      mp[i] = Map{0.0, 0.0, 0.0, 0.0, ne ? (double)val : 0.0};
    } else {
      const double m = (double)ms[i];
      const double lam = g.lam_seq != nullptr ? (double)g.lam_seq[s] : (double)g.lam;
      const double c = (double)g.discount * lam;
      Map f;
      f.a11 = (1.0 - m) + c * m;
      f.a12 = (double)g.discount * m;
      f.a22 = 1.0 - m;
      f.b1 = ((double)rw[i] - (double)val) * m;
      f.b2 = (double)val * m;
      mp[i] = f;
    }
  }
}

// Composition of the thread's maps: leftmost applied last.
DEVI Map thread_total(const Map (&mp)[GAE_ITEMS]) {
  Map r = mp[GAE_ITEMS - 1];
#pragma unroll
  for (int i = GAE_ITEMS - 2; i >= 0; --i) r = compose(mp[i], r);
  return r;
}

// Inclusive suffix scan over the block: returns for each thread the composition of the maps
// of threads tid..blockDim-1 (thread tid applied last). smem: one slot per wave.
template <class R>
DEVI MapT<R> block_suffix_scan(MapT<R> mine, MapT<R>* smem, MapT<R>& block_total) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  MapT<R> wave_total;
  const MapT<R> acc = wave_suffix_scan(mine, wave_total);
  __syncthreads();
  if (lane == 0) smem[w] = wave_total;
  __syncthreads();
  const int nw = blockDim.x >> 6;
  MapT<R> right = map_identity_t<R>();
  for (int i = nw - 1; i > w; --i) right = compose(smem[i], right);
  MapT<R> tot = right;
  for (int i = w; i >= 0; --i) tot = compose(smem[i], tot);
  block_total = tot;
  return compose(acc, right);
}

__global__ __launch_bounds__(GAE_THREADS) void gae_block_total_kernel(GaeArgs g, Map* totals) {
  __shared__ Map smem[4];
  const int64_t t0 = (int64_t)blockIdx.x * GAE_TILE + (int64_t)threadIdx.x * GAE_ITEMS;
  Map mp[GAE_ITEMS];
  float v[GAE_ITEMS];
  load_maps(g, t0, mp, v);
  Map total;
  block_suffix_scan(thread_total(mp), smem, total);
  if (threadIdx.x == 0) totals[blockIdx.x] = total;
}

// carry[b] = state (A, nv) entering block b from its right = (F_{b+1} o F_{b+2} o ...)(0, 0).
__global__ __launch_bounds__(GAE_THREADS) void gae_carry_kernel(const Map* totals, int nblocks,
                                                                double* carry) {
  __shared__ Map smem[4];
  const int per = (nblocks + GAE_THREADS - 1) / GAE_THREADS;
  const int b0 = threadIdx.x * per;
  // composition of this thread's blocks b0 .. b0+per-1
  Map mine = map_identity();
  for (int i = per - 1; i >= 0; --i) {
    const int b = b0 + i;
    if (b < nblocks) mine = compose(totals[b], mine);
  }
  Map total;
  const Map incl = block_suffix_scan(mine, smem, total);
  // exclusive: composition of everything right of this thread's range
  Map excl;
  {
    // incl = mine o right  =>  right is what enters after this thread's range; recompute it
    // from the neighbour: thread tid+1's inclusive scan equals our exclusive one.
    __shared__ Map all[GAE_THREADS];
    all[threadIdx.x] = incl;
    __syncthreads();
    excl = threadIdx.x + 1 < blockDim.x ? all[threadIdx.x + 1] : map_identity();
  }
  // walk this thread's blocks right to left
  double A = excl.b1, nv = excl.b2;  // map applied to the zero state
  for (int i = per - 1; i >= 0; --i) {
    const int b = b0 + i;
    if (b >= nblocks) continue;
    carry[2 * b] = A;
    carry[2 * b + 1] = nv;
    const Map f = totals[b];
    const double A2 = fma(f.a11, A, fma(f.a12, nv, f.b1));
    const double nv2 = fma(f.a22, nv, f.b2);
    A = A2; nv = nv2;
  }
}

__global__ __launch_bounds__(GAE_THREADS) void gae_apply_kernel(GaeArgs g, const double* carry) {
  __shared__ Map smem[4];
  __shared__ Map all[GAE_THREADS];
  const int64_t t0 = (int64_t)blockIdx.x * GAE_TILE + (int64_t)threadIdx.x * GAE_ITEMS;
  Map mp[GAE_ITEMS];
  float v[GAE_ITEMS];
  load_maps(g, t0, mp, v);
  Map total;
  const Map incl = block_suffix_scan(thread_total(mp), smem, total);
  all[threadIdx.x] = incl;
  __syncthreads();
  const Map excl = threadIdx.x + 1 < blockDim.x ? all[threadIdx.x + 1] : map_identity();
  const double A0 = carry[2 * blockIdx.x], nv0 = carry[2 * blockIdx.x + 1];
  double A = excl.a11 * A0 + excl.a12 * nv0 + excl.b1;
  double nv = excl.a22 * nv0 + excl.b2;
#pragma unroll
  for (int i = GAE_ITEMS - 1; i >= 0; --i) {
    const int64_t t = t0 + i;
    if (t >= g.n) continue;
    const Map& f = mp[i];
    const double A2 = fma(f.a11, A, fma(f.a12, nv, f.b1));
    const double nv2 = fma(f.a22, nv, f.b2);
    A = A2; nv = nv2;
    const float a = (float)A;
    g.adv[t] = a;
    g.ret[t] = a + v[i];
  }
}

// ---------------------------------------------------------------------------------------
// Single-pass GAE: one launch, every token read once and written once (20 B/token), no block
// waits for another. Sequences are independent, so nothing enters a sequence's last token from
// its right. Two kernels:
//  * padded rows (gae_owned_kernel): block b owns the rows whose END lies in the token range
//    (b*TILE, (b+1)*TILE] (one block per row when rows are at least a tile long) and walks them
//    right to left tile by tile, carrying (A, nv) across its tiles;
//  * packed sequences (gae_tile_kernel): block = tile; the state entering the tile is recomputed
//    from the crossing sequence's remaining tokens.
// Tiles are absolute multiples of TILE, so the 16-byte loads stay aligned. The host picks the
// three-launch scan above when sequences are long on average.
// ---------------------------------------------------------------------------------------

// One tile of the single-pass kernels: the block's 256 threads take 8 consecutive tokens each
// of tile `tile` (tokens [tile * TILE, (tile + 1) * TILE)), of which [t_begin, t_end) are this
// block's to write. cu_own[i] = cu[s_first + i] for i in [0, n_own] covers every sequence that
// holds one of those tokens (cu_own[0] <= t_begin, cu_own[n_own] >= t_end); with uniform rows
// cu_own is unused. (A0, nv0) is the fp64 state entering the tile from its right and is replaced
// by the state leaving it on the left. rs: the row sums of GaeArgs::row_stats (STATS only).
// oa receives the advantages of the thread's owned tokens (zero elsewhere).
// The thread's 8 consecutive tokens from t0 (a multiple of 8) as raw inputs; zeros where `want`
// is false and beyond the array.
DEVI void gae_load_items(const GaeArgs& g, int64_t t0, bool want, float (&rw)[GAE_ITEMS],
                         float (&v)[GAE_ITEMS], float (&ms)[GAE_ITEMS]) {
#pragma unroll
  for (int i = 0; i < GAE_ITEMS; ++i) { rw[i] = 0.f; v[i] = 0.f; ms[i] = 0.f; }
  if (!want) return;
  if (t0 + GAE_ITEMS <= g.n) {
#pragma unroll
    for (int q = 0; q < GAE_ITEMS / 4; ++q) {
      const f32x4 a = *(const f32x4*)(g.rewards + t0 + 4 * q);
      const f32x4 b = *(const f32x4*)(g.values + t0 + 4 * q);
      const f32x4 c = *(const f32x4*)(g.mask + t0 + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) { rw[4 * q + e] = a[e]; v[4 * q + e] = b[e]; ms[4 * q + e] = c[e]; }
    }
  } else {
#pragma unroll
    for (int i = 0; i < GAE_ITEMS; ++i) {
      const bool in = t0 + i < g.n;
      rw[i] = in ? g.rewards[t0 + i] : 0.f;
      v[i] = in ? g.values[t0 + i] : 0.f;
      ms[i] = in ? g.mask[t0 + i] : 0.f;
    }
  }
}

// local indices [i_lo, i_hi) of the thread's 8 tokens from t0 that lie in [t_begin, t_end)
DEVI void gae_owned_items(int64_t t0, int64_t t_begin, int64_t t_end, int& i_lo, int& i_hi) {
  const int64_t d_lo = t_begin - t0, d_hi = t_end - t0;
  i_lo = d_lo > 0 ? (d_lo < GAE_ITEMS ? (int)d_lo : GAE_ITEMS) : 0;
  i_hi = d_hi < GAE_ITEMS ? (d_hi > 0 ? (int)d_hi : 0) : GAE_ITEMS;
}

// How a tile finds its sequences: in cu_seqlens, as rows of uniform length, or as part of the one
// row the block walks.
enum { GAE_LAYOUT_CU = 0, GAE_LAYOUT_ROWS = 1, GAE_LAYOUT_ONE_ROW = 2 };

// (rw, v, ms): the tile's inputs as gae_load_items leaves them (at least the owned tokens).
// LAMBDAS: a lambda per sequence (GaeArgs::lam_seq).
template <bool STATS, int LAYOUT, bool LAMBDAS>
DEVI void gae_one_tile(const GaeArgs& g, int64_t tile, int64_t t_begin, int64_t t_end, int s_first,
                       int n_own, const int32_t* cu_own, double& A0, double& nv0,
                       double (&rs)[STATS ? 5 : 1], MapF* smem, MapF* all,
                       const float (&rw)[GAE_ITEMS], const float (&v)[GAE_ITEMS],
                       const float (&ms)[GAE_ITEMS], float (&oa)[GAE_ITEMS]) {
  constexpr bool uniform = LAYOUT != GAE_LAYOUT_CU;
  const int tid = threadIdx.x;
  const int64_t t0 = tile * GAE_TILE + (int64_t)tid * GAE_ITEMS;
  // The thread keeps its 8 tokens as raw inputs plus two bit masks and rebuilds a token's map
  // where it is needed (twice): holding 8 maps would cost a wave of occupancy.
  float lm[LAMBDAS ? GAE_ITEMS : 1], mm[GAE_ITEMS];
  unsigned valid = 0, ends = 0, boot = 0;  // bit i: token owned / last of its sequence / no_eos
  int i_lo, i_hi;  // owned tokens of this thread
  gae_owned_items(t0, t_begin, t_end, i_lo, i_hi);
  const bool any = i_lo < i_hi;
  if (LAMBDAS) {
#pragma unroll
    for (int i = 0; i < (LAMBDAS ? GAE_ITEMS : 1); ++i) lm[i] = g.lam;
  }
  if (any) {
    // sequence of the first owned token of this thread (index relative to s_first)
    const int64_t tf = t0 + i_lo;
    int sq;
    int e_loc;  // local index one past the last token of sequence sq (clamped)
    if (LAYOUT == GAE_LAYOUT_ONE_ROW) {
      sq = 0;
      const int64_t e = t_end - t0;
      e_loc = e < 2 * GAE_ITEMS ? (int)e : 2 * GAE_ITEMS;
    } else if (LAYOUT == GAE_LAYOUT_ROWS) {
      sq = (int)(tf / g.uniform_len) - s_first;
      const int64_t e = (int64_t)(sq + s_first + 1) * g.uniform_len - t0;
      e_loc = e < 2 * GAE_ITEMS ? (int)e : 2 * GAE_ITEMS;
    } else {
      int a = 0, b = n_own;  // cu_own[a] <= tf < cu_own[b]
      while (b - a > 1) {
        const int mid = (a + b) >> 1;
        if ((int64_t)cu_own[mid] <= tf) a = mid; else b = mid;
      }
      sq = a;
      const int64_t e = (int64_t)cu_own[sq + 1] - t0;
      e_loc = e < 2 * GAE_ITEMS ? (int)e : 2 * GAE_ITEMS;
    }
    valid = ((1u << i_hi) - 1u) & ~((1u << i_lo) - 1u);
    if (e_loc > i_hi && !LAMBDAS) {
      // common case: all owned tokens inside one sequence, none of them its last
    } else {
      // a sequence ends among these tokens (or lambda is per sequence): walk them
      for (int i = i_lo; i < i_hi; ++i) {
        while (i >= e_loc && sq + 1 < n_own) {
          ++sq;
          const int64_t e = (uniform ? (int64_t)(sq + s_first + 1) * g.uniform_len
                                     : (int64_t)cu_own[sq + 1]) - t0;
          e_loc = e < 2 * GAE_ITEMS ? (int)e : 2 * GAE_ITEMS;
        }
        if (LAMBDAS) {
          const float l = g.lam_seq[s_first + sq];
#pragma unroll
          for (int k = 0; k < (LAMBDAS ? GAE_ITEMS : 1); ++k) if (k == i) lm[k] = l;
        }
        if (i == e_loc - 1) {
          ends |= 1u << i;
          if (g.no_eos != nullptr && g.no_eos[s_first + sq] != 0) boot |= 1u << i;
        }
      }
    }
  }
  // not owned: identity (mask 0 with no offsets)
#pragma unroll
  for (int i = 0; i < GAE_ITEMS; ++i) mm[i] = ((valid >> i) & 1u) ? ms[i] : 0.f;
  const float gam = g.discount;
  const float c0 = gam * g.lam;
  // few waves hold the last token of a sequence: the others skip its constant map by a scalar branch
  const bool wave_has_end = __builtin_amdgcn_ballot_w64(ends != 0) != 0;
  auto token_map = [&](int i) -> MapF {
    const float val = v[i];
    const float m = mm[i];
    const float c = LAMBDAS ? gam * lm[LAMBDAS ? i : 0] : c0;
    MapF f;
    f.a11 = fmaf(c, m, 1.f - m);
    f.a12 = gam * m;
    f.a22 = 1.f - m;
    f.b1 = (rw[i] - val) * m;
    f.b2 = val * m;
    if (wave_has_end) {
      if ((ends >> i) & 1u) f = MapF{0.f, 0.f, 0.f, 0.f, ((boot >> i) & 1u) ? val : 0.f};
    }
    return f;
  };
  MapF mine = token_map(GAE_ITEMS - 1);
#pragma unroll
  for (int i = GAE_ITEMS - 2; i >= 0; --i) mine = compose(token_map(i), mine);
  MapF total;
  const MapF incl = block_suffix_scan(mine, smem, total);
  all[tid] = incl;
  __syncthreads();
  const MapF excl = tid + 1 < GAE_THREADS ? all[tid + 1] : map_identity_t<float>();
  // the state entering this thread's tokens: the fp32 map of everything to its right in the
  // tile applied to the fp64 state entering the tile
  float A = (float)fma((double)excl.a11, A0, fma((double)excl.a12, nv0, (double)excl.b1));
  float nv = (float)fma((double)excl.a22, nv0, (double)excl.b2);
#pragma unroll
  for (int i = 0; i < GAE_ITEMS; ++i) oa[i] = 0.f;
  if (any) {
    float orr[GAE_ITEMS];
#pragma unroll
    for (int i = GAE_ITEMS - 1; i >= 0; --i) {
      const MapF f = token_map(i);
      const float A2 = fmaf(f.a11, A, fmaf(f.a12, nv, f.b1));
      const float nv2 = fmaf(f.a22, nv, f.b2);
      A = A2; nv = nv2;
      oa[i] = A;
      orr[i] = oa[i] + v[i];
    }
    if constexpr (STATS) {
#pragma unroll
      for (int i = 0; i < GAE_ITEMS; ++i) {
        if (!((valid >> i) & 1u) || ms[i] == 0.f) continue;
        const double x = (double)oa[i];
        if (ms[i] == 1.f) {  // the usual 0/1 mask: one fp64 multiplication per token
          rs[0] += 1.0; rs[1] += x; rs[2] += 1.0; rs[3] += x; rs[4] += x * x;
        } else {
          const double m = (double)ms[i];
          const double xm = x * m, mm = m * m;
          rs[0] += m; rs[1] += xm; rs[2] += mm; rs[3] += xm * m; rs[4] += xm * xm;
        }
      }
    }
    if (valid == (1u << GAE_ITEMS) - 1u) {
#pragma unroll
      for (int q = 0; q < GAE_ITEMS / 4; ++q) {
        *(f32x4*)(g.adv + t0 + 4 * q) = f32x4{oa[4 * q], oa[4 * q + 1], oa[4 * q + 2], oa[4 * q + 3]};
        *(f32x4*)(g.ret + t0 + 4 * q) = f32x4{orr[4 * q], orr[4 * q + 1], orr[4 * q + 2], orr[4 * q + 3]};
      }
    } else {
#pragma unroll
      for (int i = 0; i < GAE_ITEMS; ++i)
        if ((valid >> i) & 1u) { g.adv[t0 + i] = oa[i]; g.ret[t0 + i] = orr[i]; }
    }
  }
  // state entering the next tile on the left
  const double A1 = fma((double)total.a11, A0, fma((double)total.a12, nv0, (double)total.b1));
  const double nv1 = fma((double)total.a22, nv0, (double)total.b2);
  A0 = A1; nv0 = nv1;
}

// (Blocks of 1024 threads, one 8192-token tile per padded row instead of four serial tiles of
// 2048, measured slower: 46.7 against 30.8 us on [1024, 8192]; one such block fills a CU's
// registers and the latency of its single pass is not covered by anything.)
// STATS: also sum each row's advantages under the mask (block = row only), see GaeArgs::row_stats.
// ONE_ROW: block = row (GaeArgs::block_per_seq); LAMBDAS: a lambda per row.
template <bool STATS, bool ONE_ROW, bool LAMBDAS>
__global__ __launch_bounds__(GAE_THREADS, 4) void gae_owned_kernel(GaeArgs g) {
  __shared__ MapF smem[GAE_THREADS / 64];
  __shared__ MapF all[GAE_THREADS];
  const int tid = threadIdx.x;
  // Workgroups go to the 8 XCDs round-robin by id. Giving XCD x the x-th eighth of the token
  // ranges keeps neighbouring ranges on one XCD.
  const int64_t per_xcd = (gridDim.x + 7) >> 3;
  const int64_t range = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  // rows of at least a tile: only every (L / TILE)-th range would own a row, so the grid is one
  // block per row instead, (lo, hi] = the range holding the row's end
  const int64_t lo = ONE_ROW ? ((int64_t)(blockIdx.x + 1) * g.uniform_len - 1)
                                     : range * GAE_TILE;
  if (!ONE_ROW && (range >= per_xcd * 8 || lo >= g.n)) return;
  const int64_t hi = ONE_ROW ? lo + 1 : (lo + GAE_TILE < g.n ? lo + GAE_TILE : g.n);
  // owned rows [s_first, s_last]: lo < end(s) <= hi
  const int s_first = (int)(lo / g.uniform_len);
  const int s_last = (int)(hi / g.uniform_len) - 1;
  if (s_first > s_last) return;  // uniform for the block
  const int n_own = s_last - s_first + 1;
  const int64_t t_begin = (int64_t)s_first * g.uniform_len;
  const int64_t t_end = (int64_t)(s_last + 1) * g.uniform_len;

  double A0 = 0.0, nv0 = 0.0;  // state entering the current tile from its right
  double rs[STATS ? 5 : 1] = {0.0};
  for (int64_t tile = (t_end - 1) / GAE_TILE; tile >= t_begin / GAE_TILE; --tile) {
    const int64_t t0 = tile * GAE_TILE + (int64_t)tid * GAE_ITEMS;
    int i_lo, i_hi;
    gae_owned_items(t0, t_begin, t_end, i_lo, i_hi);
    float rw[GAE_ITEMS], v[GAE_ITEMS], ms[GAE_ITEMS], oa[GAE_ITEMS];
    gae_load_items(g, t0, i_lo < i_hi, rw, v, ms);
    gae_one_tile<STATS, ONE_ROW ? GAE_LAYOUT_ONE_ROW : GAE_LAYOUT_ROWS, LAMBDAS>(
        g, tile, t_begin, t_end, s_first, n_own, nullptr, A0, nv0, rs, smem, all, rw, v, ms, oa);
  }
  if constexpr (STATS) {  // block = row: uniform for the block
    __shared__ double s_rs[4 * 5];
    block_sum_n<5>(rs, s_rs);
    if (tid == 0) {
#pragma unroll
      for (int k = 0; k < 5; ++k) g.row_stats[(int64_t)k * g.n_seqs + blockIdx.x] = rs[k];
    }
  }
}

// Single-pass GAE for packed sequences of ordinary length, one block per tile. What enters the
// tile from its right is the state of the sequence that crosses the tile's right edge, and it
// depends only on that sequence's tokens beyond the edge: the block reads them too (rewards,
// values, mask; nothing written), one tile's worth at a time, and composes their maps onto the
// zero state; a wave whose 512 tokens lie beyond the sequence's end skips its share. No block
// waits for another, and the remainder is read once per tile of the sequence, from L2 mostly:
// the blocks of an XCD are neighbours in the array. Against blocks that walk the sequences they
// own tile by tile, carrying the state (the padded-row kernel above, which also took cu_seqlens
// once): faster on 64 x 16384 tokens and on 4 x 32768, where a walking block has 16 tiles in a row.
// The kernel is bound by vector instruction issue (about 1150 vector and 250 scalar instructions
// per wave and tile on 1024 sequences of mean length 1760) with four blocks resident per CU, so
// that all blocks of a 1.8 M-token batch run at once; that leaves 128 registers. Two remainder
// tiles per round need 148 and spill 20 of them into scratch memory: 19.9 against 15.4 us.
constexpr int GAE_CARRY_BATCH = 1;
constexpr int GAE_CU_LDS = 16 * GAE_THREADS;  // entries of cu_seqlens the block can hold (>= TILE + 2)

// Groups of a tile for GaeArgs::seg_stats: those of the tile's first and last token and of the next
// tile's first token, each the number of group ends at or before the token. Waves 0..2 search
// (their loads go out with the tile's own); s_grp is valid after the block's next barrier.
DEVI void gae_tile_group_search(const GaeArgs& g, int64_t lo, int64_t hi, int* s_grp /* [3] */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave < 3) {
    const int64_t x = wave == 0 ? lo : (wave == 1 ? hi - 1 : hi);
    const int r = wave_count_le(g.goff + 1, g.n_groups, x, lane);
    if (lane == 0) s_grp[wave] = r;
  }
}

// Group bounds of a tile relative to its first token, kept in registers from the start of the
// kernel to its end: b[i] = goff[g_first + i] - lo for the first three bounds.
struct GaeTileGroups {
  int g_first, g_last, g_next;
  int64_t b[3];
};
DEVI GaeTileGroups gae_tile_groups(const GaeArgs& g, int64_t lo, const int* s_grp) {
  GaeTileGroups r;
  r.g_first = s_grp[0];
  r.g_last = s_grp[1] < g.n_groups ? s_grp[1] : g.n_groups - 1;
  r.g_next = s_grp[2];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int j = r.g_first + i <= g.n_groups ? r.g_first + i : g.n_groups;
    r.b[i] = g.goff[j] - lo;
  }
  return r;
}

// The five masked sums of the tile's advantages per group and wave (GaeArgs::seg_stats): x = oa
// (zero for tokens outside every sequence), m = the thread's 8 mask values (zero beyond the
// array). Every wave writes its own entry, so no wave waits for another. Every thread of the
// block calls it.
DEVI void gae_tile_group_stats(const GaeArgs& g, int64_t tile, int64_t lo, int64_t hi,
                               const GaeTileGroups& tg, const float (&oa)[GAE_ITEMS],
                               const float (&ms)[GAE_ITEMS]) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t rel = (int64_t)tid * GAE_ITEMS;  // the thread's first token relative to lo
  const int64_t st = GAE_SEG_WAVES * g.seg_slots;
  // the usual 0/1 mask (decided per wave): sum m^2 = sum m, sum m^2 x = sum m x, and sum m is a count
  bool other = false;
#pragma unroll
  for (int i = 0; i < GAE_ITEMS; ++i) other |= ms[i] != 0.f && ms[i] != 1.f;
  const bool binary = __builtin_amdgcn_ballot_w64(other) == 0;
  for (int gi = tg.g_first; gi <= tg.g_last; ++gi) {
    const int k = gi - tg.g_first;
    // the group's bounds relative to the thread's tokens, clamped to them
    // (selects, not an index: an indexed register array would live in scratch memory)
    const int64_t d0 = (k == 0 ? tg.b[0] : k == 1 ? tg.b[1] : k == 2 ? tg.b[2] : g.goff[gi] - lo) - rel;
    const int64_t d1 = (k == 0 ? tg.b[1] : k == 1 ? tg.b[2] : g.goff[gi + 1] - lo) - rel;
    const int i0 = d0 <= 0 ? 0 : (d0 >= GAE_ITEMS ? GAE_ITEMS : (int)d0);
    const int i1 = d1 <= 0 ? 0 : (d1 >= GAE_ITEMS ? GAE_ITEMS : (int)d1);
    double rs[5];
    if (binary) {
      int cnt = 0;
      double s1 = 0.0, s4 = 0.0;
#pragma unroll
      for (int i = 0; i < GAE_ITEMS; ++i) {
        const bool on = i >= i0 && i < i1 && ms[i] != 0.f;
        const double x = on ? (double)oa[i] : 0.0;
        cnt += on ? 1 : 0;
        s1 += x;
        s4 += x * x;
      }
      rs[0] = (double)wave_sum(cnt);
      rs[1] = wave_sum(s1);
      rs[4] = wave_sum(s4);
      rs[2] = rs[0];
      rs[3] = rs[1];
    } else {
#pragma unroll
      for (int q = 0; q < 5; ++q) rs[q] = 0.0;
#pragma unroll
      for (int i = 0; i < GAE_ITEMS; ++i) {
        const double m = (i >= i0 && i < i1) ? (double)ms[i] : 0.0;
        const double xm = (double)oa[i] * m, mm = m * m;
        rs[0] += m; rs[1] += xm; rs[2] += mm; rs[3] += xm * m; rs[4] += xm * xm;
      }
#pragma unroll
      for (int q = 0; q < 5; ++q) rs[q] = wave_sum(rs[q]);
    }
    if (lane == 0) {
#pragma unroll
      for (int q = 0; q < 5; ++q) g.seg_stats[(int64_t)q * st + GAE_SEG_WAVES * (tile + gi) + wave] = rs[q];
    }
  }
  // slots that no segment maps to: before the first tile's first group, between this tile's last
  // group and the next tile's first, and after the last tile's last group
  const int64_t z_lo = tile == 0 ? 0 : tile + tg.g_first;
  const int64_t r_lo = tile + tg.g_first, r_hi = tile + tg.g_last + 1;  // the slots written above
  const int64_t z_hi = hi < g.n ? tile + 1 + tg.g_next : g.seg_slots;
  for (int64_t j = GAE_SEG_WAVES * z_lo + tid; j < GAE_SEG_WAVES * z_hi; j += GAE_THREADS) {
    if (j >= GAE_SEG_WAVES * r_lo && j < GAE_SEG_WAVES * r_hi) continue;
#pragma unroll
    for (int q = 0; q < 5; ++q) g.seg_stats[(int64_t)q * st + j] = 0.0;
  }
}

// STATS: also leaves the per-(tile, group) sums of GaeArgs::seg_stats.
template <bool LAMBDAS, bool STATS>
__global__ __launch_bounds__(GAE_THREADS, 4) void gae_tile_kernel(GaeArgs g) {
  __shared__ MapF smem[GAE_THREADS / 64];
  __shared__ int s_grp[3];
  __shared__ MapF all[GAE_THREADS];
  __shared__ MapF s_part[GAE_THREADS / 64][GAE_CARRY_BATCH];
  __shared__ int32_t s_cu[GAE_CU_LDS];
  __shared__ int s_own[2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // XCD x (workgroup ids congruent to x modulo 8) takes the x-th eighth of the tiles
  const int64_t per_xcd = (gridDim.x + 7) >> 3;
  const int64_t tile = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int64_t lo = tile * GAE_TILE;
  if (tile >= per_xcd * 8 || lo >= g.n) return;
  const int64_t hi = lo + GAE_TILE < g.n ? lo + GAE_TILE : g.n;
  // The tile's inputs do not depend on the sequence layout: their loads go out first, together
  // with those of the layout.
  float rw[GAE_ITEMS], v[GAE_ITEMS], ms[GAE_ITEMS];
  gae_load_items(g, lo + (int64_t)tid * GAE_ITEMS, true, rw, v, ms);
  const bool cu_in_lds = g.n_seqs + 1 <= GAE_CU_LDS;
  int64_t cov_lo, cov_hi;
  if (cu_in_lds) {
    // the whole of cu_seqlens into LDS, every load in flight at once
    int32_t c[GAE_CU_LDS / GAE_THREADS];
#pragma unroll
    for (int k = 0; k < GAE_CU_LDS / GAE_THREADS; ++k) {
      const int i = tid + k * GAE_THREADS;
      c[k] = i <= g.n_seqs ? g.cu[i] : 0;
    }
    // (after the loads above are on their way: the search waits for its own)
    if constexpr (STATS) gae_tile_group_search(g, lo, hi, s_grp);
#pragma unroll
    for (int k = 0; k < GAE_CU_LDS / GAE_THREADS; ++k) s_cu[tid + k * GAE_THREADS] = c[k];
    if (tid < 2) s_own[tid] = 0;
    __syncthreads();
    cov_lo = (int64_t)s_cu[0];
    cov_hi = (int64_t)s_cu[g.n_seqs];
  } else {
    if constexpr (STATS) gae_tile_group_search(g, lo, hi, s_grp);
    cov_lo = (int64_t)g.cu[0];
    cov_hi = (int64_t)g.cu[g.n_seqs];
  }
  // tokens outside every sequence (none in a well-formed batch) are written as zero
  if (lo < cov_lo || hi > cov_hi) {
    for (int64_t t = lo + tid; t < hi; t += GAE_THREADS)
      if (t < cov_lo || t >= cov_hi) { g.adv[t] = 0.f; g.ret[t] = 0.f; }
  }
  const int64_t t_begin = lo > cov_lo ? lo : cov_lo;
  const int64_t t_end = hi < cov_hi ? hi : cov_hi;
  if (t_end <= t_begin) {  // uniform for the block
    if constexpr (STATS) {
      const float zero[GAE_ITEMS] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      __syncthreads();
      gae_tile_group_stats(g, tile, lo, hi, gae_tile_groups(g, lo, s_grp), zero, ms);
    }
    return;
  }

  // sequences holding the first and the last token of [t_begin, t_end): the number of sequence
  // ends at or before each
  const int32_t* cu_own;
  int s_first, s_last;
  if (cu_in_lds) {
    int n_lo = 0, n_hi = 0;
    for (int i = tid + 1; i <= g.n_seqs; i += GAE_THREADS) {
      const int64_t end = (int64_t)s_cu[i];
      n_lo += end <= t_begin;
      n_hi += end <= t_end - 1;
    }
    n_lo = wave_sum(n_lo);
    n_hi = wave_sum(n_hi);
    if (lane == 0) { atomicAdd(&s_own[0], n_lo); atomicAdd(&s_own[1], n_hi); }
    __syncthreads();
    s_first = s_own[0];
    s_last = s_own[1];
    cu_own = s_cu + s_first;
  } else {
    if (tid < 128) {  // one wave each
      const int r = wave_count_le(g.cu + 1, g.n_seqs, wave ? t_end - 1 : t_begin, lane);
      if (lane == 0) s_own[wave] = r;
    }
    __syncthreads();
    s_first = s_own[0];
    s_last = s_own[1];
    if (s_last - s_first + 2 <= GAE_CU_LDS) {
      for (int i = tid; i <= s_last - s_first + 1; i += GAE_THREADS) s_cu[i] = g.cu[s_first + i];
      __syncthreads();
      cu_own = s_cu;
    } else {
      cu_own = g.cu + s_first;  // only with many empty sequences
    }
  }
  const int n_own = s_last - s_first + 1;
  GaeTileGroups tg;
  if constexpr (STATS) tg = gae_tile_groups(g, lo, s_grp);  // a barrier has passed since the search

  // the crossing sequence's tokens [t_end, e): in whole tiles from t_end (a multiple of the tile
  // when e > t_end), the rightmost batch first
  double A0 = 0.0, nv0 = 0.0;
  const int64_t e = (int64_t)cu_own[n_own];
  if (e > t_end) {
    const float gam = g.discount;
    const float c = gam * (LAMBDAS ? g.lam_seq[s_last] : g.lam);
    const bool boot = g.no_eos != nullptr && g.no_eos[s_last] != 0;
    const int64_t n_right = (e - t_end + GAE_TILE - 1) / GAE_TILE;
    for (int64_t j = n_right; j > 0; j -= GAE_CARRY_BATCH) {
      const int64_t j0 = j > GAE_CARRY_BATCH ? j - GAE_CARRY_BATCH : 0;
      float rw[GAE_CARRY_BATCH][GAE_ITEMS], v[GAE_CARRY_BATCH][GAE_ITEMS], ms[GAE_CARRY_BATCH][GAE_ITEMS];
#pragma unroll
      for (int k = 0; k < GAE_CARRY_BATCH; ++k) {
        const int64_t t0 = t_end + (j0 + k) * GAE_TILE + (int64_t)tid * GAE_ITEMS;
        const bool live = j0 + k < j && t0 < e;
        if (live && t0 + GAE_ITEMS <= g.n) {
#pragma unroll
          for (int q = 0; q < GAE_ITEMS / 4; ++q) {
            const f32x4 a = *(const f32x4*)(g.rewards + t0 + 4 * q);
            const f32x4 b = *(const f32x4*)(g.values + t0 + 4 * q);
            const f32x4 m = *(const f32x4*)(g.mask + t0 + 4 * q);
#pragma unroll
            for (int x = 0; x < 4; ++x) { rw[k][4 * q + x] = a[x]; v[k][4 * q + x] = b[x]; ms[k][4 * q + x] = m[x]; }
          }
        } else {
#pragma unroll
          for (int i = 0; i < GAE_ITEMS; ++i) {
            const bool in = live && t0 + i < g.n;
            rw[k][i] = in ? g.rewards[t0 + i] : 0.f;
            v[k][i] = in ? g.values[t0 + i] : 0.f;
            ms[k][i] = in ? g.mask[t0 + i] : 0.f;
          }
        }
      }
      MapF part[GAE_CARRY_BATCH];
#pragma unroll
      for (int k = 0; k < GAE_CARRY_BATCH; ++k) {
        const int64_t t0 = t_end + (j0 + k) * GAE_TILE + (int64_t)tid * GAE_ITEMS;
        MapF acc = map_identity_t<float>();
        part[k] = acc;
        // a wave whose 512 tokens all lie beyond the sequence contributes the identity
        if (!(j0 + k < j && t0 - (int64_t)lane * GAE_ITEMS < e)) continue;
#pragma unroll
        for (int i = GAE_ITEMS - 1; i >= 0; --i) {
          const int64_t t = t0 + i;
          // beyond the sequence (or the batch): identity; its last token: the constant map
          const float m = (j0 + k < j && t < e) ? ms[k][i] : 0.f;
          MapF f;
          f.a11 = fmaf(c, m, 1.f - m);
          f.a12 = gam * m;
          f.a22 = 1.f - m;
          f.b1 = (rw[k][i] - v[k][i]) * m;
          f.b2 = v[k][i] * m;
          if (j0 + k < j && t == e - 1) f = MapF{0.f, 0.f, 0.f, 0.f, boot ? v[k][i] : 0.f};
          acc = compose(f, acc);
        }
        part[k] = wave_total_map(acc);
      }
      __syncthreads();  // the previous batch's readers are done
      if (lane == 0) {
#pragma unroll
        for (int k = 0; k < GAE_CARRY_BATCH; ++k) s_part[wave][k] = part[k];
      }
      __syncthreads();
#pragma unroll
      for (int k = GAE_CARRY_BATCH - 1; k >= 0; --k) {
        if (j0 + k >= j) continue;
        MapF tot = s_part[GAE_THREADS / 64 - 1][k];
#pragma unroll
        for (int w = GAE_THREADS / 64 - 2; w >= 0; --w) tot = compose(s_part[w][k], tot);
        const double A1 = fma((double)tot.a11, A0, fma((double)tot.a12, nv0, (double)tot.b1));
        const double nv1 = fma((double)tot.a22, nv0, (double)tot.b2);
        A0 = A1; nv0 = nv1;
      }
    }
  }
  double rs[1];
  float oa[GAE_ITEMS];
  gae_one_tile<false, GAE_LAYOUT_CU, LAMBDAS>(g, tile, t_begin, t_end, s_first, n_own, cu_own, A0, nv0, rs, smem,
                                              all, rw, v, ms, oa);
  if constexpr (STATS) gae_tile_group_stats(g, tile, lo, hi, tg, oa, ms);
}

// ---------------------------------------------------------------------------------------
// Normalisation
// ---------------------------------------------------------------------------------------
constexpr int NORM_THREADS = 256;
constexpr int SEG_APPLY_ELEMS = 16 * NORM_THREADS;  // elements per block of the apply pass after the packed GAE
enum { LEVEL_NONE = 0, LEVEL_BATCH = 1, LEVEL_GROUP = 2 };

struct NormArgs {
  const float* x;
  const float* mask;       // nullable
  int64_t n;
  const int64_t* goff;     // [G+1] element offsets of the groups (cover [0, n))
  const int64_t* grows;    // [G] rows in each group (for the singleton rules)
  int G;
  int tail_group;          // index of the group holding ungrouped tail rows, or -1
  int nsplit;              // blocks per group
  int mean_level, std_level;
  int leave1out, unbiased;
  double eps;
  double* part;            // [3][G][nsplit]: count, sum, sum of squared deviations; or, with
                           // closed_form, [5][G][nsplit]: sum m, sum x m, sum m^2, sum m^2 x, sum m^2 x^2
  float* out;
  int closed_form;         // the squared deviations come from the five sums of one statistics pass
  // closed form only: where the five sums of a group are. part_rows == 0: [5][G][nsplit], written
  // by norm_stats5_kernel. part_rows > 0: [5][part_rows], one entry per row of row_len elements
  // (written by the GAE kernel); group g owns the rows from goff[g] / row_len on, grows[g] of them.
  // part_tile > 0: [5][part_slots][4], four entries per (tile of part_tile tokens, group) segment
  // in slot tile + group (written by the packed GAE kernel, GaeArgs::seg_stats); unused slots are zero.
  int64_t part_rows, row_len;
  int64_t part_tile, part_slots;
};

DEVI double block_sum_d(double v, double* smem) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) smem[w] = v;
  __syncthreads();
  double r = 0.0;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) r += smem[i];
  return r;
}

DEVI void split_range(const NormArgs& a, int g, int sp, int64_t& lo, int64_t& hi) {
  const int64_t g0 = a.goff[g], g1 = a.goff[g + 1];
  const int64_t len = g1 - g0;
  const int64_t per = (len + a.nsplit - 1) / a.nsplit;
  lo = g0 + (int64_t)sp * per;
  hi = lo + per;
  if (hi > g1) hi = g1;
  if (lo > g1) lo = g1;
}

// Sum of one partial array over all splits of group g, computed cooperatively by the block
// (fixed order: the same tree whatever the launch).
DEVI double group_partial(const NormArgs& a, int which, int g, double* smem) {
  double r = 0.0;
  const double* p = a.part + ((int64_t)which * a.G + g) * a.nsplit;
  for (int i = threadIdx.x; i < a.nsplit; i += blockDim.x) r += p[i];
  return block_sum_d(r, smem);
}
// Sum over every group and split, computed cooperatively by the block.
DEVI double batch_partial(const NormArgs& a, int which, double* smem) {
  double r = 0.0;
  const double* p = a.part + (int64_t)which * a.G * a.nsplit;
  const int64_t tot = (int64_t)a.G * a.nsplit;
  for (int64_t i = threadIdx.x; i < tot; i += blockDim.x) r += p[i];
  return block_sum_d(r, smem);
}

struct MeanCtx {
  int level;      // LEVEL_*
  bool identity;  // singleton group with leave-one-out: mean = x
  bool zero;      // tail group, or leave-one-out with count <= 1, or empty: mean = 0
  bool loo;
  double cnt, sum;
};

DEVI MeanCtx make_mean_ctx(const NormArgs& a, int g, double* smem) {
  MeanCtx c;
  c.level = a.mean_level; c.identity = false; c.zero = false; c.loo = a.leave1out != 0;
  c.cnt = 0.0; c.sum = 0.0;
  if (a.mean_level == LEVEL_BATCH) {
    c.cnt = batch_partial(a, 0, smem);
    c.sum = batch_partial(a, 1, smem);
  } else if (a.mean_level == LEVEL_GROUP) {
    if (g == a.tail_group) { c.zero = true; return c; }
    if (a.grows[g] == 1 && c.loo) { c.identity = true; return c; }
    c.cnt = group_partial(a, 0, g, smem);
    c.sum = group_partial(a, 1, g, smem);
  } else {
    c.zero = true;
    return c;
  }
  if (c.loo) { if (c.cnt <= 1.0) c.zero = true; }
  else if (c.cnt == 0.0) c.zero = true;
  return c;
}

// Mean seen by one element, as the reference stores it: group-level means are rounded to
// fp32 (they are written into a zeros_like(x) tensor), batch-level means stay fp64.
DEVI double elem_mean(const MeanCtx& c, float x, float m, bool has_mask) {
  double mean;
  if (c.zero) mean = 0.0;
  else if (c.identity) mean = (double)x;
  else if (!c.loo) mean = c.sum / c.cnt;
  else if (!has_mask) mean = (c.sum - (double)x) / (c.cnt - 1.0);
  else {
    const double md = (double)m;
    if (md > 0.0) {
      double den = c.cnt - md;
      if (den < 1.0) den = 1.0;
      mean = (c.sum - (double)x * md) / den;
    } else {
      mean = c.sum / c.cnt;
    }
  }
  if (c.level != LEVEL_BATCH) mean = (double)(float)mean;
  return mean;
}

// pass 1: count and sum per (group, split)
__global__ __launch_bounds__(NORM_THREADS) void norm_stats1_kernel(NormArgs a) {
  __shared__ double smem[4];
  const int g = blockIdx.x, sp = blockIdx.y;
  int64_t lo, hi;
  split_range(a, g, sp, lo, hi);
  double cnt = 0.0, sum = 0.0;
  for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const double m = a.mask ? (double)a.mask[i] : 1.0;
    cnt += m;
    sum += (double)a.x[i] * m;
  }
  cnt = block_sum_d(cnt, smem);
  sum = block_sum_d(sum, smem);
  if (threadIdx.x == 0) {
    a.part[((int64_t)0 * a.G + g) * a.nsplit + sp] = cnt;
    a.part[((int64_t)1 * a.G + g) * a.nsplit + sp] = sum;
  }
}

// The only statistics pass of the two-launch form: five masked sums per (group, split). With a
// mean that is the same for every element of a group (no leave-one-out), the sum of squared
// deviations sum (x m - mean m)^2 is S(m^2 x^2) - 2 mean S(m^2 x) + mean^2 S(m^2), evaluated in
// fp64 by the apply pass with the mean exactly as the elements see it (rounded to fp32 at group
// level), so x and the mask are read once for the statistics instead of twice.
__global__ __launch_bounds__(NORM_THREADS) void norm_stats5_kernel(NormArgs a) {
  __shared__ double smem[4 * 5];
  const int g = blockIdx.x, sp = blockIdx.y;
  int64_t lo, hi;
  split_range(a, g, sp, lo, hi);
  double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0, s4 = 0.0;
  auto take = [&](float xf, float mf) {
    const double x = (double)xf, m = (double)mf;
    const double xm = x * m, mm = m * m;
    s0 += m; s1 += xm; s2 += mm; s3 += xm * m; s4 += xm * xm;
  };
  const bool has_mask = a.mask != nullptr;
  // scalar head up to a multiple of 4 elements, 16-byte loads in the middle, scalar tail
  int64_t mid_lo = (lo + 3) & ~(int64_t)3, mid_hi = hi & ~(int64_t)3;
  if (mid_lo > mid_hi) { mid_lo = hi; mid_hi = hi; }
  for (int64_t i = lo + threadIdx.x; i < mid_lo; i += blockDim.x) take(a.x[i], has_mask ? a.mask[i] : 1.0f);
  // four 16-byte loads of each array in flight per thread before the first sum needs them
  const int64_t step = 4 * (int64_t)blockDim.x;
  for (int64_t i = mid_lo + 4 * (int64_t)threadIdx.x; i < mid_hi; i += 4 * step) {
    f32x4 xv[4], mv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t j = i + u * step;
      xv[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      mv[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (j < mid_hi) {
        xv[u] = *(const f32x4*)(a.x + j);
        mv[u] = has_mask ? *(const f32x4*)(a.mask + j) : f32x4{1.f, 1.f, 1.f, 1.f};
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < 4; ++e) take(xv[u][e], mv[u][e]);
  }
  for (int64_t i = mid_hi + threadIdx.x; i < hi; i += blockDim.x)
    if (i >= mid_lo) take(a.x[i], has_mask ? a.mask[i] : 1.0f);
  double v[5] = {s0, s1, s2, s3, s4};
  block_sum_n<5>(v, smem);
  if (threadIdx.x == 0) {
    const int64_t o = (int64_t)g * a.nsplit + sp, st = (int64_t)a.G * a.nsplit;
#pragma unroll
    for (int k = 0; k < 5; ++k) a.part[k * st + o] = v[k];
  }
}

// Apply pass of the two-launch form. Every block first sums what it needs of the five partial
// arrays in one cooperative sweep (its group's five sums; the batch's count, or all five batch
// sums when a level is "batch") and one fused block reduction, then derives the mean and the
// deviation exactly as the three-launch kernels do, and streams its range with 16-byte accesses.
__global__ __launch_bounds__(NORM_THREADS) void norm_apply_cf_kernel(NormArgs a) {
  __shared__ double smem[4 * 10];
  const int g = blockIdx.x, sp = blockIdx.y;
  const bool has_mask = a.mask != nullptr;
  int64_t lo, hi;
  split_range(a, g, sp, lo, hi);
  const bool any_batch = a.mean_level == LEVEL_BATCH || a.std_level == LEVEL_BATCH;
  // The block's first 16 elements per thread are requested before the partial sums, which then
  // arrive while those loads are in flight.
  int64_t mid_lo = (lo + 3) & ~(int64_t)3, mid_hi = hi & ~(int64_t)3;
  if (mid_lo > mid_hi) { mid_lo = hi; mid_hi = hi; }
  const int64_t step = 4 * (int64_t)blockDim.x;
  f32x4 xv[4], mv[4];
  auto fetch = [&](int64_t i) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t j = i + u * step;
      xv[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      mv[u] = f32x4{1.f, 1.f, 1.f, 1.f};
      if (j < mid_hi) {
        xv[u] = *(const f32x4*)(a.x + j);
        if (has_mask) mv[u] = *(const f32x4*)(a.mask + j);
      }
    }
  };
  const int64_t i0 = mid_lo + 4 * (int64_t)threadIdx.x;
  fetch(i0);
  int64_t st, p0, pn;  // the group's partial sums: entries [p0, p0 + pn) of arrays of st entries
  if (a.part_tile > 0) {
    const int64_t g0 = a.goff[g], g1 = a.goff[g + 1];
    st = GAE_SEG_WAVES * a.part_slots;
    p0 = GAE_SEG_WAVES * (g0 / a.part_tile + g);
    pn = g1 > g0 ? GAE_SEG_WAVES * ((g1 - 1) / a.part_tile - g0 / a.part_tile + 1) : 0;
  } else if (a.part_rows > 0) {
    st = a.part_rows;
    p0 = a.goff[g] / a.row_len;
    pn = g == a.tail_group ? a.part_rows - p0 : a.grows[g];
  } else {
    st = (int64_t)a.G * a.nsplit;
    p0 = (int64_t)g * a.nsplit;
    pn = a.nsplit;
  }
  double v[10];  // group sums 0..4, batch sums 5..9
#pragma unroll
  for (int k = 0; k < 10; ++k) v[k] = 0.0;
  if (any_batch) {
    for (int64_t i = threadIdx.x; i < pn; i += blockDim.x) {
#pragma unroll
      for (int k = 0; k < 5; ++k) v[k] += a.part[k * st + p0 + i];
    }
    for (int64_t i = threadIdx.x; i < st; i += blockDim.x) {
#pragma unroll
      for (int k = 0; k < 5; ++k) v[5 + k] += a.part[k * st + i];
    }
    block_sum_n<10>(v, smem);
  } else {
    // group level only: the first wave sums the group's entries, the others wait for it
    if (threadIdx.x < 64) {
      for (int64_t i = threadIdx.x; i < pn; i += 64) {
#pragma unroll
        for (int k = 0; k < 5; ++k) v[k] += a.part[k * st + p0 + i];
      }
#pragma unroll
      for (int k = 0; k < 5; ++k) v[k] = wave_sum(v[k]);
      if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < 5; ++k) smem[k] = v[k];
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 5; ++k) v[k] = smem[k];
    v[5] = v[0];
    if (has_mask && v[0] == 0.0) {  // nothing active in the group: is anything active at all?
      double c = 0.0;
      for (int64_t i = threadIdx.x; i < st; i += blockDim.x) c += a.part[i];
      v[5] = block_sum_d(c, smem + 8);
    }
  }
  if (has_mask && v[5] == 0.0) {  // nothing active: the input is returned unchanged
    for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) a.out[i] = a.x[i];
    return;
  }
  // mean context (see make_mean_ctx; no leave-one-out here)
  MeanCtx mc;
  mc.level = a.mean_level; mc.identity = false; mc.zero = false; mc.loo = false; mc.cnt = 0.0; mc.sum = 0.0;
  if (a.mean_level == LEVEL_BATCH) { mc.cnt = v[5]; mc.sum = v[6]; if (mc.cnt == 0.0) mc.zero = true; }
  else if (a.mean_level == LEVEL_GROUP) {
    if (g == a.tail_group) mc.zero = true;
    else { mc.cnt = v[0]; mc.sum = v[1]; if (mc.cnt == 0.0) mc.zero = true; }
  } else mc.zero = true;
  const double mean = elem_mean(mc, 0.f, 1.f, false);  // one value for the whole group
  auto ss_of = [&](int base) {
    const double ss = v[base + 4] - 2.0 * mean * v[base + 3] + mean * mean * v[base + 2];
    return ss > 0.0 ? ss : 0.0;
  };
  double std_d = 1.0;
  double eps = a.eps;
  if (a.std_level == LEVEL_BATCH) {
    const double cnt = v[5], ss = ss_of(5);
    if (a.unbiased) std_d = cnt <= 1.0 ? 1.0 : sqrt(ss / (cnt - 1.0));
    else std_d = cnt == 0.0 ? 1.0 : sqrt(ss / cnt);
  } else if (a.std_level == LEVEL_GROUP) {
    if (g == a.tail_group) std_d = 0.0;
    else if (a.grows[g] == 1 && a.unbiased) std_d = 1.0;
    else {
      const double cnt = v[0], ss = ss_of(0);
      if (a.unbiased) std_d = cnt <= 1.0 ? 1.0 : sqrt(ss / (cnt - 1.0));
      else std_d = cnt == 0.0 ? 1.0 : sqrt(ss / cnt);
    }
    std_d = (double)(float)std_d;
  } else {
    eps = 0.0;
  }
  const bool mean64 = a.mean_level == LEVEL_BATCH, std64 = a.std_level == LEVEL_BATCH;
  auto one = [&](float x, float m) -> float {
    if (mean64 || std64) {
      double c = mean64 ? ((double)x - mean) : (double)(x - (float)mean);
      if (has_mask) c = mean64 ? c * (double)m : (double)((float)c * m);
      const double den = std64 ? (std_d + eps) : (double)((float)std_d + (float)eps);
      return (float)(c / den);
    }
    float c = x - (float)mean;
    if (has_mask) c = c * m;
    return c / ((float)std_d + (float)eps);
  };
  for (int64_t i = lo + threadIdx.x; i < mid_lo; i += blockDim.x) a.out[i] = one(a.x[i], has_mask ? a.mask[i] : 1.0f);
  for (int64_t i = i0; i < mid_hi; i += 4 * step) {
    if (i != i0) fetch(i);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t j = i + u * step;
      if (j >= mid_hi) break;
      f32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = one(xv[u][e], mv[u][e]);
      *(f32x4*)(a.out + j) = r;
    }
  }
  for (int64_t i = mid_hi + threadIdx.x; i < hi; i += blockDim.x)
    if (i >= mid_lo) a.out[i] = one(a.x[i], has_mask ? a.mask[i] : 1.0f);
}

// pass 2: sum of squared masked deviations per (group, split)
__global__ __launch_bounds__(NORM_THREADS) void norm_stats2_kernel(NormArgs a) {
  __shared__ double smem[4];
  const int g = blockIdx.x, sp = blockIdx.y;
  const MeanCtx mc = make_mean_ctx(a, g, smem);
  int64_t lo, hi;
  split_range(a, g, sp, lo, hi);
  double ss = 0.0;
  const bool has_mask = a.mask != nullptr;
  for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const float x = a.x[i];
    const float m = has_mask ? a.mask[i] : 1.0f;
    const double mean = elem_mean(mc, x, m, has_mask);
    const double d = has_mask ? ((double)x * (double)m - mean * (double)m) : ((double)x - mean);
    ss += d * d;
  }
  ss = block_sum_d(ss, smem);
  if (threadIdx.x == 0) a.part[((int64_t)2 * a.G + g) * a.nsplit + sp] = ss;
}

// pass 3: normalise
__global__ __launch_bounds__(NORM_THREADS) void norm_apply_kernel(NormArgs a) {
  __shared__ double smem[4];
  const int g = blockIdx.x, sp = blockIdx.y;
  const bool has_mask = a.mask != nullptr;
  int64_t lo, hi;
  split_range(a, g, sp, lo, hi);
  if (has_mask) {
    const double total = batch_partial(a, 0, smem);
    if (total == 0.0) {  // nothing active: the input is returned unchanged
      for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) a.out[i] = a.x[i];
      return;
    }
  }
  const MeanCtx mc = make_mean_ctx(a, g, smem);
  // standard deviation
  double std_d = 1.0;
  double eps = a.eps;
  if (a.std_level == LEVEL_BATCH) {
    const double cnt = batch_partial(a, 0, smem);
    const double ss = batch_partial(a, 2, smem);
    if (a.unbiased) std_d = cnt <= 1.0 ? 1.0 : sqrt(ss / (cnt - 1.0));
    else std_d = cnt == 0.0 ? 1.0 : sqrt(ss / cnt);
  } else if (a.std_level == LEVEL_GROUP) {
    if (g == a.tail_group) std_d = 0.0;
    else if (a.grows[g] == 1 && a.unbiased) std_d = 1.0;
    else {
      const double cnt = group_partial(a, 0, g, smem);
      const double ss = group_partial(a, 2, g, smem);
      if (a.unbiased) std_d = cnt <= 1.0 ? 1.0 : sqrt(ss / (cnt - 1.0));
      else std_d = cnt == 0.0 ? 1.0 : sqrt(ss / cnt);
    }
    std_d = (double)(float)std_d;
  } else {
    eps = 0.0;
  }
  const bool mean64 = a.mean_level == LEVEL_BATCH, std64 = a.std_level == LEVEL_BATCH;
  for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const float x = a.x[i];
    const float m = has_mask ? a.mask[i] : 1.0f;
    const double mean = elem_mean(mc, x, m, has_mask);
    float r;
    if (mean64 || std64) {
      double c = mean64 ? ((double)x - mean) : (double)(x - (float)mean);
      if (has_mask) c = mean64 ? c * (double)m : (double)((float)c * m);
      const double den = std64 ? (std_d + eps) : (double)((float)std_d + (float)eps);
      r = (float)(c / den);
    } else {
      float c = x - (float)mean;
      if (has_mask) c = c * m;
      r = c / ((float)std_d + (float)eps);
    }
    a.out[i] = r;
  }
}

// masked_normalization (functional.py:16-53): one group, var = E[x^2] - E[x]^2 in fp64,
// (x*mask - mean) / (sqrt(var) + eps); the centred value is not re-masked.
__global__ __launch_bounds__(NORM_THREADS) void masked_norm_stats_kernel(const float* x,
                                                                          const float* mask,
                                                                          int64_t n, double* part) {
  __shared__ double smem[4];
  double cnt = 0.0, s = 0.0, s2 = 0.0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const double m = mask ? (double)mask[i] : 1.0;
    const double v = (double)x[i] * m;
    cnt += m; s += v; s2 += v * v;
  }
  cnt = block_sum_d(cnt, smem); s = block_sum_d(s, smem); s2 = block_sum_d(s2, smem);
  if (threadIdx.x == 0) {
    part[blockIdx.x] = cnt; part[gridDim.x + blockIdx.x] = s; part[2 * gridDim.x + blockIdx.x] = s2;
  }
}
__global__ __launch_bounds__(NORM_THREADS) void masked_norm_apply_kernel(
    const float* x, const float* mask, int64_t n, const double* part, int nparts, int unbiased,
    double eps, float* out) {
  __shared__ double smem[4];
  double cnt = 0.0, s = 0.0, s2 = 0.0;
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) {
    cnt += part[i]; s += part[nparts + i]; s2 += part[2 * nparts + i];
  }
  cnt = block_sum_d(cnt, smem); s = block_sum_d(s, smem); s2 = block_sum_d(s2, smem);
  const double mean = s / cnt;
  double var = s2 / cnt - mean * mean;
  if (unbiased) var *= cnt / (cnt - 1.0);
  const double den = sqrt(var) + eps;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const double v = (double)x[i] * (mask ? (double)mask[i] : 1.0);
    out[i] = (float)((v - mean) / den);
  }
}

// The same over each row of a [rows, cols] array (masked_normalization with dim = the trailing
// dimensions): one block per row, statistics then the apply pass over the row.
__global__ __launch_bounds__(NORM_THREADS) void masked_norm_rows_kernel(
    const float* x, const float* mask, int64_t cols, int unbiased, double eps, float* out) {
  __shared__ double smem[4];
  const float* xr = x + (int64_t)blockIdx.x * cols;
  const float* mr = mask ? mask + (int64_t)blockIdx.x * cols : nullptr;
  float* o = out + (int64_t)blockIdx.x * cols;
  double cnt = 0.0, s = 0.0, s2 = 0.0;
  for (int64_t i = threadIdx.x; i < cols; i += blockDim.x) {
    const double m = mr ? (double)mr[i] : 1.0;
    const double v = (double)xr[i] * m;
    cnt += m; s += v; s2 += v * v;
  }
  cnt = block_sum_d(cnt, smem); s = block_sum_d(s, smem); s2 = block_sum_d(s2, smem);
  const double mean = s / cnt;
  double var = s2 / cnt - mean * mean;
  if (unbiased) var *= cnt / (cnt - 1.0);
  const double den = sqrt(var) + eps;
  for (int64_t i = threadIdx.x; i < cols; i += blockDim.x) {
    const double v = (double)xr[i] * (mr ? (double)mr[i] : 1.0);
    o[i] = (float)((v - mean) / den);
  }
}

// ---------------------------------------------------------------------------------------
// Reward shaping in front of GAE (PPOActor.compute_advantages, areal/trainer/ppo/actor.py:224-283):
// one pass over a padded [bs, L] batch instead of some twenty elementwise tensor ops. One block
// per row; the row's sequence length (sum of the attention mask) first, then per token t:
//   lm[t]   = float(loss_mask[(t + 1) % L])                       (torch.roll(..., -1))
//   old[t]  = logp[(t + 1) % L] * lm[t]   (logp[t] * lm[t] when the log-probs are not rolled)
//   ref[t]  = ref_logp[t] * lm[t]         (0 when there is no reference policy)
//   kl[t]   = -kl_ctl * estimator(old[t] - ref[t])                (data.py:1662-1698)
//   gkl[t]  = kl[t], zero at t = seqlen - 1
//   out[t]  = reward_score at t = max(seqlen - 2, 0), else 0 (0 everywhere for a truncated
//             row when mask_no_eos_with_zero)
//   tot[t]  = gkl[t] + out[t]
// The arithmetic follows the reference's tensor ops in their order (this file is compiled
// without floating-point contraction). Index -1 of an empty row addresses the last slot, as
// Python indexing does.
// ---------------------------------------------------------------------------------------
struct PrepArgs {
  const uint8_t* loss_mask;  // [bs, L] nonzero = 1
  const uint8_t* attn_mask;  // [bs, L]
  const float* logp;         // [bs, L]
  float* ref_logp;           // [bs, L] or null; masked in place when ref_in_place
  const float* reward_score; // [bs]
  int64_t L;
  int roll_logp;             // 1: old = roll(logp, -1); 0: old = logp
  int estimator;             // 1, 2, 3
  int apply_clamp;
  int mask_no_eos_with_zero;
  int ref_in_place;
  float kl_ctl;
  float* lm_out;             // [bs, L]
  float* old_out;            // [bs, L]
  float* kl_out;             // [bs, L]  kl rewards before the end-of-sequence zero
  float* gkl_out;            // [bs, L] or null
  float* outcome_out;        // [bs, L] or null
  float* tot_out;            // [bs, L]
  int64_t* seqlens_out;      // [bs]
  uint8_t* no_eos_out;       // [bs]
};

DEVI void adv_prep_token(const PrepArgs& a, float lm, float lp, float rf_in, bool has_ref, bool at_end,
                         bool at_out, float score, float neg_ctl, float& old, float& ref, float& kl,
                         float& gkl, float& oc) {
  old = lp * lm;
  ref = has_ref ? rf_in * lm : 0.f * lm;
  const float diff = old - ref;
  float est;
  if (a.estimator == 1) est = diff;
  else if (a.estimator == 2) est = diff * diff / 2.0f;
  else { const float neg = -diff; est = expf(neg) - 1.f - neg; }
  if (a.apply_clamp) est = fminf(fmaxf(est, -10.f), 10.f);
  kl = neg_ctl * est;
  gkl = at_end ? 0.f : kl;
  oc = at_out ? score : 0.f;
}

// VEC: L % 16 == 0 and every array 16-byte aligned: four tokens per thread and step, 16-byte
// loads and stores (the rolled neighbour of a group's last token is one extra scalar load).
template <bool VEC>
__global__ __launch_bounds__(NORM_THREADS) void adv_prep_kernel(PrepArgs a) {
  __shared__ double smem[4];
  const int64_t b = blockIdx.x, L = a.L;
  const uint8_t* am = a.attn_mask + b * L;
  const uint8_t* lmk = a.loss_mask + b * L;
  const float* lp = a.logp + b * L;
  float* rf = a.ref_logp ? a.ref_logp + b * L : nullptr;
  double cnt = 0.0;
  if (VEC) {
    for (int64_t t = (int64_t)threadIdx.x * 16; t < L; t += (int64_t)blockDim.x * 16) {
      const u32x4 w = *(const u32x4*)(am + t);
      int c = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) c += ((w[i] >> (8 * k)) & 0xffu) ? 1 : 0;
      cnt += (double)c;
    }
  } else {
    for (int64_t t = threadIdx.x; t < L; t += blockDim.x) cnt += am[t] ? 1.0 : 0.0;
  }
  const int64_t seqlen = (int64_t)block_sum_d(cnt, smem);
  const bool no_eos = seqlen == L;
  if (threadIdx.x == 0) { a.seqlens_out[b] = seqlen; a.no_eos_out[b] = no_eos ? 1 : 0; }
  const int64_t t_end = seqlen - 1 >= 0 ? seqlen - 1 : seqlen - 1 + L;  // rewards[b, seqlen - 1] = 0
  const int64_t t_out = seqlen - 2 > 0 ? seqlen - 2 : 0;                 // clip(seqlen - 2, min = 0)
  float score = a.reward_score[b];
  if (a.mask_no_eos_with_zero && no_eos) score = 0.f;
  const float neg_ctl = -a.kl_ctl;
  const bool has_ref = rf != nullptr;
  if (VEC) {
    for (int64_t t = (int64_t)threadIdx.x * 4; t < L; t += (int64_t)blockDim.x * 4) {
      const int64_t tn = t + 4 < L ? t + 4 : 0;  // the roll's neighbour of the group's last token
      const uint32_t mw = *(const uint32_t*)(lmk + t);
      const float lmv[4] = {((mw >> 8) & 0xffu) ? 1.f : 0.f, ((mw >> 16) & 0xffu) ? 1.f : 0.f,
                            (mw >> 24) ? 1.f : 0.f, lmk[tn] ? 1.f : 0.f};
      const f32x4 lv = *(const f32x4*)(lp + t);
      const float lpv[4] = {a.roll_logp ? lv[1] : lv[0], a.roll_logp ? lv[2] : lv[1],
                            a.roll_logp ? lv[3] : lv[2], a.roll_logp ? lp[tn] : lv[3]};
      f32x4 rv = {0.f, 0.f, 0.f, 0.f};
      if (has_ref) rv = *(const f32x4*)(rf + t);
      f32x4 o_lm, o_old, o_ref, o_kl, o_gkl, o_oc, o_tot;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float old, ref, kl, gkl, oc;
        adv_prep_token(a, lmv[i], lpv[i], rv[i], has_ref, t + i == t_end, t + i == t_out, score, neg_ctl,
                       old, ref, kl, gkl, oc);
        o_lm[i] = lmv[i]; o_old[i] = old; o_ref[i] = ref; o_kl[i] = kl; o_gkl[i] = gkl; o_oc[i] = oc;
        o_tot[i] = gkl + oc;
      }
      if (has_ref && a.ref_in_place) *(f32x4*)(rf + t) = o_ref;
      *(f32x4*)(a.lm_out + b * L + t) = o_lm;
      *(f32x4*)(a.old_out + b * L + t) = o_old;
      *(f32x4*)(a.kl_out + b * L + t) = o_kl;
      if (a.gkl_out) *(f32x4*)(a.gkl_out + b * L + t) = o_gkl;
      if (a.outcome_out) *(f32x4*)(a.outcome_out + b * L + t) = o_oc;
      *(f32x4*)(a.tot_out + b * L + t) = o_tot;
    }
    return;
  }
  for (int64_t t = threadIdx.x; t < L; t += blockDim.x) {
    const int64_t tn = t + 1 < L ? t + 1 : 0;
    const float lm = lmk[tn] ? 1.f : 0.f;
    float old, ref, kl, gkl, oc;
    adv_prep_token(a, lm, a.roll_logp ? lp[tn] : lp[t], has_ref ? rf[t] : 0.f, has_ref, t == t_end,
                   t == t_out, score, neg_ctl, old, ref, kl, gkl, oc);
    if (has_ref && a.ref_in_place) rf[t] = ref;
    a.lm_out[b * L + t] = lm;
    a.old_out[b * L + t] = old;
    a.kl_out[b * L + t] = kl;
    if (a.gkl_out) a.gkl_out[b * L + t] = gkl;
    if (a.outcome_out) a.outcome_out[b * L + t] = oc;
    a.tot_out[b * L + t] = gkl + oc;
  }
}

// ---------------------------------------------------------------------------------------
// Turn-level GAE (areal/trainer/ppo/gae.py:82-163): every generated turn is one timestep.
// One block per padded row. Active tokens carry non-decreasing turn ids (checked; a violation
// sets *status), so a turn starts at the first active token whose id exceeds every active id on
// its left. Pass 1 compacts the turns: start position's value, and the fp64 prefix sum of the
// active rewards taken just before the start (turn reward = difference of consecutive
// prefixes). Thread 0 then runs the recurrence over the compact turns right to left, and pass
// 2 hands every token its turn's advantage and return.
// Per row workspace: prefix [L+1] double, value/adv/ret [L] float each.
// ---------------------------------------------------------------------------------------
constexpr int TURN_THREADS = 256;
constexpr int TURN_ITEMS = 4;

struct TurnArgs {
  const float* rewards;
  const float* values;
  const float* mask;       // float loss mask, nonzero = active
  const int32_t* turn_ids;
  const uint8_t* no_eos;   // [bs] or null
  const float* lam_seq;    // [bs] or null
  int64_t bs, L;
  float discount, lam;
  float* adv;
  float* ret;
  double* ws_prefix;       // [bs][L + 1]
  float* ws_val;           // [bs][L]
  float* ws_adv;           // [bs][L]
  float* ws_ret;           // [bs][L]
  int* status;             // bit 0: negative id, bit 1: id >= L, bit 2: ids go backwards
};

struct TurnCarry { int count; int maxid; double sum; };

// Exclusive scan over the block of (start count, running max id, reward sum), chunk carry
// included. smem: [TURN_THREADS] of each.
DEVI TurnCarry turn_block_exclusive(int cnt, int mx, double sm, const TurnCarry& carry, int* s_cnt,
                                    int* s_max, double* s_sum, TurnCarry& chunk_total) {
  // s_cnt / s_max / s_sum: one entry per wave. Scans inside a wave through DPP, the waves' totals
  // through LDS: two barriers.
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int ic = wave_inclusive_scan(cnt, 0, [](int a, int b) { return a + b; });
  const int im = wave_inclusive_scan(mx, -1, [](int a, int b) { return a > b ? a : b; });
  const double is = wave_inclusive_scan(sm, 0.0, [](double a, double b) { return a + b; });
  __syncthreads();  // the previous chunk's readers are done
  if (lane == 63) { s_cnt[w] = ic; s_max[w] = im; s_sum[w] = is; }
  __syncthreads();
  TurnCarry ex = carry;
  for (int i = 0; i < w; ++i) {
    ex.count += s_cnt[i];
    ex.maxid = ex.maxid > s_max[i] ? ex.maxid : s_max[i];
    ex.sum += s_sum[i];
  }
  chunk_total = carry;
  for (int i = 0; i < TURN_THREADS / 64; ++i) {
    chunk_total.count += s_cnt[i];
    chunk_total.maxid = chunk_total.maxid > s_max[i] ? chunk_total.maxid : s_max[i];
    chunk_total.sum += s_sum[i];
  }
  // the lanes before this one in its wave
  const int pc = wave_shift_up(ic, 0), pm = wave_shift_up(im, -1);
  const double ps = wave_shift_up(is, 0.0);
  ex.count += pc;
  ex.maxid = ex.maxid > pm ? ex.maxid : pm;
  ex.sum += ps;
  return ex;
}

__global__ __launch_bounds__(TURN_THREADS) void turn_gae_kernel(TurnArgs a) {
  __shared__ int s_cnt[TURN_THREADS];
  __shared__ int s_max[TURN_THREADS];
  __shared__ double s_sum[TURN_THREADS];
  __shared__ int s_k;
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x, L = a.L;
  const float* rw = a.rewards + row * L;
  const float* vl = a.values + row * L;
  const float* ms = a.mask + row * L;
  const int32_t* id = a.turn_ids + row * L;
  double* prefix = a.ws_prefix + row * (L + 1);
  float* tval = a.ws_val + row * L;
  float* tadv = a.ws_adv + row * L;
  float* tret = a.ws_ret + row * L;
  int bad = 0;

  // ---- pass 1: compact the turns
  TurnCarry carry{0, -1, 0.0};
  for (int64_t base = 0; base < L; base += TURN_THREADS * TURN_ITEMS) {
    const int64_t t0 = base + (int64_t)tid * TURN_ITEMS;
    int ids[TURN_ITEMS]; bool act[TURN_ITEMS]; float r[TURN_ITEMS];
    int cnt = 0, mx = -1; double sm = 0.0;
    // thread-local: starts relative to the maximum seen inside the thread's own items
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      const int64_t t = t0 + i;
      act[i] = t < L && ms[t] != 0.0f;
      ids[i] = act[i] ? id[t] : -1;
      r[i] = act[i] ? rw[t] : 0.0f;
      if (act[i]) {
        if (ids[i] < 0) bad |= 1;
        if ((int64_t)ids[i] >= L) bad |= 2;
        mx = mx > ids[i] ? mx : ids[i];
        sm += (double)r[i];
      }
    }
    (void)cnt;
    // the number of starts in a thread depends on the maximum to its left, so scan the maximum
    // and the reward sums first, then count starts, then scan the counts
    TurnCarry tot1;
    const TurnCarry ex1 = turn_block_exclusive(0, mx, sm, carry, s_cnt, s_max, s_sum, tot1);
    int run_max = ex1.maxid;
    bool start[TURN_ITEMS];
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      start[i] = act[i] && ids[i] > run_max;
      if (act[i] && ids[i] < run_max) bad |= 4;
      if (act[i]) run_max = run_max > ids[i] ? run_max : ids[i];
      cnt += start[i];
    }
    TurnCarry tot2;
    const TurnCarry ex2 = turn_block_exclusive(cnt, -1, 0.0, TurnCarry{carry.count, -1, 0.0}, s_cnt,
                                               s_max, s_sum, tot2);
    int k = ex2.count;
    double run_sum = ex1.sum;
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      if (start[i]) {
        prefix[k] = run_sum;            // active rewards strictly before this turn
        tval[k] = vl[t0 + i];           // the turn's state value: value at its first token
        ++k;
      }
      run_sum += (double)r[i];
    }
    carry.count = tot2.count; carry.maxid = tot1.maxid; carry.sum = tot1.sum;
  }
  if (tid == 0) { prefix[carry.count] = carry.sum; s_k = carry.count; }
  if (bad) atomicOr(a.status, bad);
  __syncthreads();
  __threadfence_block();
  const int K = s_k;

  // ---- recurrence over the turns, right to left (gae.py:139-150)
  if (tid == 0) {
    const float gam = a.discount;
    const float lam = a.lam_seq ? a.lam_seq[row] : a.lam;
    const float c = gam * lam;
    float nextv = (a.no_eos && a.no_eos[row]) ? vl[L - 1] : 0.0f;
    float last = 0.0f;
    for (int k = K - 1; k >= 0; --k) {
      const float R = (float)(prefix[k + 1] - prefix[k]);
      const float V = tval[k];
      const float delta = (R + gam * nextv) - V;
      const float g = delta + c * last;
      tadv[k] = g;
      tret[k] = g + V;
      nextv = V;
      last = g;
    }
  }
  __syncthreads();
  __threadfence_block();

  // ---- pass 2: every token takes the result of its turn (gae.py:152-157)
  TurnCarry carry2{0, -1, 0.0};
  for (int64_t base = 0; base < L; base += TURN_THREADS * TURN_ITEMS) {
    const int64_t t0 = base + (int64_t)tid * TURN_ITEMS;
    int ids[TURN_ITEMS]; bool act[TURN_ITEMS]; float m[TURN_ITEMS];
    int mx = -1;
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      const int64_t t = t0 + i;
      m[i] = t < L ? ms[t] : 0.0f;
      act[i] = m[i] != 0.0f;
      ids[i] = act[i] ? id[t] : -1;
      if (act[i]) mx = mx > ids[i] ? mx : ids[i];
    }
    TurnCarry tot1;
    const TurnCarry ex1 = turn_block_exclusive(0, mx, 0.0, carry2, s_cnt, s_max, s_sum, tot1);
    int run_max = ex1.maxid, cnt = 0;
    bool start[TURN_ITEMS];
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      start[i] = act[i] && ids[i] > run_max;
      if (act[i]) run_max = run_max > ids[i] ? run_max : ids[i];
      cnt += start[i];
    }
    TurnCarry tot2;
    const TurnCarry ex2 = turn_block_exclusive(cnt, -1, 0.0, TurnCarry{carry2.count, -1, 0.0}, s_cnt,
                                               s_max, s_sum, tot2);
    int k = ex2.count;  // turns started strictly before this thread's first token
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      const int64_t t = t0 + i;
      if (start[i]) ++k;
      if (t >= L) continue;
      if (act[i] && k > 0) {
        const float mm = m[i];
        a.adv[row * L + t] = tadv[k - 1] * mm;
        a.ret[row * L + t] = tret[k - 1] * mm + vl[t] * (1.0f - mm);
      } else {
        a.adv[row * L + t] = 0.0f;
        a.ret[row * L + t] = vl[t];
      }
    }
    carry2.count = tot2.count; carry2.maxid = tot1.maxid;
  }
}

// Per-row lengths for the per-sample lambda functions (_build_gae_lambda_context,
// areal/trainer/ppo/gae.py:166-205): number of active tokens, and number of distinct turn ids
// among them (= turn starts, ids being non-decreasing over the active tokens; violations are
// reported through *status as in turn_gae_kernel). turn_ids may be null (turn count 0).
__global__ __launch_bounds__(TURN_THREADS) void gae_context_kernel(const float* mask,
                                                                   const int32_t* turn_ids, int64_t L,
                                                                   int64_t* token_len,
                                                                   int64_t* turn_cnt, int* status) {
  __shared__ int s_cnt[TURN_THREADS];
  __shared__ int s_max[TURN_THREADS];
  __shared__ double s_sum[TURN_THREADS];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const float* ms = mask + row * L;
  const int32_t* id = turn_ids ? turn_ids + row * L : nullptr;
  int bad = 0;
  TurnCarry carry{0, -1, 0.0};
  int64_t starts = 0;
  for (int64_t base = 0; base < L; base += TURN_THREADS * TURN_ITEMS) {
    const int64_t t0 = base + (int64_t)tid * TURN_ITEMS;
    int ids[TURN_ITEMS]; bool act[TURN_ITEMS];
    int mx = -1, nact = 0;
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      const int64_t t = t0 + i;
      act[i] = t < L && ms[t] != 0.0f;
      ids[i] = (act[i] && id) ? id[t] : -1;
      nact += act[i];
      if (act[i] && id) {
        if (ids[i] < 0) bad |= 1;
        if ((int64_t)ids[i] >= L) bad |= 2;
        mx = mx > ids[i] ? mx : ids[i];
      }
    }
    TurnCarry tot;
    // count: active tokens; max: running turn id; sum unused
    const TurnCarry ex = turn_block_exclusive(nact, mx, 0.0, carry, s_cnt, s_max, s_sum, tot);
    int run_max = ex.maxid;
#pragma unroll
    for (int i = 0; i < TURN_ITEMS; ++i) {
      if (!act[i] || !id) continue;
      if (ids[i] > run_max) ++starts;
      if (ids[i] < run_max) bad |= 4;
      run_max = run_max > ids[i] ? run_max : ids[i];
    }
    carry = tot;
  }
  // total of the per-thread start counts
  __syncthreads();
  s_cnt[tid] = (int)starts;
  __syncthreads();
  if (tid == 0) {
    long long tot = 0;
    for (int i = 0; i < TURN_THREADS; ++i) tot += s_cnt[i];
    token_len[row] = carry.count;
    turn_cnt[row] = tot;
  }
  if (bad) atomicOr(status, bad);
}

// gae_owned_kernel's instance for the batch (STATS needs block = row)
template <bool STATS>
void launch_gae_owned(const GaeArgs& g, int64_t grid, hipStream_t stream) {
  const dim3 gr((unsigned)grid), bl(GAE_THREADS);
  if (g.block_per_seq) {
    if (g.lam_seq != nullptr) hipLaunchKernelGGL((gae_owned_kernel<STATS, true, true>), gr, bl, 0, stream, g);
    else hipLaunchKernelGGL((gae_owned_kernel<STATS, true, false>), gr, bl, 0, stream, g);
  } else if constexpr (!STATS) {
    if (g.lam_seq != nullptr) hipLaunchKernelGGL((gae_owned_kernel<false, false, true>), gr, bl, 0, stream, g);
    else hipLaunchKernelGGL((gae_owned_kernel<false, false, false>), gr, bl, 0, stream, g);
  }
}

}  // namespace

extern "C" {

size_t areal_gae_workspace_bytes(int64_t n_tokens) {
  if (n_tokens <= 0) return 0;
  const int64_t nb = ceil_div_i64(n_tokens, GAE_TILE);
  return (size_t)nb * (sizeof(Map) + 2 * sizeof(double)) + 256;
}

// Generalised advantage estimation over packed sequences.
//   sequences: cu_seqlens [n_seqs+1] (int32), or uniform_len > 0 for a padded [n_seqs, L] array
//   no_eos [n_seqs] (uint8, nullable): bootstrap from the last value of the sequence
//   lambda_seq [n_seqs] (nullable): per-sequence lambda, else the scalar gae_lambda
int areal_gae_packed(const float* rewards, const float* values, const float* loss_mask,
                     const int32_t* cu_seqlens, const uint8_t* no_eos, const float* lambda_seq,
                     int64_t n_tokens, int64_t n_seqs, int64_t uniform_len, float discount,
                     float gae_lambda, float* advantages, float* returns, void* workspace,
                     size_t workspace_bytes, hipStream_t stream) {
  if (n_tokens < 0 || n_seqs < 0) return AREAL_ERR_BAD_ARG;
  if (n_tokens == 0) return AREAL_OK;
  if (!rewards || !values || !loss_mask || !advantages || !returns) return AREAL_ERR_BAD_ARG;
  if (n_seqs == 0 || (uniform_len <= 0 && cu_seqlens == nullptr)) return AREAL_ERR_BAD_ARG;
  if (uniform_len > 0 && uniform_len * n_seqs != n_tokens) return AREAL_ERR_BAD_ARG;
  if (n_seqs > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  if (workspace == nullptr || workspace_bytes < areal_gae_workspace_bytes(n_tokens))
    return AREAL_ERR_WORKSPACE;
  const int64_t nb = ceil_div_i64(n_tokens, GAE_TILE);
  if (nb > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  char* wp = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  Map* totals = (Map*)wp;
  double* carry = (double*)(wp + (size_t)nb * sizeof(Map));
  GaeArgs g{rewards, values, loss_mask, cu_seqlens, no_eos, lambda_seq, n_tokens, (int)n_seqs,
            uniform_len, discount, gae_lambda, advantages, returns, 0, nullptr};
  // Measured on 1024 lognormal sequences (1.8 M tokens) / 64 x 16384 / 128 long-tailed up to
  // 32768 / 4 x 32768: tile kernel 19 / 19 / 28 / 24 us, three launches 32 / 21 / 21 / 15 us.
  const int64_t mean_len = n_tokens / n_seqs;
  if (uniform_len <= 0 && mean_len <= 8 * GAE_TILE) {
    // packed sequences: block = tile, the state entering from the right recomputed per tile
    const dim3 grid((unsigned)(ceil_div_i64(nb, 8) * 8));
    if (lambda_seq != nullptr)
      hipLaunchKernelGGL((gae_tile_kernel<true, false>), grid, dim3(GAE_THREADS), 0, stream, g);
    else
      hipLaunchKernelGGL((gae_tile_kernel<false, false>), grid, dim3(GAE_THREADS), 0, stream, g);
    AREAL_CHECK_LAUNCH();
    return AREAL_OK;
  }
  // padded rows: blocks that own whole rows, as long as there are rows enough to fill the chip
  // or the rows are short (a block walks its row's tiles one after the other)
  if (uniform_len > 0 && uniform_len <= 64 * (int64_t)GAE_TILE &&
      (n_seqs >= 256 || uniform_len <= 4 * GAE_TILE)) {
    g.block_per_seq = uniform_len >= GAE_TILE;
    const int64_t grid = g.block_per_seq ? n_seqs : ceil_div_i64(nb, 8) * 8;
    launch_gae_owned<false>(g, grid, stream);
    AREAL_CHECK_LAUNCH();
    return AREAL_OK;
  }
  // long sequences: reduce-then-scan over all tokens
  hipLaunchKernelGGL(gae_block_total_kernel, dim3((unsigned)nb), dim3(GAE_THREADS), 0, stream, g,
                     totals);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(gae_carry_kernel, dim3(1), dim3(GAE_THREADS), 0, stream, totals, (int)nb,
                     carry);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(gae_apply_kernel, dim3((unsigned)nb), dim3(GAE_THREADS), 0, stream, g, carry);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// areal_gae_packed on a padded [n_seqs, uniform_len] batch whose rows are at least one tile (2048
// tokens) long, which also leaves in row_stats [5][n_seqs] (fp64) the masked sums of each row's
// advantages that areal_group_norm_from_row_stats turns into means and deviations: the
// statistics pass of a normalisation of the advantages under the same mask, at no extra traffic.
int areal_gae_padded_row_stats(const float* rewards, const float* values, const float* loss_mask,
                               const uint8_t* no_eos, const float* lambda_seq, int64_t n_seqs,
                               int64_t uniform_len, float discount, float gae_lambda,
                               float* advantages, float* returns, double* row_stats,
                               hipStream_t stream) {
  if (n_seqs < 0 || uniform_len < 0) return AREAL_ERR_BAD_ARG;
  if (n_seqs == 0 || uniform_len == 0) return AREAL_OK;
  if (!rewards || !values || !loss_mask || !advantages || !returns || !row_stats) return AREAL_ERR_BAD_ARG;
  if (uniform_len < GAE_TILE || uniform_len > 64 * (int64_t)GAE_TILE || n_seqs > (1 << 30))
    return AREAL_ERR_UNSUPPORTED;
  GaeArgs g{rewards, values, loss_mask, nullptr, no_eos, lambda_seq, n_seqs * uniform_len, (int)n_seqs,
            uniform_len, discount, gae_lambda, advantages, returns, 1, row_stats};
  launch_gae_owned<true>(g, n_seqs, stream);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// Packed GAE that also leaves the statistics pass of a group normalisation of its advantages:
// groups are runs of whole sequences, group_offsets [n_groups + 1] (int64, device) their token
// offsets (group_offsets[0] = 0, group_offsets[n_groups] = n_tokens). segment_stats receives
// [5][slots][4] fp64 sums (slots = 2048-token tiles + groups) for
// areal_group_norm_from_segment_stats. One launch. AREAL_ERR_UNSUPPORTED when the batch is not one
// for the single-pass kernel (sequences longer than 16384 tokens on average) or the groups are
// shorter than 256 tokens on average: the caller then runs areal_gae_packed and areal_group_norm.
size_t areal_gae_segment_stats_bytes(int64_t n_tokens, int64_t n_groups) {
  if (n_tokens <= 0 || n_groups <= 0) return 0;
  return (size_t)5 * GAE_SEG_WAVES * (size_t)(ceil_div_i64(n_tokens, GAE_TILE) + n_groups) * sizeof(double);
}

int areal_gae_packed_group_stats(const float* rewards, const float* values, const float* loss_mask,
                                 const int32_t* cu_seqlens, const uint8_t* no_eos,
                                 const float* lambda_seq, int64_t n_tokens, int64_t n_seqs,
                                 float discount, float gae_lambda, const int64_t* group_offsets,
                                 int64_t n_groups, float* advantages, float* returns,
                                 double* segment_stats, size_t segment_stats_bytes,
                                 hipStream_t stream) {
  if (n_tokens < 0 || n_seqs < 0 || n_groups < 0) return AREAL_ERR_BAD_ARG;
  if (n_tokens == 0) return AREAL_OK;
  if (!rewards || !values || !loss_mask || !advantages || !returns || !cu_seqlens || !group_offsets ||
      !segment_stats || n_seqs == 0 || n_groups == 0)
    return AREAL_ERR_BAD_ARG;
  if (n_seqs > (1 << 30) || n_groups > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  const int64_t nb = ceil_div_i64(n_tokens, GAE_TILE);
  if (nb > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  if (n_tokens / n_seqs > 8 * GAE_TILE || n_tokens / n_groups < 256) return AREAL_ERR_UNSUPPORTED;
  if (segment_stats_bytes < areal_gae_segment_stats_bytes(n_tokens, n_groups)) return AREAL_ERR_WORKSPACE;
  GaeArgs g{rewards, values, loss_mask, cu_seqlens, no_eos, lambda_seq, n_tokens, (int)n_seqs,
            0, discount, gae_lambda, advantages, returns, 0, nullptr};
  g.goff = group_offsets; g.n_groups = (int)n_groups; g.seg_stats = segment_stats;
  g.seg_slots = nb + n_groups;
  const dim3 grid((unsigned)(ceil_div_i64(nb, 8) * 8));
  if (lambda_seq != nullptr)
    hipLaunchKernelGGL((gae_tile_kernel<true, true>), grid, dim3(GAE_THREADS), 0, stream, g);
  else
    hipLaunchKernelGGL((gae_tile_kernel<false, true>), grid, dim3(GAE_THREADS), 0, stream, g);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

size_t areal_turn_gae_workspace_bytes(int64_t bs, int64_t max_seqlen) {
  if (bs <= 0 || max_seqlen <= 0) return 0;
  return (size_t)bs * ((size_t)(max_seqlen + 1) * sizeof(double) + (size_t)max_seqlen * 3 * sizeof(float)) + 256;
}

// Turn-level GAE on padded [bs, max_seqlen] tensors: rewards, values, loss_mask fp32, turn_ids
// int32 (-1 in prompt / tool gaps), no_eos [bs] (nullable), lambda_seq [bs] (nullable, else the
// scalar). status (device int, zeroed by the caller) receives a bit mask of malformed turn ids
// at active tokens: 1 negative, 2 not smaller than max_seqlen, 4 decreasing.
int areal_turn_gae(const float* rewards, const float* values, const float* loss_mask,
                   const int32_t* turn_ids, const uint8_t* no_eos, const float* lambda_seq,
                   int64_t bs, int64_t max_seqlen, float discount, float gae_lambda,
                   float* advantages, float* returns, int* status, void* workspace,
                   size_t workspace_bytes, hipStream_t stream) {
  if (bs < 0 || max_seqlen < 0) return AREAL_ERR_BAD_ARG;
  if (bs == 0 || max_seqlen == 0) return AREAL_OK;
  if (!rewards || !values || !loss_mask || !turn_ids || !advantages || !returns || !status)
    return AREAL_ERR_BAD_ARG;
  if (bs > (1 << 30) || max_seqlen > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  if (workspace == nullptr || workspace_bytes < areal_turn_gae_workspace_bytes(bs, max_seqlen))
    return AREAL_ERR_WORKSPACE;
  char* wp = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  TurnArgs a;
  a.rewards = rewards; a.values = values; a.mask = loss_mask; a.turn_ids = turn_ids;
  a.no_eos = no_eos; a.lam_seq = lambda_seq; a.bs = bs; a.L = max_seqlen;
  a.discount = discount; a.lam = gae_lambda; a.adv = advantages; a.ret = returns;
  a.ws_prefix = (double*)wp;
  a.ws_val = (float*)(wp + (size_t)bs * (size_t)(max_seqlen + 1) * sizeof(double));
  a.ws_adv = a.ws_val + (size_t)bs * max_seqlen;
  a.ws_ret = a.ws_adv + (size_t)bs * max_seqlen;
  a.status = status;
  hipLaunchKernelGGL(turn_gae_kernel, dim3((unsigned)bs), dim3(TURN_THREADS), 0, stream, a);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// token_lengths[b] = active tokens of row b; turn_counts[b] = distinct turn ids among them (0
// when turn_ids is null). status as in areal_turn_gae.
int areal_gae_lambda_context(const float* loss_mask, const int32_t* turn_ids, int64_t bs,
                             int64_t max_seqlen, int64_t* token_lengths, int64_t* turn_counts,
                             int* status, hipStream_t stream) {
  if (bs < 0 || max_seqlen < 0) return AREAL_ERR_BAD_ARG;
  if (bs == 0) return AREAL_OK;
  if (!loss_mask || !token_lengths || !turn_counts || !status) return AREAL_ERR_BAD_ARG;
  hipLaunchKernelGGL(gae_context_kernel, dim3((unsigned)bs), dim3(TURN_THREADS), 0, stream,
                     loss_mask, turn_ids, max_seqlen, token_lengths, turn_counts, status);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// Blocks per group: 4096 to 8192 elements per block, and at most 2048 partials per array in all
// (every block of the later passes sums them) unless there are more groups than that.
// (5 blocks of these kernels fit a CU at a time: beyond 1280 blocks a second, partly empty round
// starts, so larger inputs take 8192 elements per block.)
static int norm_nsplit(int64_t n_groups, int64_t max_group_len) {
  int64_t s = ceil_div_i64(max_group_len, 4096);
  if (s * n_groups > 1280) s = ceil_div_i64(max_group_len, 8192);
  const int64_t cap = n_groups >= 2048 ? 1 : 2048 / n_groups;
  if (s > cap) s = cap;
  if (s < 1) s = 1;
  return (int)s;
}

size_t areal_group_norm_workspace_bytes(int64_t n_groups, int64_t max_group_len) {
  if (n_groups <= 0) return 0;
  return (size_t)5 * n_groups * norm_nsplit(n_groups, max_group_len) * sizeof(double) + 256;
}

// Normalization(x, mask, groups): levels 0 = none, 1 = batch, 2 = group.
//   group_offsets [G+1] int64 element offsets (device) partitioning [0, n);
//   group_rows [G] int64 (device): number of rows (samples) of each group;
//   tail_group: index of a group made of rows that belong to no group (mean 0, std 0 at group
//   level, still part of batch statistics), or -1.
int areal_group_norm(const float* x, const float* mask, int64_t n, const int64_t* group_offsets,
                     const int64_t* group_rows, int64_t n_groups, int64_t max_group_len,
                     int tail_group, int mean_level, int std_level, int leave_one_out,
                     int unbiased, double eps, float* out, void* workspace,
                     size_t workspace_bytes, hipStream_t stream) {
  if (n < 0 || n_groups < 0) return AREAL_ERR_BAD_ARG;
  if (n == 0) return AREAL_OK;
  if (!x || !out || !group_offsets || !group_rows || n_groups == 0) return AREAL_ERR_BAD_ARG;
  if (mean_level < 0 || mean_level > 2 || std_level < 0 || std_level > 2) return AREAL_ERR_BAD_ARG;
  if (n_groups > 65535 * 16) return AREAL_ERR_UNSUPPORTED;
  if (workspace == nullptr ||
      workspace_bytes < areal_group_norm_workspace_bytes(n_groups, max_group_len))
    return AREAL_ERR_WORKSPACE;
  NormArgs a;
  a.x = x; a.mask = mask; a.n = n; a.goff = group_offsets; a.grows = group_rows;
  a.G = (int)n_groups; a.tail_group = tail_group; a.nsplit = norm_nsplit(n_groups, max_group_len);
  a.mean_level = mean_level; a.std_level = std_level; a.leave1out = leave_one_out;
  a.unbiased = unbiased; a.eps = eps;
  a.part = (double*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  a.out = out;
  // Two launches (one statistics pass) whenever every element of a group sees the same mean and a
  // batch-level deviation does not sit on top of per-group means; otherwise the deviations need
  // a pass of their own.
  a.closed_form = (!leave_one_out && !(mean_level == LEVEL_GROUP && std_level == LEVEL_BATCH)) ? 1 : 0;
  a.part_rows = 0; a.row_len = 0; a.part_tile = 0; a.part_slots = 0;
  const dim3 grid((unsigned)n_groups, (unsigned)a.nsplit);
  if (a.closed_form) {
    hipLaunchKernelGGL(norm_stats5_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
    AREAL_CHECK_LAUNCH();
  } else {
    hipLaunchKernelGGL(norm_stats1_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
    AREAL_CHECK_LAUNCH();
    hipLaunchKernelGGL(norm_stats2_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
    AREAL_CHECK_LAUNCH();
  }
  if (a.closed_form)
    hipLaunchKernelGGL(norm_apply_cf_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
  else
    hipLaunchKernelGGL(norm_apply_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// The apply pass of areal_group_norm alone, on a [n_rows, row_len] array whose per-row sums
// (row_stats [5][n_rows], as areal_gae_padded_row_stats leaves them) are already known: one
// launch. Groups are runs of whole rows (group_offsets in elements, multiples of row_len).
// Only for the level combinations that need no second statistics pass: no leave-one-out, and
// not a group-level mean under a batch-level deviation (AREAL_ERR_UNSUPPORTED otherwise).
int areal_group_norm_from_row_stats(const float* x, const float* mask, int64_t n_rows, int64_t row_len,
                                    const int64_t* group_offsets, const int64_t* group_rows,
                                    int64_t n_groups, int64_t max_group_len, int tail_group,
                                    int mean_level, int std_level, int unbiased, double eps,
                                    const double* row_stats, float* out, hipStream_t stream) {
  if (n_rows < 0 || row_len < 0 || n_groups < 0) return AREAL_ERR_BAD_ARG;
  if (n_rows == 0 || row_len == 0) return AREAL_OK;
  if (!x || !out || !group_offsets || !group_rows || !row_stats || n_groups == 0) return AREAL_ERR_BAD_ARG;
  if (mean_level < 0 || mean_level > 2 || std_level < 0 || std_level > 2) return AREAL_ERR_BAD_ARG;
  if (mean_level == LEVEL_GROUP && std_level == LEVEL_BATCH) return AREAL_ERR_UNSUPPORTED;
  if (n_groups > 65535 * 16) return AREAL_ERR_UNSUPPORTED;
  NormArgs a;
  a.x = x; a.mask = mask; a.n = n_rows * row_len; a.goff = group_offsets; a.grows = group_rows;
  a.G = (int)n_groups; a.tail_group = tail_group; a.nsplit = norm_nsplit(n_groups, max_group_len);
  a.mean_level = mean_level; a.std_level = std_level; a.leave1out = 0;
  a.unbiased = unbiased; a.eps = eps;
  a.part = const_cast<double*>(row_stats);
  a.out = out;
  a.closed_form = 1;
  a.part_rows = n_rows; a.row_len = row_len; a.part_tile = 0; a.part_slots = 0;
  const dim3 grid((unsigned)n_groups, (unsigned)a.nsplit);
  hipLaunchKernelGGL(norm_apply_cf_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// The apply pass of areal_group_norm alone on a packed array whose per-segment sums
// (segment_stats, as areal_gae_packed_group_stats leaves them for the same n and group_offsets)
// are already known: one launch. Same level restrictions as areal_group_norm_from_row_stats.
int areal_group_norm_from_segment_stats(const float* x, const float* mask, int64_t n,
                                        const int64_t* group_offsets, const int64_t* group_rows,
                                        int64_t n_groups, int64_t max_group_len, int tail_group,
                                        int mean_level, int std_level, int unbiased, double eps,
                                        const double* segment_stats, float* out, hipStream_t stream) {
  if (n < 0 || n_groups < 0) return AREAL_ERR_BAD_ARG;
  if (n == 0) return AREAL_OK;
  if (!x || !out || !group_offsets || !group_rows || !segment_stats || n_groups == 0) return AREAL_ERR_BAD_ARG;
  if (mean_level < 0 || mean_level > 2 || std_level < 0 || std_level > 2) return AREAL_ERR_BAD_ARG;
  if (mean_level == LEVEL_GROUP && std_level == LEVEL_BATCH) return AREAL_ERR_UNSUPPORTED;
  if (n_groups > 65535 * 16) return AREAL_ERR_UNSUPPORTED;
  NormArgs a;
  a.x = x; a.mask = mask; a.n = n; a.goff = group_offsets; a.grows = group_rows;
  a.G = (int)n_groups; a.tail_group = tail_group;
  // the partial sums do not depend on the split: one round of 16 elements per thread
  int64_t ns = ceil_div_i64(max_group_len, (int64_t)SEG_APPLY_ELEMS);
  if (ns > 65535) ns = 65535;
  if (ns < 1) ns = 1;
  a.nsplit = (int)ns;
  a.mean_level = mean_level; a.std_level = std_level; a.leave1out = 0;
  a.unbiased = unbiased; a.eps = eps;
  a.part = const_cast<double*>(segment_stats);
  a.out = out;
  a.closed_form = 1;
  a.part_rows = 0; a.row_len = 0;
  a.part_tile = GAE_TILE; a.part_slots = ceil_div_i64(n, GAE_TILE) + n_groups;
  const dim3 grid((unsigned)n_groups, (unsigned)a.nsplit);
  hipLaunchKernelGGL(norm_apply_cf_kernel, grid, dim3(NORM_THREADS), 0, stream, a);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

size_t areal_masked_norm_workspace_bytes(int64_t n) {
  (void)n;
  return (size_t)3 * 256 * sizeof(double) + 256;
}

int areal_masked_norm(const float* x, const float* mask, int64_t n, int unbiased, double eps,
                      float* out, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (n < 0) return AREAL_ERR_BAD_ARG;
  if (n == 0) return AREAL_OK;
  if (!x || !out) return AREAL_ERR_BAD_ARG;
  if (workspace == nullptr || workspace_bytes < areal_masked_norm_workspace_bytes(n))
    return AREAL_ERR_WORKSPACE;
  double* part = (double*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  int64_t nb = ceil_div_i64(n, NORM_THREADS * 8);
  if (nb > 256) nb = 256;
  hipLaunchKernelGGL(masked_norm_stats_kernel, dim3((unsigned)nb), dim3(NORM_THREADS), 0, stream, x,
                     mask, n, part);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(masked_norm_apply_kernel, dim3((unsigned)nb), dim3(NORM_THREADS), 0, stream, x,
                     mask, n, (const double*)part, (int)nb, unbiased, eps, out);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// masked_normalization over the trailing dimensions: x, mask (nullable), out are [rows, cols].
int areal_masked_norm_rows(const float* x, const float* mask, int64_t rows, int64_t cols,
                           int unbiased, double eps, float* out, hipStream_t stream) {
  if (rows < 0 || cols < 0 || rows > 0x7fffffffLL) return AREAL_ERR_BAD_ARG;
  if (rows == 0 || cols == 0) return AREAL_OK;
  if (!x || !out) return AREAL_ERR_BAD_ARG;
  hipLaunchKernelGGL(masked_norm_rows_kernel, dim3((unsigned)rows), dim3(NORM_THREADS), 0, stream, x,
                     mask, cols, unbiased, eps, out);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// Reward shaping in front of GAE on a padded [bs, L] batch; see adv_prep_kernel. loss_mask and
// attn_mask are bytes (nonzero = set); ref_logp, gkl_out and outcome_out may be null. With
// ref_in_place the masked reference log-probs are written back (the reference's `ref_logp *=
// loss_mask`); old_out may be logp itself when roll_logp is 0 (its `old_logp *= loss_mask`).
int areal_advantage_prep(const uint8_t* loss_mask, const uint8_t* attn_mask, const float* logp,
                         float* ref_logp, const float* reward_score, int64_t bs, int64_t L,
                         int roll_logp, int estimator, int apply_clamp, int mask_no_eos_with_zero,
                         int ref_in_place, float kl_ctl, float* lm_out, float* old_out,
                         float* kl_out, float* gkl_out, float* outcome_out, float* tot_out,
                         int64_t* seqlens_out, uint8_t* no_eos_out, hipStream_t stream) {
  if (bs < 0 || L < 0 || bs > 0x7fffffffLL) return AREAL_ERR_BAD_ARG;
  if (estimator < 1 || estimator > 3) return AREAL_ERR_BAD_ARG;
  if (bs == 0) return AREAL_OK;
  if (L == 0) return AREAL_ERR_BAD_ARG;
  if (!loss_mask || !attn_mask || !logp || !reward_score || !lm_out || !old_out || !kl_out ||
      !tot_out || !seqlens_out || !no_eos_out)
    return AREAL_ERR_BAD_ARG;
  PrepArgs a{loss_mask, attn_mask, logp, ref_logp, reward_score, L, roll_logp, estimator,
             apply_clamp, mask_no_eos_with_zero, ref_in_place, kl_ctl, lm_out, old_out, kl_out,
             gkl_out, outcome_out, tot_out, seqlens_out, no_eos_out};
  auto al16 = [](const void* q) { return q == nullptr || ((uintptr_t)q & 15) == 0; };
  const bool vec = L % 16 == 0 && al16(loss_mask) && al16(attn_mask) && al16(logp) && al16(ref_logp) &&
                   al16(lm_out) && al16(old_out) && al16(kl_out) && al16(gkl_out) && al16(outcome_out) &&
                   al16(tot_out);
  if (vec) hipLaunchKernelGGL(adv_prep_kernel<true>, dim3((unsigned)bs), dim3(NORM_THREADS), 0, stream, a);
  else hipLaunchKernelGGL(adv_prep_kernel<false>, dim3((unsigned)bs), dim3(NORM_THREADS), 0, stream, a);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // extern "C"
