// Fused lm_head -> log-softmax -> label log-prob + entropy, forward and backward, for gfx950.
//
// Every matrix product of the path is one bf16 MFMA contraction D[i][j] = sum_k A[.]*B[.] over
// 256 x 256 x 64 tiles, by one kernel template in three operand layouts, with the epilogue (what
// happens to the accumulators) as a template parameter:
//   gemm16_sweep<VAR_NT>  (A[i][k], B[j][k], both k-contiguous)
//     forward   : A = W [V,H],       B = hidden [T,H]     -> softmax statistics; the saving variant
//                                                            also writes the bf16 exponentials e [T,V]
//     recompute : A = W [V,H],       B = hidden [Tc,H]    -> dlogits (bf16)
//   gemm16_sweep<VAR_MIX> (A[k][i] k-major, B[j][k] k-contiguous)
//     dHidden   : A = W [V,H] as stored, B = e or dlogits [T,V'] -> bf16 store, rows scaled
//                 (VAR_NT on a zero-padded W^T when V is not a multiple of 64)
//   gemm16_sweep<VAR_TN>  (A[k][i], B[k][j], both k-major)
//     dWeight   : A = hidden [T,H] (scaled per row in the saved mode), B = e or dlogits [T,V']
//                 -> bf16 store, or fp32 store / accumulate
// Its k-loop is the hand-scheduled v_mfma_f32_16x16x32_bf16 loop that gen_mainloop16.py writes into
// mainloop16.inc (any K that is a multiple of 64, at least 128). gemm_nt_generic (both operands
// k-contiguous, any K % 8 == 0, 32x32x16 MFMA, register-staged loads) takes every other shape,
// with epilogues of the same arithmetic written for its accumulator layout.
// The vocabulary is put on the MFMA "A" side of the forward: in a block column of the
// accumulators 16 lanes own 16 tokens and four lane groups own 4 of every 16 vocabulary entries,
// so the softmax reductions over the vocabulary run inside a lane and across four lanes, and the
// fp32 logits never leave registers.
//
// Follows the algorithm of the reference's chunked LM head
// (areal/models/mcore/vocab_parallel_head.py:564-735 forward, :737-938 backward) and the
// backward formula of areal/utils/functional/vocab_parallel_kernels.py:99-137.
#include "common.hpp"
#include "mainloop16.inc"

namespace {

constexpr int TILE = 256;        // rows of A and of B per workgroup tile
constexpr int BK = 64;           // k extent of one LDS stage
constexpr int LDK = BK + 8;      // LDS row pitch in elements (144 B: conflict-free b128 reads)
constexpr int OPER = TILE * LDK; // elements of one operand stage
constexpr int NTHREADS = 256;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

struct GemmArgs {
  const u16* A; int64_t lda; int M;   // A rows (index i)
  const u16* B; int64_t ldb; int N;   // B rows (index j)
  int K;                              // multiple of 8
  int acols, bcols;                   // k-major operands only: readable columns of A and B
                                      // (a k-major operand must have K readable rows)
  // split-K (gemm16_sweep with a store epilogue only): the grid is ksplit
  // copies of the tile schedule; copy z contracts k-tiles [z*kt_per_split, (z+1)*kt_per_split)
  // and writes its partial result zstride bytes after the previous copy's. ksplit <= 1: off.
  int ksplit, kt_per_split;
  int64_t zstride;
  // When set and the int it points to is non-zero, the launch does nothing (every workgroup
  // returns at once): lets the host queue a launch sequence before it knows a device-side status.
  // With run_if_set != 0 the sense is inverted: the launch only does something when the int is
  // non-zero (a fallback queued behind the launch that may raise the status).
  const int* skip_if_set;
  int run_if_set;
  // gemm16_sweep, both operands k-contiguous: when M is not a multiple of the tile, the last A tile
  // is rows [M - 256, M) (it overlaps its predecessor) instead of a ragged tile; the epilogue is
  // told which of its rows are new. Needs M >= 256.
  int overlap_last_a;
  // Workgroups per super-block of the schedule (32 or 8; 0 = 32), see Sched.
  int sb_wgs;
};
DEVI bool gate_closed(const int* flag, int run_if_set) {
  return flag != nullptr && ((*flag != 0) != (run_if_set != 0));
}
DEVI bool gemm_skipped(const GemmArgs& g) { return gate_closed(g.skip_if_set, g.run_if_set); }

// Mapping of workgroup ids onto (B tile, A-range split). Workgroup ids go round-robin over
// the 8 XCDs, so the 32 workgroups resident on one XCD are id = xcd + 8*q for 32 consecutive
// q. They are laid out as an RB x RS block of (B tiles) x (splits) so that they share operand
// tiles through that XCD's L2. A launch with fewer workgroups than the chip has CUs can use
// super-blocks of 8 instead, which spread over the XCDs more evenly (several share an XCD's round).
struct Sched {
  int bj0, nbj;  // B tiles [bj0, bj0 + nbj)
  int ai0, nai;  // A tiles [ai0, ai0 + nai)
  int S;         // splits of the A-tile range
  int RB, RS;    // RB * RS == 1 << sb_log2
  int sb_log2;   // log2 of the workgroups per super-block: 5 or 3
  int n_sb_j;    // super-blocks along j
  int n_sb;      // total super-blocks
};

DEVI bool sched_decode(const Sched& sc, int id, int& bj, int& split, int& ai_begin, int& ai_end) {
  const int xcd = id & 7, q = id >> 3;
  const int sb = (q >> sc.sb_log2) * 8 + xcd;
  const int r = q & ((1 << sc.sb_log2) - 1);
  if (sb >= sc.n_sb) return false;
  const int sbj = sb % sc.n_sb_j, sbs = sb / sc.n_sb_j;
  const int bl = sbj * sc.RB + (r % sc.RB);
  split = sbs * sc.RS + (r / sc.RB);
  if (bl >= sc.nbj || split >= sc.S) return false;
  bj = sc.bj0 + bl;
  ai_begin = sc.ai0 + (int)(((int64_t)split * sc.nai) / sc.S);
  ai_end = sc.ai0 + (int)(((int64_t)(split + 1) * sc.nai) / sc.S);
  return ai_begin < ai_end;
}

static Sched make_sched(int bj0, int nbj, int ai0, int nai, int S, int sb_wgs = 32) {
  Sched sc;
  sc.bj0 = bj0; sc.nbj = nbj; sc.ai0 = ai0; sc.nai = nai; sc.S = S;
  sc.sb_log2 = sb_wgs == 8 ? 3 : 5;
  const int rs_max = sb_wgs == 8 ? 4 : 8;
  sc.RS = S >= 8 ? 8 : (S >= 4 ? 4 : (S >= 2 ? 2 : 1));
  if (sc.RS > rs_max) sc.RS = rs_max;
  sc.RB = (1 << sc.sb_log2) / sc.RS;
  sc.n_sb_j = (nbj + sc.RB - 1) / sc.RB;
  const int n_sb_s = (S + sc.RS - 1) / sc.RS;
  sc.n_sb = sc.n_sb_j * n_sb_s;
  return sc;
}
static int sched_grid(const Sched& sc) { return ((sc.n_sb + 7) / 8) * 8 * (1 << sc.sb_log2); }

// ---------------------------------------------------------------------------------------
// Main loop pieces
// ---------------------------------------------------------------------------------------

// Each thread moves 8 chunks of 16 B per operand per stage: chunk c = tid + 256*i covers
// row c/8 (= 32*i + tid/8), k offset (c%8)*8.
struct TileLoader {
  const u32x4* ptr[8];
  bool kvalid;  // recomputed per stage
  DEVI void init(const u16* base, int64_t ld, int row0, int nrows, int tid) {
    const int kc = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int row = row0 + i * 32 + (tid >> 3);
      row = row < nrows ? row : nrows - 1;  // clamp: out-of-range rows are discarded later
      ptr[i] = (const u32x4*)(base + (int64_t)row * ld + kc);
    }
  }
};

DEVI void global_load_stage(const TileLoader& ld, u32x4 (&regs)[8], int k0, int K, int tid) {
  const bool ok = (k0 + (tid & 7) * 8 + 8) <= K;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (ok) v = ld.ptr[i][k0 >> 3];
    regs[i] = v;
  }
}

DEVI void lds_store_stage(u16* stage, const u32x4 (&regs)[8], int tid) {
  u16* p = stage + (tid >> 3) * LDK + (tid & 7) * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i) *(u32x4*)(p + i * 32 * LDK) = regs[i];
}

DEVI void mma_ksteps(const u16* pa, const u16* pb, f32x16 (&acc)[4][4], int s_begin, int s_end) {
#pragma unroll
  for (int s = s_begin; s < s_end; ++s) {
    bf16x8 af[4], bf[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) af[a] = *(const bf16x8*)(pa + a * 32 * LDK + s * 16);
#pragma unroll
    for (int b = 0; b < 4; ++b) bf[b] = *(const bf16x8*)(pb + b * 32 * LDK + s * 16);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[b], acc[a][b], 0, 0, 0);
  }
}

// Workgroup (4 waves as 2x2, each wave a 128x128 block of 4x4 MFMA 32x32 blocks) sweeps the
// A tiles [ai_begin, ai_end) against one fixed B tile. Epi::tile() consumes each finished
// accumulator block.
//
// Accumulator layout inside a wave: acc[a][b][r] holds
//   i = a*32 + 8*(r/4) + 4*(lane/32) + (r%4)   (A row inside the wave's 128)
//   j = b*32 + (lane%32)                        (B row inside the wave's 128)
//
// gemm_nt_generic: any K that is a multiple of 8 (k tail zero-filled); operands staged through
// registers into a padded LDS layout. Used for small or odd shapes.
template <class Epi>
__global__ __launch_bounds__(NTHREADS) void gemm_nt_generic(GemmArgs g, Sched sc,
                                                            typename Epi::Params ep) {
  __shared__ __attribute__((aligned(16))) u16 lds[2 * 2 * OPER];
  int bj, split, ai_begin, ai_end;
  if (gemm_skipped(g)) return;
  if (!sched_decode(sc, blockIdx.x, bj, split, ai_begin, ai_end)) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wa = wave >> 1, wb = wave & 1;
  const int nk = (g.K + BK - 1) / BK;

  TileLoader lb;
  lb.init(g.B, g.ldb, bj * TILE, g.N, tid);

  typename Epi::State st;
  Epi::begin(st, ep, bj * TILE + wb * 128, split, wa, lane);

  const int frag_off = (lane & 31) * LDK + (lane >> 5) * 8;

  for (int ai = ai_begin; ai < ai_end; ++ai) {
    TileLoader la;
    la.init(g.A, g.lda, ai * TILE, g.M, tid);

    f32x16 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

    u32x4 ra[8], rb[8];
    global_load_stage(la, ra, 0, g.K, tid);
    global_load_stage(lb, rb, 0, g.K, tid);
    __syncthreads();  // every wave is done reading LDS of the previous tile
    lds_store_stage(lds, ra, tid);
    lds_store_stage(lds + OPER, rb, tid);
    if (nk > 1) {
      global_load_stage(la, ra, BK, g.K, tid);
      global_load_stage(lb, rb, BK, g.K, tid);
    }
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      const u16* sA = lds + cur * 2 * OPER;
      const u16* sB = sA + OPER;
      const u16* pa = sA + wa * 128 * LDK + frag_off;
      const u16* pb = sB + wb * 128 * LDK + frag_off;
      mma_ksteps(pa, pb, acc, 0, 2);
      if (kt + 1 < nk) {
        u16* nA = lds + (cur ^ 1) * 2 * OPER;
        lds_store_stage(nA, ra, tid);
        lds_store_stage(nA + OPER, rb, tid);
        if (kt + 2 < nk) {
          global_load_stage(la, ra, (kt + 2) * BK, g.K, tid);
          global_load_stage(lb, rb, (kt + 2) * BK, g.K, tid);
        }
      }
      mma_ksteps(pa, pb, acc, 2, 4);
      __syncthreads();
    }
    Epi::tile(st, ep, acc, ai * TILE + wa * 128, bj * TILE + wb * 128, lane);
  }
  Epi::end(st, ep, bj * TILE + wb * 128, split, wa, lane);
}

#define LDS_AS(p) ((void __attribute__((address_space(3)))*)(p))

// ---------------------------------------------------------------------------------------
// Epilogues. Each is a template on EDGE: the interior of the tile grid (every tile fully inside
// M x N) runs the EDGE = false instance, which carries no bounds predicates; ragged last tiles
// are launched separately with EDGE = true. Keeping one variant per kernel keeps the
// accumulators in registers (several variants behind run-time branches made the compiler spill
// them, which showed up as tens of GB of scratch traffic per launch).
//
// Epilogue 0: plain store (bf16 store, fp32 store, fp32 accumulate). Used for dHidden and
// dWeight and for the stand-alone GEMM entry point. Output is indexed out[j * ldo + i]
// (B row major, A row contiguous), so a lane's 4 consecutive i values are contiguous.
// ---------------------------------------------------------------------------------------
struct StoreParams {
  void* out; int64_t ldo; int M; int N;  // M % 4 == 0
  const float* jscale;                   // MODE 3: [N] factors of the output rows j
};

// MODE 0: bf16 store, 1: fp32 store, 2: fp32 accumulate, 3: bf16 store of jscale[j] * value
template <bool EDGE, int MODE>
struct StoreEpi {
  typedef StoreParams Params;
  struct State {};
  static DEVI void begin(State&, const Params&, int, int, int, int) {}
  static DEVI void end(State&, const Params&, int, int, int, int) {}
  static DEVI void split_output(Params& p, int64_t bytes) { p.out = (char*)p.out + bytes; }
  static DEVI void tile(State&, const Params& p, f32x16 (&acc)[4][4], int i0, int j0, int lane) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int j = j0 + b * 32 + (lane & 31);
      float js = 1.f;
      if (MODE == 3) js = (!EDGE || j < p.N) ? p.jscale[j] : 0.f;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int i = i0 + a * 32 + 8 * rq + 4 * (lane >> 5);
          if (!EDGE || (j < p.N && i < p.M)) {
            float x0 = acc[a][b][rq * 4 + 0], x1 = acc[a][b][rq * 4 + 1];
            float x2 = acc[a][b][rq * 4 + 2], x3 = acc[a][b][rq * 4 + 3];
            if (MODE == 3) { x0 *= js; x1 *= js; x2 *= js; x3 *= js; }
            const int64_t off = (int64_t)j * p.ldo + i;
            if (MODE == 0 || MODE == 3) {
              u32x2 v;
              v[0] = (uint32_t)f32_to_bf16_bits(x0) | ((uint32_t)f32_to_bf16_bits(x1) << 16);
              v[1] = (uint32_t)f32_to_bf16_bits(x2) | ((uint32_t)f32_to_bf16_bits(x3) << 16);
              *(u32x2*)((u16*)p.out + off) = v;
            } else {
              f32x4* dst = (f32x4*)((float*)p.out + off);
              f32x4 v = {x0, x1, x2, x3};
              if (MODE == 2) v += *dst;
              *dst = v;
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the accumulator reads of one block together
      }
    }
  }
};
template <bool E> using StoreBf16 = StoreEpi<E, 0>;
template <bool E> using StoreF32 = StoreEpi<E, 1>;
template <bool E> using AccumF32 = StoreEpi<E, 2>;
template <bool E> using StoreBf16Scaled = StoreEpi<E, 3>;

// Row reference of the saved exponentials e = 2^(c2 x - ref): ref[t] = c2 * (the largest of NREF
// logits of token t: its label's and a fixed stride sample of the vocabulary) + REF_MARGIN. The
// estimate does not exceed the row maximum (up to rounding), so the largest exponential of a row is
// at least 2^-REF_MARGIN and everything within 2^-(126 - REF_MARGIN) of it is a normal bf16
// number. The saving forward takes ALL its sums relative to this reference (no running maximum to
// rescale by), so a row is only usable while its maximum is within REF_WINDOW binades above the
// estimate: the largest exponential is then at most 2^(REF_WINDOW - REF_MARGIN), small enough for
// fp32 accumulation over the vocabulary and for the row factor of the backward (its inverse times
// the loss gradient) to stay a normal bf16 number. lmhead_merge_kernel checks that with the exact
// row maximum and raises *status otherwise; the forward then runs again without saving.
// One wave per REF_TOK tokens (the sampled weight rows are fetched once for all of them), bf16
// pairs multiplied by v_dot2c_f32_bf16; also clears *status.
constexpr int NREF = 8;
constexpr int REF_TOK = 4;
constexpr float REF_MARGIN = 16.f;
constexpr float REF_WINDOW = 100.f;

DEVI float dot8_bf16(u32x4 a, u32x4 b, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // (the elements go through scalars: a bit cast applied to a vector element directly reads
    // element 0 whatever the index in this toolchain)
    const uint32_t x = a[i], y = b[i];
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, y), acc, false);
  }
  return acc;
}

__global__ __launch_bounds__(256) void lmhead_rowref_kernel(
    const u16* __restrict__ hidden, const u16* __restrict__ weight, const float* __restrict__ bias,
    const int64_t* __restrict__ labels, int T, int H, int V, float scale, float c2,
    float* __restrict__ row_ref, int* __restrict__ status) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *status = 0;
  const int t0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * REF_TOK;
  const int lane = threadIdx.x & 63;
  if (t0 >= T) return;
  int ids[NREF];  // ids[0]: replaced per token by its label
#pragma unroll
  for (int k = 0; k < NREF; ++k) ids[k] = (int)(((int64_t)k * V) / NREF);
  int lab[REF_TOK];
  const u16* hrow[REF_TOK];
#pragma unroll
  for (int j = 0; j < REF_TOK; ++j) {
    const int t = t0 + j < T ? t0 + j : T - 1;  // a short last group repeats the last token
    const int64_t l = labels[t];
    lab[j] = (l >= 0 && l < V) ? (int)l : ids[0];
    hrow[j] = hidden + (int64_t)t * H;
  }
  float acc[REF_TOK][NREF];
#pragma unroll
  for (int j = 0; j < REF_TOK; ++j)
#pragma unroll
    for (int k = 0; k < NREF; ++k) acc[j][k] = 0.f;
  for (int h = lane * 8; h < H; h += 512) {  // H % 8 == 0
    u32x4 wf[NREF];
#pragma unroll
    for (int k = 1; k < NREF; ++k) wf[k] = *(const u32x4*)(weight + (int64_t)ids[k] * H + h);
#pragma unroll
    for (int j = 0; j < REF_TOK; ++j) {
      const u32x4 hv = *(const u32x4*)(hrow[j] + h);
      const u32x4 lv = *(const u32x4*)(weight + (int64_t)lab[j] * H + h);
      acc[j][0] = dot8_bf16(hv, lv, acc[j][0]);
#pragma unroll
      for (int k = 1; k < NREF; ++k) acc[j][k] = dot8_bf16(hv, wf[k], acc[j][k]);
    }
  }
#pragma unroll
  for (int j = 0; j < REF_TOK; ++j) {
    float mx = neg_inf();
#pragma unroll
    for (int k = 0; k < NREF; ++k) {
      const int id = k == 0 ? lab[j] : ids[k];
      const float x = (wave_sum(acc[j][k]) + (bias != nullptr ? bias[id] : 0.f)) * scale;
      mx = fmaxf(mx, x);
    }
    if (lane == 0 && t0 + j < T) row_ref[t0 + j] = fmaf(mx, c2, REF_MARGIN);
  }
}

// ---------------------------------------------------------------------------------------
// Epilogue 1: online softmax statistics over the vocabulary (forward).
// Per token the lane keeps: running max m of the logits x, s = sum exp((x-m)/T),
// q = sum ((x-m)/T * log2e) * exp((x-m)/T), the label's logit, min and (MOMENTS) sum x,
// sum x^2. One token (its 64 logits in this lane) at a time: the logits are read from the
// accumulators twice (statistics pass, exponential pass) and never written back.
// ---------------------------------------------------------------------------------------
// c2 * m rounded to fp32, and sums / differences with such products, kept out of fma
// contraction: the softmax sums are relative to this ROUNDED reference (the exponent of a logit
// is fma(x, c2, -ref): exact product minus the rounded reference), so whatever re-references
// them has to use the same rounded value or the rounding error of c2 * m (up to ulp(c2 m) / 2
// binades) enters the result.
DEVI float ref_of(float m, float c2) {
#pragma clang fp contract(off)
  return m * c2;
}
DEVI float ref_diff(float a, float b, float c2) {  // fl(a c2) - fl(b c2)
#pragma clang fp contract(off)
  const float x = a * c2, y = b * c2;
  return x - y;
}
DEVI float ref_plus(float m, float c2, float add) {  // fl(m c2) + add
#pragma clang fp contract(off)
  const float x = m * c2;
  return x + add;
}

constexpr int NSTAT = 7;  // m, s, q, xlabel, min, sumx, sumx2

struct FwdParams {
  const int64_t* labels; int T; int V;
  float scale;        // logit_scale
  float c2;           // inv_temperature * log2(e)
  const float* bias;  // nullable, [V]
  float* ws;          // [NSTAT][P][T]
  int P;              // total partial slots
  int slot_base;      // first slot written by this launch
  // SAVE: e[t][v] = exp2(c2 * x[t][v] - ref[t]) in bf16, ref = the row reference that
  // lmhead_rowref_kernel prepared; columns [V, ldv) are written as zero.
  u16* probs; int64_t ldv;
  const float* probs_ref;  // [T]
};

template <bool EDGE, bool AFFINE, bool MOMENTS, bool SAVE>
struct FwdEpi {
  typedef FwdParams Params;
  struct State {
    float m[4], s[4], q[4], xl[4], mn[4], sx[4], sx2[4];
    int lab[4];
  };
  static DEVI void split_output(Params&, int64_t) {}
  static DEVI void begin(State& st, const Params& p, int t0, int, int, int lane) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      st.m[b] = neg_inf(); st.s[b] = 0.f; st.q[b] = 0.f; st.xl[b] = 0.f;
      st.mn[b] = pos_inf(); st.sx[b] = 0.f; st.sx2[b] = 0.f;
      const int t = t0 + b * 32 + (lane & 31);
      int64_t l = (!EDGE || t < p.T) ? p.labels[t] : -1;
      st.lab[b] = (l >= 0 && l < p.V) ? (int)l : -1;
    }
  }

  static DEVI void tile(State& st, const Params& p, const f32x16 (&acc)[4][4], int v0, int t0, int lane) {
    const int vl = v0 + 4 * (lane >> 5);
    auto vidx = [&](int a, int r) { return vl + a * 32 + 8 * (r >> 2) + (r & 3); };
    auto logit = [&](int a, int b, int r) -> float {
      float x = acc[a][b][r];
      if (AFFINE) {
        float bv = 0.f;
        if (p.bias != nullptr && (!EDGE || vidx(a, r) < p.V)) bv = p.bias[vidx(a, r)];
        x = (x + bv) * p.scale;
      }
      return x;
    };
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int tok = t0 + b * 32 + (lane & 31);
      float rr = 0.f;  // SAVE: the token's row reference, needed after the statistics pass
      if (SAVE && (!EDGE || tok < p.T)) rr = p.probs_ref[tok];
      float tmax = neg_inf(), tmin = pos_inf(), sx = 0.f, sx2 = 0.f;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float x = logit(a, b, r);
          if (!EDGE || vidx(a, r) < p.V) {
            tmax = fmaxf(tmax, x);
            tmin = fminf(tmin, x);
            if (MOMENTS) { sx += x; sx2 = fmaf(x, x, sx2); }
          }
        }
        if (SAVE) __builtin_amdgcn_sched_barrier(0);  // 16 accumulator reads at a time
      }
      st.mn[b] = fminf(st.mn[b], tmin);
      if (MOMENTS) { st.sx[b] += sx; st.sx2[b] += sx2; }
      const float m_old = st.m[b];
      const float m_new = fmaxf(m_old, tmax);
      // rescale the running sums to the new reference (see ref_of); on the first tile
      // m_old = -inf and s = q = 0, so the factor is taken as 2^0 instead of evaluating -inf - x
      float s = st.s[b], q = st.q[b];
      const float mc = (!EDGE || m_new > neg_inf()) ? ref_of(m_new, p.c2) : 0.f;
      const float dl = (m_old > neg_inf()) ? ref_diff(m_old, m_new, p.c2) : 0.f;
      const float alpha = fast_exp2(dl);
      q = alpha * fmaf(dl, s, q);
      s = alpha * s;
      if (!SAVE) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float t = fmaf(logit(a, b, r), p.c2, -mc);
            const float e = fast_exp2(t);
            if (!EDGE || vidx(a, r) < p.V) { s += e; q = fmaf(t, e, q); }
          }
      } else {
        // The sums take the exponentials relative to the running maximum, as above (in (0, 1]
        // whatever the row reference is); what is stored is the same exponential moved to the
        // row reference by one factor per (token, tile). That factor over- or underflows only
        // where the stored value is not used: rows outside the reference window, and tiles
        // whose maximum lies 126 binades below the row's.
        const float gamma = fast_exp2(mc - rr);
        u16* row = p.probs + (int64_t)tok * p.ldv;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            const int vq = vl + a * 32 + 8 * rq;
            u16 d[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const float t = fmaf(logit(a, b, rq * 4 + k), p.c2, -mc);
              const float e = fast_exp2(t);
              float es = e * gamma;
              if (EDGE && vq + k >= p.V) es = 0.f;
              else { s += e; q = fmaf(t, e, q); }
              d[k] = f32_to_bf16_bits(es);
            }
            if (!EDGE || (tok < p.T && vq < p.ldv)) {
              u32x2 pk;
              pk[0] = (uint32_t)d[0] | ((uint32_t)d[1] << 16);
              pk[1] = (uint32_t)d[2] | ((uint32_t)d[3] << 16);
              *(u32x2*)(row + vq) = pk;
            }
          }
          // pins the partial sums here: without it the compiler sinks the whole summation
          // chain below the stores of all four token blocks and spills every term
          asm volatile("" : "+v"(s), "+v"(q));
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      st.s[b] = s; st.q[b] = q; st.m[b] = m_new;
      const int lab = st.lab[b];
      const bool hit = (lab >= v0) && (lab < v0 + 128);
      if (__builtin_amdgcn_ballot_w64(hit) != 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (vidx(a, r) == lab) st.xl[b] = logit(a, b, r);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  static DEVI void end(State& st, const Params& p, int t0, int split, int wa, int lane) {
    const int slot = p.slot_base + split * 4 + wa * 2 + (lane >> 5);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int t = t0 + b * 32 + (lane & 31);
      if (EDGE && t >= p.T) continue;
      const int64_t PT = (int64_t)p.P * p.T;
      float* w = p.ws + (int64_t)slot * p.T + t;
      w[0 * PT] = st.m[b]; w[1 * PT] = st.s[b]; w[2 * PT] = st.q[b]; w[3 * PT] = st.xl[b];
      w[4 * PT] = st.mn[b];
      if (MOMENTS) { w[5 * PT] = st.sx[b]; w[6 * PT] = st.sx2[b]; }
    }
  }
};
template <bool E> using FwdPlain = FwdEpi<E, false, false, false>;
template <bool E> using FwdPlainMom = FwdEpi<E, false, true, false>;
template <bool E> using FwdAffine = FwdEpi<E, true, false, false>;
template <bool E> using FwdAffineMom = FwdEpi<E, true, true, false>;
template <bool E> using FwdPlainSave = FwdEpi<E, false, false, true>;
template <bool E> using FwdPlainMomSave = FwdEpi<E, false, true, true>;
template <bool E> using FwdAffineSave = FwdEpi<E, true, false, true>;
template <bool E> using FwdAffineMomSave = FwdEpi<E, true, true, true>;

// Merge the partial statistics of one token over all slots. A block is 64 tokens (lanes) x
// MERGE_WAVES waves; wave w takes slots w, w + MERGE_WAVES, ... (loads stay coalesced along the
// tokens, and a launch with few tokens and many slots still has enough threads in flight), the
// partial results meet in LDS and wave 0 adds them in a fixed order.
// ref_sums: the slots' sums S, Q are relative to row_ref[t] (the saving forward of the
// hand-scheduled kernels) instead of to each slot's own maximum; the final expressions are then
// evaluated in fp64, where c2 x - ref and log S (each up to REF_WINDOW binades) cancel.
// gate / gate_run_if_set: as GemmArgs::skip_if_set / run_if_set.
constexpr int MERGE_WAVES = 8;
__global__ __launch_bounds__(64 * MERGE_WAVES) void lmhead_merge_kernel(
    const float* __restrict__ ws, int P, int T, int V, int ref_sums, float c2,
    float* __restrict__ logprobs, float* __restrict__ entropy, float* __restrict__ vmin,
    float* __restrict__ vmax, float* __restrict__ vmean, float* __restrict__ vnorm,
    float* __restrict__ row_max, float* __restrict__ sum_exp, const float* __restrict__ row_ref,
    int* __restrict__ status, const int* __restrict__ gate, int gate_run_if_set) {
  if (gate_closed(gate, gate_run_if_set)) return;
  __shared__ float sh_f[5][MERGE_WAVES][64];   // max, S, Q, label logit, min
  __shared__ double sh_d[2][MERGE_WAVES][64];  // sum x, sum x^2
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * 64 + lane;
  const int tt = t < T ? t : T - 1;  // lanes past the end repeat the last token and write nothing
  const int64_t PT = (int64_t)P * T;
  const bool moments = vmean != nullptr || vnorm != nullptr;
  float M = neg_inf();
  for (int p = wv; p < P; p += MERGE_WAVES) M = fmaxf(M, ws[(int64_t)p * T + tt]);
  sh_f[0][wv][lane] = M;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MERGE_WAVES; ++i) M = fmaxf(M, sh_f[0][i][lane]);
  float S = 0.f, Q = 0.f, xl = 0.f, mn = pos_inf();
  double sx = 0.0, sx2 = 0.0;
  for (int p = wv; p < P; p += MERGE_WAVES) {
    const float* w = ws + (int64_t)p * T + tt;
    const float m = w[0];
    if (ref_sums) {
      S += w[1 * PT];
      Q += w[2 * PT];
    } else if (m > neg_inf()) {
      const float dl = ref_diff(m, M, c2);  // as in the epilogue
      const float alpha = exp2f(dl);
      S += alpha * w[1 * PT];
      Q += alpha * fmaf(dl, w[1 * PT], w[2 * PT]);
    }
    xl += w[3 * PT];
    mn = fminf(mn, w[4 * PT]);
    if (moments) { sx += (double)w[5 * PT]; sx2 += (double)w[6 * PT]; }
  }
  sh_f[1][wv][lane] = S; sh_f[2][wv][lane] = Q; sh_f[3][wv][lane] = xl; sh_f[4][wv][lane] = mn;
  sh_d[0][wv][lane] = sx; sh_d[1][wv][lane] = sx2;
  __syncthreads();
  if (wv != 0 || t >= T) return;
  S = 0.f; Q = 0.f; xl = 0.f; mn = pos_inf(); sx = 0.0; sx2 = 0.0;
#pragma unroll
  for (int i = 0; i < MERGE_WAVES; ++i) {
    S += sh_f[1][i][lane]; Q += sh_f[2][i][lane]; xl += sh_f[3][i][lane];
    mn = fminf(mn, sh_f[4][i][lane]);
    sx += sh_d[0][i][lane]; sx2 += sh_d[1][i][lane];
  }
  if (ref_sums) {
    const double ln2 = 0.6931471805599453094;
    const double rr = (double)row_ref[t];
    const double lnS = log((double)S);
    if (logprobs) {
      const float lp = (float)(((double)xl * (double)c2 - rr) * ln2 - lnS);
      logprobs[t] = xl <= M ? fminf(lp, 0.f) : lp;
    }
    if (entropy) entropy[t] = (float)(lnS - ln2 * (double)Q / (double)S);
    // what the backward kernels expect: the sum relative to the rounded product fl(c2 * max)
    if (sum_exp) sum_exp[t] = (float)((double)S * exp2(rr - (double)ref_of(M, c2)));
    // usable only if the row maximum was inside the window (then no sum overflowed either)
    if (!(fmaf(M, c2, -row_ref[t]) <= REF_WINDOW - REF_MARGIN) || !(S < pos_inf())) atomicMax(status, 1);
  } else {
    const float logS = logf(S);
    // label exponent against the same rounded reference the sums use. For a label inside the
    // vocabulary (xl <= M) the result is <= 0 in exact arithmetic; the last rounding may leave
    // +1e-8 when p = 1 to fp32 precision.
    if (logprobs) {
      const float lp = fmaf(xl, c2, -ref_of(M, c2)) * LN2 - logS;
      logprobs[t] = xl <= M ? fminf(lp, 0.f) : lp;
    }
    if (entropy) entropy[t] = logS - (Q * LN2) / S;
    if (sum_exp) sum_exp[t] = S;
    // the saved exponentials of this row are usable if its largest one is at most 2^(window - margin)
    if (row_ref != nullptr && !(fmaf(M, c2, -row_ref[t]) <= REF_WINDOW - REF_MARGIN)) atomicMax(status, 1);
  }
  if (vmin) vmin[t] = mn;
  if (vmax) vmax[t] = M;
  if (vmean) vmean[t] = (float)(sx / (double)V);
  if (vnorm) vnorm[t] = (float)sqrt(sx2);
  if (row_max) row_max[t] = M;
}

// ---------------------------------------------------------------------------------------
// Epilogue 2: recompute logits and emit dlogits = (onehot - p) * g * invT * scale in bf16,
// in two layouts: dl [Tc, ldv] (vocabulary contiguous) and dlT [V, ldt] (token contiguous).
// ---------------------------------------------------------------------------------------
struct BwdParams {
  const int64_t* labels;     // [Tc]
  const float* row_max;      // [Tc]
  const float* sum_exp;      // [Tc]
  const float* grad;         // [Tc] dLoss/dlogprob
  int T; int V;
  float scale; float c2; float inv_temp;
  const float* bias;
  u16* dl; int64_t ldv;      // ldv = V rounded up to 64; columns [V, ldv) are written as zero
  u16* dlT; int64_t ldt;     // ldt = T rounded up to 64; columns [T, ldt) are written as zero
};

template <bool EDGE, bool AFFINE, bool WT>  // WT: also write the token-contiguous copy dlT
struct BwdEpi {
  typedef BwdParams Params;
  struct State {
    float nb[4], gs[4];
    int lab[4];
  };
  static DEVI void begin(State& st, const Params& p, int t0, int, int, int lane) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int t = t0 + b * 32 + (lane & 31);
      if (!EDGE || t < p.T) {
        const int64_t l = p.labels[t];
        st.lab[b] = (l >= 0 && l < p.V) ? (int)l : -1;
        st.nb[b] = -ref_plus(p.row_max[t], p.c2, fast_log2(p.sum_exp[t]));
        st.gs[b] = p.grad[t] * p.inv_temp * p.scale;
      } else {
        st.lab[b] = -1; st.nb[b] = 0.f; st.gs[b] = 0.f;
      }
    }
  }
  static DEVI void end(State&, const Params&, int, int, int, int) {}
  static DEVI void split_output(Params&, int64_t) {}

  static DEVI void tile(State& st, const Params& p, const f32x16 (&acc)[4][4], int v0, int t0, int lane) {
    const int vl = v0 + 4 * (lane >> 5);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int t = t0 + b * 32 + (lane & 31);
      const float nb = st.nb[b], gs = st.gs[b];
      const int lab = st.lab[b];
      u16* row = p.dl + (int64_t)t * p.ldv;
      u16* col = p.dlT + t;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int vq = vl + a * 32 + 8 * rq;
          u16 d[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int v = vq + e;
            float x = acc[a][b][rq * 4 + e];
            if (AFFINE) {
              float bv = 0.f;
              if (p.bias != nullptr && (!EDGE || v < p.V)) bv = p.bias[v];
              x = (x + bv) * p.scale;
            }
            const float pr = fast_exp2(fmaf(x, p.c2, nb));
            float dv = -pr * gs;
            if (v == lab) dv += gs;
            if (EDGE && (v >= p.V || t >= p.T)) dv = 0.f;
            d[e] = f32_to_bf16_bits(dv);
          }
          if (!EDGE || (t < p.T && vq < p.ldv)) {
            u32x2 pk;
            pk[0] = (uint32_t)d[0] | ((uint32_t)d[1] << 16);
            pk[1] = (uint32_t)d[2] | ((uint32_t)d[3] << 16);
            *(u32x2*)(row + vq) = pk;
          }
          if (WT && (!EDGE || t < p.ldt)) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (!EDGE || vq + e < p.V) col[(int64_t)(vq + e) * p.ldt] = d[e];
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
};
template <bool E> using BwdPlain = BwdEpi<E, false, false>;
template <bool E> using BwdAffine = BwdEpi<E, true, false>;
template <bool E> using BwdPlainT = BwdEpi<E, false, true>;
template <bool E> using BwdAffineT = BwdEpi<E, true, true>;

// Operands of the backward from the exponentials the forward saved, e[t][v] = 2^(c2 x - ref[t]):
//   dlogits[t][v] = f[t] * e'[t][v],   f[t] = -g[t] * invT * scale * 2^(ref[t] - lse2[t]),
// with lse2 = fl(c2 * row_max) + log2(sum_exp) and e' = e except at the label, where
// e' = expm1(logprob) * 2^(lse2 - ref) taken from the fp32 label log-probability (so that
// f * e' = -g' * expm1(logprob) = g' * (1 - p) keeps its precision when p is close to 1).
// The row factor f never multiplies the [T, V] buffer: dHidden scales its output rows by it and
// dWeight contracts e' with hs = bf16(f[t] * hidden[t][:]). One block per row of probs:
// rows < T write f[t], hs[t][:] and the label's entry; rows [T, Tpad) of probs and hs are cleared.
__global__ __launch_bounds__(256) void saved_prep_kernel(
    u16* __restrict__ probs, int64_t ldv, const float* __restrict__ ref,
    const int64_t* __restrict__ labels, const float* __restrict__ row_max,
    const float* __restrict__ sum_exp, const float* __restrict__ grad,
    const float* __restrict__ logprobs, const u16* __restrict__ hidden, int T, int H, int V,
    float c2, float gscale, float* __restrict__ rowfac, u16* __restrict__ hs,
    const int* __restrict__ skip_if_set) {
  if (skip_if_set != nullptr && *skip_if_set != 0) return;
  const int t = blockIdx.x;
  if (t >= T) {
    u16* row = probs + (int64_t)t * ldv;
    for (int64_t v = (int64_t)threadIdx.x * 8; v < ldv; v += 2048) *(u32x4*)(row + v) = u32x4{0u, 0u, 0u, 0u};
    if (hs != nullptr)
      for (int h = threadIdx.x * 8; h < H; h += 2048) *(u32x4*)(hs + (int64_t)t * H + h) = u32x4{0u, 0u, 0u, 0u};
    return;
  }
  const float lse2 = ref_plus(row_max[t], c2, fast_log2(sum_exp[t]));
  const float f = -(grad[t] * gscale) * fast_exp2(ref[t] - lse2);
  if (threadIdx.x == 0) {
    rowfac[t] = f;
    const int64_t lab = labels[t];
    if (lab >= 0 && lab < V) {
      u16* e = probs + (int64_t)t * ldv + lab;
      const float unit = fast_exp2(lse2 - ref[t]);  // a probability of 1 in the units of e
      const float el = logprobs ? expm1f(logprobs[t]) * unit : bf16_bits_to_f32(*e) - unit;
      *e = f32_to_bf16_bits(el);
    }
  }
  if (hs != nullptr) {
    const u16* src = hidden + (int64_t)t * H;
    u16* dst = hs + (int64_t)t * H;
    for (int h = threadIdx.x * 8; h < H; h += 2048) {  // H % 8 == 0
      const u32x4 in = *(const u32x4*)(src + h);
      u32x4 out;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float lo = bf16_bits_to_f32((u16)(in[k] & 0xffffu)) * f;
        const float hi = bf16_bits_to_f32((u16)(in[k] >> 16)) * f;
        out[k] = (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
      }
      *(u32x4*)(dst + h) = out;
    }
  }
}

// out[v] (+)= sum over rows of w[row] * dl[row][v] (w = 1 when null), fp32: the lm_head bias
// gradient. One block per 64 columns: 4 row lanes x 64 columns per pass (128-byte row pieces),
// LDS reduce over the lanes.
__global__ __launch_bounds__(256) void colsum_bf16_kernel(const u16* __restrict__ dl, int64_t ld,
                                                          int64_t rows, int V, int accumulate,
                                                          const float* __restrict__ w,
                                                          float* __restrict__ out,
                                                          const int* __restrict__ skip_if_set) {
  if (skip_if_set != nullptr && *skip_if_set != 0) return;
  __shared__ float sm[4][64];
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int lane_row = threadIdx.x >> 6;
  float acc = 0.f;
  if (c < V)
    for (int64_t r = lane_row; r < rows; r += 4) {
      const float x = bf16_bits_to_f32(dl[r * ld + c]);
      acc = w != nullptr ? fmaf(w[r], x, acc) : acc + x;
    }
  sm[lane_row][threadIdx.x & 63] = acc;
  __syncthreads();
  if (lane_row == 0 && c < V) {
    const float s = (sm[0][threadIdx.x] + sm[1][threadIdx.x]) + (sm[2][threadIdx.x] + sm[3][threadIdx.x]);
    out[c] = accumulate ? out[c] + s : s;
  }
}

// dst[c][r] = src[r][c] for r < R, c < C; dst[c][r] = 0 for R <= r < ldd. 64x64 tiles.
__global__ __launch_bounds__(256) void transpose_pad_bf16_kernel(const u16* __restrict__ src,
                                                                 int64_t lds_, int R, int C,
                                                                 u16* __restrict__ dst,
                                                                 int64_t ldd) {
  __shared__ u16 tile[64][66];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < R && c < C) ? src[(int64_t)r * lds_ + c] : (u16)0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, r = r0 + tx;
    if (c < C && r < ldd) dst[(int64_t)c * ldd + r] = tile[tx][i];
  }
}

// out[i] = bf16(scale[i / row_len] * sum_z part[z * zstride + i]) (scale = 1 when null): the
// split-K partial results of dHidden. row_len % 4 == 0.
__global__ void splitk_reduce_bf16_kernel(const float* __restrict__ part, int Z, int64_t zstride,
                                          int64_t n, const float* __restrict__ scale,
                                          int64_t row_len, u16* __restrict__ out,
                                          const int* __restrict__ skip_if_set) {
  if (skip_if_set != nullptr && *skip_if_set != 0) return;
  int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x * 4;
  for (; i < n; i += stride) {  // n % 4 == 0
    f32x4 a = *(const f32x4*)(part + i);
    for (int z = 1; z < Z; ++z) {
      const f32x4 b = *(const f32x4*)(part + (int64_t)z * zstride + i);
      a[0] += b[0]; a[1] += b[1]; a[2] += b[2]; a[3] += b[3];
    }
    if (scale != nullptr) {
      const float f = scale[i / row_len];
      a[0] *= f; a[1] *= f; a[2] *= f; a[3] *= f;
    }
    u32x2 o;
    o[0] = (uint32_t)f32_to_bf16_bits(a[0]) | ((uint32_t)f32_to_bf16_bits(a[1]) << 16);
    o[1] = (uint32_t)f32_to_bf16_bits(a[2]) | ((uint32_t)f32_to_bf16_bits(a[3]) << 16);
    *(u32x2*)(out + i) = o;
  }
}

__global__ void cast_f32_to_bf16_kernel(const float* __restrict__ src, u16* __restrict__ dst,
                                        int64_t n) {
  int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x * 4;
  for (; i + 3 < n; i += stride) {
    const f32x4 v = *(const f32x4*)(src + i);
    u32x2 o;
    o[0] = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
    o[1] = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
    *(u32x2*)(dst + i) = o;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (int64_t j = n & ~(int64_t)3; j < n; ++j) dst[j] = f32_to_bf16_bits(src[j]);
}


// =======================================================================================
// The contraction with the hand-scheduled main loop (mainloop16.inc, written by
// gen_mainloop16.py): v_mfma_f32_16x16x32_bf16, accumulators in a[0:255], k-loop as one assembly
// block per output tile: a 256 x 256 x 64 tile, four waves of 128 x 128, three operand layouts
// (nt / tn / mix), any K that is a multiple of 64 and at least 128.
//
// Accumulator layout of a wave: block (ia, jb) of 16 x 16, register r of a lane:
//   i = ia*16 + 4*(lane/16) + r     (A row inside the wave's 128)
//   j = jb*16 + (lane%16)           (B row inside the wave's 128)
// and block (ia, jb) sits in tuple t[ia*2 + jb/4], elements (jb%4)*4 .. +3.
// =======================================================================================
//
// The compiler does not know that values live in a[0:255] between the main loop's block (which
// lists them as clobbered) and the blocks with which the epilogues fetch them, one block column
// (fixed jb: 16 output rows j) at a time, x[ia * 4 + r]. The build checks on the generated
// assembly that no compiler-emitted instruction of these kernels touches an accumulator register.
template <int JB>
DEVI void acc_col(float (&x)[32]) {
  if constexpr (JB == 0) asm volatile(ML16_READ_COL0 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else if constexpr (JB == 1) asm volatile(ML16_READ_COL1 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else if constexpr (JB == 2) asm volatile(ML16_READ_COL2 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else if constexpr (JB == 3) asm volatile(ML16_READ_COL3 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else if constexpr (JB == 4) asm volatile(ML16_READ_COL4 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else if constexpr (JB == 5) asm volatile(ML16_READ_COL5 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else if constexpr (JB == 6) asm volatile(ML16_READ_COL6 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
  else asm volatile(ML16_READ_COL7 : ML16_COL_OUTPUTS(x) : : ML16_ACC_CLOBBERS);
}
// Nothing the compiler allocates may sit in an accumulator register across this point. Its
// register allocator treats free accumulator registers as good homes for long-lived values, and
// it believes them free after the main loop; with these fences (and the same clobber list on
// every acc_col block) only a value defined and last used between two neighbouring fences could
// still land there, which the build's check of the assembly would report.
#define ML16_AGPR_FENCE() asm volatile("" ::: ML16_ACC_CLOBBERS)
template <int N> struct IntC { static constexpr int value = N; };
template <int JB = 0, class F>
DEVI void for_each_col(F&& f) {
  if constexpr (JB < 8) {
    f(IntC<JB>{});
    for_each_col<JB + 1>(f);
  }
}

constexpr int RING16_BYTES = 2 * ML16_OPER_BYTES;  // [A stage 0][A stage 1][B stage 0][B stage 1]
// Per-wave staging area behind the ring: one block column of the wave's sub-tile (16 output rows
// j x 128 values i in bf16) is transposed through it so that global stores cover whole lines.
constexpr int STAGE16_PITCH = 272;                 // bytes per j row: 256 + 16 (conflict-free)
constexpr int STAGE16_BYTES = 16 * STAGE16_PITCH;  // per wave
enum { VAR_NT = 0, VAR_TN = 1, VAR_MIX = 2 };

// chunk swizzle of a k-contiguous stage row (measured: 0 LDS bank conflicts for the 16-row
// fragment reads, lane l on row l % 16 at chunk ks * 4 + l / 16)
DEVI int swz16(int r) { return r & 7; }

// Per-lane byte offsets of the 8 direct loads of one operand half, and the LDS read addresses
// (stage 0) of its fragments. KM: k-major operand (`first` = its tile of 32 nblk columns, nvalid =
// readable columns; the loads fetch 256 columns from the tile's first one whatever nblk is, and
// wave row / column W reads the nblk blocks of 16 columns from block W * nblk on); otherwise
// k-contiguous (`first` = the tile's first row, nvalid = rows; nblk = 8).
template <bool KM>
DEVI void setup_operand16(int64_t ld, int first, int nvalid, int W, int oper, int wave, int lane,
                          uint32_t lds_base, uint32_t (&off)[8], uint32_t (&rd)[8], int nblk = 8) {
  if (!KM) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = wave * 64 + i * 8 + (lane >> 3);
      const int rr = first + r < nvalid ? r : nvalid - 1 - first;  // clamped rows are discarded later
      off[i] = 2u * ((uint32_t)rr * (uint32_t)ld + (uint32_t)(((lane & 7) ^ swz16(r)) * 8));
    }
    const int rl = lane & 15, kg = lane >> 4, sw = swz16(rl);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      rd[ks] = lds_base + oper * ML16_OPER_BYTES + (W * 128 + rl) * 128 + (((ks * 4 + kg) ^ sw) * 16);
  } else {
    // instruction i of a wave fills k-rows wave*16 + 2*i + (lane >> 5); the 64-byte chunks of a
    // row are swizzled with k & 3 and the halves of a chunk swapped in rows with k & 8
    const int hl = lane >> 5, piece = lane & 31;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int kr = wave * 16 + 2 * i + hl;
      const int k3 = kr & 3, cf = ((kr >> 3) & 1) * 2;
      int gp = first * (nblk * 4) + (((piece >> 2) ^ k3) << 2) + ((piece & 3) ^ cf);
      const int last = nvalid / 8 - 1;
      gp = gp < last ? gp : last;  // columns past the end are discarded later
      off[i] = 2u * ((uint32_t)kr * (uint32_t)ld + (uint32_t)(gp * 8));
    }
    const int G = lane >> 4, q = lane & 15, r4 = q >> 2;
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      const int y = W * nblk + x;  // block of 16 columns inside the 256 loaded ones
      rd[x] = lds_base + oper * ML16_OPER_BYTES + (G * 8 + r4) * 512 + ((((y >> 1) & 7) ^ r4) << 6) +
              ((((y & 1) ^ G) & 1) << 5) + (q & 3) * 8;
    }
  }
}

// A workgroup sweeps the A tiles [ai_begin, ai_end) against one B tile. Requirements checked by
// the host: K % 64 == 0 and K >= 128; a sweep of more than one A tile has only full A tiles (a
// ragged last one as rows [M - 256, M), see GemmArgs::overlap_last_a) and a k-contiguous A (the
// loader's lane offsets are those of the first tile); every copy of a split-K launch has at least
// two k-tiles (an even number in all but the last, see split_ktiles).
// Epi::tile gets the first row of the tile's sub-block of this wave and, last, the first row of the
// tile that no earlier tile of the sweep covered.
// NA < 8 (k-major A only): A tiles of 32 NA columns, each wave row taking NA blocks of 16; the MFMAs
// of the missing blocks are not issued (a tile costs NA / 8 of a full one), so an M that fills its
// last 256-wide tile badly (896 = 3.5 x 256 = 4 x 224) wastes nothing. NA is the epilogue's (Epi::NA).
template <int VAR, class Epi>
__global__ __launch_bounds__(NTHREADS) void gemm16_sweep(GemmArgs g, Sched sc, typename Epi::Params ep) {
  __shared__ __attribute__((aligned(1024))) unsigned char lds[RING16_BYTES + 4 * STAGE16_BYTES];
  constexpr bool A_KM = VAR != VAR_NT, B_KM = VAR == VAR_TN;
  constexpr int NA = Epi::NA;
  static_assert(NA == 8 || (NA == 7 && A_KM), "narrow A tiles need a k-major A");
  constexpr int TM = NA * 32;  // A rows (output index i) per tile
  int bj, split, ai_begin, ai_end;
  int wg = blockIdx.x, nk = g.K / BK;
  if (g.ksplit > 1) {
    const int per_copy = gridDim.x / g.ksplit;  // a multiple of 8 super-blocks
    const int z = wg / per_copy;
    wg -= z * per_copy;
    wg = (wg & ~7) | ((wg - z * sc.n_sb) & 7);  // copies start on different XCDs
    const int kt0 = z * g.kt_per_split;
    nk -= kt0;
    nk = nk < g.kt_per_split ? nk : g.kt_per_split;
    g.A += A_KM ? (int64_t)kt0 * BK * g.lda : (int64_t)kt0 * BK;
    g.B += B_KM ? (int64_t)kt0 * BK * g.ldb : (int64_t)kt0 * BK;
    Epi::split_output(ep, (int64_t)z * g.zstride);
    if (nk <= 0) return;
  }
  if (gemm_skipped(g)) return;
  if (!sched_decode(sc, wg, bj, split, ai_begin, ai_end)) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave >> 1, wb = wave & 1;
  const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_AS(lds);

  // first row of A tile ai (k-contiguous A): the last tile of a ragged M may overlap its predecessor
  auto a_row0 = [&](int ai) -> int {
    const int r = ai * TM;
    return (VAR == VAR_NT && g.overlap_last_a != 0 && r + TILE > g.M) ? g.M - TILE : r;
  };
  uint32_t oa[8], ob[8], ra[8], rb[8];
  setup_operand16<A_KM>(g.lda, A_KM ? ai_begin : a_row0(ai_begin), A_KM ? g.acols : g.M, wa, 0, wave, lane,
                        lds_base, oa, ra, NA);
  setup_operand16<B_KM>(g.ldb, B_KM ? bj : bj * TILE, B_KM ? g.bcols : g.N, wb, 1, wave, lane, lds_base, ob, rb);

  // pointers to the next k-tile to fetch and their advance per k-tile in bytes. A k-major
  // operand's tile column is part of the lane offsets, so its pointer only carries the k offset.
  const uint32_t stride_a = A_KM ? (uint32_t)(BK * g.lda * 2) : 128u;
  const uint32_t stride_b = B_KM ? (uint32_t)(BK * g.ldb * 2) : 128u;
  auto a_tile_ptr = [&](int ai) -> const char* {
    return (const char*)(A_KM ? g.A : g.A + (int64_t)a_row0(ai) * g.lda);
  };
  const char* pa = a_tile_ptr(ai_begin);
  const char* pb = (const char*)(B_KM ? g.B : g.B + (int64_t)bj * TILE * g.ldb);
  const char* pb_next = pb;
  const uint32_t ldsw = lds_base + (uint32_t)wave * 8192u;
  // an odd number of k-tiles: one more pair whose second k-tile is dead (see gen_mainloop16.py)
  const int npairs = (nk + 1) >> 1;
  const int odd = nk & 1;
  const uint32_t pen_a = odd ? 0u : stride_a, pen_b = odd ? 0u : stride_b;
  u16* stage = (u16*)(lds + RING16_BYTES + wave * STAGE16_BYTES);

  if (VAR == VAR_NT)
    asm volatile(ML16_NT_PROLOGUE
                 : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb)
                 : ML16_S_LDSW(ldsw), ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b),
                   ML16_NT_VGPR_INPUTS(oa, ob, ra, rb)
                 : "memory", "scc");
  else if (VAR == VAR_TN)
    asm volatile(ML16_TN_PROLOGUE
                 : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb)
                 : ML16_S_LDSW(ldsw), ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b),
                   ML16_TN_VGPR_INPUTS(oa, ob, ra, rb)
                 : "memory", "scc");
  else
    asm volatile(ML16_MIX_PROLOGUE
                 : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb)
                 : ML16_S_LDSW(ldsw), ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b),
                   ML16_MIX_VGPR_INPUTS(oa, ob, ra, rb)
                 : "memory", "scc");

  // What an epilogue carries from tile to tile of a sweep has to be small: over the main loop the
  // compiler only has v[0:ML16_*_FIRST_VGPR) for it.
  typename Epi::State st;
  for (int ai = ai_begin; ai < ai_end; ++ai) {
    // where the loader goes when this tile's k range is exhausted: the next A tile of the
    // sweep, or (after the last tile) this tile again, whose first k-tiles are loaded and never used
    const char* pa_next = a_tile_ptr(ai + 1 < ai_end ? ai + 1 : ai);
    int cnt = npairs;
    if (npairs == 1) { pa = pa_next; pb = pb_next; }
    if (VAR == VAR_NT)
      asm volatile(ML16_NT_TILE
                   : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb), "+" ML16_S_CNT(cnt)
                   : ML16_S_PA_NEXT(pa_next), ML16_S_PB_NEXT(pb_next), ML16_S_LDSW(ldsw),
                     ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b), ML16_S_ODD(odd),
                     ML16_S_PEN_A(pen_a), ML16_S_PEN_B(pen_b), ML16_NT_VGPR_INPUTS(oa, ob, ra, rb)
                   : "memory", "scc", ML16_S_SCRATCH_CLOBBERS, ML16_NT_CLOBBERS, ML16_ACC_CLOBBERS);
    else if (VAR == VAR_TN && NA == 7)
      asm volatile(ML16_TN_TILE7
                   : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb), "+" ML16_S_CNT(cnt)
                   : ML16_S_PA_NEXT(pa_next), ML16_S_PB_NEXT(pb_next), ML16_S_LDSW(ldsw),
                     ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b), ML16_S_ODD(odd),
                     ML16_S_PEN_A(pen_a), ML16_S_PEN_B(pen_b), ML16_TN_VGPR_INPUTS(oa, ob, ra, rb)
                   : "memory", "scc", ML16_S_SCRATCH_CLOBBERS, ML16_TN_CLOBBERS, ML16_ACC_CLOBBERS);
    else if (VAR == VAR_TN)
      asm volatile(ML16_TN_TILE
                   : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb), "+" ML16_S_CNT(cnt)
                   : ML16_S_PA_NEXT(pa_next), ML16_S_PB_NEXT(pb_next), ML16_S_LDSW(ldsw),
                     ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b), ML16_S_ODD(odd),
                     ML16_S_PEN_A(pen_a), ML16_S_PEN_B(pen_b), ML16_TN_VGPR_INPUTS(oa, ob, ra, rb)
                   : "memory", "scc", ML16_S_SCRATCH_CLOBBERS, ML16_TN_CLOBBERS, ML16_ACC_CLOBBERS);
    else if (NA == 7)
      asm volatile(ML16_MIX_TILE7
                   : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb), "+" ML16_S_CNT(cnt)
                   : ML16_S_PA_NEXT(pa_next), ML16_S_PB_NEXT(pb_next), ML16_S_LDSW(ldsw),
                     ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b), ML16_S_ODD(odd),
                     ML16_S_PEN_A(pen_a), ML16_S_PEN_B(pen_b), ML16_MIX_VGPR_INPUTS(oa, ob, ra, rb)
                   : "memory", "scc", ML16_S_SCRATCH_CLOBBERS, ML16_MIX_CLOBBERS, ML16_ACC_CLOBBERS);
    else
      asm volatile(ML16_MIX_TILE
                   : "+" ML16_S_PA(pa), "+" ML16_S_PB(pb), "+" ML16_S_CNT(cnt)
                   : ML16_S_PA_NEXT(pa_next), ML16_S_PB_NEXT(pb_next), ML16_S_LDSW(ldsw),
                     ML16_S_STRIDE_A(stride_a), ML16_S_STRIDE_B(stride_b), ML16_S_ODD(odd),
                     ML16_S_PEN_A(pen_a), ML16_S_PEN_B(pen_b), ML16_MIX_VGPR_INPUTS(oa, ob, ra, rb)
                   : "memory", "scc", ML16_S_SCRATCH_CLOBBERS, ML16_MIX_CLOBBERS, ML16_ACC_CLOBBERS);
    // The lane number goes through an empty block so that nothing of the epilogue's per-lane
    // address arithmetic is computed ahead of the main loop, which leaves the compiler only
    // v[0:ML16_*_FIRST_VGPR) for values that live across it.
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    Epi::open(st, ep, bj * TILE + wb * 128, split, wa, lane_e, ai == ai_begin);
    Epi::tile(st, ep, a_row0(ai) + wa * (NA * 16), bj * TILE + wb * 128, lane_e, stage, ai * TM);
    Epi::close(st, ep, bj * TILE + wb * 128, split, wa, lane_e);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // drain the trailing (unused) loads before LDS is released
  Epi::end(st, ep, bj * TILE + wb * 128, split, wa, lane);
}

// One block column of the wave's sub-tile (16 rows j x 128 bf16 values i) from the staging area
// to global memory: lane -> (row 4*p + lane/16, 16-byte piece lane%16), so 16 lanes write the
// 256 contiguous bytes of a row. out_row0 points at element (j0, i0) of the output.
// STREAM: the output is a [T, V]-sized buffer that nothing reads before the kernel ends; its
// stores carry the non-temporal hint so that they do not push the operand tiles the XCD's other
// workgroups share out of L2.
// EDGE: only rows < rows_valid and columns [cols_from, cols_valid) are written (both multiples of 8).
template <bool EDGE, bool STREAM = false>
DEVI void flush_stage16(const u16* stage, u16* out_row0, int64_t ld, int rows_valid, int cols_valid,
                        int cols_from, int lane) {
  const int piece = lane & 15;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int row = p * 4 + (lane >> 4);
    const u32x4 v = *(const u32x4*)((const char*)stage + row * STAGE16_PITCH + piece * 16);
    if (!EDGE || (row < rows_valid && piece * 8 < cols_valid && piece * 8 >= cols_from)) {
      u32x4* dst = (u32x4*)(out_row0 + (int64_t)row * ld + piece * 8);
      if (STREAM) __builtin_nontemporal_store(v, dst);
      else *dst = v;
    }
  }
}
DEVI void stage16_put(u16* stage, int lane, int ia, u32x2 v) {
  *(u32x2*)((char*)stage + (lane & 15) * STAGE16_PITCH + (ia * 16 + 4 * (lane >> 4)) * 2) = v;
}

// ---- plain store (dHidden, dWeight, stand-alone GEMM): out[j * ldo + i]
// NA < 8: the wave's sub-tile has only NA blocks of 16 values i (gemm16_sweep's narrow A tiles); the
// bounds of the EDGE instance then also stop at the sub-tile's width.
template <bool EDGE, int MODE, int NA_>
struct Store16Impl {
  static_assert(NA_ == 8 || EDGE, "narrow tiles use the bounds-checked instance");
  static constexpr int NA = NA_;
  typedef StoreParams Params;
  struct State {};
  static DEVI void open(State&, const Params&, int, int, int, int, bool) {}
  static DEVI void close(State&, const Params&, int, int, int, int) {}
  static DEVI void end(State&, const Params&, int, int, int, int) {}
  static DEVI void split_output(Params& p, int64_t bytes) { p.out = (char*)p.out + bytes; }
  static DEVI void tile(State&, const Params& p, int i0, int j0, int lane, u16* stage, int) {
    for_each_col([&](auto bc) {
      constexpr int b = decltype(bc)::value;
      float x[32];
      acc_col<b>(x);
      const int j = j0 + b * 16 + (lane & 15);
      if (MODE == 0 || MODE == 3) {
        // bf16: through the staging area, whole lines out (needs 16-byte aligned rows: the host
        // only takes this path when ldo % 8 == 0 and the output is 16-byte aligned)
        float js = 1.f;
        if (MODE == 3) js = (!EDGE || j < p.N) ? p.jscale[j] : 0.f;
#pragma unroll
        for (int a = 0; a < NA; ++a) {
          float x0 = x[a * 4], x1 = x[a * 4 + 1], x2 = x[a * 4 + 2], x3 = x[a * 4 + 3];
          if (MODE == 3) { x0 *= js; x1 *= js; x2 *= js; x3 *= js; }
          u32x2 v;
          v[0] = pack_bf16x2(x0, x1);
          v[1] = pack_bf16x2(x2, x3);
          stage16_put(stage, lane, a, v);
        }
        int cols_valid = p.M - i0;
        if (NA < 8) cols_valid = cols_valid < NA * 16 ? cols_valid : NA * 16;
        flush_stage16<EDGE>(stage, (u16*)p.out + (int64_t)(j0 + b * 16) * p.ldo + i0, p.ldo,
                            p.N - (j0 + b * 16), cols_valid, 0, lane);
      } else {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
          const int i = i0 + a * 16 + 4 * (lane >> 4);
          if (!EDGE || (j < p.N && i < p.M)) {
            f32x4* dst = (f32x4*)((float*)p.out + (int64_t)j * p.ldo + i);
            f32x4 v = {x[a * 4], x[a * 4 + 1], x[a * 4 + 2], x[a * 4 + 3]};
            if (MODE == 2) v += *dst;
            *dst = v;
          }
        }
      }
    });
  }
};
template <bool EDGE, int MODE> struct Store16 : Store16Impl<EDGE, MODE, 8> {};
template <int MODE> struct Store16Narrow : Store16Impl<true, MODE, 7> {};
template <bool E> using Store16Bf16 = Store16<E, 0>;
template <bool E> using Store16F32 = Store16<E, 1>;
template <bool E> using Accum16F32 = Store16<E, 2>;
template <bool E> using Store16Bf16Scaled = Store16<E, 3>;


// ---- forward: online softmax statistics (see FwdEpi). In a block column the 16 lanes l % 16 own
// the 16 tokens and the four lane groups l / 16 own 4 of every 16 vocabulary entries, so a token's
// 128 entries of the wave's sub-tile sit in four lanes. Per column those four lanes agree on the
// column's maximum, sum their exponentials relative to it, and lane group jb % 4 folds the result
// into the running statistics of token column jb, of which it keeps two (jb and jb + 4): ten to
// fourteen registers per lane live across the main loop. Partial statistics go to slot
// split * 2 + wa at the end of the sweep.
// The four lanes that share a token are 16 and 32 lanes apart. v_permlane16_swap exchanges the
// odd rows (of 16 lanes) of its first register with the even rows of its second, v_permlane32_swap
// rows 2-3 of the first with rows 0-1 of the second: applied to two copies of a value they leave
// (own, partner 16 / 32 lanes away) in every lane, as vector operations of a few cycles where a
// shuffle goes through the LDS crossbar (about a hundred cycles that nothing overlaps here: the
// wave is alone on its SIMD). The leading wait states are those a vector write needs before
// these instructions read it. (The compiler's own builtin for them returns one register for
// both results in this toolchain, hence the assembly.)
DEVI void swap_rows16(float& a, float& b) {
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
DEVI void swap_rows32(float& a, float& b) {
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
DEVI float group_max(float v) {
  float a = v, b = v;
  swap_rows16(a, b);
  a = b = fmaxf(a, b);
  swap_rows32(a, b);
  return fmaxf(a, b);
}
DEVI float group_min(float v) {
  float a = v, b = v;
  swap_rows16(a, b);
  a = b = fminf(a, b);
  swap_rows32(a, b);
  return fminf(a, b);
}
DEVI float group_sum(float v) {
  float a = v, b = v;
  swap_rows16(a, b);
  a = b = a + b;
  swap_rows32(a, b);
  return a + b;
}

// A logit that takes no part (past the vocabulary, or a row that an earlier tile of the sweep
// already covered): far below every real logit, finite so that 0 * it stays 0 in the entropy sum.
constexpr float MASKED_LOGIT = -1e30f;

template <bool EDGE, bool AFFINE, bool MOMENTS, bool SAVE>
struct Fwd16 {
  static constexpr int NA = 8;
  typedef FwdParams Params;
  // SAVE: s and q are relative to the row reference of the saved exponentials (fixed for the whole
  // sweep: nothing is rescaled); otherwise relative to the running maximum m.
  struct State {
    float m[2], s[2], q[2], xl[2], mn[2], sx[MOMENTS ? 2 : 1], sx2[MOMENTS ? 2 : 1];
  };
  static DEVI void split_output(Params&, int64_t) {}
  static DEVI void open(State& st, const Params&, int, int, int, int, bool first) {
    if (first) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        st.m[k] = neg_inf(); st.s[k] = 0.f; st.q[k] = 0.f; st.xl[k] = 0.f; st.mn[k] = pos_inf();
        if (MOMENTS) { st.sx[k] = 0.f; st.sx2[k] = 0.f; }
      }
    }
  }
  static DEVI void close(State&, const Params&, int, int, int, int) {}

  // v_new: the first vocabulary entry of the tile that no earlier tile of the sweep covered (the
  // last tile of a ragged vocabulary overlaps its predecessor); entries below it take no part.
  static DEVI void tile(State& st, const Params& p, int v0, int t0, int lane, u16* stage, int v_new) {
    if (v_new >= v0 + 128) return;    // every row of this wave's sub-tile is a repeat
    const bool overlap = v_new > v0;  // wave-uniform
    const int vl = v0 + 4 * (lane >> 4);
    const int group = lane >> 4;
    auto vidx = [&](int a, int r) { return vl + a * 16 + r; };
    // labels and row references of the 8 tokens this lane sees, fetched ahead of the columns
    int lab[8];
    float rr[SAVE ? 8 : 1];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const int t = t0 + b * 16 + (lane & 15);
      const bool live = !EDGE || t < p.T;
      const int64_t l = live ? p.labels[t] : -1;
      lab[b] = (l >= v_new && l < p.V) ? (int)l : -1;
      if (SAVE) rr[b] = live ? p.probs_ref[t] : 0.f;
    }
    ML16_AGPR_FENCE();
    for_each_col([&](auto bc) {
      constexpr int b = decltype(bc)::value;
      constexpr int k = b >> 2;
      float x[32];
      acc_col<b>(x);
      if (AFFINE) {
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float bv = 0.f;
            if (p.bias != nullptr && (!EDGE || vidx(a, r) < p.V)) bv = p.bias[vidx(a, r)];
            x[a * 4 + r] = (x[a * 4 + r] + bv) * p.scale;
          }
      }
      float tmax = neg_inf(), tmin = pos_inf(), sx = 0.f, sx2 = 0.f;
      if (!EDGE && !overlap) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
          tmax = fmaxf(tmax, x[i]);
          tmin = fminf(tmin, x[i]);
          if (MOMENTS) { sx += x[i]; sx2 = fmaf(x[i], x[i], sx2); }
        }
      } else {
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float xv = x[a * 4 + r];
            if ((!EDGE || vidx(a, r) < p.V) && vidx(a, r) >= v_new) {
              tmax = fmaxf(tmax, xv);
              tmin = fminf(tmin, xv);
              if (MOMENTS) { sx += xv; sx2 = fmaf(xv, xv, sx2); }
            } else {
              x[a * 4 + r] = MASKED_LOGIT;
            }
          }
      }
      float s = 0.f, q = 0.f;
      if (!SAVE) {
        // the column's reference: the maximum over the token's 128 entries in this sub-tile (see
        // ref_of); -inf only if every entry lies past the vocabulary
        tmax = group_max(tmax);
        const float mc = (!EDGE || tmax > neg_inf()) ? ref_of(tmax, p.c2) : 0.f;
        ML16_AGPR_FENCE();
#pragma unroll
        for (int a = 0; a < 8; ++a) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float t = fmaf(x[a * 4 + r], p.c2, -mc);
            const float e = fast_exp2(t);
            s += e;
            q = fmaf(t, e, q);
          }
          __builtin_amdgcn_sched_barrier(0);
          ML16_AGPR_FENCE();
        }
      } else {
        // Exponentials relative to the row reference, summed and stored as they are: one fma, one
        // v_exp_f32, two sums and half a packed conversion per logit. The 16 tokens x 128 entries of
        // the column go through the staging area and leave as whole lines.
        const float nr = -rr[b];
#pragma unroll
        for (int a = 0; a < 8; ++a) {
          float d[4];
#pragma unroll
          for (int e4 = 0; e4 < 4; ++e4) {
            const float t = fmaf(x[a * 4 + e4], p.c2, nr);
            const float e = fast_exp2(t);
            s += e;
            q = fmaf(t, e, q);
            d[e4] = e;
          }
          u32x2 pk;
          pk[0] = pack_bf16x2(d[0], d[1]);
          pk[1] = pack_bf16x2(d[2], d[3]);
          stage16_put(stage, lane, a, pk);
          // keeps the exponentials of one block next to the sums that consume them (left alone,
          // the scheduler computes all 32 first and spills them)
          __builtin_amdgcn_sched_barrier(0);
          ML16_AGPR_FENCE();
        }
        u16* out = p.probs + (int64_t)(t0 + b * 16) * p.ldv + v0;
        if (!EDGE && !overlap)
          flush_stage16<false, true>(stage, out, p.ldv, 16, 128, 0, lane);
        else
          flush_stage16<true, true>(stage, out, p.ldv, EDGE ? p.T - (t0 + b * 16) : 16, (int)p.ldv - v0,
                                    overlap ? v_new - v0 : 0, lane);
      }
      // the label's logit, if it is one of this lane's 32 entries
      float xl = 0.f;
      const bool hit = (lab[b] >= v0) && (lab[b] < v0 + 128);
      if (__builtin_amdgcn_ballot_w64(hit) != 0) {
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (vidx(a, r) == lab[b]) xl = x[a * 4 + r];
      }
      // The partial results pass through an empty block here: their readers come later (the last
      // one after the last column), and the compiler otherwise moves the summation chains of
      // every column down there, keeping all the exponentials alive in scratch memory until then.
      asm volatile("" : "+v"(s), "+v"(q), "+v"(tmin), "+v"(xl) : : ML16_ACC_CLOBBERS);
      s = group_sum(s);
      q = group_sum(q);
      tmin = group_min(tmin);
      xl = group_sum(xl);
      if (SAVE) tmax = group_max(tmax);
      if (MOMENTS) {
        asm volatile("" : "+v"(sx), "+v"(sx2));
        sx = group_sum(sx);
        sx2 = group_sum(sx2);
      }
      // lane group b % 4 folds the column into the running statistics of token column b
      if (group == (b & 3)) {
        if (SAVE) {
          st.s[k] += s;
          st.q[k] += q;
          st.m[k] = fmaxf(st.m[k], tmax);
        } else {
          // both sets of sums move to the reference of the larger maximum
          const float m_old = st.m[k];
          const float m_new = fmaxf(m_old, tmax);
          const float d_old = (m_old > neg_inf()) ? ref_diff(m_old, m_new, p.c2) : 0.f;
          const float d_col = (!EDGE || tmax > neg_inf()) ? ref_diff(tmax, m_new, p.c2) : 0.f;
          const float a_old = fast_exp2(d_old), a_col = fast_exp2(d_col);
          st.q[k] = a_old * fmaf(d_old, st.s[k], st.q[k]) + a_col * fmaf(d_col, s, q);
          st.s[k] = a_old * st.s[k] + a_col * s;
          st.m[k] = m_new;
        }
        st.mn[k] = fminf(st.mn[k], tmin);
        st.xl[k] += xl;
        if (MOMENTS) { st.sx[k] += sx; st.sx2[k] += sx2; }
      }
      asm volatile("" : "+v"(st.m[k]), "+v"(st.s[k]), "+v"(st.q[k]), "+v"(st.xl[k]), "+v"(st.mn[k])
                   : : ML16_ACC_CLOBBERS);
      if (MOMENTS) asm volatile("" : "+v"(st.sx[k]), "+v"(st.sx2[k]));
      __builtin_amdgcn_sched_barrier(0);
    });
  }

  static DEVI void end(State& st, const Params& p, int t0, int split, int wa, int lane) {
    const int slot = p.slot_base + split * 2 + wa;
    const int64_t PT = (int64_t)p.P * p.T;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int t = t0 + ((lane >> 4) + 4 * k) * 16 + (lane & 15);
      if (EDGE && t >= p.T) continue;
      float* w = p.ws + (int64_t)slot * p.T + t;
      w[0 * PT] = st.m[k]; w[1 * PT] = st.s[k]; w[2 * PT] = st.q[k]; w[3 * PT] = st.xl[k];
      w[4 * PT] = st.mn[k];
      if (MOMENTS) { w[5 * PT] = st.sx[k]; w[6 * PT] = st.sx2[k]; }
    }
  }
};
template <bool E> using Fwd16Plain = Fwd16<E, false, false, false>;
template <bool E> using Fwd16PlainMom = Fwd16<E, false, true, false>;
template <bool E> using Fwd16Affine = Fwd16<E, true, false, false>;
template <bool E> using Fwd16AffineMom = Fwd16<E, true, true, false>;
template <bool E> using Fwd16PlainSave = Fwd16<E, false, false, true>;
template <bool E> using Fwd16PlainMomSave = Fwd16<E, false, true, true>;
template <bool E> using Fwd16AffineSave = Fwd16<E, true, false, true>;
template <bool E> using Fwd16AffineMomSave = Fwd16<E, true, true, true>;

// ---- recompute: dlogits = (onehot - p) * g * invT * scale in bf16, [Tc, ldv] (see BwdEpi)
template <bool EDGE, bool AFFINE>
struct Bwd16 {
  static constexpr int NA = 8;
  typedef BwdParams Params;
  struct State {
    float nb[8], gs[8];
    int lab[8];
  };
  static DEVI void open(State& st, const Params& p, int t0, int, int, int lane, bool) {
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const int t = t0 + b * 16 + (lane & 15);
      if (!EDGE || t < p.T) {
        const int64_t l = p.labels[t];
        st.lab[b] = (l >= 0 && l < p.V) ? (int)l : -1;
        st.nb[b] = -ref_plus(p.row_max[t], p.c2, fast_log2(p.sum_exp[t]));
        st.gs[b] = p.grad[t] * p.inv_temp * p.scale;
      } else {
        st.lab[b] = -1; st.nb[b] = 0.f; st.gs[b] = 0.f;
      }
    }
  }
  static DEVI void close(State&, const Params&, int, int, int, int) {}
  static DEVI void end(State&, const Params&, int, int, int, int) {}
  static DEVI void split_output(Params&, int64_t) {}

  // (a tile that overlaps its predecessor rewrites the shared rows with the same values)
  static DEVI void tile(State& st, const Params& p, int v0, int t0, int lane, u16* stage, int) {
    const int vl = v0 + 4 * (lane >> 4);
    for_each_col([&](auto bc) {
      constexpr int b = decltype(bc)::value;
      float x[32];
      acc_col<b>(x);
      const int t = t0 + b * 16 + (lane & 15);
      const float nb = st.nb[b], gs = st.gs[b];
      const int lab = st.lab[b];
#pragma unroll
      for (int a = 0; a < 8; ++a) {
        const int vq = vl + a * 16;
        float d[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = vq + e;
          float xv = x[a * 4 + e];
          if (AFFINE) {
            float bv = 0.f;
            if (p.bias != nullptr && (!EDGE || v < p.V)) bv = p.bias[v];
            xv = (xv + bv) * p.scale;
          }
          const float pr = fast_exp2(fmaf(xv, p.c2, nb));
          float dv = -pr * gs;
          if (v == lab) dv += gs;
          if (EDGE && (v >= p.V || t >= p.T)) dv = 0.f;
          d[e] = dv;
        }
        u32x2 pk;
        pk[0] = pack_bf16x2(d[0], d[1]);
        pk[1] = pack_bf16x2(d[2], d[3]);
        stage16_put(stage, lane, a, pk);
      }
      flush_stage16<EDGE, true>(stage, p.dl + (int64_t)(t0 + b * 16) * p.ldv + v0, p.ldv, p.T - (t0 + b * 16),
                          (int)p.ldv - v0, 0, lane);
    });
  }
};
template <bool E> using Bwd16Plain = Bwd16<E, false>;
template <bool E> using Bwd16Affine = Bwd16<E, true>;

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Splits of the A range per B tile: enough workgroups to fill the chip, and at least 4 so that
// the 32 workgroups sharing an XCD's L2 form an 8 x 4 block (12 distinct operand tiles per sweep
// step) rather than 32 x 1 (33 tiles: with many B tiles that re-reads every B tile from HBM for
// every A tile).
int pick_splits(int nbj, int nai, int target_wgs) {
  int S = 1;
  while ((nbj * S < target_wgs || S < 4) && S * 2 <= nai && S < 64) S *= 2;
  return S;
}

enum { KERNEL_GENERIC = 0, KERNEL16_NT = 4, KERNEL16_TN = 5, KERNEL16_MIX = 6 };

// K ranges the hand-scheduled main loop takes: at least two whole k-tiles.
bool k16_ok(int64_t K) { return K >= 2 * BK && K % BK == 0; }

template <class Epi, int KERNEL>
int launch_region(const GemmArgs& g, int bj0, int nbj, int ai0, int nai, int S,
                  const typename Epi::Params& ep, hipStream_t stream) {
  if (nbj <= 0 || nai <= 0) return AREAL_OK;
  if (S > nai) S = nai;
  if (S < 1) S = 1;
  const Sched sc = make_sched(bj0, nbj, ai0, nai, S, g.sb_wgs == 8 ? 8 : 32);
  if constexpr (KERNEL >= KERNEL16_NT) {
    constexpr int VAR = KERNEL == KERNEL16_NT ? VAR_NT : KERNEL == KERNEL16_TN ? VAR_TN : VAR_MIX;
    // the loader addresses a tile as a 64-bit base plus 32-bit byte offsets per lane
    if (g.lda > (VAR == VAR_NT ? (1 << 22) : (1 << 24)) || g.ldb > (VAR == VAR_TN ? (1 << 24) : (1 << 22)))
      return AREAL_ERR_UNSUPPORTED;
    // every copy of a split-K launch needs two k-tiles too (split_ktiles() sees to the last one)
    if (!k16_ok(g.K) || (g.ksplit > 1 && (g.kt_per_split < 2 || g.K / BK - (g.ksplit - 1) * g.kt_per_split < 2)))
      return AREAL_ERR_UNSUPPORTED;
    // a k-major A operand carries its tile column in the lane offsets: one A tile per workgroup
    if (VAR != VAR_NT && S != nai) return AREAL_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gemm16_sweep<VAR, Epi>), dim3(sched_grid(sc) * (g.ksplit > 1 ? g.ksplit : 1)),
                       dim3(NTHREADS), 0, stream, g, sc, ep);
  } else {
    if (g.ksplit > 1) return AREAL_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gemm_nt_generic<Epi>), dim3(sched_grid(sc)), dim3(NTHREADS), 0, stream, g,
                       sc, ep);
  }
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// How a GEMM is cut into launches. The hand-scheduled kernel (k16: K a multiple of 64, at least
// 128, and the caller's epilogue and operand layout allow it) runs the interior tiles with the
// predicate-free epilogue, then the ragged last B tile and the ragged last A tile with the EDGE
// epilogue. Everything else is one launch of the generic kernel over all tiles.
struct Regions {
  bool k16;
  int nai_full, nbj_full;  // tiles entirely inside M and N (k16), else all tiles
  bool ragged_a, ragged_b;
  int S;                   // splits used for the interior and the ragged-B launch
  bool fold_a;             // the ragged last A tile runs as rows [M - 256, M) at the end of the last
                           // split's sweep (GemmArgs::overlap_last_a) instead of a launch of its own;
                           // set by fold_ragged_a() for the epilogues that support it
};
// The hand-scheduled forward and recompute launches take a ragged last vocabulary tile into the
// main launch when there is a full tile for it to overlap and whole 64-column groups (the stores
// of the saved buffers are 16-byte pieces, and columns [V, round_up(V, 64)) would stay unwritten).
void fold_ragged_a(Regions& r, int64_t M) {
  r.fold_a = r.k16 && r.ragged_a && r.nai_full >= 1 && M % BK == 0;
}
Regions plan_regions(int64_t M, int64_t N, int64_t K, int target_wgs, int S_fixed, bool allow16 = true) {
  Regions r;
  r.k16 = allow16 && k16_ok(K);
  r.fold_a = false;
  if (r.k16) {
    r.nai_full = (int)(M / TILE); r.nbj_full = (int)(N / TILE);
    r.ragged_a = (M % TILE) != 0; r.ragged_b = (N % TILE) != 0;
  } else {
    r.nai_full = (int)ceil_div_i64(M, TILE); r.nbj_full = (int)ceil_div_i64(N, TILE);
    r.ragged_a = false; r.ragged_b = false;
  }
  const int nbj_all = r.nbj_full + (r.ragged_b ? 1 : 0);
  r.S = r.nai_full > 0 ? (S_fixed > 0 ? S_fixed : pick_splits(nbj_all, r.nai_full, target_wgs)) : 0;
  if (r.S > r.nai_full) r.S = r.nai_full;
  return r;
}

// Epi16<EDGE> is the epilogue written for the hand-scheduled kernel's accumulator layout, Epi32<EDGE>
// the same arithmetic for the generic kernel's; ep_edge_a is the parameter block of the ragged-A
// launch (it may differ from ep in where it writes its partial results).
// MERGE_EDGES: epilogues whose bounds predicates are cheap (plain stores) run ONE launch of the
// EDGE = true instance over all tiles when any tile is ragged: a separate launch for the last
// row of tiles has too few workgroups to fill the chip and each walks the whole K range.
template <template <bool> class Epi16, template <bool> class Epi32, class P, int KERNEL16, bool MERGE_EDGES = false>
int launch_gemm(const GemmArgs& g, const Regions& r, const P& ep, const P& ep_edge_a,
                hipStream_t stream) {
  int rc;
  if (!r.k16) {
    if constexpr (KERNEL16 != KERNEL16_NT) return AREAL_ERR_UNSUPPORTED;  // the generic kernel reads k-contiguous operands
    return launch_region<Epi32<true>, KERNEL_GENERIC>(g, 0, r.nbj_full, 0, r.nai_full, r.S, ep, stream);
  }
  if (MERGE_EDGES && (r.ragged_a || r.ragged_b)) {
    const int nai = r.nai_full + (r.ragged_a ? 1 : 0);
    return launch_region<Epi16<true>, KERNEL16>(g, 0, r.nbj_full + (r.ragged_b ? 1 : 0), 0, nai,
                                                r.S == r.nai_full ? nai : r.S, ep, stream);
  }
  GemmArgs gm = g;
  int nai_main = r.nai_full;
  if constexpr (KERNEL16 == KERNEL16_NT) {
    if (r.fold_a) { gm.overlap_last_a = 1; ++nai_main; }
  }
  if ((rc = launch_region<Epi16<false>, KERNEL16>(gm, 0, r.nbj_full, 0, nai_main, r.S, ep, stream)) != AREAL_OK)
    return rc;
  if (r.ragged_b &&
      (rc = launch_region<Epi16<true>, KERNEL16>(gm, r.nbj_full, 1, 0, nai_main, r.S, ep, stream)) != AREAL_OK)
    return rc;
  if (r.ragged_a && nai_main == r.nai_full &&
      (rc = launch_region<Epi16<true>, KERNEL16>(g, 0, r.nbj_full + (r.ragged_b ? 1 : 0), r.nai_full, 1, 1,
                                                 ep_edge_a, stream)) != AREAL_OK)
    return rc;
  return AREAL_OK;
}

int check_operand(const void* p, int64_t ld) {
  if (p == nullptr) return AREAL_ERR_BAD_ARG;
  if (!aligned16(p) || (ld % 8) != 0) return AREAL_ERR_ALIGNMENT;
  return AREAL_OK;
}

// Slots of partial softmax statistics per token written by the forward launches: per split of
// the vocabulary range, 2 wave rows x (in the 32x32 kernels) the 2 lane groups that share a
// token; the hand-scheduled kernels combine their 4 lane groups in registers.
int fwd_slots_per_split(const Regions& r) { return r.k16 ? 2 : 4; }
int fwd_slots(const Regions& r) { return fwd_slots_per_split(r) * (r.S + ((r.ragged_a && !r.fold_a) ? 1 : 0)); }

// The four plain-store epilogues over either kernel. mode: 0 bf16, 1 fp32, 2 fp32 accumulate,
// 3 bf16 with a factor per output row. The hand-scheduled kernel writes bf16 as 16-byte pieces of
// whole rows, which needs aligned output rows; the generic kernel (k-contiguous operands only)
// takes what it cannot. S_fixed as plan_regions (stores want one A tile per workgroup).
// A k-major A whose n = ceil(M / 256) tiles are filled to 7 / 8 at most (M <= 224 n, e.g. 896 =
// 3.5 x 256): n tiles of 224 cover M too and each costs 7 / 8 of a full tile.
bool narrow_a_tiles(int64_t M) {
  const int64_t n = ceil_div_i64(M, TILE);
  return M % TILE != 0 && M <= n * (TILE - 32);
}
template <int KERNEL16>
int launch_store(const GemmArgs& g, const StoreParams& ep, int mode, hipStream_t stream) {
  bool allow16 = true;
  if (mode == 0 || mode == 3) allow16 = ep.ldo % 8 == 0 && aligned16(ep.out) && ep.M % 8 == 0;
  const Regions r = plan_regions(ep.M, ep.N, g.K, 0, 1 << 20, allow16);
  if constexpr (KERNEL16 != KERNEL16_NT) {
    // the modes the two backward contractions use: dWeight 0 - 2, dHidden 0, 1 and 3
    constexpr int UNUSED_MODE = KERNEL16 == KERNEL16_TN ? 3 : 2;
    if (r.k16 && mode != UNUSED_MODE && narrow_a_tiles(ep.M)) {
      const int nai = (int)ceil_div_i64(ep.M, TILE), nbj = (int)ceil_div_i64(ep.N, TILE);
      if (mode == 0) return launch_region<Store16Narrow<0>, KERNEL16>(g, 0, nbj, 0, nai, nai, ep, stream);
      if (mode == 1) return launch_region<Store16Narrow<1>, KERNEL16>(g, 0, nbj, 0, nai, nai, ep, stream);
      constexpr int LAST_MODE = KERNEL16 == KERNEL16_TN ? 2 : 3;
      return launch_region<Store16Narrow<LAST_MODE>, KERNEL16>(g, 0, nbj, 0, nai, nai, ep, stream);
    }
  }
  switch (mode) {
    case 0: return launch_gemm<Store16Bf16, StoreBf16, StoreParams, KERNEL16, true>(g, r, ep, ep, stream);
    case 1: return launch_gemm<Store16F32, StoreF32, StoreParams, KERNEL16, true>(g, r, ep, ep, stream);
    case 2: return launch_gemm<Accum16F32, AccumF32, StoreParams, KERNEL16, true>(g, r, ep, ep, stream);
    default: return launch_gemm<Store16Bf16Scaled, StoreBf16Scaled, StoreParams, KERNEL16, true>(g, r, ep, ep, stream);
  }
}

// dHidden [T, H] has few output tiles when the model is small (H / 256 x T / 256). When the
// tile count does not fill whole rounds of 256 workgroups, the vocabulary (K) range is split
// over copies of the schedule, each writing an fp32 partial result that
// splitk_reduce_bf16_kernel sums.
// The launch is a schedule of super-blocks of up to 32 workgroups; super-block sb of copy c
// runs on XCD (sb + c * n_sb) % 8, whose 32 CUs take its workgroups as they free up. Cost of
// z copies in units of one workgroup's full K range = the busiest XCD's rounds of 32
// workgroups, each K / z long, plus a small charge per split for the reduction of the partial
// results.
double sched_cost(const Sched& sc, int z) {
  int64_t load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int c = 0; c < z; ++c)
    for (int sb = 0; sb < sc.n_sb; ++sb) {
      const int sbj = sb % sc.n_sb_j, sbs = sb / sc.n_sb_j;
      const int nb = sc.nbj - sbj * sc.RB < sc.RB ? sc.nbj - sbj * sc.RB : sc.RB;
      const int ns = sc.S - sbs * sc.RS < sc.RS ? sc.S - sbs * sc.RS : sc.RS;
      load[(sb + c * sc.n_sb) & 7] += (int64_t)(nb > 0 ? nb : 0) * (ns > 0 ? ns : 0);
    }
  int64_t worst = 0;
  for (int x = 0; x < 8; ++x) worst = load[x] > worst ? load[x] : worst;
  return (double)ceil_div_i64(worst, 32) / z + 0.03 * (z - 1);
}

// k-tiles per copy of a launch whose nk k-tiles are split over (up to) z copies: whole pairs (an
// even count runs without a dead k-tile), no empty copy, and at least two k-tiles in the last one.
void split_ktiles(int nk, int& z, int& kps) {
  kps = (int)ceil_div_i64(nk, z);
  kps += kps & 1;
  z = (int)ceil_div_i64(nk, kps);
  if (z > 1 && nk - (z - 1) * kps < 2) {  // a single k-tile left over: the last copy but one takes it
    kps += 2;
    z = (int)ceil_div_i64(nk, kps);
  }
}

int dh_ksplit(int64_t H, int64_t T, int64_t K) {
  const int64_t tiles = ceil_div_i64(H, TILE) * ceil_div_i64(T, TILE);
  if (tiles >= 2048 || K % BK != 0) return 1;
  const int64_t nk = K / BK;
  const int nai = (int)ceil_div_i64(H, TILE), nbj = (int)ceil_div_i64(T, TILE);
  const Sched sc = make_sched(0, nbj, 0, nai, nai);
  int best = 1;
  double best_cost = sched_cost(sc, 1);
  for (int z = 2; z <= 16 && z <= nk / 8; ++z) {
    const double cost = sched_cost(sc, z);
    if (cost < best_cost - 1e-9) { best_cost = cost; best = z; }
  }
  return best;
}
size_t dh_partial_bytes(int64_t H, int64_t T, int64_t K) {
  const int z = dh_ksplit(H, T, K);
  return z > 1 ? (size_t)z * (size_t)(T * H) * sizeof(float) + 256 : 0;
}

// The weight can be contracted as stored ([V, H], k-major for dHidden) when its V rows cover the
// K = round_up(V, 64) rows the kernel reads (and make two k-tiles, which the kernel that reads
// k-major operands needs); otherwise a zero-padded transposed copy is used.
bool dh_weight_in_place(int64_t V) { return V % BK == 0 && V >= 2 * BK; }

// dHidden[t, h] = tscale[t] * sum_v dl[t, v] * W[v, h] (tscale = 1 when null), bf16 out;
// split-K through `partial` when it pays. w is the weight itself [V, H] when
// dh_weight_in_place(V), else its transposed copy W^T [H, ldv].
template <int KERNEL16>
int launch_dhidden_k(const GemmArgs& g0, int64_t H, int64_t T, int64_t ldv, void* dhidden,
                     float* partial, const float* tscale, hipStream_t stream) {
  GemmArgs g = g0;
  int z = dh_ksplit(H, T, ldv);
  int kps = 0;
  if (z > 1) split_ktiles((int)(ldv / BK), z, kps);
  if (z <= 1 || partial == nullptr) {
    const StoreParams ep{dhidden, H, (int)H, (int)T, tscale};
    return launch_store<KERNEL16>(g, ep, tscale != nullptr ? 3 : 0, stream);
  }
  g.ksplit = z;
  g.kt_per_split = kps;
  g.zstride = T * H * (int64_t)sizeof(float);
  const StoreParams ep{partial, H, (int)H, (int)T, nullptr};
  int rc = launch_store<KERNEL16>(g, ep, 1, stream);
  if (rc != AREAL_OK) return rc;
  int64_t blocks = ceil_div_i64(T * H, 256 * 4);
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(splitk_reduce_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, partial,
                     z, T * H, T * H, tscale, H, (u16*)dhidden, g.skip_if_set);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}
int launch_dhidden(const u16* w, int64_t V, const u16* dl, int64_t ldv, int64_t H, int64_t T,
                   void* dhidden, float* partial, const float* tscale, const int* skip_if_set,
                   hipStream_t stream) {
  if (dh_weight_in_place(V)) {
    GemmArgs g{w, H, (int)H, dl, ldv, (int)T, (int)ldv, (int)H, 0};
    g.skip_if_set = skip_if_set;
    return launch_dhidden_k<KERNEL16_MIX>(g, H, T, ldv, dhidden, partial, tscale, stream);
  }
  GemmArgs g{w, ldv, (int)H, dl, ldv, (int)T, (int)ldv, 0, 0};
  g.skip_if_set = skip_if_set;
  return launch_dhidden_k<KERNEL16_NT>(g, H, T, ldv, dhidden, partial, tscale, stream);
}

// dWeight [V, H] in bf16 has ceil(V / 256) x ceil(H / 256) output tiles, one per workgroup, in
// super-blocks of 32 that go round-robin to the XCDs. When their number is not a multiple of 8 the
// last round occupies a few XCDs for a whole K range while the others idle (594 x 16 tiles: 298
// super-blocks, 38 rounds on two XCDs against 37 on six). The B tiles of that last partial round
// are then contracted by a second launch that splits the token (K) range over z copies of its
// schedule, fp32 partial results summed by splitk_reduce_bf16_kernel.
struct DwTail {
  int nbj_main;  // B tiles of the first launch
  int z, kps;    // copies and k-tiles per copy of the second (z <= 1: there is none)
  int64_t rows;  // vocabulary rows of the second launch
  int sb_wgs;    // workgroups per super-block of the second launch's schedule
};
DwTail plan_dw_tail(int64_t H, int64_t V, int64_t Tpad) {
  const int nai = (int)ceil_div_i64(H, TILE), nbj = (int)ceil_div_i64(V, TILE);
  DwTail t{nbj, 1, 0, 0, 32};
  if (!k16_ok(Tpad) || H % 8 != 0) return t;
  const Sched sc = make_sched(0, nbj, 0, nai, nai);
  if (sc.n_sb % 8 == 0) return t;
  const int n_sb_s = sc.n_sb / sc.n_sb_j;
  int nj = sc.n_sb_j;
  while (nj > 0 && (nj * n_sb_s) % 8 != 0) --nj;
  if (nj == 0) return t;
  const int64_t nk = Tpad / BK;
  int best = 1, best_sb = 32;
  double best_cost = sched_cost(make_sched(nj * sc.RB, nbj - nj * sc.RB, 0, nai, nai), 1);
  for (int sb_wgs = 32; sb_wgs >= 8; sb_wgs -= 24) {
    const Sched st = make_sched(nj * sc.RB, nbj - nj * sc.RB, 0, nai, nai, sb_wgs);
    for (int z = 2; z <= 8 && z <= nk / 8; ++z) {
      const double cost = sched_cost(st, z);
      if (cost < best_cost - 1e-9) { best_cost = cost; best = z; best_sb = sb_wgs; }
    }
  }
  // rounds of a whole K range: before, and after with the first launch's even rounds. A k-tile
  // takes about a microsecond; the two extra launches have to be paid for.
  const double before = (double)ceil_div_i64(sc.n_sb, 8), after = (double)(nj * n_sb_s / 8) + best_cost;
  if (best <= 1 || (before - after) * (double)nk < 16.0) return t;
  t.nbj_main = nj * sc.RB;
  t.z = best;
  t.sb_wgs = best_sb;
  split_ktiles((int)nk, t.z, t.kps);
  t.rows = V - (int64_t)t.nbj_main * TILE;
  if (t.z <= 1) t = DwTail{nbj, 1, 0, 0, 32};
  return t;
}
size_t dw_tail_bytes(int64_t H, int64_t V, int64_t Tpad) {
  const DwTail t = plan_dw_tail(H, V, Tpad);
  return t.z > 1 ? (size_t)t.z * (size_t)(t.rows * H) * sizeof(float) + 256 : 0;
}

// dWeight [V, H] in bf16 = B^T A over the K token rows of the k-major operands g.A [K, H] and
// g.B [K, ldv]: whole rounds of super-blocks in one launch, then (plan_dw_tail) the remaining
// vocabulary rows with the token range split, through dw_part (dw_tail_bytes(H, V, K) bytes).
int launch_dweight_bf16(GemmArgs g, int64_t H, int64_t V, int64_t ldv, void* dweight, float* dw_part,
                        hipStream_t stream) {
  const int64_t K = g.K;
  const DwTail tail = dw_part != nullptr ? plan_dw_tail(H, V, K) : DwTail{0, 1, 0, 0, 32};
  int rc;
  if (tail.z <= 1) {
    const StoreParams ep{dweight, H, (int)H, (int)V, nullptr};
    return launch_store<KERNEL16_TN>(g, ep, 0, stream);
  }
  const int64_t v0 = (int64_t)tail.nbj_main * TILE;
  GemmArgs gm = g;
  gm.N = (int)v0;
  const StoreParams ep{dweight, H, (int)H, (int)v0, nullptr};
  rc = launch_store<KERNEL16_TN>(gm, ep, 0, stream);
  if (rc != AREAL_OK) return rc;
  GemmArgs gt = g;
  gt.B = g.B + v0;
  gt.N = (int)tail.rows;
  gt.bcols = (int)(ldv - v0);
  gt.ksplit = tail.z;
  gt.kt_per_split = tail.kps;
  gt.sb_wgs = tail.sb_wgs;
  gt.zstride = tail.rows * H * (int64_t)sizeof(float);
  const StoreParams ept{dw_part, H, (int)H, (int)tail.rows, nullptr};
  rc = launch_store<KERNEL16_TN>(gt, ept, 1, stream);
  if (rc != AREAL_OK) return rc;
  int64_t blocks = ceil_div_i64(tail.rows * H, 256 * 4);
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(splitk_reduce_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, dw_part,
                     tail.z, tail.rows * H, tail.rows * H, (const float*)nullptr, H,
                     (u16*)dweight + v0 * H, g.skip_if_set);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // namespace

// =======================================================================================
// C ABI
// =======================================================================================
extern "C" {

// out[j*ldo + i] = sum_k A[i*lda + k] * B[j*ldb + k]; A, B bf16; K % 8 == 0, M % 4 == 0.
int areal_gemm_nt_bf16(const void* A, int64_t lda, const void* B, int64_t ldb, void* out,
                       int64_t ldo, int64_t M, int64_t N, int64_t K, int out_mode,
                       hipStream_t stream) {
  if (M < 0 || N < 0 || K < 0 || out == nullptr || out_mode < 0 || out_mode > 2)
    return AREAL_ERR_BAD_ARG;
  if (M == 0 || N == 0) return AREAL_OK;
  if (K % 8 != 0 || M % 4 != 0) return AREAL_ERR_ALIGNMENT;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  int rc;
  if ((rc = check_operand(A, lda)) != AREAL_OK) return rc;
  if ((rc = check_operand(B, ldb)) != AREAL_OK) return rc;
  if (out_mode == 0 ? (ldo % 4 != 0 || ((uintptr_t)out & 7)) : (ldo % 4 != 0 || !aligned16(out)))
    return AREAL_ERR_ALIGNMENT;
  GemmArgs g{(const u16*)A, lda, (int)M, (const u16*)B, ldb, (int)N, (int)K, 0, 0};
  const StoreParams ep{out, ldo, (int)M, (int)N};
  return launch_store<KERNEL16_NT>(g, ep, out_mode, stream);
}

int areal_abi_version(void) { return 3; }  // AREAL_HIP_ABI_VERSION of include/areal_hip.h

size_t areal_lmhead_probs_bytes(int64_t T, int64_t V) {
  if (T <= 0 || V <= 0) return 0;
  return (size_t)round_up_i64(T, 2 * BK) * (size_t)round_up_i64(V, BK) * 2;
}

static Regions fwd_regions(int64_t T, int64_t H, int64_t V) {
  Regions r = plan_regions(V, T, H, 512, 0);
  fold_ragged_a(r, V);
  return r;
}

size_t areal_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (T <= 0 || V <= 0 || H <= 0) return 0;
  return (size_t)NSTAT * fwd_slots(fwd_regions(T, H, V)) * (size_t)T * sizeof(float);
}

// Forward. hidden [T,H] bf16, weight [V,H] bf16, labels [T] int64 (labels outside [0, V) give
// a label logit of 0). Outputs are fp32 [T]; any output pointer other than row_max / sum_exp
// may be null; vocab_mean and vocab_norm cost two extra operations per logit and are computed
// only when one of them is requested.
//
// probs / probs_ref / probs_status (all null or all set) keep the exponentials of the softmax
// for areal_lmhead_bwd_saved: probs bf16 [round_up(T, 128)][round_up(V, 64)] (rows >= T are not
// written) holds e = 2^(c2 x - probs_ref[t]); probs_ref fp32 [T] is a per-row reference taken
// from a few logits of the row before the sweep; *probs_status (one int) is set to 0 when every
// row's exponentials are in range and to 1 when some row's maximum lies more than REF_WINDOW
// binades above its estimate: then probs must not be used and the backward has to recompute
// (the per-token outputs are right either way).
int areal_lmhead_fwd(const void* hidden, const void* weight, const float* bias,
                     const int64_t* labels, int64_t T, int64_t H, int64_t V,
                     float inv_temperature, float logit_scale, float* logprobs, float* entropy,
                     float* vocab_min, float* vocab_max, float* vocab_mean, float* vocab_norm,
                     float* row_max, float* sum_exp, void* probs, size_t probs_bytes,
                     float* probs_ref, int* probs_status, void* workspace, size_t workspace_bytes,
                     hipStream_t stream) {
  if (T < 0 || H <= 0 || V <= 0 || labels == nullptr) return AREAL_ERR_BAD_ARG;
  if ((probs == nullptr) != (probs_ref == nullptr) || (probs == nullptr) != (probs_status == nullptr))
    return AREAL_ERR_BAD_ARG;
  if (probs != nullptr && probs_bytes < areal_lmhead_probs_bytes(T, V)) return AREAL_ERR_WORKSPACE;
  if (probs != nullptr && !aligned16(probs)) return AREAL_ERR_ALIGNMENT;
  if (!(inv_temperature > 0.f) || !(logit_scale > 0.f)) return AREAL_ERR_BAD_ARG;
  if (T == 0) return AREAL_OK;
  if (T > (1 << 30) || V > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  int rc;
  if ((rc = check_operand(hidden, H)) != AREAL_OK) return rc;
  if ((rc = check_operand(weight, H)) != AREAL_OK) return rc;
  const size_t need = areal_lmhead_fwd_workspace_bytes(T, H, V);
  if (workspace == nullptr || workspace_bytes < need) return AREAL_ERR_WORKSPACE;
  const Regions r = fwd_regions(T, H, V);
  const int P = fwd_slots(r);
  GemmArgs g{(const u16*)weight, H, (int)V, (const u16*)hidden, H, (int)T, (int)H, 0, 0};
  FwdParams ep{labels, (int)T, (int)V, logit_scale, inv_temperature * LOG2E, bias,
               (float*)workspace, P, 0, (u16*)probs, round_up_i64(V, BK), probs_ref};
  FwdParams ep_a = ep;
  ep_a.slot_base = fwd_slots_per_split(r) * r.S;
  const bool affine = (logit_scale != 1.0f) || (bias != nullptr);
  const bool moments = (vocab_mean != nullptr) || (vocab_norm != nullptr);
  const float c2 = inv_temperature * LOG2E;
  if (probs != nullptr) {
    hipLaunchKernelGGL(lmhead_rowref_kernel, dim3((unsigned)ceil_div_i64(T, 4 * REF_TOK)), dim3(256), 0, stream,
                       (const u16*)hidden, (const u16*)weight, bias, labels, (int)T, (int)H, (int)V,
                       logit_scale, c2, probs_ref, probs_status);
    AREAL_CHECK_LAUNCH();
  }
  // (each launch_gemm names the epilogue for the hand-scheduled kernel and the one for the generic kernel)
  auto fwd_plain = [&](const GemmArgs& gg) {
    if (!affine && !moments) return launch_gemm<Fwd16Plain, FwdPlain, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
    if (!affine) return launch_gemm<Fwd16PlainMom, FwdPlainMom, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
    if (!moments) return launch_gemm<Fwd16Affine, FwdAffine, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
    return launch_gemm<Fwd16AffineMom, FwdAffineMom, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
  };
  auto fwd_save = [&](const GemmArgs& gg) {
    if (!affine && !moments) return launch_gemm<Fwd16PlainSave, FwdPlainSave, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
    if (!affine) return launch_gemm<Fwd16PlainMomSave, FwdPlainMomSave, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
    if (!moments) return launch_gemm<Fwd16AffineSave, FwdAffineSave, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
    return launch_gemm<Fwd16AffineMomSave, FwdAffineMomSave, FwdParams, KERNEL16_NT>(gg, r, ep, ep_a, stream);
  };
  auto merge = [&](int ref_sums, const float* ref, const int* gate, int gate_run_if_set) {
    hipLaunchKernelGGL(lmhead_merge_kernel, dim3((unsigned)ceil_div_i64(T, 64)), dim3(64 * MERGE_WAVES),
                       0, stream, (const float*)workspace, P, (int)T, (int)V, ref_sums, c2, logprobs,
                       entropy, vocab_min, vocab_max, vocab_mean, vocab_norm, row_max, sum_exp, ref,
                       probs_status, gate, gate_run_if_set);
  };
  if (probs == nullptr) {
    if ((rc = fwd_plain(g)) != AREAL_OK) return rc;
    merge(0, nullptr, nullptr, 0);
  } else if (r.k16) {
    // The saving sweep takes its sums relative to the row references, which is only right for rows
    // whose maximum is within the window above the estimate. The merge raises *probs_status if
    // some row is outside; the plain sweep and its merge are queued behind it and do their work
    // only in that case (otherwise every workgroup of them returns at once), so the outputs are
    // right either way without the host looking at the status in between.
    if ((rc = fwd_save(g)) != AREAL_OK) return rc;
    merge(1, probs_ref, nullptr, 0);
    AREAL_CHECK_LAUNCH();
    GemmArgs gf = g;
    gf.skip_if_set = probs_status;
    gf.run_if_set = 1;
    if ((rc = fwd_plain(gf)) != AREAL_OK) return rc;
    merge(0, nullptr, probs_status, 1);
  } else {
    // the generic kernel's saving epilogue keeps its sums relative to each tile's maximum: the
    // outputs do not depend on the row reference, only the saved buffer does
    if ((rc = fwd_save(g)) != AREAL_OK) return rc;
    merge(0, probs_ref, nullptr, 0);
  }
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// Backward workspace (bf16): W^T [H, ldv] + dl [Tc, ldv] per token chunk; chunks that are not a
// multiple of 64 tokens (or shorter than 128) also need hidden^T [H, ldt] and dlT [V, ldt]
// (token_chunk a multiple of 64 and T a multiple of 64, both at least 128, avoid them).
size_t areal_lmhead_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t token_chunk) {
  if (T <= 0 || H <= 0 || V <= 0 || token_chunk <= 0) return 0;
  const int64_t Tc = token_chunk < T ? token_chunk : T;
  const int64_t ldv = round_up_i64(V, BK), ldt = round_up_i64(Tc, BK);
  int64_t elems = (dh_weight_in_place(V) ? 0 : H * ldv) + Tc * ldv;
  const bool ragged = !k16_ok(Tc) || ((T % Tc) != 0 && !k16_ok(T % Tc));  // some chunk cannot be read k-major
  if (ragged) elems += H * ldt + V * ldt;
  // slack for 256-byte sub-buffer alignment
  // (the last term: partial results of the bf16 dWeight store, one chunk covering the batch)
  return (size_t)elems * 2 + dh_partial_bytes(H, Tc, ldv) + (Tc >= T ? dw_tail_bytes(H, V, Tc) : 0) + 6 * 256;
}

// Backward. grad_logprobs [T] fp32 = dLoss/dlogprobs. Writes dhidden [T,H] bf16 and the weight
// gradient into dweight [V,H]: fp32, overwritten (accumulate == 0) or added to (accumulate == 1),
// or bf16 written by the contraction itself (accumulate == 2; one token chunk only, i.e.
// token_chunk >= T: several chunks need the fp32 sum).
int areal_lmhead_bwd(const void* hidden, const void* weight, const float* bias,
                     const int64_t* labels, const float* row_max, const float* sum_exp,
                     const float* grad_logprobs, int64_t T, int64_t H, int64_t V,
                     float inv_temperature, float logit_scale, void* dhidden, void* dweight,
                     float* dbias, int accumulate, int64_t token_chunk, void* workspace,
                     size_t workspace_bytes, hipStream_t stream) {
  if (T < 0 || H <= 0 || V <= 0 || token_chunk <= 0) return AREAL_ERR_BAD_ARG;
  if (accumulate < 0 || accumulate > 2) return AREAL_ERR_BAD_ARG;
  // accumulate == 2: dweight is bf16 and written by the contraction itself, which a single chunk allows
  const bool dw_bf16 = accumulate == 2;
  if (dw_bf16 && token_chunk < T) return AREAL_ERR_UNSUPPORTED;
  float* const dweight_f32 = (float*)dweight;
  if (labels == nullptr || row_max == nullptr || sum_exp == nullptr || grad_logprobs == nullptr)
    return AREAL_ERR_BAD_ARG;
  if (dhidden == nullptr && dweight_f32 == nullptr) return AREAL_ERR_BAD_ARG;
  if (T == 0) return AREAL_OK;
  if (T > (1 << 30) || V > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  int rc;
  if ((rc = check_operand(hidden, H)) != AREAL_OK) return rc;
  if ((rc = check_operand(weight, H)) != AREAL_OK) return rc;
  if (dhidden != nullptr && !aligned16(dhidden)) return AREAL_ERR_ALIGNMENT;
  if (dweight_f32 != nullptr && !aligned16(dweight_f32)) return AREAL_ERR_ALIGNMENT;
  if (workspace == nullptr ||
      workspace_bytes < areal_lmhead_bwd_workspace_bytes(T, H, V, token_chunk))
    return AREAL_ERR_WORKSPACE;

  const int64_t Tc_max = token_chunk < T ? token_chunk : T;
  const int64_t ldv = round_up_i64(V, BK), ldt = round_up_i64(Tc_max, BK);
  auto carve = [](char*& p, int64_t bytes) {
    char* r = (char*)(((uintptr_t)p + 255) & ~(uintptr_t)255);
    p = r + bytes;
    return (u16*)r;
  };
  char* wp = (char*)workspace;
  const bool ragged = !k16_ok(Tc_max) || ((T % Tc_max) != 0 && !k16_ok(T % Tc_max));
  const bool w_in_place = dh_weight_in_place(V);
  u16* wT = w_in_place ? nullptr : carve(wp, H * ldv * 2);
  u16* dl = carve(wp, Tc_max * ldv * 2);
  u16* hT = ragged ? carve(wp, H * ldt * 2) : nullptr;
  u16* dlT = ragged ? carve(wp, V * ldt * 2) : nullptr;
  float* dh_part = dh_partial_bytes(H, Tc_max, ldv) ? (float*)carve(wp, dh_partial_bytes(H, Tc_max, ldv)) : nullptr;
  float* dw_part = (dw_bf16 && dw_tail_bytes(H, V, Tc_max)) ? (float*)carve(wp, dw_tail_bytes(H, V, Tc_max)) : nullptr;

  const float c2 = inv_temperature * LOG2E;
  const bool affine = (logit_scale != 1.0f) || (bias != nullptr);
  if (dhidden != nullptr && !w_in_place) {
    // W^T [H, ldv]: rows = h, columns = v (zero padded to ldv).
    hipLaunchKernelGGL(transpose_pad_bf16_kernel,
                       dim3((unsigned)ceil_div_i64(H, 64), (unsigned)ceil_div_i64(ldv, 64)),
                       dim3(256), 0, stream, (const u16*)weight, H, (int)V, (int)H, wT, ldv);
    AREAL_CHECK_LAUNCH();
  }
  for (int64_t t0 = 0; t0 < T; t0 += Tc_max) {
    const int64_t Tc = (T - t0) < Tc_max ? (T - t0) : Tc_max;
    const int64_t ldt_c = round_up_i64(Tc, BK);
    const u16* hid_c = (const u16*)hidden + t0 * H;
    // dWeight reads dl and hidden k-major (no transposed copies) when the chunk is a multiple
    // of 64 tokens (at least 128); otherwise it goes through dlT and hidden^T.
    const bool tn = k16_ok(Tc) && dweight_f32 != nullptr;
    const bool need_dlT = dweight_f32 != nullptr && !tn;
    // 1. recompute logits of the chunk, emit dlogits
    {
      GemmArgs g{(const u16*)weight, H, (int)V, hid_c, H, (int)Tc, (int)H, 0, 0};
      BwdParams ep{labels + t0, row_max + t0, sum_exp + t0, grad_logprobs + t0, (int)Tc,
                   (int)V, logit_scale, c2, inv_temperature, bias, dl, ldv, dlT, ldt_c};
      // the token-contiguous copy dlT is written by the generic kernel's epilogue only
      Regions r = plan_regions(V, Tc, H, 512, 0, !need_dlT);
      fold_ragged_a(r, V);
      if (need_dlT)
        rc = affine ? launch_gemm<Bwd16Affine, BwdAffineT, BwdParams, KERNEL16_NT>(g, r, ep, ep, stream)
                    : launch_gemm<Bwd16Plain, BwdPlainT, BwdParams, KERNEL16_NT>(g, r, ep, ep, stream);
      else
        rc = affine ? launch_gemm<Bwd16Affine, BwdAffine, BwdParams, KERNEL16_NT>(g, r, ep, ep, stream)
                    : launch_gemm<Bwd16Plain, BwdPlain, BwdParams, KERNEL16_NT>(g, r, ep, ep, stream);
      if (rc != AREAL_OK) return rc;
    }
    // 2. dHidden[t, h] = sum_v dl[t, v] * W^T[h, v]
    if (dhidden != nullptr) {
      if ((rc = launch_dhidden(w_in_place ? (const u16*)weight : wT, V, dl, ldv, H, Tc,
                               (u16*)dhidden + t0 * H, dh_part, nullptr, nullptr, stream)) != AREAL_OK)
        return rc;
    }
    // dBias[v] += sum_t dl[t, v]
    if (dbias != nullptr) {
      hipLaunchKernelGGL(colsum_bf16_kernel, dim3((unsigned)ceil_div_i64(V, 64)), dim3(256), 0, stream,
                         dl, ldv, Tc, (int)V, (accumulate == 1 || t0 > 0) ? 1 : 0, nullptr, dbias, nullptr);
      AREAL_CHECK_LAUNCH();
    }
    // 3. dWeight[v, h] += sum_t dl[t, v] * hidden[t, h]
    if (tn) {
      GemmArgs g{hid_c, H, (int)H, dl, ldv, (int)V, (int)Tc, (int)H, (int)ldv};
      const StoreParams ep{dweight_f32, H, (int)H, (int)V};
      rc = dw_bf16 ? launch_dweight_bf16(g, H, V, ldv, dweight, dw_part, stream)
                   : launch_store<KERNEL16_TN>(g, ep, (accumulate == 1 || t0 > 0) ? 2 : 1, stream);
      if (rc != AREAL_OK) return rc;
    } else if (dweight_f32 != nullptr) {
      hipLaunchKernelGGL(transpose_pad_bf16_kernel,
                         dim3((unsigned)ceil_div_i64(H, 64), (unsigned)ceil_div_i64(ldt_c, 64)),
                         dim3(256), 0, stream, hid_c, H, (int)Tc, (int)H, hT, ldt_c);
      AREAL_CHECK_LAUNCH();
      GemmArgs g{hT, ldt_c, (int)H, dlT, ldt_c, (int)V, (int)ldt_c, 0, 0};
      const StoreParams ep{dweight_f32, H, (int)H, (int)V};
      rc = launch_store<KERNEL16_NT>(g, ep, dw_bf16 ? 0 : (accumulate == 1 || t0 > 0) ? 2 : 1, stream);
      if (rc != AREAL_OK) return rc;
    }
  }
  return AREAL_OK;
}

// Workspace of the backward from saved exponentials: row factors [T] fp32, scaled hidden states
// [round_up(T, 128), H] bf16, W^T [H, round_up(V, 64)] bf16 (only when V is not a multiple of 64)
// and the split-K partials of dHidden and of dWeight's last partial round.
size_t areal_lmhead_bwd_saved_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (T <= 0 || H <= 0 || V <= 0) return 0;
  const size_t wt = dh_weight_in_place(V) ? 0 : (size_t)(H * round_up_i64(V, BK)) * 2;
  return (size_t)T * 4 + (size_t)(round_up_i64(T, 2 * BK) * H) * 2 + wt +
         dh_partial_bytes(H, T, round_up_i64(V, BK)) + dw_tail_bytes(H, V, round_up_i64(T, 2 * BK)) + 5 * 256;
}

// Backward from the exponentials areal_lmhead_fwd saved (probs, probs_ref, with *probs_status
// read back as 0): no logits are recomputed and no pass rewrites the [T, V] buffer. Per row,
// dlogits = f[t] * e' with a row factor f; dHidden scales its output rows by f and dWeight
// contracts e' with f[t] * hidden[t]. Only the label's entry of each row of probs is rewritten
// (and rows [T, round_up(T, 128)) are cleared: dWeight contracts over that padded token range, so
// that any T takes the hand-scheduled main loop), so probs can be used once. logprobs (nullable)
// are the label log-probabilities of the forward; with them the label's entry is evaluated in
// fp32. dweight [V,H]: dweight_mode 0 = fp32 store, 1 = fp32 accumulate, 2 = bf16 store (the
// whole batch is one contraction, so no fp32 staging is needed). probs_status (nullable): the
// device int areal_lmhead_fwd set; when it reads non-zero at execution time every kernel of this
// call returns at once and no output is touched, so the call can be queued before the host has
// seen the status (which it then checks, and runs areal_lmhead_bwd instead if it was set).
int areal_lmhead_bwd_saved(const void* hidden, const void* weight, const int64_t* labels,
                           const float* row_max, const float* sum_exp, const float* logprobs,
                           const float* grad_logprobs, int64_t T, int64_t H, int64_t V,
                           float inv_temperature, float logit_scale, void* probs, size_t probs_bytes,
                           const float* probs_ref, const int* probs_status, void* dhidden, void* dweight,
                           int dweight_mode, float* dbias, void* workspace,
                           size_t workspace_bytes, hipStream_t stream) {
  if (T < 0 || H <= 0 || V <= 0) return AREAL_ERR_BAD_ARG;
  if (probs != nullptr && probs_bytes < areal_lmhead_probs_bytes(T, V)) return AREAL_ERR_WORKSPACE;
  if (labels == nullptr || row_max == nullptr || sum_exp == nullptr || grad_logprobs == nullptr ||
      probs == nullptr || probs_ref == nullptr)
    return AREAL_ERR_BAD_ARG;
  if (dhidden == nullptr && dweight == nullptr) return AREAL_ERR_BAD_ARG;
  if (dweight_mode < 0 || dweight_mode > 2) return AREAL_ERR_BAD_ARG;
  if (T == 0) return AREAL_OK;
  if (T > (1 << 30) || V > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  int rc;
  if ((rc = check_operand(hidden, H)) != AREAL_OK) return rc;
  if ((rc = check_operand(weight, H)) != AREAL_OK) return rc;
  if (!aligned16(probs)) return AREAL_ERR_ALIGNMENT;
  if (dhidden != nullptr && !aligned16(dhidden)) return AREAL_ERR_ALIGNMENT;
  if (dweight != nullptr && !aligned16(dweight)) return AREAL_ERR_ALIGNMENT;
  if (workspace == nullptr || workspace_bytes < areal_lmhead_bwd_saved_workspace_bytes(T, H, V))
    return AREAL_ERR_WORKSPACE;
  const int64_t ldv = round_up_i64(V, BK), Tpad = round_up_i64(T, 2 * BK);
  auto align256 = [](void* q) { return (void*)(((uintptr_t)q + 255) & ~(uintptr_t)255); };
  float* rowfac = (float*)align256(workspace);
  u16* hs = (u16*)align256(rowfac + T);
  const bool w_in_place = dh_weight_in_place(V);
  u16* wT = (u16*)align256(hs + Tpad * H);
  float* dh_part = dh_partial_bytes(H, T, ldv) ? (float*)align256(wT + (w_in_place ? 0 : H * ldv)) : nullptr;
  float* dw_part = (float*)align256((char*)align256(wT + (w_in_place ? 0 : H * ldv)) + dh_partial_bytes(H, T, ldv));
  u16* e = (u16*)probs;
  hipLaunchKernelGGL(saved_prep_kernel, dim3((unsigned)Tpad), dim3(256), 0, stream, e, ldv, probs_ref,
                     labels, row_max, sum_exp, grad_logprobs, logprobs, (const u16*)hidden, (int)T,
                     (int)H, (int)V, inv_temperature * LOG2E, inv_temperature * logit_scale, rowfac,
                     dweight != nullptr ? hs : nullptr, probs_status);
  AREAL_CHECK_LAUNCH();
  if (dhidden != nullptr) {
    if (!w_in_place) {
      hipLaunchKernelGGL(transpose_pad_bf16_kernel,
                         dim3((unsigned)ceil_div_i64(H, 64), (unsigned)ceil_div_i64(ldv, 64)),
                         dim3(256), 0, stream, (const u16*)weight, H, (int)V, (int)H, wT, ldv);
      AREAL_CHECK_LAUNCH();
    }
    if ((rc = launch_dhidden(w_in_place ? (const u16*)weight : wT, V, e, ldv, H, T, dhidden, dh_part,
                             rowfac, probs_status, stream)) != AREAL_OK)
      return rc;
  }
  if (dbias != nullptr) {
    hipLaunchKernelGGL(colsum_bf16_kernel, dim3((unsigned)ceil_div_i64(V, 64)), dim3(256), 0, stream,
                       e, ldv, T, (int)V, dweight_mode == 1 ? 1 : 0, (const float*)rowfac, dbias, probs_status);
    AREAL_CHECK_LAUNCH();
  }
  if (dweight != nullptr) {
    // dWeight[v, h] += sum_t e'[t, v] * hs[t, h], k-major over the Tpad rows of both (rows past
    // T are cleared)
    GemmArgs g{hs, H, (int)H, e, ldv, (int)V, (int)Tpad, (int)H, (int)ldv};
    g.skip_if_set = probs_status;
    if (dweight_mode == 2) return launch_dweight_bf16(g, H, V, ldv, dweight, dw_part, stream);
    const StoreParams ep{dweight, H, (int)H, (int)V, nullptr};
    rc = launch_store<KERNEL16_TN>(g, ep, dweight_mode == 1 ? 2 : 1, stream);
    if (rc != AREAL_OK) return rc;
  }
  return AREAL_OK;
}

int areal_cast_f32_to_bf16(const float* src, void* dst, int64_t n, hipStream_t stream) {
  if (n < 0 || (n > 0 && (src == nullptr || dst == nullptr))) return AREAL_ERR_BAD_ARG;
  if (n == 0) return AREAL_OK;
  if (!aligned16(src) || ((uintptr_t)dst & 7)) return AREAL_ERR_ALIGNMENT;
  int64_t blocks = ceil_div_i64(n, 256 * 4);
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(cast_f32_to_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src,
                     (u16*)dst, n);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // extern "C"
