// Data movement and logging reductions either side of the loss: packing padded [B, S] batches
// into the packed layout by cu_seqlens and back, re-aligning a packed batch, and the masked
// sum / count / min / max of many per-token statistics in one launch.
//
// Follows areal/utils/data.py: pack_tensor_dict (:496-545), pad_packed_tensor_dict (:822-982),
// unpack_sequence + pad_and_stack_tensors_along_first_dim as used by reorder_and_pad_outputs
// (areal/engine/core/train_engine.py:110-144); and areal/utils/stats_tracker.py: _avg_of,
// _min_of, _max_of (:455-560), which reduce every logged tensor under its denominator mask.
#include "common.hpp"

namespace {

constexpr int PK_THREADS = 256;

// 16 bytes at any address. The compiler picks the access the target allows for the alignment
// (gfx950 runs with unaligned access enabled, where this is still one 16-byte instruction).
struct __attribute__((packed, aligned(1))) Bytes16 { uint32_t w[4]; };

// number of nonzero bytes among the four of x
DEVI int nonzero_bytes(uint32_t x) {
  x = (x | (x >> 4)) & 0x0f0f0f0fu;
  x = (x | (x >> 2)) & 0x03030303u;
  x = (x | (x >> 1)) & 0x01010101u;
  return __popc(x);
}

// lens[b] = number of nonzero entries of mask row b (one block per row), 16 mask bytes per load.
__global__ __launch_bounds__(PK_THREADS) void rowlens_kernel(const uint8_t* mask, int64_t S,
                                                             int32_t* lens) {
  __shared__ int sm[4];
  const uint8_t* row = mask + (int64_t)blockIdx.x * S;
  int len = 0;
  const int64_t n16 = S >> 4;
  for (int64_t i = threadIdx.x; i < n16; i += blockDim.x) {
    const Bytes16 v = *(const Bytes16*)(row + 16 * i);
#pragma unroll
    for (int k = 0; k < 4; ++k) len += nonzero_bytes(v.w[k]);
  }
  for (int64_t s = 16 * n16 + threadIdx.x; s < S; s += blockDim.x) len += row[s] != 0;
  len = wave_sum(len);
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = len;
  __syncthreads();
  if (threadIdx.x == 0) lens[blockIdx.x] = sm[0] + sm[1] + sm[2] + sm[3];
}

// Inclusive prefix sum over the wave's 64 lanes: inside each row of 16 through DPP, then the
// totals of the rows to the left (lanes 15, 31, 47) are added.
DEVI int wave_inclusive_sum(int v) {
  v += dpp_move<DPP_ROW_SHR + 1>(0, v);
  v += dpp_move<DPP_ROW_SHR + 2>(0, v);
  v += dpp_move<DPP_ROW_SHR + 4>(0, v);
  v += dpp_move<DPP_ROW_SHR + 8>(0, v);
  const int t0 = lane_value(v, 15), t1 = lane_value(v, 31), t2 = lane_value(v, 47);
  const int row = (threadIdx.x & 63) >> 4;
  return v + (row == 0 ? 0 : row == 1 ? t0 : row == 2 ? t0 + t1 : t0 + t1 + t2);
}

// cu = exclusive prefix sums of lens, *max_len = max(lens) (one block; 4 entries per thread and
// round, two barriers per round).
constexpr int SCAN_ITEMS = 4;
__global__ __launch_bounds__(PK_THREADS) void cu_scan_kernel(const int32_t* lens, int64_t B,
                                                             int32_t* cu, int32_t* max_len) {
  __shared__ int sm_sum[PK_THREADS / 64], sm_max[PK_THREADS / 64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int carry = 0, mx = 0;
  if (threadIdx.x == 0) cu[0] = 0;
  for (int64_t b0 = 0; b0 < B; b0 += PK_THREADS * SCAN_ITEMS) {
    const int64_t b = b0 + (int64_t)threadIdx.x * SCAN_ITEMS;
    int len[SCAN_ITEMS];
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) len[i] = b + i < B ? lens[b + i] : 0;
    int tot = 0;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) { tot += len[i]; mx = len[i] > mx ? len[i] : mx; }
    const int incl = wave_inclusive_sum(tot);
    __syncthreads();  // the previous round's readers are done
    if (lane == 63) sm_sum[w] = incl;
    __syncthreads();
    int base = carry + incl - tot;
    for (int i = 0; i < w; ++i) base += sm_sum[i];
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
      base += len[i];
      if (b + i < B) cu[b + i + 1] = base;
    }
    for (int i = 0; i < PK_THREADS / 64; ++i) carry += sm_sum[i];
  }
  mx = wave_reduce(mx, [](int a, int b) { return a > b ? a : b; });
  __syncthreads();
  if (lane == 0) sm_max[w] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < PK_THREADS / 64; ++i) mx = sm_max[i] > mx ? sm_max[i] : mx;
    *max_len = mx;
  }
}

// Copy of n contiguous bytes by the whole block: 16 bytes per thread and access, whatever the
// two addresses' alignment, four loads in flight per thread before the first store; then the
// last n % 16 bytes one by one.
DEVI void block_copy_bytes(char* dst, const char* src, int64_t n) {
  const int64_t n16 = n >> 4;
  for (int64_t i0 = threadIdx.x; i0 < n16; i0 += 4 * (int64_t)blockDim.x) {
    Bytes16 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = i0 + u * (int64_t)blockDim.x;
      if (i < n16) v[u] = *(const Bytes16*)(src + 16 * i);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = i0 + u * (int64_t)blockDim.x;
      if (i < n16) *(Bytes16*)(dst + 16 * i) = v[u];
    }
  }
  for (int64_t i = 16 * n16 + threadIdx.x; i < n; i += blockDim.x) dst[i] = src[i];
}

// Several tensors packed in one launch. Block (c, k) writes packed tokens [c * chunk, (c + 1) *
// chunk) of tensor k: it finds the sequence of its first token (every wave searches cu_seqlens
// with 64 probes per round) and then walks the sequences its chunk touches, each one contiguous
// run of a padded row to one contiguous run of the packed array. No block is empty. The chunk is
// 16 KiB of the widest tensor (at most 2048 tokens), so a thread has four loads of 16 bytes in
// flight at once.
constexpr int PK_MAX_TENSORS = 8;
constexpr int PK_CHUNK_BYTES = 16384, PK_CHUNK_MAX = 2048;
struct PackArgs {
  const char* src[PK_MAX_TENSORS];
  char* dst[PK_MAX_TENSORS];
  int64_t eb[PK_MAX_TENSORS];  // bytes of one token's trailing dimensions
  const int32_t* cu;
  int n_seqs;
  int64_t S, total;
  int chunk;  // tokens per block
};
__global__ __launch_bounds__(PK_THREADS) void pack_rows_kernel(PackArgs a) {
  const int k = blockIdx.y;
  int64_t t = (int64_t)blockIdx.x * a.chunk;
  const int64_t t1 = t + a.chunk < a.total ? t + a.chunk : a.total;
  // (selects, not an index into the argument arrays: those would be copied to scratch memory)
  const char* src = a.src[0]; char* dst = a.dst[0]; int64_t eb = a.eb[0];
#pragma unroll
  for (int i = 1; i < PK_MAX_TENSORS; ++i)
    if (k == i) { src = a.src[i]; dst = a.dst[i]; eb = a.eb[i]; }
  // sequence of token t: the number of sequence ends at or before it (same value in every wave)
  int b = wave_count_le(a.cu + 1, a.n_seqs, t, threadIdx.x & 63);
  while (t < t1 && b < a.n_seqs) {
    const int64_t start = a.cu[b], end = a.cu[b + 1];
    const int64_t stop = end < t1 ? end : t1;
    if (stop > t) block_copy_bytes(dst + t * eb, src + ((int64_t)b * a.S + (t - start)) * eb, (stop - t) * eb);
    t = stop > t ? stop : t;
    ++b;
  }
}

struct Fill { char bytes[16]; int n; };

// n bytes at dst (the start of an element) filled with the pattern by the whole block: 16-byte
// stores of the repeated pattern when its length divides 16, byte by byte otherwise and at the end.
DEVI void block_fill_bytes(char* dst, int64_t n, const Fill& f) {
  int64_t done = 0;
  if ((16 % f.n) == 0) {
    Bytes16 pat;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t x = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) x |= (uint32_t)(uint8_t)f.bytes[(4 * w + k) % f.n] << (8 * k);
      pat.w[w] = x;
    }
    const int64_t n16 = n >> 4;
    for (int64_t i = threadIdx.x; i < n16; i += blockDim.x) *(Bytes16*)(dst + 16 * i) = pat;
    done = 16 * n16;
  }
  for (int64_t i = done + threadIdx.x; i < n; i += blockDim.x) dst[i] = f.bytes[i % f.n];
}

// Tokens per block of the row-wise kernels below: 16 KiB of an element, at most 2048 tokens.
static int64_t pk_chunk_tokens(int64_t eb) {
  const int64_t c = PK_CHUNK_BYTES / eb;
  return c < 1 ? 1 : (c > PK_CHUNK_MAX ? PK_CHUNK_MAX : c);
}

// padded[row][j] = j < len_b ? packed[cu[b] + j] : fill, b = row_seq[row] (or row). Block
// (row, c) writes tokens [c * chunk, (c + 1) * chunk) of its row: one contiguous copy, one fill.
__global__ __launch_bounds__(PK_THREADS) void unpack_kernel(const char* packed, char* padded,
                                                            const int32_t* cu, const int32_t* row_seq,
                                                            int64_t S, int64_t eb, Fill fill, int chunks,
                                                            int chunk) {
  const int64_t row = blockIdx.x / chunks;
  const int64_t j0 = (int64_t)(blockIdx.x % chunks) * chunk;
  const int64_t nj = S - j0 < chunk ? S - j0 : chunk;
  const int64_t b = row_seq ? row_seq[row] : row;  // packed sequence shown in this row
  const int64_t start = cu[b], len = (int64_t)cu[b + 1] - start;
  int64_t ncopy = len - j0;
  ncopy = ncopy < 0 ? 0 : (ncopy > nj ? nj : ncopy);
  char* d = padded + (row * S + j0) * eb;
  if (ncopy > 0) block_copy_bytes(d, packed + (start + j0) * eb, ncopy * eb);
  if (ncopy < nj) block_fill_bytes(d + ncopy * eb, (nj - ncopy) * eb, fill);
}

// dst[cu_new[s] + j] = j < old length of s ? src[cu_old[s] + j] : fill; sequences of cu_new
// beyond n_old (a trailing pad segment) are all fill. arange != 0: dst is int64 position ids,
// and the fill is j (position inside the new sequence, src == NULL) or j - old length instead.
// Block c writes tokens [c * chunk, (c + 1) * chunk) of dst, sequence by sequence as pack_rows_kernel.
__global__ __launch_bounds__(PK_THREADS) void realign_kernel(const char* src, char* dst,
                                                             const int32_t* cu_old, int n_old,
                                                             const int32_t* cu_new, int n_new,
                                                             int64_t eb, Fill fill, int arange,
                                                             int64_t total_new, int chunk) {
  int64_t t = (int64_t)blockIdx.x * chunk;
  const int64_t t1 = t + chunk < total_new ? t + chunk : total_new;
  int s = wave_count_le(cu_new + 1, n_new, t, threadIdx.x & 63);
  while (t < t1 && s < n_new) {
    const int64_t start = cu_new[s], end = cu_new[s + 1];
    const int64_t stop = end < t1 ? end : t1;
    if (stop > t) {
      const int64_t j0 = t - start, j1 = stop - start;  // positions inside the new sequence
      const int64_t len = (s < n_old && src != nullptr) ? (int64_t)cu_old[s + 1] - cu_old[s] : 0;
      const int64_t jc = j1 < len ? j1 : len;            // copied positions are [j0, jc)
      if (jc > j0) block_copy_bytes(dst + t * eb, src + ((int64_t)cu_old[s] + j0) * eb, (jc - j0) * eb);
      const int64_t jf = j0 > len ? j0 : len;            // filled positions are [jf, j1)
      if (jf < j1) {
        char* d = dst + (start + jf) * eb;
        if (arange) {
          const int64_t shift = src == nullptr ? 0 : (s < n_old ? (int64_t)cu_old[s + 1] - cu_old[s] : 0);
          const int64_t per = eb >> 3;  // int64 channels per token
          for (int64_t i = threadIdx.x; i < (j1 - jf) * per; i += blockDim.x)
            ((int64_t*)d)[i] = jf + i / per - shift;
        } else {
          block_fill_bytes(d, (j1 - jf) * eb, fill);
        }
      }
      t = stop;
    }
    ++s;
  }
}

// ---------------------------------------------------------------------------------------
// Masked statistics of K tensors in one launch.
// ---------------------------------------------------------------------------------------
constexpr int STATS_MAX_K = 32;
constexpr int STATS_BLOCKS = 256;
struct StatsArgs {
  const float* v[STATS_MAX_K];
  const uint8_t* m[STATS_MAX_K];  // denominator mask of tensor k (null: all ones)
  int K;
  int64_t n;
};
struct StatPart { double sum, cnt; float mn, mx; };

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
DEVI float block_minmax(float v, float* smem, bool is_min) {
  v = is_min ? wave_min(v) : wave_max(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) smem[w] = v;
  __syncthreads();
  float r = smem[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) r = is_min ? fminf(r, smem[i]) : fmaxf(r, smem[i]);
  return r;
}

// grid (STATS_BLOCKS, K): partial over a slice of tensor blockIdx.y
__global__ __launch_bounds__(PK_THREADS) void stats_partial_kernel(StatsArgs a, StatPart* parts) {
  __shared__ double sm_d[4];
  __shared__ float sm_f[4];
  const int k = blockIdx.y;
  const float* v = a.v[k];
  const uint8_t* m = a.m[k];
  double sum = 0.0, cnt = 0.0;
  float mn = pos_inf(), mx = neg_inf();
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n;
       i += (int64_t)gridDim.x * blockDim.x) {
    if (m != nullptr && m[i] == 0) continue;
    const float x = v[i];
    sum += (double)x; cnt += 1.0;
    mn = fminf(mn, x); mx = fmaxf(mx, x);
  }
  sum = block_sum_d(sum, sm_d);
  cnt = block_sum_d(cnt, sm_d);
  mn = block_minmax(mn, sm_f, true);
  mx = block_minmax(mx, sm_f, false);
  if (threadIdx.x == 0) parts[(int64_t)k * gridDim.x + blockIdx.x] = StatPart{sum, cnt, mn, mx};
}
// out[k] = {sum, count, min, max} (min = +inf, max = -inf when the mask is empty)
__global__ __launch_bounds__(PK_THREADS) void stats_final_kernel(const StatPart* parts, int nparts,
                                                                 double* out) {
  __shared__ double sm_d[4];
  __shared__ float sm_f[4];
  const int k = blockIdx.x;
  double sum = 0.0, cnt = 0.0;
  float mn = pos_inf(), mx = neg_inf();
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) {
    const StatPart p = parts[(int64_t)k * nparts + i];
    sum += p.sum; cnt += p.cnt; mn = fminf(mn, p.mn); mx = fmaxf(mx, p.mx);
  }
  sum = block_sum_d(sum, sm_d);
  cnt = block_sum_d(cnt, sm_d);
  mn = block_minmax(mn, sm_f, true);
  mx = block_minmax(mx, sm_f, false);
  if (threadIdx.x == 0) {
    out[4 * k] = sum; out[4 * k + 1] = cnt; out[4 * k + 2] = (double)mn; out[4 * k + 3] = (double)mx;
  }
}

bool make_fill(const void* fill, int fill_bytes, Fill& f) {
  if (fill_bytes < 0 || fill_bytes > 16) return false;
  f.n = fill_bytes > 0 ? fill_bytes : 1;
  for (int i = 0; i < 16; ++i) f.bytes[i] = 0;
  if (fill_bytes > 0 && fill != nullptr)
    for (int i = 0; i < fill_bytes; ++i) f.bytes[i] = ((const char*)fill)[i];
  return true;
}

}  // namespace

extern "C" {

// attention_mask [B, S] bytes (nonzero = token) -> lens [B], cu_seqlens [B+1], *max_len, all
// int32 on the device (data.py:513-517).
int areal_seqlens_from_mask(const uint8_t* attention_mask, int64_t B, int64_t S, int32_t* lens,
                            int32_t* cu_seqlens, int32_t* max_len, hipStream_t stream) {
  if (B < 0 || S < 0) return AREAL_ERR_BAD_ARG;
  if (!cu_seqlens || !max_len || (B > 0 && (!attention_mask || !lens))) return AREAL_ERR_BAD_ARG;
  if (B > (1 << 30) || B * S >= ((int64_t)1 << 31)) return AREAL_ERR_UNSUPPORTED;
  if (B > 0) {
    hipLaunchKernelGGL(rowlens_kernel, dim3((unsigned)B), dim3(PK_THREADS), 0, stream,
                       attention_mask, S, lens);
    AREAL_CHECK_LAUNCH();
  }
  hipLaunchKernelGGL(cu_scan_kernel, dim3(1), dim3(PK_THREADS), 0, stream, lens, B, cu_seqlens,
                     max_len);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// packed [total, E] <- the first len_b tokens of every row of padded [B, S, E]; elem_bytes = bytes
// of one token's trailing dimensions (data.py:535-541). Up to 8 tensors of one batch (host
// arrays of device pointers and of element sizes) in one launch.
int areal_pack_padded_multi(const void* const* padded, void* const* packed, const int64_t* elem_bytes,
                            int n_tensors, const int32_t* cu_seqlens, int64_t B, int64_t S,
                            int64_t total, hipStream_t stream) {
  if (B < 0 || S < 0 || total < 0 || n_tensors < 0 || n_tensors > PK_MAX_TENSORS) return AREAL_ERR_BAD_ARG;
  if (total == 0 || n_tensors == 0) return AREAL_OK;
  if (!padded || !packed || !elem_bytes || !cu_seqlens || B == 0) return AREAL_ERR_BAD_ARG;
  PackArgs a;
  for (int k = 0; k < PK_MAX_TENSORS; ++k) { a.src[k] = nullptr; a.dst[k] = nullptr; a.eb[k] = 0; }
  for (int k = 0; k < n_tensors; ++k) {
    if (!padded[k] || !packed[k] || elem_bytes[k] <= 0) return AREAL_ERR_BAD_ARG;
    a.src[k] = (const char*)padded[k]; a.dst[k] = (char*)packed[k]; a.eb[k] = elem_bytes[k];
  }
  int64_t max_eb = 1;
  for (int k = 0; k < n_tensors; ++k) max_eb = elem_bytes[k] > max_eb ? elem_bytes[k] : max_eb;
  const int64_t chunk = pk_chunk_tokens(max_eb);
  const int64_t chunks = ceil_div_i64(total, chunk);
  if (chunks >= ((int64_t)1 << 31) || B > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  a.cu = cu_seqlens; a.n_seqs = (int)B; a.S = S; a.total = total; a.chunk = (int)chunk;
  const dim3 grid((unsigned)chunks, (unsigned)n_tensors);
  hipLaunchKernelGGL(pack_rows_kernel, grid, dim3(PK_THREADS), 0, stream, a);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

int areal_pack_padded(const void* padded, void* packed, const int32_t* cu_seqlens, int64_t B,
                      int64_t S, int64_t elem_bytes, int64_t total, hipStream_t stream) {
  if (elem_bytes <= 0) return AREAL_ERR_BAD_ARG;
  if (total > 0 && (!padded || !packed)) return AREAL_ERR_BAD_ARG;
  return areal_pack_padded_multi(&padded, &packed, &elem_bytes, 1, cu_seqlens, B, S, total, stream);
}

// padded [B, S, E] <- packed sequences, the rest filled with the fill pattern (fill_bytes <= 16
// bytes repeated over the element; NULL = zero bytes): unpack_sequence + reorder_list +
// pad_and_stack. row_seq [B] (nullable): row r shows packed sequence row_seq[r].
int areal_unpack_to_padded(const void* packed, void* padded, const int32_t* cu_seqlens,
                           const int32_t* row_seq, int64_t B, int64_t S, int64_t elem_bytes,
                           const void* fill, int fill_bytes, hipStream_t stream) {
  if (B < 0 || S < 0 || elem_bytes <= 0) return AREAL_ERR_BAD_ARG;
  if (B == 0 || S == 0) return AREAL_OK;
  if (!padded || !cu_seqlens) return AREAL_ERR_BAD_ARG;
  Fill f;
  if (!make_fill(fill, fill_bytes, f)) return AREAL_ERR_BAD_ARG;
  const int64_t chunk = pk_chunk_tokens(elem_bytes), chunks = ceil_div_i64(S, chunk);
  if (chunks * B >= ((int64_t)1 << 31)) return AREAL_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(unpack_kernel, dim3((unsigned)(chunks * B)), dim3(PK_THREADS), 0, stream,
                     (const char*)packed, (char*)padded, cu_seqlens, row_seq, S, elem_bytes, f, (int)chunks,
                     (int)chunk);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

// Re-layout of a packed batch (data.py:848-911, :927-969): sequence s moves from cu_old to
// cu_new (new length >= old length, the tail filled); cu_new may hold extra trailing
// sequences (the batch pad), filled entirely. position_ids != 0: elem_bytes is a multiple of 8
// (int64 channels); src == NULL writes 0..len-1 per new sequence, otherwise the pads continue
// with 0, 1, 2, ... after the copied part.
int areal_realign_packed(const void* src, void* dst, const int32_t* cu_old, int64_t n_old,
                         const int32_t* cu_new, int64_t n_new, int64_t elem_bytes,
                         const void* fill, int fill_bytes, int position_ids, int64_t total_new,
                         hipStream_t stream) {
  if (n_old < 0 || n_new < 0 || elem_bytes <= 0 || total_new < 0) return AREAL_ERR_BAD_ARG;
  if (total_new == 0) return AREAL_OK;
  if (!dst || !cu_new || n_new == 0 || (n_old > 0 && !cu_old)) return AREAL_ERR_BAD_ARG;
  if (position_ids && (elem_bytes % 8 != 0 || ((uintptr_t)dst & 7))) return AREAL_ERR_ALIGNMENT;
  if (!position_ids && src == nullptr && n_old > 0) return AREAL_ERR_BAD_ARG;
  Fill f;
  if (!make_fill(fill, fill_bytes, f)) return AREAL_ERR_BAD_ARG;
  const int64_t chunk = pk_chunk_tokens(elem_bytes), chunks = ceil_div_i64(total_new, chunk);
  if (chunks >= ((int64_t)1 << 31) || n_new > (1 << 30)) return AREAL_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(realign_kernel, dim3((unsigned)chunks), dim3(PK_THREADS), 0, stream,
                     (const char*)src, (char*)dst, cu_old, (int)n_old, cu_new, (int)n_new,
                     elem_bytes, f, position_ids, total_new, (int)chunk);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

size_t areal_masked_stats_workspace_bytes(int K) {
  if (K <= 0) return 0;
  return (size_t)K * STATS_BLOCKS * sizeof(StatPart) + 256;
}

// out [K][4] double = {sum, count, min, max} of values[k][i] over mask[k][i] != 0 (mask[k] NULL:
// every element). values / masks are HOST arrays of K device pointers, K <= 32.
int areal_masked_stats(const float* const* values, const uint8_t* const* masks, int K, int64_t n,
                       double* out, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (K < 0 || K > STATS_MAX_K || n < 0) return AREAL_ERR_BAD_ARG;
  if (K == 0) return AREAL_OK;
  if (!values || !masks || !out) return AREAL_ERR_BAD_ARG;
  if (workspace == nullptr || workspace_bytes < areal_masked_stats_workspace_bytes(K))
    return AREAL_ERR_WORKSPACE;
  StatsArgs a;
  a.K = K; a.n = n;
  for (int k = 0; k < STATS_MAX_K; ++k) { a.v[k] = nullptr; a.m[k] = nullptr; }
  for (int k = 0; k < K; ++k) {
    if (values[k] == nullptr && n > 0) return AREAL_ERR_BAD_ARG;
    a.v[k] = values[k]; a.m[k] = masks[k];
  }
  StatPart* parts = (StatPart*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  int blocks = (int)ceil_div_i64(n > 0 ? n : 1, PK_THREADS * 8);
  if (blocks > STATS_BLOCKS) blocks = STATS_BLOCKS;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(stats_partial_kernel, dim3(blocks, K), dim3(PK_THREADS), 0, stream, a, parts);
  AREAL_CHECK_LAUNCH();
  hipLaunchKernelGGL(stats_final_kernel, dim3(K), dim3(PK_THREADS), 0, stream, parts, blocks, out);
  AREAL_CHECK_LAUNCH();
  return AREAL_OK;
}

}  // extern "C"
