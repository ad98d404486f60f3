// get_valid_counts and non_max_suppression for gfx950.
//
// Both are order-sensitive on the CPU; here the order is reproduced with
// wavefront ballots / prefix sums (stream compaction) and a rank sort whose key
// (score descending, original index ascending) is unique, so the result does
// not depend on scheduling.  Nothing is copied back to the host: valid_count is
// read on the device and every launch shape depends only on (batches, n, k).
#include <mutex>

#include "hip_common.h"

namespace cvmhip {

constexpr int GVC_CHUNK = 256;

// number of rows in this 256-row chunk whose score passes the threshold
__global__ void __launch_bounds__(GVC_CHUNK)
k_gvc_count(const int32_t* __restrict__ x, int32_t* __restrict__ counts, int n, int k, int32_t thr, int nchunks) {
  __shared__ int wsum[GVC_CHUNK / 64];
  const int b = blockIdx.y, chunk = blockIdx.x;
  const int row = chunk * GVC_CHUNK + threadIdx.x;
  const bool keep = row < n && x[((int64_t)b * n + row) * k + 1] > thr;
  const unsigned long long m = __ballot(keep);
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = __popcll(m);
  __syncthreads();
  if (threadIdx.x == 0) {
    int t = 0;
    for (int i = 0; i < GVC_CHUNK / 64; ++i) t += wsum[i];
    counts[b * nchunks + chunk] = t;
  }
}

// Each chunk derives its output offset from the counts of the chunks before it,
// then places its surviving rows in their original order; rows at or past the
// batch total are filled with -1.
__global__ void __launch_bounds__(GVC_CHUNK)
k_gvc_scatter(const int32_t* __restrict__ x, const int32_t* __restrict__ counts, int32_t* __restrict__ valid_count,
              int32_t* __restrict__ y, int n, int k, int32_t thr, int nchunks) {
  __shared__ int wsum[GVC_CHUNK / 64];
  __shared__ int s_bef[GVC_CHUNK / 64], s_tot[GVC_CHUNK / 64];
  __shared__ int s_before, s_total;
  const int b = blockIdx.y, chunk = blockIdx.x;
  {
    // the counts are summed by all threads (one thread walking a hundred of them is a chain of a hundred loads)
    int before = 0, total = 0;
    for (int c = threadIdx.x; c < nchunks; c += GVC_CHUNK) {
      const int v = counts[b * nchunks + c];
      before += c < chunk ? v : 0;
      total += v;
    }
    for (int d = 32; d >= 1; d >>= 1) {
      before += __shfl_xor(before, d, 64);
      total += __shfl_xor(total, d, 64);
    }
    if ((threadIdx.x & 63) == 0) { s_bef[threadIdx.x >> 6] = before; s_tot[threadIdx.x >> 6] = total; }
    __syncthreads();
    if (threadIdx.x == 0) {
      before = total = 0;
      for (int w = 0; w < GVC_CHUNK / 64; ++w) { before += s_bef[w]; total += s_tot[w]; }
      s_before = before;
      s_total = total;
      if (chunk == 0) valid_count[b] = total;
    }
  }
  const int row = chunk * GVC_CHUNK + threadIdx.x;
  const int32_t* src = x + ((int64_t)b * n + row) * k;
  const bool keep = row < n && src[1] > thr;
  const unsigned long long m = __ballot(keep);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int in_wave = __popcll(m & ((1ull << lane) - 1ull));
  if (lane == 0) wsum[wv] = __popcll(m);
  __syncthreads();
  int pos = s_before + in_wave;
  for (int i = 0; i < wv; ++i) pos += wsum[i];
  int32_t* yb = y + (int64_t)b * n * k;
  if (keep)
    for (int c = 0; c < k; ++c) yb[(int64_t)pos * k + c] = src[c];
  if (row < n && row >= s_total)
    for (int c = 0; c < k; ++c) yb[(int64_t)row * k + c] = -1;
}

// ------------------------------------------------------------------ NMS
// int64 IoU*100 of two corner-format boxes, same arithmetic as the reference
// (src/runtime/cpu/ops/nms.cc:4-40).
__device__ __forceinline__ int64_t iou100(const int32_t* r1, const int32_t* r2) {
  const int64_t a1 = (int64_t)wsub(r1[2], r1[0]) * wsub(r1[3], r1[1]);
  const int64_t a2 = (int64_t)wsub(r2[2], r2[0]) * wsub(r2[3], r2[1]);
  const int64_t sum_area = (int64_t)((uint64_t)a1 + (uint64_t)a2);
  if (sum_area <= 0) return 0;
  const int32_t xr = r1[2] < r2[2] ? r1[2] : r2[2], xl = r1[0] > r2[0] ? r1[0] : r2[0];
  const int32_t yb = r1[3] < r2[3] ? r1[3] : r2[3], yt = r1[1] > r2[1] ? r1[1] : r2[1];
  int32_t w = wsub(xr, xl), h = wsub(yb, yt);
  if (w < 0) w = 0;
  if (h < 0) h = 0;
  int64_t overlap = (int64_t)h * w;
  int64_t uni = sum_area - overlap;
  if (uni <= 0) return 0;
  if (INT64_MAX / 100 < overlap) uni /= 100; else overlap *= 100;
  return overlap / uni;
}

// iou100(r1, r2) >= thr without the 64-bit division when the products are small
// enough to compare exactly: floor(100*o/u) >= t  <=>  100*o >= t*u  for u > 0.
__device__ __forceinline__ bool iou_at_least(const int32_t* r1, const int32_t* r2, int thr) {
  const int64_t a1 = (int64_t)wsub(r1[2], r1[0]) * wsub(r1[3], r1[1]);
  const int64_t a2 = (int64_t)wsub(r2[2], r2[0]) * wsub(r2[3], r2[1]);
  const int64_t sum_area = (int64_t)((uint64_t)a1 + (uint64_t)a2);
  const int32_t xr = r1[2] < r2[2] ? r1[2] : r2[2], xl = r1[0] > r2[0] ? r1[0] : r2[0];
  const int32_t yb = r1[3] < r2[3] ? r1[3] : r2[3], yt = r1[1] > r2[1] ? r1[1] : r2[1];
  int32_t w = wsub(xr, xl), h = wsub(yb, yt);
  if (w < 0) w = 0;
  if (h < 0) h = 0;
  const int64_t overlap = (int64_t)h * w;
  const int64_t uni = sum_area - overlap;
  const int64_t small = (int64_t)1 << 40;
  if (sum_area > 0 && sum_area < small && overlap < small && uni > 0 && thr > 0 && thr < (1 << 20))
    return overlap * 100 >= (int64_t)thr * uni;
  return iou100(r1, r2) >= thr;
}

__device__ __forceinline__ int clamp_vc(int vc, int n) { return vc > n ? n : (vc < 0 ? 0 : vc); }

// The reference returns from the whole call at the first batch without valid
// rows (nms.cc:76-79): that batch is filled with -1 and later batches are left
// untouched.  0 = process normally, 1 = this is that batch, 2 = skipped.
__device__ __forceinline__ int batch_state(const int32_t* valid_count, int b, int n) {
  for (int i = 0; i < b; ++i)
    if (clamp_vc(valid_count[i], n) <= 0) return 2;
  return clamp_vc(valid_count[b], n) <= 0 ? 1 : 0;
}

// Rank of row i among the first vc rows under (score descending, index
// ascending) -- the order std::stable_sort gives (nms.cc:89-91).
// Also gathers the row into its sorted slot.
constexpr int RANK_JT = 1024;  // candidate rows one workgroup compares its 256 rows against

__global__ void __launch_bounds__(256) k_zero32(int32_t* __restrict__ p, int64_t count) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) p[i] = 0;
}

// rank[i] += number of rows j of this workgroup's chunk that sort before row i.
// The chunks of all workgroups add up with integer atomics, so the result does
// not depend on their order.
__global__ void __launch_bounds__(256)
k_nms_rank(const int32_t* __restrict__ x, const int32_t* __restrict__ valid_count, int32_t* __restrict__ rank,
           int n, int k, int score_index) {
  __shared__ __attribute__((aligned(16))) int32_t tile[RANK_JT];
  const int b = blockIdx.z;
  if (batch_state(valid_count, b, n) != 0) return;
  const int vc = clamp_vc(valid_count[b], n);
  const int base = blockIdx.y * RANK_JT;
  if (blockIdx.x * 256 >= vc || base >= vc) return;
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int32_t* xb = x + (int64_t)b * n * k;
  const int32_t si = i < vc ? xb[(int64_t)i * k + score_index] : 0;
#pragma unroll
  for (int t = 0; t < RANK_JT / 256; ++t) {
    const int j = base + t * 256 + threadIdx.x;
    tile[t * 256 + threadIdx.x] = j < vc ? xb[(int64_t)j * k + score_index] : INT32_MIN;
  }
  __syncthreads();
  const int lim = vc - base < RANK_JT ? vc - base : RANK_JT;
  int r = 0;
  for (int t = 0; t < lim; t += 4) {  // entries past vc hold INT32_MIN and an index above every row: they lose both tests
    const int4 s4 = *reinterpret_cast<const int4*>(&tile[t]);
    const int j = base + t;
    r += (s4.x > si) || (s4.x == si && j < i);
    r += (s4.y > si) || (s4.y == si && j + 1 < i);
    r += (s4.z > si) || (s4.z == si && j + 2 < i);
    r += (s4.w > si) || (s4.w == si && j + 3 < i);
  }
  if (i < vc && r) atomicAdd(&rank[(int64_t)b * n + i], r);
}

// ---- ranks by a stable sort, for many rows without a usable top_k.  Counting, for every row, the rows that sort
// before it costs n^2 comparisons (hours at the 2^24 rows the operator accepts); a least-significant-digit radix
// sort is the same stable order in four passes over the keys.  key = ~(score ^ 0x80000000) sorts ascending as the
// score sorts descending, and equal keys keep their order of arrival, i.e. ascending row index -- the order
// std::stable_sort gives (nms.cc:89-91).  A pass over one 8-bit digit is three launches:
//   k_radix_hist     every workgroup counts the digits of its RADIX_CHUNK consecutive elements
//   k_radix_scan     one workgroup per batch turns hist[digit][workgroup] into first positions (exclusive sum in
//                    digit-major order)
//   k_radix_scatter  every workgroup moves its elements, in their order, to first position + what came before
// Everything is integer counts: no float, no order-dependent atomics, so the result is the same on every run.
// Pass 0 reads the scores from the tensor (row i is element i); the last pass writes rank[row] = position.
constexpr int RADIX_CHUNK = 2048, RADIX_THREADS = 256, RADIX_ROUNDS = RADIX_CHUNK / RADIX_THREADS;
constexpr int RADIX_MIN_ROWS = 8192;   // below this the all-pairs count is faster

__device__ __forceinline__ uint32_t radix_key(int32_t score) { return ~((uint32_t)score ^ 0x80000000u); }

__global__ void __launch_bounds__(RADIX_THREADS)
k_radix_hist(const int32_t* __restrict__ x, const int32_t* __restrict__ valid_count, const uint32_t* __restrict__ keys_in,
             int32_t* __restrict__ hist, int n, int k, int score_index, int pass, int nblocks, int64_t key_stride) {
  __shared__ int s_hist[256];
  const int b = blockIdx.y, blk = blockIdx.x, tid = threadIdx.x;
  if (batch_state(valid_count, b, n) != 0) return;
  const int vc = clamp_vc(valid_count[b], n);
  s_hist[tid] = 0;
  __syncthreads();
  const int base = blk * RADIX_CHUNK;
  const int32_t* xb = x + (int64_t)b * n * k;
  const uint32_t* kin = keys_in + b * key_stride;
  for (int r = 0; r < RADIX_ROUNDS; ++r) {
    const int i = base + r * RADIX_THREADS + tid;
    if (i < vc) {
      const uint32_t key = pass == 0 ? radix_key(xb[(int64_t)i * k + score_index]) : kin[i];
      atomicAdd(&s_hist[(key >> (8 * pass)) & 255u], 1);
    }
  }
  __syncthreads();
  hist[((int64_t)b * 256 + tid) * nblocks + blk] = s_hist[tid];
}

// exclusive prefix sum over the 256 * nblocks counts of a batch, in place
__global__ void __launch_bounds__(1024)
k_radix_scan(const int32_t* __restrict__ valid_count, int32_t* __restrict__ hist, int n, int nblocks) {
  __shared__ int s_sum[1024];
  const int b = blockIdx.x, tid = threadIdx.x;
  if (batch_state(valid_count, b, n) != 0) return;
  int32_t* h = hist + (int64_t)b * 256 * nblocks;
  const int total = 256 * nblocks;
  const int per = (total + 1023) / 1024;
  const int lo = tid * per < total ? tid * per : total, hi = lo + per < total ? lo + per : total;
  int sum = 0;
  for (int i = lo; i < hi; ++i) sum += h[i];
  s_sum[tid] = sum;
  __syncthreads();
  // inclusive scan of the 1024 partial sums
  for (int d = 1; d < 1024; d <<= 1) {
    const int v = tid >= d ? s_sum[tid - d] : 0;
    __syncthreads();
    s_sum[tid] += v;
    __syncthreads();
  }
  int run = s_sum[tid] - sum;
  for (int i = lo; i < hi; ++i) {
    const int c = h[i];
    h[i] = run;
    run += c;
  }
}

__global__ void __launch_bounds__(RADIX_THREADS)
k_radix_scatter(const int32_t* __restrict__ x, const int32_t* __restrict__ valid_count, const uint32_t* __restrict__ keys_in,
                const int32_t* __restrict__ idx_in, uint32_t* __restrict__ keys_out, int32_t* __restrict__ idx_out,
                const int32_t* __restrict__ hist, int32_t* __restrict__ rank, int n, int k, int score_index, int pass,
                int nblocks, int64_t key_stride, int last) {
  __shared__ int s_first[256];      // next free position of every digit for this workgroup
  __shared__ int s_cnt[4][256];     // elements of the current round per wavefront and digit
  const int b = blockIdx.y, blk = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (batch_state(valid_count, b, n) != 0) return;
  const int vc = clamp_vc(valid_count[b], n);
  const int base = blk * RADIX_CHUNK;
  if (base >= vc) return;
  s_first[tid] = hist[((int64_t)b * 256 + tid) * nblocks + blk];
  const int32_t* xb = x + (int64_t)b * n * k;
  const uint32_t* kin = keys_in + b * key_stride;
  const int32_t* iin = idx_in + b * key_stride;
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int r = 0; r < RADIX_ROUNDS; ++r) {
    for (int w = 0; w < 4; ++w) s_cnt[w][tid] = 0;
    __syncthreads();
    const int i = base + r * RADIX_THREADS + tid;
    const bool live = i < vc;
    uint32_t key = 0;
    int row = 0;
    if (live) {
      key = pass == 0 ? radix_key(xb[(int64_t)i * k + score_index]) : kin[i];
      row = pass == 0 ? i : iin[i];
    }
    const unsigned digit = (key >> (8 * pass)) & 255u;
    // lanes of this wavefront that are live and hold the same digit
    unsigned long long same = __ballot(live);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const unsigned long long set = __ballot((digit >> bit) & 1u);
      same &= ((digit >> bit) & 1u) ? set : ~set;
    }
    const int before = __popcll(same & lt);
    if (live && before == 0) s_cnt[wave][digit] = __popcll(same);   // the first lane of every group of equal digits
    __syncthreads();
    if (live) {
      int pos = s_first[digit] + before;
      for (int w = 0; w < wave; ++w) pos += s_cnt[w][digit];
      if (last) {
        rank[(int64_t)b * n + row] = pos;
      } else {
        keys_out[b * key_stride + pos] = key;
        idx_out[b * key_stride + pos] = row;
      }
    }
    __syncthreads();
    s_first[tid] += s_cnt[0][tid] + s_cnt[1][tid] + s_cnt[2][tid] + s_cnt[3][tid];
    __syncthreads();
  }
}

// With 0 < top_k <= TOPK_MAX_K only the top_k best rows are ever looked at again, so only they need a
// rank.  One workgroup per batch keeps every score in registers (thread t owns rows t, t + 1024, ...),
// finds the top_k-th largest score T by bisection on the bits in which scores differ (ballot counts, no
// atomics on data), and ranks: rows above T among themselves (fewer than top_k; listed in LDS as
// (score, ~index) words so one 64-bit compare orders them as the stable sort would); rows equal to T
// by their position among the equal rows in index order; every other row gets the marker rank top_k,
// which only says "not among the first top_k".  With top_k >= valid rows every row is ranked in the list.
// All counts are integers, so the result is exact.
constexpr int TOPK_THREADS = 1024, TOPK_ROWS = 32, TOPK_WAVES = TOPK_THREADS / 64;  // rows per thread
constexpr int TOPK_MAX_N = TOPK_THREADS * TOPK_ROWS, TOPK_MAX_K = 2048;

// rows of this wavefront whose key is at least `cand`, over the first RB rows of every lane
template <int RB>
__device__ __forceinline__ int topk_count_ge(const uint32_t (&key)[TOPK_ROWS], uint32_t cand) {
  int c = 0;
#pragma unroll
  for (int r = 0; r < RB; ++r) c += __popcll(__ballot(key[r] >= cand));
  return c;
}

__global__ void __launch_bounds__(TOPK_THREADS)
k_nms_topk_rank(const int32_t* __restrict__ x, const int32_t* __restrict__ valid_count, int32_t* __restrict__ rank,
                int n, int k, int score_index, int topk) {
  __shared__ __attribute__((aligned(16))) unsigned long long s_comp[TOPK_MAX_K];
  __shared__ int s_cnt[TOPK_MAX_K];
  __shared__ int s_tab[TOPK_ROWS * TOPK_WAVES], s_part[2][TOPK_WAVES], s_wsum[TOPK_WAVES];
  __shared__ uint32_t s_and[TOPK_WAVES], s_or[TOPK_WAVES];
  __shared__ int s_gcount;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (batch_state(valid_count, b, n) != 0) return;
  const int vc = clamp_vc(valid_count[b], n);
  const int R = (vc + TOPK_THREADS - 1) / TOPK_THREADS;
  int32_t* rk = rank + (int64_t)b * n;
  // top_k >= valid rows (at most TOPK_MAX_K of them then): every row is "above" and is ranked in the list
  const bool all = topk >= vc;
  const int32_t* xb = x + (int64_t)b * n * k;
  for (int i = tid; i < TOPK_MAX_K; i += TOPK_THREADS) { s_cnt[i] = 0; s_comp[i] = 0; }
  if (tid == 0) s_gcount = 0;
  // scores as unsigned keys that compare like the signed values; rows past the end hold key 0 and are
  // told apart by their index wherever a real key could be 0 too
  uint32_t key[TOPK_ROWS];
  // All loads are issued before the first result is used (rows past the end re-read the last valid row):
  // a load under a condition, or with its select right behind it, waits for the one before it, and a
  // dozen round trips to memory in a row were a third of this kernel.
#pragma unroll
  for (int r = 0; r < TOPK_ROWS; ++r) {
    const int i = r * TOPK_THREADS + tid, ic = i < vc ? i : vc - 1;
    key[r] = (uint32_t)xb[(int64_t)ic * k + score_index];
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < TOPK_ROWS; ++r) key[r] = r * TOPK_THREADS + tid < vc ? key[r] ^ 0x80000000u : 0u;
  // Bits above the highest bit in which two live keys differ are common to all keys: the bisection
  // only walks the bits below (8 steps for scores that span 8 bits, whatever their offset).
  uint32_t kand = 0xffffffffu, kor = 0;
#pragma unroll
  for (int r = 0; r < TOPK_ROWS; ++r) {
    if (r >= R) break;
    if (r * TOPK_THREADS + tid < vc) { kand &= key[r]; kor |= key[r]; }
  }
  for (int d = 32; d >= 1; d >>= 1) {
    kand &= (uint32_t)__shfl_xor((int)kand, d, 64);
    kor |= (uint32_t)__shfl_xor((int)kor, d, 64);
  }
  if (lane == 0) { s_and[wave] = kand; s_or[wave] = kor; }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < TOPK_WAVES; ++w) { kand &= s_and[w]; kor |= s_or[w]; }
  const uint32_t diff = kand ^ kor;
  const int top_bit = diff ? 31 - __clz((int)diff) : -1;
  // T becomes the top_k-th largest key: the largest T with at least top_k keys >= T
  uint32_t T = top_bit >= 0 ? (kor & ~((2u << top_bit) - 1u)) : kor;
  for (int bit = all ? -1 : top_bit; bit >= 0; --bit) {
    const uint32_t cand = T | (1u << bit);
    // rows past R hold key 0 < cand; counting in blocks of four rows keeps row tests out of the loop (the
    // scalar unit, shared by the 16 wavefronts, is what this loop waits for)
    int c;
    switch ((R + 3) >> 2) {
      case 0: c = 0; break;
      case 1: c = topk_count_ge<4>(key, cand); break;
      case 2: c = topk_count_ge<8>(key, cand); break;
      case 3: c = topk_count_ge<12>(key, cand); break;
      case 4: c = topk_count_ge<16>(key, cand); break;
      case 5: c = topk_count_ge<20>(key, cand); break;
      case 6: c = topk_count_ge<24>(key, cand); break;
      case 7: c = topk_count_ge<28>(key, cand); break;
      default: c = topk_count_ge<32>(key, cand); break;
    }
    int* part = s_part[bit & 1];
    if (lane == 0) part[wave] = c;
    __syncthreads();
    int tot = 0;
#pragma unroll
    for (int w = 0; w < TOPK_WAVES; ++w) tot += part[w];
    if (tot >= topk) T = cand;
  }
  // rows above T: listed in any order (the 64-bit word carries the index); rows equal to T: counted
  // per (row block r, wavefront), which is index order
  const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
  for (int r = 0; r < TOPK_ROWS; ++r) {
    if (r >= R) break;
    const int i = r * TOPK_THREADS + tid;
    const bool up = all ? i < vc : key[r] > T;
    const unsigned long long bu = __ballot(up), be = __ballot(!all && i < vc && key[r] == T);
    int base = 0;
    if (lane == 0) {
      s_tab[r * TOPK_WAVES + wave] = __popcll(be);
      if (bu) base = atomicAdd(&s_gcount, __popcll(bu));
    }
    base = __shfl(base, 0, 64);
    if (up) s_comp[base + __popcll(bu & lt)] = ((unsigned long long)key[r] << 32) | (uint32_t)~(uint32_t)i;
  }
  __syncthreads();
  const int g = s_gcount;           // rows above T: fewer than top_k
  const int from_equal = topk - g;  // this many of the equal rows, in index order, complete the top_k
  // exclusive prefix of the equal-row counts over (r, wavefront)
  {
    const int cells = R * TOPK_WAVES;
    const int v = tid < cells ? s_tab[tid] : 0;
    int inc = v;
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(inc, d, 64);
      if (lane >= d) inc += o;
    }
    if (lane == 63) s_wsum[wave] = inc;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w) before += s_wsum[w];
    if (tid < cells) s_tab[tid] = before + inc - v;
  }
  // ranks among the rows above T: element p counts the words larger than its own, its q range split
  // over `slices` threads whose partial counts add up in LDS
  const int P = (g + 63) & ~63;
  const int slices = P > 0 && P < TOPK_THREADS ? TOPK_THREADS / P : 1;
  const int chunk = ((g + slices - 1) / slices + 1) & ~1;
  for (int item = tid; item < P * slices; item += TOPK_THREADS) {
    const int p = item % P, sl = item / P;
    if (p >= g) continue;
    const unsigned long long me = s_comp[p];
    int q0 = sl * chunk, q1 = q0 + chunk;   // the list is zero-padded past g: zeros are below every real word
    if (q1 > TOPK_MAX_K) q1 = TOPK_MAX_K;
    int c = 0;
    for (int q = q0; q < q1 && q < g; q += 2) {
      const ulonglong2 o = *reinterpret_cast<const ulonglong2*>(&s_comp[q]);
      c += (o.x > me) + (o.y > me);
    }
    if (c) atomicAdd(&s_cnt[p], c);
  }
  __syncthreads();
  for (int p = tid; p < g; p += TOPK_THREADS) rk[(int)~(uint32_t)s_comp[p]] = s_cnt[p];
#pragma unroll
  for (int r = 0; r < TOPK_ROWS; ++r) {
    if (r >= R) break;
    const int i = r * TOPK_THREADS + tid;
    const bool eq = !all && i < vc && key[r] == T;
    const unsigned long long be = __ballot(eq);
    if (all || i >= vc || key[r] > T) continue;
    if (eq) {
      const int e = s_tab[r * TOPK_WAVES + wave] + __popcll(be & lt);
      rk[i] = e < from_equal ? g + e : topk;
    } else {
      rk[i] = topk;
    }
  }
}

// Row i moves to its sorted slot; rows ranked at or past top_k are then overwritten with -1 in the input
// tensor (nms.cc:92-96).  Every output row starts as -1: k_nms_select writes the kept rows over the front.
__global__ void __launch_bounds__(256)
k_nms_scatter(int32_t* __restrict__ x, const int32_t* __restrict__ valid_count, const int32_t* __restrict__ rank,
              int32_t* __restrict__ order, int32_t* __restrict__ sorted, int32_t* __restrict__ y, int n, int k,
              int topk, int64_t ws_stride) {
  const int b = blockIdx.y;
  const int state = batch_state(valid_count, b, n);
  if (state == 2) return;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  int32_t* yrow = y + ((int64_t)b * n + i) * k;
  for (int c = 0; c < k; ++c) yrow[c] = -1;
  if (state == 1) return;
  const int vc = clamp_vc(valid_count[b], n);
  if (i >= vc) return;
  int32_t* xrow = x + ((int64_t)b * n + i) * k;
  const int r = rank[(int64_t)b * n + i];
  if (topk > 0 && r >= topk) {  // never looked at again (its rank may be the marker top_k, shared by many rows)
    for (int c = 0; c < k; ++c) xrow[c] = -1;
    return;
  }
  order[b * ws_stride + r] = i;
  int32_t* dst = sorted + b * ws_stride * k + (int64_t)r * k;
  for (int c = 0; c < k; ++c) dst[c] = xrow[c];
}

constexpr int NMS_BM_ROWS = 512, NMS_BM_WORDS = 16;  // rows of the suppression bit matrix and its words per row

// Suppression bit matrix for the first `keep` sorted rows, when they are few enough: bit j of row i says
// that row i, if it survives, removes row j (j > i, matching id unless forced, overlap at the threshold).
// One wavefront per (row, 64 candidates); the ballot is the two mask words.
__global__ void __launch_bounds__(256)
k_nms_mask(const int32_t* __restrict__ valid_count, const int32_t* __restrict__ sorted, uint32_t* __restrict__ mask,
           int n, int k, int iou_threshold, int topk, int coord_start, int id_index, int force_suppress,
           int64_t ws_stride) {
  const int b = blockIdx.z;
  if (batch_state(valid_count, b, n) != 0) return;
  const int vc = clamp_vc(valid_count[b], n);
  const int keep = (topk >= 0 && topk < vc) ? topk : vc;
  if (keep > NMS_BM_ROWS) return;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (i >= keep) return;
  const int j = blockIdx.y * 64 + lane;
  const int32_t* srt = sorted + b * ws_stride * k;
  bool hit = false;
  if (j > i && j < keep) {
    const int32_t* r1 = srt + (int64_t)i * k;
    const int32_t* r2 = srt + (int64_t)j * k;
    if (force_suppress || id_index < 0 || r1[id_index] == r2[id_index])
      hit = iou_at_least(r1 + coord_start, r2 + coord_start, iou_threshold);
  }
  const unsigned long long bits = __ballot(hit);
  if (lane == 0) {
    uint32_t* m = mask + ((int64_t)b * NMS_BM_ROWS + i) * NMS_BM_WORDS + blockIdx.y * 2;
    m[0] = (uint32_t)bits;
    m[1] = (uint32_t)(bits >> 32);
  }
}

constexpr int NMS_THREADS = 1024;
constexpr int NMS_LDS_ROWS = 1024, NMS_LDS_K = 6;  // rows x columns of the LDS copy in k_nms_select (24 KiB)

// One workgroup per batch walks the sorted rows in order.  Row i is emitted if
// it survived and has id >= 0; a surviving row then suppresses, in parallel,
// the rows after it up to (not including) the first row with a negative id.
__global__ void __launch_bounds__(NMS_THREADS)
k_nms_select(const int32_t* __restrict__ valid_count, int32_t* __restrict__ y,
             const int32_t* __restrict__ sorted, int32_t* __restrict__ nextneg,
             int32_t* __restrict__ removed, const uint32_t* __restrict__ mask, int n, int k, int max_output_size,
             int iou_threshold, int topk, int coord_start, int id_index, int force_suppress, int64_t ws_stride) {
  __shared__ int s_wmin[NMS_THREADS / 64];
  __shared__ int s_carry;
  const int b = blockIdx.x, tid = threadIdx.x;
  const int state = batch_state(valid_count, b, n);
  if (state == 2) return;
  if (state == 1) return;  // k_nms_scatter has already filled the output with -1
  int32_t* yb = y + (int64_t)b * n * k;
  const int vc = clamp_vc(valid_count[b], n);
  const int32_t* srt = sorted + b * ws_stride * k;
  int32_t* nn = nextneg + b * (ws_stride + 1);
  int32_t* rem = removed + b * ws_stride;
  const int keep = (topk >= 0 && topk < vc) ? topk : vc;

  // The greedy walk is a chain of dependent steps: when the candidate rows fit (top_k bounds them in
  // practice) they, the cut points and the removal flags live in LDS, whose latency is a tenth of HBM's.
  __shared__ int32_t s_rows[NMS_LDS_ROWS * NMS_LDS_K];
  __shared__ int32_t s_nn[NMS_LDS_ROWS + 1];
  __shared__ uint32_t s_mask[NMS_BM_ROWS * NMS_BM_WORDS];  // the loop path keeps its removal flags here instead
  static_assert(NMS_BM_ROWS * NMS_BM_WORDS >= NMS_LDS_ROWS, "removal flags share the bit matrix's storage");
  const bool staged = keep <= NMS_LDS_ROWS && k <= NMS_LDS_K;
  if (staged) {
    for (int i = tid; i < keep * k; i += NMS_THREADS) s_rows[i] = srt[i];
    srt = s_rows;
    rem = reinterpret_cast<int32_t*>(s_mask);
    nn = s_nn;
    __syncthreads();
  }

  // nn[j] = smallest j' >= j with a negative id (keep if none): suffix minimum,
  // computed chunk by chunk from the back.
  if (tid == 0) { s_carry = keep; nn[keep] = keep; }
  for (int i = tid; i < keep; i += NMS_THREADS) rem[i] = 0;
  __syncthreads();
  for (int base = ((keep - 1) / NMS_THREADS) * NMS_THREADS; base >= 0 && keep > 0; base -= NMS_THREADS) {
    const int j = base + tid;
    int v = (j < keep && srt[(int64_t)j * k] < 0) ? j : keep;
    // inclusive suffix-min inside the wavefront
    const int lane = tid & 63, wv = tid >> 6;
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_down(v, d, 64);
      if (lane + d < 64) v = o < v ? o : v;
    }
    if (lane == 0) s_wmin[wv] = v;
    __syncthreads();
    int later = s_carry;
    for (int w = wv + 1; w < NMS_THREADS / 64; ++w) later = s_wmin[w] < later ? s_wmin[w] : later;
    v = later < v ? later : v;
    if (j < keep) nn[j] = v;
    __syncthreads();
    if (tid == 0) s_carry = v;  // thread 0 holds the minimum of the whole chunk and everything after it
    __syncthreads();
  }

  int yi = 0;
  // With few enough rows k_nms_mask has tested every pair up front, and the walk only has to find the set
  // of removed rows: a row is removed by rows before it only, so whether it acts is known when the walk
  // reaches it.  One wavefront holds the set in registers (lane l: bits 32l..32l+31, repeated every 16
  // lanes) and ORs in the matrix row of each row that is still there, cut at the first later row with a
  // negative id.  The rows emitted are then the surviving ones whose id is not negative, in order.  Same
  // decisions as the loop below.
  __shared__ uint32_t s_pos[NMS_BM_WORDS], s_emit[NMS_BM_WORDS];
  __shared__ int s_before[NMS_BM_WORDS], s_yi;
  if (staged && keep <= NMS_BM_ROWS) {
    const uint32_t* mb = mask + (int64_t)b * NMS_BM_ROWS * NMS_BM_WORDS;
    for (int t = tid; t < keep * NMS_BM_WORDS; t += NMS_THREADS) {
      const int live = s_nn[(t / NMS_BM_WORDS) + 1] - (t % NMS_BM_WORDS) * 32;  // bits of this word below the cut
      s_mask[t] = mb[t] & (live >= 32 ? 0xffffffffu : live <= 0 ? 0u : (1u << live) - 1u);
    }
    if (tid < NMS_BM_ROWS) {
      const unsigned long long pos = __ballot(tid < keep && s_rows[tid * k] >= 0);
      if ((tid & 63) == 0) {
        s_pos[tid >> 5] = (uint32_t)pos;
        s_pos[(tid >> 5) + 1] = (uint32_t)(pos >> 32);
      }
    }
    __syncthreads();
    if (tid < 64) {
      const int l16 = tid & (NMS_BM_WORDS - 1);
      // The walk goes block by block (32 rows = one word of the set).  Inside a block only the bits of that word
      // matter, and they are a chain of scalar steps over the block's rows, using the diagonal block (lane j of
      // diagv: row 32 B + j, word B).  The rows that acted then OR their whole matrix rows into the set for the
      // blocks to come -- independent LDS reads spread over the four groups of 16 lanes, off the chain.
      // (One step per row through the vector registers -- read the set's word, test, OR the row -- took 88 clocks a
      // row, 16 of the kernel's 21 us for 400 candidates.)
      uint32_t remw = 0;
      const int keep_u = __builtin_amdgcn_readfirstlane(keep);   // the chain below is scalar: say so
      const int nblocks = (keep_u + 31) >> 5;
      for (int B = 0; B < nblocks; ++B) {
        const int rowj = B * 32 + (tid & 31);
        const uint32_t diagv = rowj < keep ? s_mask[rowj * NMS_BM_WORDS + B] : 0u;
        uint32_t cur = (uint32_t)__builtin_amdgcn_readlane((int)remw, B);
        const int here = keep_u - B * 32 < 32 ? keep_u - B * 32 : 32;
        const uint32_t valid = here >= 32 ? 0xffffffffu : (1u << here) - 1u;
        // 32 steps of three scalar instructions each (test the row's bit, select its diagonal bits or nothing, OR), the
        // diagonal rows fetched from the lanes beforehand with constant lane numbers.  Only bits behind a row count
        // (a row never removes an earlier one), so a row's bit is final when the walk passes it and the rows that
        // acted are the ones whose bit is still clear at the end.
        uint32_t d[32];
#pragma unroll
        for (int jj = 0; jj < 32; ++jj) d[jj] = (uint32_t)__builtin_amdgcn_readlane((int)diagv, jj) & ~((2u << jj) - 1u);
#pragma unroll
        for (int jj = 0; jj < 32; ++jj) cur |= ((cur >> jj) & 1u) ? 0u : d[jj];
        const uint32_t acted = ~cur & valid;
        // lane (q, l16), q = lane / 16: word l16 of the rows q, q + 4, ... of the block, eight reads in flight
        uint32_t acc = 0;
        const int q = tid >> 4;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int jj = q + 4 * u;
          const uint32_t w = s_mask[(B * 32 + jj) * NMS_BM_WORDS + l16];   // rows past `keep` lie inside the matrix and never act
          acc |= ((acted >> jj) & 1u) ? w : 0u;
        }
        acc |= (uint32_t)__shfl_xor((int)acc, 16, 64);
        acc |= (uint32_t)__shfl_xor((int)acc, 32, 64);
        remw |= acc;
      }
      const int live = keep - l16 * 32;
      const uint32_t e = ~remw & s_pos[l16] & (live >= 32 ? 0xffffffffu : live <= 0 ? 0u : (1u << live) - 1u);
      const int c = __popc(e);
      int p = c;  // inclusive prefix over the 16 words
      for (int d = 1; d < NMS_BM_WORDS; d <<= 1) {
        const int o = __shfl_up(p, d, NMS_BM_WORDS);
        if (l16 >= d) p += o;
      }
      if (tid < NMS_BM_WORDS) { s_emit[tid] = e; s_before[tid] = p - c; }
      if (tid == NMS_BM_WORDS - 1) s_yi = p;
    }
    __syncthreads();
    yi = s_yi;
    // max_output_size keeps the first `max_output_size` emitted rows (nms.cc:126-137)
    if (max_output_size > 0 && yi > max_output_size) yi = max_output_size;
    if (tid < NMS_BM_ROWS) {
      const uint32_t e = s_emit[tid >> 5];
      if ((e >> (tid & 31)) & 1u) {
        const int at = s_before[tid >> 5] + __popc(e & ((1u << (tid & 31)) - 1u));
        if (at < yi)
          for (int c = 0; c < k; ++c) yb[(int64_t)at * k + c] = s_rows[tid * k + c];
      }
    }
    return;
  }
  for (int i = 0; i < keep; ++i) {
    __syncthreads();  // removals from the previous row (and the staging above) are visible
    if (rem[i]) continue;
    const int32_t* r1 = srt + (int64_t)i * k;
    if (r1[0] >= 0) {
      if (tid < k) yb[(int64_t)yi * k + tid] = r1[tid];
      ++yi;
    }
    const int limit = nn[i + 1];
    const int32_t id1 = id_index >= 0 ? r1[id_index] : 0;
    for (int j = i + 1 + tid; j < limit; j += NMS_THREADS) {
      if (rem[j]) continue;
      const int32_t* r2 = srt + (int64_t)j * k;
      if (force_suppress || id_index < 0 || id1 == r2[id_index])
        if (iou_at_least(r1 + coord_start, r2 + coord_start, iou_threshold)) rem[j] = 1;
    }
  }
  // max_output_size keeps the first `max_output_size` emitted rows (nms.cc:126-137)
  if (max_output_size > 0 && yi > max_output_size) yi = max_output_size;
  __syncthreads();
  for (int64_t i = (int64_t)yi * k + tid; i < (int64_t)n * k; i += NMS_THREADS) yb[i] = -1;
}

// ---- scratch of the entry point that allocates nothing (cvmhip_non_max_suppression_static).
// One array per GPU, part of the code object, held until the process ends.  In host code its name is only a
// handle for hipGetSymbolAddress: the device address is looked up once per device, with that device
// current, and only that address is ever passed to a kernel.
constexpr size_t NMS_STATIC_WORDS = (size_t)1 << 19;   // 2 MiB: e.g. one batch of 37 000 rows of 6 values
static __device__ __align__(256) int32_t g_nms_scratch[NMS_STATIC_WORDS];

constexpr int NMS_MAX_DEVICES = 64;
static std::mutex g_nms_scratch_mu;
static void* g_nms_scratch_ptr[NMS_MAX_DEVICES] = {};

// device address of the current device's copy of the array
static int nms_static_scratch(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= NMS_MAX_DEVICES) {
    set_error("non_max_suppression_static: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return CVMHIP_ERR_RUNTIME;
  }
  std::lock_guard<std::mutex> lock(g_nms_scratch_mu);
  if (!g_nms_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_nms_scratch));
    if (e != hipSuccess || !p) {
      set_error("non_max_suppression_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return CVMHIP_ERR_RUNTIME;
    }
    g_nms_scratch_ptr[dev] = p;
  }
  *ptr = g_nms_scratch_ptr[dev];
  return CVMHIP_OK;
}

static int nms_check_args(const int32_t* x, const int32_t* valid_count, const int32_t* y, int batches, int n, int k,
                          int iou_threshold, int coord_start, int score_index, int id_index, int topk) {
  if (!x || !valid_count || !y || x == y || batches < 1 || n < 1 || k < 2 || batches > 65535)
    return arg_error("non_max_suppression");
  if (iou_threshold <= 0) return arg_error("non_max_suppression.iou_threshold must be positive");
  if (coord_start < 0 || coord_start + 4 > k || score_index < 0 || score_index >= k || id_index >= k)
    return arg_error("non_max_suppression indices");
  // 2^24 is the largest dimension the reference's shape check accepts (src/runtime/infer_attr.cc).  Ranking is a sort, but
  // the greedy walk over the candidate rows (the first top_k in sorted order, or all valid rows) compares every kept
  // row with every later one, as the reference's does: one workgroup needs about 0.8 s for 100 000 candidate rows of
  // which most are kept, and the time grows with the square.  More than 2^18 candidates (about 5 s at worst) are
  // refused rather than launched as a kernel that runs for minutes.
  if (n > (1 << 24)) return arg_error("non_max_suppression: more than 2^24 anchors per batch");
  if (n > (1 << 18) && !(topk >= 0 && topk <= (1 << 18)))
    return arg_error("non_max_suppression: more than 2^18 candidate rows per batch (set top_k to bound the greedy walk)");
  return CVMHIP_OK;
}

// Validation and launches shared by the two entry points; `workspace` holds cvmhip_nms_workspace_bytes() bytes.
static int nms_launch(int32_t* x, const int32_t* valid_count, int32_t* y,
                      int batches, int n, int k, int max_output_size,
                      int iou_threshold, int topk, int coord_start,
                      int score_index, int id_index, int force_suppress,
                      void* workspace, hipStream_t s) {
  int32_t* order = reinterpret_cast<int32_t*>(workspace);
  int32_t* nextneg = order + (size_t)batches * n;
  int32_t* removed = nextneg + (size_t)batches * (n + 1);
  int32_t* sorted = removed + (size_t)batches * n;
  int32_t* rank = sorted + (size_t)batches * n * k;
  uint32_t* mask = reinterpret_cast<uint32_t*>(rank + (size_t)batches * n);
  int rc;
  if (topk > 0 && topk <= TOPK_MAX_K && n <= TOPK_MAX_N) {
    k_nms_topk_rank<<<batches, TOPK_THREADS, 0, s>>>(x, valid_count, rank, n, k, score_index, topk);
    rc = check_launch("nms.topk_rank");
  } else if (n >= RADIX_MIN_ROWS) {
    // stable radix sort: two key and two index buffers and the digit counts, behind the bit matrix
    const int nblocks = (n + RADIX_CHUNK - 1) / RADIX_CHUNK;
    uint32_t* keys[2];
    int32_t* idx[2];
    keys[0] = mask + (size_t)batches * NMS_BM_ROWS * NMS_BM_WORDS;
    keys[1] = keys[0] + (size_t)batches * n;
    idx[0] = reinterpret_cast<int32_t*>(keys[1] + (size_t)batches * n);
    idx[1] = idx[0] + (size_t)batches * n;
    int32_t* hist = idx[1] + (size_t)batches * n;
    rc = CVMHIP_OK;
    for (int pass = 0; pass < 4 && !rc; ++pass) {
      const int in = (pass + 1) & 1, out = pass & 1;   // pass 0 reads the tensor itself
      dim3 grid(nblocks, batches);
      k_radix_hist<<<grid, RADIX_THREADS, 0, s>>>(x, valid_count, keys[in], hist, n, k, score_index, pass, nblocks, (int64_t)n);
      k_radix_scan<<<batches, 1024, 0, s>>>(valid_count, hist, n, nblocks);
      k_radix_scatter<<<grid, RADIX_THREADS, 0, s>>>(x, valid_count, keys[in], idx[in], keys[out], idx[out], hist, rank, n, k,
                                                     score_index, pass, nblocks, (int64_t)n, pass == 3 ? 1 : 0);
      rc = check_launch("nms.radix_sort");
    }
  } else {
    k_zero32<<<grid_for((int64_t)batches * n, 256), 256, 0, s>>>(rank, (int64_t)batches * n);
    dim3 rgrid((n + 255) / 256, (n + RANK_JT - 1) / RANK_JT, batches);
    k_nms_rank<<<rgrid, 256, 0, s>>>(x, valid_count, rank, n, k, score_index);
    rc = check_launch("nms.rank");
  }
  if (rc) return rc;
  dim3 grid((n + 255) / 256, batches);
  k_nms_scatter<<<grid, 256, 0, s>>>(x, valid_count, rank, order, sorted, y, n, k, topk, (int64_t)n);
  rc = check_launch("nms.scatter");
  if (rc) return rc;
  int rows = n < NMS_BM_ROWS ? n : NMS_BM_ROWS;  // upper bound of the rows the walk can see, when the matrix is used
  if (topk >= 0 && topk < rows) rows = topk;
  if (rows > 0 && k <= NMS_LDS_K) {
    dim3 mgrid((rows + 3) / 4, (rows + 63) / 64, batches);
    k_nms_mask<<<mgrid, 256, 0, s>>>(valid_count, sorted, mask, n, k, iou_threshold, topk, coord_start, id_index,
                                     force_suppress, (int64_t)n);
    rc = check_launch("nms.mask");
    if (rc) return rc;
  }
  k_nms_select<<<batches, NMS_THREADS, 0, s>>>(valid_count, y, sorted, nextneg, removed, mask, n, k,
                                               max_output_size, iou_threshold, topk, coord_start, id_index,
                                               force_suppress, (int64_t)n);
  return check_launch("nms.select");
}


}  // namespace cvmhip

using namespace cvmhip;

extern "C" {

size_t cvmhip_get_valid_counts_workspace_bytes(int batches, int n) {
  const int nchunks = (n + GVC_CHUNK - 1) / GVC_CHUNK;
  return (size_t)batches * nchunks * sizeof(int32_t);
}

int cvmhip_get_valid_counts(const int32_t* x, int32_t* valid_count, int32_t* y,
                            int batches, int n, int k, int32_t score_threshold,
                            void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !valid_count || !y || batches < 1 || n < 1 || k < 2 || batches > 65535) return arg_error("get_valid_counts");
  if (!workspace || workspace_bytes < cvmhip_get_valid_counts_workspace_bytes(batches, n))
    return arg_error("get_valid_counts workspace");
  const int nchunks = (n + GVC_CHUNK - 1) / GVC_CHUNK;
  int32_t* counts = reinterpret_cast<int32_t*>(workspace);
  hipStream_t s = as_stream(stream);
  dim3 grid(nchunks, batches);
  k_gvc_count<<<grid, GVC_CHUNK, 0, s>>>(x, counts, n, k, score_threshold, nchunks);
  int rc = check_launch("get_valid_counts.count");
  if (rc) return rc;
  k_gvc_scatter<<<grid, GVC_CHUNK, 0, s>>>(x, counts, valid_count, y, n, k, score_threshold, nchunks);
  return check_launch("get_valid_counts.scatter");
}

// per batch: order[n], nextneg[n+1], removed[n], sorted[n*k], rank[n], suppression bit matrix; from RADIX_MIN_ROWS rows on
// also the radix sort's two key buffers, two index buffers and digit counts
size_t cvmhip_nms_workspace_bytes(int batches, int n, int k) {
  size_t per = (size_t)n * (4 + (size_t)k) + 2 + (size_t)NMS_BM_ROWS * NMS_BM_WORDS;
  if (n >= RADIX_MIN_ROWS) per += (size_t)n * 4 + (size_t)256 * ((n + RADIX_CHUNK - 1) / RADIX_CHUNK);
  return (size_t)batches * per * sizeof(int32_t);
}

int cvmhip_non_max_suppression(int32_t* x, const int32_t* valid_count, int32_t* y,
                               int batches, int n, int k, int max_output_size,
                               int iou_threshold, int topk, int coord_start,
                               int score_index, int id_index, int force_suppress,
                               void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = nms_check_args(x, valid_count, y, batches, n, k, iou_threshold, coord_start, score_index, id_index, topk);
  if (rc) return rc;
  if (!workspace || workspace_bytes < cvmhip_nms_workspace_bytes(batches, n, k)) return arg_error("non_max_suppression workspace");
  return nms_launch(x, valid_count, y, batches, n, k, max_output_size, iou_threshold, topk, coord_start, score_index,
                    id_index, force_suppress, workspace, as_stream(stream));
}

size_t cvmhip_nms_static_capacity_bytes(void) { return sizeof(int32_t) * NMS_STATIC_WORDS; }

int cvmhip_non_max_suppression_static(int32_t* x, const int32_t* valid_count, int32_t* y,
                                      int batches, int n, int k, int max_output_size,
                                      int iou_threshold, int topk, int coord_start,
                                      int score_index, int id_index, int force_suppress, void* stream) {
  const int rc = nms_check_args(x, valid_count, y, batches, n, k, iou_threshold, coord_start, score_index, id_index, topk);
  if (rc) return rc;
  const size_t need = cvmhip_nms_workspace_bytes(batches, n, k);
  if (need > cvmhip_nms_static_capacity_bytes()) {
    set_error("invalid argument: non_max_suppression_static: batches=%d n=%d k=%d needs %zu bytes of scratch, the static "
              "buffer holds %zu; use cvmhip_non_max_suppression with a caller workspace",
              batches, n, k, need, cvmhip_nms_static_capacity_bytes());
    return CVMHIP_ERR_ARG;
  }
  void* scratch = nullptr;
  const int rs = nms_static_scratch(&scratch);
  if (rs) return rs;
  return nms_launch(x, valid_count, y, batches, n, k, max_output_size, iou_threshold, topk, coord_start, score_index,
                    id_index, force_suppress, scratch, as_stream(stream));
}

}  // extern "C"
