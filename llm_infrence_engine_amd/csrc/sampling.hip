// Token choice from float logits:
//   temperature <= 0 : the first index of the maximum
//   otherwise        : logits / temperature, then top-k (ties at the k-th value kept), then top-p
//                      (a token is dropped when the mass of the strictly larger ones reaches top_p; the
//                      largest is always kept), then a draw from the softmax of what is left.
// The k-th value and the top-p threshold are found over an order-preserving integer image of the floats, by a
// radix descent that spreads every row over many blocks (see below), so no sort is needed.  The uniform number
// of a draw is Philox4x32-10(seed, draw index): the same seed and index give the same token.
#include "common.h"
#include "api.h"
#include <algorithm>
#include <mutex>

namespace {

constexpr int THREADS = 1024;

__device__ __forceinline__ unsigned order_key(float f) {  // a < b  <=>  key(a) < key(b)
  const unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ unsigned mulhi32(unsigned a, unsigned b) { return __umulhi(a, b); }

__device__ float philox_uniform(unsigned long long seed, unsigned counter) {
  unsigned c0 = counter, c1 = 0, c2 = 0, c3 = 0;
  unsigned k0 = (unsigned)seed, k1 = (unsigned)(seed >> 32);
  for (int r = 0; r < 10; ++r) {
    const unsigned hi0 = mulhi32(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const unsigned hi1 = mulhi32(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const unsigned n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return (float)(c0 >> 8) * (1.0f / 16777216.0f);  // [0, 1)
}

struct MaxIdx { float v; int i; };

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {  // larger value, then smaller index; NaN never wins
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ MaxIdx block_argmax(const float* __restrict__ row, int V, MaxIdx* red) {
  MaxIdx best = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < V; i += blockDim.x) best = better(best, MaxIdx{row[i], i});
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) {
    MaxIdx other = {__shfl_xor(best.v, o, MS_WAVE), __shfl_xor(best.i, o, MS_WAVE)};
    best = better(best, other);
  }
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = best;
  __syncthreads();
  MaxIdx r = red[0];
  for (int w = 1; w < (int)(blockDim.x / MS_WAVE); ++w) r = better(r, red[w]);
  if (r.i == 0x7fffffff) r.i = 0;  // a row of NaN or -inf only
  return r;
}

// ------------------------------------------------------------------------------------------------
// The draw.  A row is spread over n_chunks blocks, and the two thresholds are found by a radix descent over the
// 32-bit keys in three levels (11 + 11 + 10 bits) instead of a bitwise search of 32 + 32 passes by one block:
//
//   top-k: the key v with count{key >= v} >= k > count{key > v}   (ties at the k-th value are kept)
//   top-p: the key v with mass{key >= v} >= p * total > mass{key > v}, total = mass{key >= the top-k key}
//          (a token is dropped when the mass of the strictly larger ones reaches p; the largest always stays)
//
// Per level one kernel makes the histogram (counts and masses per digit) of the keys that share the digits
// found so far, and the next kernel finds the digit at which the running count or mass, taken from the top,
// reaches what is asked for.  Masses are exp(s - max) in fixed point (44 binary places), so sums are exact,
// do not depend on the order in which blocks add them (integer atomics), and every kernel that works one out
// again gets the same bits.  Last, the kept mass of every chunk and one block per row that walks the chunk
// where u * total falls, in index order.
constexpr int RADIX_BINS = 2048;
constexpr int MAX_CHUNKS = 64;
constexpr int N_HIST = 5;            // levels 1 to 3 of the top-k descent, levels 2 and 3 of the top-p descent
constexpr int FIX_PLACES = 44;

struct RowWork {                     // one per row, in the workspace the caller brings
  // Every field is written by one kernel (block 0 of the row) and read by later kernels only.
  unsigned chunk_max[MAX_CHUNKS];    // key of the largest scaled logit of every chunk
  unsigned k_digits[2];              // digits of the top-k key after the searches of levels 1 and 2
  unsigned p_digits[2];              // and of the top-p key
  unsigned top_k_key;                // the top-k key itself (0: top-k keeps everything)
  unsigned floor_key;                // tokens with key >= floor_key are kept
  unsigned pad;
  unsigned long long k_count_above[2];  // tokens with larger digits than those found so far
  unsigned long long k_mass_above[2];
  unsigned long long p_mass_above[2];
  unsigned long long total;          // mass of the tokens that top-k keeps
  unsigned long long chunk_mass[MAX_CHUNKS];
  unsigned count[N_HIST][RADIX_BINS];
  unsigned long long mass[N_HIST][RADIX_BINS];
};

__device__ __forceinline__ unsigned long long fixed_mass(float s, float zmax) {
  return (unsigned long long)(expf(s - zmax) * (float)(1ull << FIX_PLACES));   // at most 2^44: exact for a float
}

__device__ __forceinline__ float key_value(unsigned key) {   // the float whose key this is
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

__device__ __forceinline__ unsigned row_max_key(const RowWork& w, int n_chunks) {
  unsigned best = 0;
  for (int c = 0; c < n_chunks; ++c) best = max(best, w.chunk_max[c]);
  return best;
}

__device__ __forceinline__ int level_shift(int level) { return level == 1 ? 21 : (level == 2 ? 10 : 0); }
__device__ __forceinline__ int level_bins(int level) { return level == 3 ? 1024 : RADIX_BINS; }

struct Found { int bin; unsigned long long count_above, mass_above, count_in, mass_in; };

// The first bin, from the top, at which the running count (by_mass = false) or mass of the bins so far reaches
// `need`; with it the count and mass of the bins above it and of the bin itself.  If none does, the lowest
// bin that holds anything (or bin 0).  Every thread of the block calls this and gets the same answer.
__device__ Found first_bin_reaching(const unsigned* __restrict__ count, const unsigned long long* __restrict__ mass,
                                    int bins, bool by_mass, unsigned long long need) {
  __shared__ unsigned long long wave_c[THREADS / MS_WAVE], wave_m[THREADS / MS_WAVE];
  __shared__ Found found;
  __shared__ int lowest;
  const int t = threadIdx.x, lane = t & (MS_WAVE - 1), wave = t / MS_WAVE;
  // thread t owns bins hi and hi - 1, hi = bins - 1 - 2 t: thread 0 the two topmost
  const int hi = bins - 1 - 2 * t;
  unsigned long long c[2] = {0, 0}, m[2] = {0, 0};
#pragma unroll
  for (int j = 0; j < 2; ++j)
    if (hi - j >= 0) { c[j] = count[hi - j]; m[j] = mass[hi - j]; }
  unsigned long long sc = c[0] + c[1], sm = m[0] + m[1];     // inclusive scan over threads, from the top
  for (int o = 1; o < MS_WAVE; o <<= 1) {
    const unsigned long long oc = __shfl_up(sc, o, MS_WAVE), om = __shfl_up(sm, o, MS_WAVE);
    if (lane >= o) { sc += oc; sm += om; }
  }
  if (t == 0) { found.bin = -1; lowest = bins; }
  __syncthreads();
  if (lane == MS_WAVE - 1) { wave_c[wave] = sc; wave_m[wave] = sm; }
  __syncthreads();
  unsigned long long before_c = 0, before_m = 0;
  for (int w = 0; w < wave; ++w) { before_c += wave_c[w]; before_m += wave_m[w]; }
  unsigned long long run_c = before_c + sc - (c[0] + c[1]), run_m = before_m + sm - (m[0] + m[1]);   // above bin hi
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (hi - j < 0) break;
    const unsigned long long upto = (by_mass ? run_m + m[j] : run_c + c[j]), above = by_mass ? run_m : run_c;
    if (above < need && upto >= need) found = Found{hi - j, run_c, run_m, c[j], m[j]};   // one thread at most
    if (c[j]) atomicMin(&lowest, hi - j);
    run_c += c[j]; run_m += m[j];
  }
  __syncthreads();
  if (found.bin < 0 && t == 0) {   // fewer tokens (or less mass) than asked for: everything is kept
    const int b = lowest < bins ? lowest : 0;
    unsigned long long tc = 0, tm = 0;
    for (int w = 0; w < THREADS / MS_WAVE; ++w) { tc += wave_c[w]; tm += wave_m[w]; }
    found = Found{b, tc - count[b], tm - mass[b], count[b], mass[b]};
  }
  __syncthreads();
  const Found f = found;
  __syncthreads();
  return f;
}

__device__ __forceinline__ void chunk_range(int V, int n_chunks, int c, int* begin, int* end) {
  const int len = (V + n_chunks - 1) / n_chunks;
  *begin = min(V, c * len);
  *end = min(V, *begin + len);
}

// Stage 0: every chunk's largest key, and the workspace made ready (histograms and sums zero).
__global__ void __launch_bounds__(THREADS)
sample_max_kernel(const float* __restrict__ logits, size_t ld, int V, const float* __restrict__ temperature,
                  RowWork* __restrict__ work, int n_chunks) {
  __shared__ unsigned red[THREADS / MS_WAVE];
  const int r = blockIdx.y, c = blockIdx.x;
  RowWork& w = work[r];
  // this block's share of the row's histograms
  unsigned* zc = &w.count[0][0];
  unsigned long long* zm = &w.mass[0][0];
  for (int i = c * THREADS + threadIdx.x; i < N_HIST * RADIX_BINS; i += n_chunks * THREADS) { zc[i] = 0u; zm[i] = 0ull; }
  if (threadIdx.x == 0) { w.chunk_mass[c] = 0ull; w.chunk_max[c] = 0u; }
  const float T = temperature[r];
  if (!(T > 0.f)) return;
  const float inv_t = 1.0f / T;
  const float* row = logits + (size_t)r * ld;
  int begin, end;
  chunk_range(V, n_chunks, c, &begin, &end);
  unsigned best = 0;
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float s = row[i] * inv_t;
    if (s == s) best = max(best, order_key(s));     // NaN never wins
  }
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) best = max(best, (unsigned)__shfl_xor((int)best, o, MS_WAVE));
  if ((threadIdx.x & (MS_WAVE - 1)) == 0) red[threadIdx.x / MS_WAVE] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < THREADS / MS_WAVE; ++k) best = max(best, red[k]);
    w.chunk_max[c] = best;
  }
}

// One level of a descent.  WHAT 0: level 1 of every key (no search before it).  WHAT 1: top-k levels 2 and 3.
// WHAT 2: the last top-k search, the first top-p search, and top-p level 2.  WHAT 3: top-p level 3.
// Block 0 of a row also writes down what the searches found, for the kernels that follow.
template <int WHAT>
__global__ void __launch_bounds__(THREADS)
sample_level_kernel(const float* __restrict__ logits, size_t ld, int V, const float* __restrict__ temperature,
                    const int* __restrict__ top_k, const float* __restrict__ top_p, RowWork* __restrict__ work,
                    int n_chunks, int level) {
  __shared__ unsigned lc[RADIX_BINS];
  __shared__ unsigned long long lm[RADIX_BINS];
  const int r = blockIdx.y, c = blockIdx.x;
  RowWork& w = work[r];
  const float T = temperature[r];
  if (!(T > 0.f)) return;
  const int k = top_k ? top_k[r] : 0;
  const bool use_k = k > 0 && k < V;
  const float p = top_p ? top_p[r] : 1.f;
  const bool use_p = p < 1.f;
  const bool first_block = c == 0 && threadIdx.x == 0;

  int hist = 0;              // which histogram this kernel fills
  unsigned digits = 0;       // the digits a key must share to be counted at this level
  if (WHAT == 1) {
    if (!use_k) return;
    hist = level - 1;
    // the search of the level above
    const unsigned long long count_so_far = level == 2 ? 0ull : w.k_count_above[0];
    const unsigned long long mass_so_far = level == 2 ? 0ull : w.k_mass_above[0];
    const Found f = first_bin_reaching(w.count[level - 2], w.mass[level - 2], level_bins(level - 1), false,
                                       (unsigned long long)k - count_so_far);
    digits = level == 2 ? (unsigned)f.bin : ((w.k_digits[0] << 11) | (unsigned)f.bin);
    if (first_block) {
      w.k_digits[level - 2] = digits;
      w.k_count_above[level - 2] = count_so_far + f.count_above;
      w.k_mass_above[level - 2] = mass_so_far + f.mass_above;
    }
  } else if (WHAT == 2) {
    unsigned floor_k = 0;
    unsigned long long total;
    if (use_k) {
      const Found f = first_bin_reaching(w.count[2], w.mass[2], level_bins(3), false,
                                         (unsigned long long)k - w.k_count_above[1]);
      floor_k = (w.k_digits[1] << 10) | (unsigned)f.bin;
      total = w.k_mass_above[1] + f.mass_above + f.mass_in;
    } else {   // everything is kept: the sum of level 1
      const Found f = first_bin_reaching(w.count[0], w.mass[0], RADIX_BINS, false, ~0ull);
      total = f.mass_above + f.mass_in;
    }
    if (first_block) { w.top_k_key = floor_k; w.total = total; }
    if (!use_p) return;
    const unsigned long long target = (unsigned long long)((double)p * (double)total);
    const Found g = first_bin_reaching(w.count[0], w.mass[0], RADIX_BINS, true, target > 0 ? target : 1ull);
    digits = (unsigned)g.bin;
    hist = 3;
    if (first_block) { w.p_digits[0] = digits; w.p_mass_above[0] = g.mass_above; }
  } else if (WHAT == 3) {
    if (!use_p) return;
    const unsigned long long target = (unsigned long long)((double)p * (double)w.total);
    const unsigned long long need = (target > 0 ? target : 1ull) - w.p_mass_above[0];
    const Found g = first_bin_reaching(w.count[3], w.mass[3], RADIX_BINS, true, need);
    digits = (w.p_digits[0] << 11) | (unsigned)g.bin;
    hist = 4;
    if (first_block) { w.p_digits[1] = digits; w.p_mass_above[1] = w.p_mass_above[0] + g.mass_above; }
  }

  const int shift = level_shift(level), bins = level_bins(level);
  for (int i = threadIdx.x; i < bins; i += blockDim.x) { lc[i] = 0u; lm[i] = 0ull; }
  __syncthreads();
  const float inv_t = 1.0f / T;
  const float zmax = key_value(row_max_key(w, n_chunks));
  const float* row = logits + (size_t)r * ld;
  int begin, end;
  chunk_range(V, n_chunks, c, &begin, &end);
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float s = row[i] * inv_t;
    if (!(s == s)) continue;
    const unsigned key = order_key(s);
    if (level > 1 && (key >> (shift + (level == 2 ? 11 : 10))) != digits) continue;
    const int bin = (int)((key >> shift) & (unsigned)(bins - 1));
    atomicAdd(&lc[bin], 1u);
    atomicAdd(&lm[bin], fixed_mass(s, zmax));
  }
  __syncthreads();
  for (int i = threadIdx.x; i < bins; i += blockDim.x)
    if (lc[i]) {
      atomicAdd(&w.count[hist][i], lc[i]);
      atomicAdd(&w.mass[hist][i], lm[i]);
    }
}

// The floor below which nothing is kept, then every chunk's kept mass.
__global__ void __launch_bounds__(THREADS)
sample_chunk_mass_kernel(const float* __restrict__ logits, size_t ld, int V, const float* __restrict__ temperature,
                         const float* __restrict__ top_p, RowWork* __restrict__ work, int n_chunks, int thresholds) {
  __shared__ unsigned long long red[THREADS / MS_WAVE];
  const int r = blockIdx.y, c = blockIdx.x;
  RowWork& w = work[r];
  const float T = temperature[r];
  if (!(T > 0.f)) return;
  unsigned floor_key = 0;
  if (thresholds) {
    floor_key = w.top_k_key;
    const float p = top_p ? top_p[r] : 1.f;
    if (p < 1.f) {
      const unsigned long long target = (unsigned long long)((double)p * (double)w.total);
      const Found g = first_bin_reaching(w.count[4], w.mass[4], level_bins(3), true,
                                         (target > 0 ? target : 1ull) - w.p_mass_above[1]);
      const unsigned p_key = (w.p_digits[1] << 10) | (unsigned)g.bin;
      if (p_key > floor_key) floor_key = p_key;
    }
  }
  const float inv_t = 1.0f / T;
  const float zmax = key_value(row_max_key(w, n_chunks));
  const float* row = logits + (size_t)r * ld;
  int begin, end;
  chunk_range(V, n_chunks, c, &begin, &end);
  unsigned long long mine = 0;
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float s = row[i] * inv_t;
    if (s == s && order_key(s) >= floor_key) mine += fixed_mass(s, zmax);
  }
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) mine += __shfl_xor(mine, o, MS_WAVE);
  if ((threadIdx.x & (MS_WAVE - 1)) == 0) red[threadIdx.x / MS_WAVE] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long sum = 0;
    for (int k = 0; k < THREADS / MS_WAVE; ++k) sum += red[k];
    w.chunk_mass[c] = sum;
    if (c == 0) w.floor_key = floor_key;    // handed to the last kernel
  }
}

// One block per row: the chunk in which u * total falls, then the first token of it, in index order, at which
// the running mass passes that mark.  A row without temperature takes the first index of its maximum.
__global__ void __launch_bounds__(THREADS)
sample_draw_kernel(const float* __restrict__ logits, size_t ld, int V, const float* __restrict__ temperature,
                   const unsigned long long* __restrict__ seeds, const int* __restrict__ draw_index,
                   RowWork* __restrict__ work, int n_chunks, int* __restrict__ out) {
  __shared__ MaxIdx red_mi[THREADS / MS_WAVE];
  __shared__ unsigned long long scan[THREADS / MS_WAVE];
  __shared__ int chosen;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * ld;
  const float T = temperature[r];
  if (!(T > 0.f)) {
    const MaxIdx top = block_argmax(row, V, red_mi);
    if (threadIdx.x == 0) out[r] = top.i;
    return;
  }
  RowWork& w = work[r];
  const unsigned floor_key = w.floor_key;
  unsigned long long total = 0;
  for (int c = 0; c < n_chunks; ++c) total += w.chunk_mass[c];
  const float u = philox_uniform(seeds ? seeds[r] : 0ull, draw_index ? (unsigned)draw_index[r] : 0u);
  unsigned long long target = (unsigned long long)((double)u * (double)total);     // u < 1: below the total
  if (total > 0 && target >= total) target = total - 1;
  int c = 0;
  unsigned long long before = 0;
  while (c + 1 < n_chunks && before + w.chunk_mass[c] <= target) { before += w.chunk_mass[c]; ++c; }
  int begin, end;
  chunk_range(V, n_chunks, c, &begin, &end);
  const float inv_t = 1.0f / T;
  const float zmax = key_value(row_max_key(w, n_chunks));
  const int per = (end - begin + (int)blockDim.x - 1) / (int)blockDim.x;
  const int lo = min(end, begin + (int)threadIdx.x * per), hi = min(end, lo + per);
  unsigned long long mine = 0;
  for (int i = lo; i < hi; ++i) {
    const float s = row[i] * inv_t;
    if (s == s && order_key(s) >= floor_key) mine += fixed_mass(s, zmax);
  }
  // exclusive sums over the threads, in thread (that is, index) order
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  unsigned long long incl = mine;
  for (int o = 1; o < MS_WAVE; o <<= 1) {
    const unsigned long long v = __shfl_up(incl, o, MS_WAVE);
    if (lane >= o) incl += v;
  }
  if (lane == MS_WAVE - 1) scan[wave] = incl;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  unsigned long long mine_before = before + incl - mine;
  for (int k = 0; k < wave; ++k) mine_before += scan[k];
  if (mine > 0 && mine_before <= target && target < mine_before + mine) {
    unsigned long long run = mine_before;
    for (int i = lo; i < hi; ++i) {
      const float s = row[i] * inv_t;
      if (!(s == s) || order_key(s) < floor_key) continue;
      run += fixed_mass(s, zmax);
      if (run > target) { chosen = i; break; }
    }
  }
  __syncthreads();
  const int pick = chosen;
  if (pick >= 0) {
    if (threadIdx.x == 0) out[r] = pick;
    return;
  }
  const MaxIdx top = block_argmax(row, V, red_mi);   // no mass at all (a row of NaN or -inf): as the greedy choice
  if (threadIdx.x == 0) out[r] = top.i;
}

// First maximum of a row in two stages, so that a few rows still use the whole chip: stage 1 finds the best
// of each of n_chunks slices of the row, stage 2 the best of those (larger value, then smaller index).
__global__ void __launch_bounds__(256)
argmax_chunks_kernel(const float* __restrict__ logits, size_t ld, int V, int n_chunks, float* __restrict__ val,
                     int* __restrict__ idx) {
  __shared__ MaxIdx red[4];
  const int r = blockIdx.y, c = blockIdx.x;
  const int len = ((V + n_chunks - 1) / n_chunks + 3) & ~3;   // slices start at a multiple of four logits
  const int begin = min(V, c * len), end = min(V, begin + len);
  const float* row = logits + (size_t)r * ld;
  MaxIdx best = {-INFINITY, 0x7fffffff};
  if ((((uintptr_t)row) & 15) == 0) {   // four logits a load, and a thread's loads all asked for before the first is used
    for (int i = begin + threadIdx.x * 4; i < end; i += blockDim.x * 4) {
      if (i + 3 < end) {
        const float4 v = *reinterpret_cast<const float4*>(row + i);
        best = better(best, MaxIdx{v.x, i});
        best = better(best, MaxIdx{v.y, i + 1});
        best = better(best, MaxIdx{v.z, i + 2});
        best = better(best, MaxIdx{v.w, i + 3});
      } else {
        for (int j = i; j < end; ++j) best = better(best, MaxIdx{row[j], j});
      }
    }
  } else {
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) best = better(best, MaxIdx{row[i], i});
  }
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) {
    MaxIdx other = {__shfl_xor(best.v, o, MS_WAVE), __shfl_xor(best.i, o, MS_WAVE)};
    best = better(best, other);
  }
  if ((threadIdx.x & (MS_WAVE - 1)) == 0) red[threadIdx.x / MS_WAVE] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) best = better(best, red[w]);
    val[(size_t)r * n_chunks + c] = best.v;
    idx[(size_t)r * n_chunks + c] = best.i;
  }
}

__global__ void __launch_bounds__(MS_WAVE)
argmax_final_kernel(const float* __restrict__ val, const int* __restrict__ idx, int n_chunks, int* __restrict__ out) {
  const int r = blockIdx.x;
  MaxIdx best = {-INFINITY, 0x7fffffff};
  for (int c = threadIdx.x; c < n_chunks; c += MS_WAVE)
    best = better(best, MaxIdx{val[(size_t)r * n_chunks + c], idx[(size_t)r * n_chunks + c]});
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) {
    MaxIdx other = {__shfl_xor(best.v, o, MS_WAVE), __shfl_xor(best.i, o, MS_WAVE)};
    best = better(best, other);
  }
  if (threadIdx.x == 0) out[r] = best.i == 0x7fffffff ? 0 : best.i;
}

}  // namespace

// ---- the stage-1 results of ms_argmax_static: values first, then indices.  A file-scope array: every GPU the
// library runs on holds its own copy (256 KB) at its own address until the process ends.
constexpr int STATIC_MAX_ROWS = 256, STATIC_MAX_CHUNKS = 128, STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[(size_t)STATIC_MAX_ROWS * STATIC_MAX_CHUNKS * (sizeof(float) + sizeof(int))];
// In host code `scratch` is only a handle for the symbol; what kernels may dereference is the address
// that hipGetSymbolAddress returns for the current device, looked up once per device and kept here.
static void* scratch_addr[STATIC_MAX_DEVICES] = {};
static std::mutex scratch_mutex;

// Device address of `scratch` on the current device (nullptr: the lookup failed or the device index is too large).
static void* scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_addr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    scratch_addr[dev] = p;
  }
  return scratch_addr[dev];
}

// out[r] = first index of the maximum of logits[r, :].  scratch_val / scratch_idx: [n_rows, n_chunks].
extern "C" int ms_argmax(const float* logits, long long ld, int n_rows, int vocab, float* scratch_val,
                         int* scratch_idx, int n_chunks, int* out, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (vocab <= 0 || ld < vocab || n_chunks <= 0 || n_rows > 65535) return MS_BAD_ARG;
  argmax_chunks_kernel<<<dim3(n_chunks, n_rows), dim3(256), 0, stream>>>(logits, (size_t)ld, vocab, n_chunks,
                                                                          scratch_val, scratch_idx);
  argmax_final_kernel<<<dim3(n_rows), dim3(MS_WAVE), 0, stream>>>(scratch_val, scratch_idx, n_chunks, out);
  return ms_launch_status();
}

extern "C" int ms_argmax_static_init() { return scratch_of_current_device() ? MS_OK : MS_LAUNCH_FAILED; }

extern "C" void ms_argmax_static_limits(int* max_rows, int* max_chunks) {
  if (max_rows) *max_rows = STATIC_MAX_ROWS;
  if (max_chunks) *max_chunks = STATIC_MAX_CHUNKS;
}

// ms_argmax with the stage-1 results in the library's own static device array instead of caller-provided
// buffers: nothing is allocated or freed here.  Nothing in the array has to start at zero (stage 2 reads only
// what stage 1 of the same call wrote, with this call's row stride), so the last call's contents are harmless.
extern "C" int ms_argmax_static(const float* logits, long long ld, int n_rows, int vocab, int n_chunks, int* out,
                                hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (vocab <= 0 || ld < vocab || n_chunks <= 0 || logits == nullptr || out == nullptr) return MS_BAD_ARG;
  if (n_rows > STATIC_MAX_ROWS || n_chunks > STATIC_MAX_CHUNKS) return MS_UNSUPPORTED;
  unsigned char* base = (unsigned char*)scratch_of_current_device();
  if (base == nullptr) return MS_LAUNCH_FAILED;
  float* val = (float*)base;
  int* idx = (int*)(base + (size_t)STATIC_MAX_ROWS * STATIC_MAX_CHUNKS * sizeof(float));
  argmax_chunks_kernel<<<dim3(n_chunks, n_rows), dim3(256), 0, stream>>>(logits, (size_t)ld, vocab, n_chunks, val, idx);
  argmax_final_kernel<<<dim3(n_rows), dim3(MS_WAVE), 0, stream>>>(val, idx, n_chunks, out);
  return ms_launch_status();
}

// Bytes of workspace ms_sample needs for n_rows rows (any contents: the first kernel makes it ready).
extern "C" long long ms_sample_workspace_bytes(int n_rows) { return (long long)sizeof(RowWork) * (n_rows > 0 ? n_rows : 0); }

// One token per row.  Rows with temperature <= 0 (or a null temperature) take the first maximum.  use_top_k /
// use_top_p: 0 if no row has a top_k in (0, vocab) / a top_p below 1 (their kernels are then left out; when in
// doubt pass 1).  workspace: ms_sample_workspace_bytes(n_rows) bytes, 8-byte aligned.
extern "C" int ms_sample(const float* logits, long long ld, int n_rows, int vocab, const float* temperature,
                         const int* top_k, const float* top_p, const unsigned long long* seeds,
                         const int* draw_index, int* out, void* workspace, int use_top_k, int use_top_p,
                         hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (vocab <= 0 || ld < vocab || n_rows > 65535) return MS_BAD_ARG;
  if (temperature == nullptr) return MS_BAD_ARG;      // all rows greedy: ms_argmax is the entry for that
  if (workspace == nullptr || ((uintptr_t)workspace % 8)) return MS_BAD_ARG;
  RowWork* work = (RowWork*)workspace;
  // About one block for every CU, but 8 to 24 to a row: every block of a row adds its histogram to the row's with
  // atomics on the same few bins, and reads the histogram of the level before whole, so more blocks to a row cost
  // more than they spread (8 rows of 151,936: 113 us with 64 blocks a row, 71 with 24; 64 rows: 141 us with 8,
  // 179 with 4, 182 with 16).
  int n_chunks = ms_compute_units() / n_rows;
  n_chunks = std::max(8, std::min(n_chunks, 24));
  n_chunks = std::max(1, std::min(std::min(n_chunks, MAX_CHUNKS), (vocab + 2047) / 2048));
  const dim3 grid(n_chunks, n_rows), block(THREADS);
  if (top_k == nullptr) use_top_k = 0;
  if (top_p == nullptr) use_top_p = 0;
  const int thresholds = use_top_k || use_top_p;
  sample_max_kernel<<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, work, n_chunks);
  if (thresholds) {
    sample_level_kernel<0><<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, top_k, top_p, work, n_chunks, 1);
    if (use_top_k) {
      sample_level_kernel<1><<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, top_k, top_p, work, n_chunks, 2);
      sample_level_kernel<1><<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, top_k, top_p, work, n_chunks, 3);
    }
    sample_level_kernel<2><<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, use_top_k ? top_k : nullptr, top_p, work, n_chunks, 2);
    if (use_top_p)
      sample_level_kernel<3><<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, top_k, top_p, work, n_chunks, 3);
  }
  sample_chunk_mass_kernel<<<grid, block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, use_top_p ? top_p : nullptr, work, n_chunks, thresholds);
  sample_draw_kernel<<<dim3(n_rows), block, 0, stream>>>(logits, (size_t)ld, vocab, temperature, seeds, draw_index, work, n_chunks, out);
  return ms_launch_status();
}
