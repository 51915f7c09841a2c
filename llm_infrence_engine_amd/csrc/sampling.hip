// Token choice from float logits, one block per row:
//   temperature <= 0 : the first index of the maximum
//   otherwise        : logits / temperature, then top-k (ties at the k-th value kept), then top-p
//                      (a token is dropped when the mass of the strictly larger ones reaches top_p; the
//                      largest is always kept), then a draw from the softmax of what is left.
// The k-th value and the top-p threshold are found by a bitwise search over an order-preserving integer
// image of the floats (32 passes over the row each), so no sort and no workspace are needed.  The
// uniform number of a draw is Philox4x32-10(seed, draw index): the same seed and index give the same token.
#include "common.h"
#include "api.h"
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

__global__ void __launch_bounds__(THREADS)
sample_kernel(const float* __restrict__ logits, size_t ld, int V, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const unsigned long long* __restrict__ seeds, const int* __restrict__ draw_index,
              int* __restrict__ out) {
  __shared__ MaxIdx red_mi[THREADS / MS_WAVE];
  __shared__ float red_f[16];
  __shared__ float scan[THREADS];
  __shared__ int chosen;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * ld;
  const float T = temperature ? temperature[r] : 0.f;
  const MaxIdx top = block_argmax(row, V, red_mi);
  if (!(T > 0.f)) {
    if (threadIdx.x == 0) out[r] = top.i;
    return;
  }
  const float inv_t = 1.0f / T;
  const float zmax = top.v * inv_t;

  // ---- top-k: key of the k-th largest scaled logit
  unsigned floor_key = 0;  // tokens with key >= floor_key are kept
  const int k = top_k ? top_k[r] : 0;
  if (k > 0 && k < V) {
    unsigned prefix = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = prefix | (1u << bit);
      float cnt = 0.f;
      for (int i = threadIdx.x; i < V; i += blockDim.x) cnt += (order_key(row[i] * inv_t) >= cand) ? 1.f : 0.f;
      if (block_sum(cnt, red_f) >= (float)k) prefix = cand;
    }
    floor_key = prefix;
  }

  // ---- top-p: the smallest key t such that the mass strictly above t is below top_p
  const float p = top_p ? top_p[r] : 1.f;
  if (p < 1.f) {
    float z = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float s = row[i] * inv_t;
      if (order_key(s) >= floor_key) z += expf(s - zmax);
    }
    const float total = block_sum(z, red_f);
    // predicate(t) = mass{key > t} < p * total is false below some key and true from it on; find that key
    unsigned lo = 0, hi = order_key(zmax);  // predicate(hi) holds: nothing lies above the maximum
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo) / 2;
      float above = 0.f;
      for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float s = row[i] * inv_t;
        const unsigned key = order_key(s);
        if (key > mid && key >= floor_key) above += expf(s - zmax);
      }
      if (block_sum(above, red_f) < p * total) hi = mid; else lo = mid + 1;
    }
    if (lo > floor_key) floor_key = lo;
  }

  // ---- draw: first index whose running mass exceeds u * total, scanning in index order
  const int per = (V + blockDim.x - 1) / blockDim.x;
  const int begin = min(V, (int)threadIdx.x * per), end = min(V, begin + per);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) {
    const float s = row[i] * inv_t;
    if (order_key(s) >= floor_key) mine += expf(s - zmax);
  }
  scan[threadIdx.x] = mine;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  if (threadIdx.x == 0) {  // serial prefix over 1024 partial sums: fixed order, fixed result
    float run = 0.f;
    for (int t = 0; t < (int)blockDim.x; ++t) { const float v = scan[t]; scan[t] = run; run += v; }
    red_f[0] = run;
  }
  __syncthreads();
  const float total = red_f[0];
  const float u = philox_uniform(seeds ? seeds[r] : 0ull, draw_index ? (unsigned)draw_index[r] : 0u);
  const float target = u * total;
  const float before = scan[threadIdx.x];
  if (mine > 0.f && before <= target && target < before + mine) {
    float run = before;
    int pick = -1, last = -1;
    for (int i = begin; i < end; ++i) {
      const float s = row[i] * inv_t;
      if (order_key(s) < floor_key) continue;
      run += expf(s - zmax);
      last = i;
      if (run > target) { pick = i; break; }
    }
    chosen = pick >= 0 ? pick : last;
  }
  __syncthreads();
  if (threadIdx.x == 0) out[r] = chosen >= 0 ? chosen : top.i;  // rounding left no owner: the maximum is always kept
}

// First maximum of a row in two stages, so that a few rows still use the whole chip: stage 1 finds the best
// of each of n_chunks slices of the row, stage 2 the best of those (larger value, then smaller index).
__global__ void __launch_bounds__(256)
argmax_chunks_kernel(const float* __restrict__ logits, size_t ld, int V, int n_chunks, float* __restrict__ val,
                     int* __restrict__ idx) {
  __shared__ MaxIdx red[4];
  const int r = blockIdx.y, c = blockIdx.x;
  const int len = (V + n_chunks - 1) / n_chunks;
  const int begin = c * len, end = min(V, begin + len);
  const float* row = logits + (size_t)r * ld;
  MaxIdx best = {-INFINITY, 0x7fffffff};
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) best = better(best, MaxIdx{row[i], i});
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

extern "C" int ms_sample(const float* logits, long long ld, int n_rows, int vocab, const float* temperature,
                         const int* top_k, const float* top_p, const unsigned long long* seeds,
                         const int* draw_index, int* out, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (vocab <= 0 || ld < vocab) return MS_BAD_ARG;
  sample_kernel<<<dim3(n_rows), dim3(THREADS), 0, stream>>>(logits, (size_t)ld, vocab, temperature, top_k, top_p,
                                                             seeds, draw_index, out);
  return ms_launch_status();
}
