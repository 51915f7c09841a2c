// Row-wise kernels: embedding gather, RMS norm (with the residual sum fused), gated activation,
// rotary position encoding fused with the write of keys and values into cache pages.
// The residual stream is float in every mode; sums of squares, the normalisation, rotation angles
// and the activation are computed in float.
#include "common.h"
#include "api.h"
#include <algorithm>

// ------------------------------------------------------------------------------------------------
// out[n, :] = float(table[ids[n], :])
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out, int H) {
  const int n = blockIdx.x;
  const T* row = table + (size_t)ids[n] * H;
  float* o = out + (size_t)n * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_float(row[i]);
}

extern "C" int ms_embed(const int* ids, const void* table, float* out, int n_tokens, int hidden, int dtype,
                        hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (hidden <= 0) return MS_BAD_ARG;
  dim3 grid(n_tokens), block(256);
  if (dtype == MS_F32) embed_kernel<float><<<grid, block, 0, stream>>>(ids, (const float*)table, out, hidden);
  else if (dtype == MS_BF16) embed_kernel<bf16><<<grid, block, 0, stream>>>(ids, (const bf16*)table, out, hidden);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Row r of the output is the norm of row rows[r] (or r) of x.  With `delta`, x[row] += delta[row]
// first (written back), which is the residual sum of the layer before; delta may come as n_partials
// partial sums [n_partials, N, H], added in order.
// y = w * (x * rsqrt(mean(x^2) + eps)), all in float, rounded once on store.
template <typename T, typename TD>
__global__ void rms_norm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int n_partials,
                                size_t partial_stride, const float* __restrict__ w,
                                const int* __restrict__ rows, T* __restrict__ out, int H, float eps, int write_back,
                                int staged) {
  __shared__ float red[16];
  extern __shared__ float buf[];  // H floats: the row after the residual sum (a row too wide for it is read twice)
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + (size_t)src * H;
  T* o = out + (size_t)r * H;
  float ss = 0.f;
  if (H % 4 == 0 && n_partials == 1 && staged) {  // four values at a time (rows start 16-byte aligned when H % 4 == 0)
    const TD* dr = delta ? delta + (size_t)src * H : nullptr;
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      float4 v = *reinterpret_cast<const float4*>(xr + i);
      if (dr) {
        v.x += to_float(dr[i]); v.y += to_float(dr[i + 1]); v.z += to_float(dr[i + 2]); v.w += to_float(dr[i + 3]);
        if (write_back) *reinterpret_cast<float4*>(xr + i) = v;
      }
      *reinterpret_cast<float4*>(buf + i) = v;
      ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      const float4 v = *reinterpret_cast<const float4*>(buf + i);
      const float4 g = *reinterpret_cast<const float4*>(w + i);
      o[i] = from_float<T>(g.x * (v.x * inv));
      o[i + 1] = from_float<T>(g.y * (v.y * inv));
      o[i + 2] = from_float<T>(g.z * (v.z * inv));
      o[i + 3] = from_float<T>(g.w * (v.w * inv));
    }
    return;
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = xr[i];
    if (delta) {
      for (int p = 0; p < n_partials; ++p) v += to_float(delta[p * partial_stride + (size_t)src * H + i]);
      if (write_back) xr[i] = v;
    }
    if (staged) buf[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  if (staged) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = from_float<T>(w[i] * (buf[i] * inv));
    return;
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) {   // the same sum again, in the same order: the same value
    float v = xr[i];                                     // (each thread reads back what it wrote itself)
    if (delta && !write_back)
      for (int p = 0; p < n_partials; ++p) v += to_float(delta[p * partial_stride + (size_t)src * H + i]);
    o[i] = from_float<T>(w[i] * (v * inv));
  }
}

extern "C" int ms_rms_norm(float* x, const void* delta, int delta_dtype, int n_partials, long long partial_stride,
                           const float* weight, const int* rows, void* out, int n_rows, int hidden, float eps,
                           int write_back, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (delta && (n_partials < 1 || partial_stride < 0)) return MS_BAD_ARG;
  if (hidden <= 0) return MS_BAD_ARG;
  dim3 grid(n_rows), block(hidden >= 1024 ? 256 : 128);
  // the row is staged in LDS while it fits what a launch may ask for without more ado (64 KB with the 64 bytes
  // of the reduction); a wider row is read from memory a second time instead
  const int staged = (size_t)hidden * sizeof(float) + 64 <= 65536 ? 1 : 0;
  size_t lds = staged ? (size_t)hidden * sizeof(float) : 0;
#define LAUNCH(T, TD) rms_norm_kernel<T, TD><<<grid, block, lds, stream>>>(x, (const TD*)delta, n_partials, (size_t)partial_stride, weight, rows, (T*)out, hidden, eps, write_back, staged)
  if (dtype == MS_F32) {
    if (delta && delta_dtype == MS_BF16) return MS_BAD_ARG;
    LAUNCH(float, float);
  } else if (dtype == MS_BF16) {
    if (delta && delta_dtype == MS_F32) LAUNCH(bf16, float);
    else LAUNCH(bf16, bf16);
  } else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// x[n, :] += delta[n, :]  (the residual sum alone, for arrangements that do not fuse it into a norm)
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ x, const TD* __restrict__ delta, size_t total) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) x[i] += to_float(delta[i]);
}

extern "C" int ms_residual_add(float* x, const void* delta, long long total, int dtype, hipStream_t stream) {
  if (total <= 0) return MS_OK;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 4096) blocks = 4096;
  if (dtype == MS_F32) residual_add_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)delta, (size_t)total);
  else if (dtype == MS_BF16) residual_add_kernel<bf16><<<blocks, 256, 0, stream>>>(x, (const bf16*)delta, (size_t)total);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// x[n, :] += bias[:]  (for a product that came without its bias)
template <typename T>
__global__ void bias_add_kernel(T* __restrict__ x, const float* __restrict__ bias, int width, size_t total) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) x[i] = from_float<T>(to_float(x[i]) + bias[i % width]);
}

extern "C" int ms_bias_add(void* x, const float* bias, int n_rows, int width, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (width <= 0) return MS_BAD_ARG;
  const size_t total = (size_t)n_rows * width;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 8192) blocks = 8192;
  if (dtype == MS_F32) bias_add_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, bias, width, total);
  else if (dtype == MS_BF16) bias_add_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)x, bias, width, total);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// out[n, i] = silu(gu[n, 2i]) * gu[n, 2i + 1],  silu(z) = z / (1 + exp(-z)): gate and up interleaved
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    // out[n, i] sits at idx and its (gate, up) pair at 2 * idx: rows are contiguous, so no division is needed
    const float g = to_float(gu[2 * idx]);
    const float u = to_float(gu[2 * idx + 1]);
    out[idx] = from_float<T>(g / (1.0f + expf(-g)) * u);
  }
}

// bfloat16, eight outputs per thread: two 16-byte loads, one 16-byte store
__global__ void silu_mul_bf16x8_kernel(const uint4* __restrict__ gu, uint4* __restrict__ out, size_t total8) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total8; idx += stride) {
    const uint4 a = gu[2 * idx], b = gu[2 * idx + 1];
    const unsigned in[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};  // each word: gate (low half), up (high half)
    unsigned short r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float g = __uint_as_float(in[i] << 16), u = __uint_as_float(in[i] & 0xffff0000u);
      const bf16 h = __float2bfloat16(g / (1.0f + expf(-g)) * u);
      r[i] = *reinterpret_cast<const unsigned short*>(&h);
    }
    uint4 o;
    o.x = r[0] | ((unsigned)r[1] << 16); o.y = r[2] | ((unsigned)r[3] << 16);
    o.z = r[4] | ((unsigned)r[5] << 16); o.w = r[6] | ((unsigned)r[7] << 16);
    out[idx] = o;
  }
}

extern "C" int ms_silu_mul(const void* gate_up, void* out, int n_tokens, int intermediate, int dtype,
                           hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (intermediate <= 0) return MS_BAD_ARG;
  const size_t total = (size_t)n_tokens * intermediate;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 8192) blocks = 8192;
  if (dtype == MS_F32) silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, intermediate, total);
  else if (dtype == MS_BF16 && total % 8 == 0 && (uintptr_t)gate_up % 16 == 0 && (uintptr_t)out % 16 == 0) {
    int b8 = (int)((total / 8 + 255) / 256);
    if (b8 > 16384) b8 = 16384;
    silu_mul_bf16x8_kernel<<<b8, 256, 0, stream>>>((const uint4*)gate_up, (uint4*)out, total / 8);
  }
  else if (dtype == MS_BF16) silu_mul_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out, intermediate, total);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// One block per token.  qkv[n] = [q heads | k heads | v heads], head_dim values each.
// The first rot_dim values of every q and k head are rotated with half-split pairing (j, j + rot_dim/2):
//   x1' = x1 cos - x2 sin,  x2' = x2 cos + x1 sin,  angle = float(position) * inv_freq[j]
// With `bias` ([(nh + 2 nkv) d] float) it is added to q, k and v first, for a projection that came without it.
// q is rotated in place.  With pages given, the rotated k and v go to
// pages[slot / page_size][kv head][slot % page_size][:] for slot = slot_mapping[n] (slot < 0: not stored;
// with v_transposed the value goes to v_pages[page][kv head][:][slot % page_size]);
// k is also rotated in place so that a caller without pages sees it.
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, const int* __restrict__ slot_mapping,
                                  T* __restrict__ k_pages, T* __restrict__ v_pages, int nh, int nkv, int d,
                                  int rot_dim, int page_size, int v_transposed) {
  const int n = blockIdx.x;
  T* row = qkv + (size_t)n * (nh + 2 * nkv) * d;
  const float pos = (float)positions[n];
  const int half = rot_dim / 2;
  long long slot = -1;
  if (k_pages) slot = slot_mapping[n];
  const long long page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? (int)(slot % page_size) : 0;

  // rotate q and k heads: work item = (head, j)
  const int n_rot_heads = nh + nkv;
  for (int w = threadIdx.x; w < n_rot_heads * half; w += blockDim.x) {
    const int h = w / half, j = w - h * half;
    T* x = row + (size_t)h * d;
    float s, c;
    sincosf(pos * inv_freq[j], &s, &c);
    float x1 = to_float(x[j]), x2 = to_float(x[j + half]);
    if (bias) { x1 += bias[h * d + j]; x2 += bias[h * d + j + half]; }
    x[j] = from_float<T>(x1 * c - x2 * s);
    x[j + half] = from_float<T>(x2 * c + x1 * s);
  }
  if (bias) {  // what is not rotated still gets its bias: the tails of q and k heads beyond rot_dim, and v
    const int tail = d - rot_dim;
    for (int w = threadIdx.x; w < n_rot_heads * tail; w += blockDim.x) {
      const int idx = (w / tail) * d + rot_dim + w % tail;
      row[idx] = from_float<T>(to_float(row[idx]) + bias[idx]);
    }
    for (int w = threadIdx.x; w < nkv * d; w += blockDim.x) {
      const int idx = (nh + nkv) * d + w;
      row[idx] = from_float<T>(to_float(row[idx]) + bias[idx]);
    }
  }
  if (slot < 0) return;
  __syncthreads();
  // copy k and v heads into the page
  const T* k = row + (size_t)nh * d;
  const T* v = k + (size_t)nkv * d;
  for (int w = threadIdx.x; w < nkv * d; w += blockDim.x) {
    const int h = w / d, i = w - h * d;
    const size_t dst = (((size_t)page * nkv + h) * page_size + off) * d + i;
    k_pages[dst] = k[w];
    // value pages may be stored transposed, [page][kv head][dim][page_size], for the matrix-core attention
    v_pages[v_transposed ? (((size_t)page * nkv + h) * d + i) * page_size + off : dst] = v[w];
  }
}

// The same work 16 bytes at a time, four tokens to a block (64 threads each): the angles of a token are worked
// out once and shared by all its heads, a thread rotates VEC pairs of one head and, for a key head, puts them
// into the page from its registers; so one barrier (after the angles) is all.  Needs rot_dim / 2 and head_dim
// to be multiples of VEC = 16 / sizeof(T) and rot_dim / 2 <= ROPE_MAX_HALF.
constexpr int ROPE_TOKENS = 4, ROPE_GROUP = 64, ROPE_MAX_HALF = 128;

template <typename T, int VEC>
struct alignas(16) Packet { T v[VEC]; };

template <typename T, int VEC>
__global__ void __launch_bounds__(ROPE_TOKENS * ROPE_GROUP)
rope_store_vec_kernel(T* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ positions,
                      const float* __restrict__ inv_freq, const int* __restrict__ slot_mapping,
                      T* __restrict__ k_pages, T* __restrict__ v_pages, int n_tokens, int nh, int nkv, int d,
                      int rot_dim, int page_size, int v_transposed) {
  typedef Packet<T, VEC> Vec;
  typedef Packet<float, VEC> FVec;
  __shared__ float sm_cos[ROPE_TOKENS][ROPE_MAX_HALF], sm_sin[ROPE_TOKENS][ROPE_MAX_HALF];
  const int tg = threadIdx.x / ROPE_GROUP, tl = threadIdx.x % ROPE_GROUP;
  const int n = blockIdx.x * ROPE_TOKENS + tg;
  const bool live = n < n_tokens;
  const int half = rot_dim / 2;
  if (live && half > 0) {
    const float pos = (float)positions[n];
    // bfloat16 results: the short routine that the fused decode kernel uses too (error 2e-7), so a key gets the
    // same rotation whether a portion or a decode step stores it
    for (int j = tl; j < half; j += ROPE_GROUP) {
      if (sizeof(T) == 2) ms_sincos_rot(pos * inv_freq[j], &sm_sin[tg][j], &sm_cos[tg][j]);
      else sincosf(pos * inv_freq[j], &sm_sin[tg][j], &sm_cos[tg][j]);
    }
  }
  __syncthreads();
  if (!live) return;
  T* row = qkv + (size_t)n * (nh + 2 * nkv) * d;
  long long slot = -1;
  if (k_pages) slot = slot_mapping[n];
  const long long page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? (int)(slot % page_size) : 0;

  // rotated pairs of q and k heads: work item = (head, VEC consecutive j)
  const int per_head = half / VEC;
  for (int w = tl; w < (nh + nkv) * per_head; w += ROPE_GROUP) {
    const int h = w / per_head, j = (w - h * per_head) * VEC;
    T* x = row + (size_t)h * d;
    Vec a = *reinterpret_cast<const Vec*>(x + j), b = *reinterpret_cast<const Vec*>(x + j + half);
    FVec ba = {}, bb = {};
    if (bias) {
      ba = *reinterpret_cast<const FVec*>(bias + h * d + j);
      bb = *reinterpret_cast<const FVec*>(bias + h * d + j + half);
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float x1 = to_float(a.v[i]) + ba.v[i], x2 = to_float(b.v[i]) + bb.v[i];
      const float c = sm_cos[tg][j + i], sn = sm_sin[tg][j + i];
      a.v[i] = from_float<T>(x1 * c - x2 * sn);
      b.v[i] = from_float<T>(x2 * c + x1 * sn);
    }
    *reinterpret_cast<Vec*>(x + j) = a;
    *reinterpret_cast<Vec*>(x + j + half) = b;
    if (h >= nh && slot >= 0) {
      T* dst = k_pages + (((size_t)page * nkv + (h - nh)) * page_size + off) * d;
      *reinterpret_cast<Vec*>(dst + j) = a;
      *reinterpret_cast<Vec*>(dst + j + half) = b;
    }
  }
  // what is not rotated: the tails of q and k heads beyond rot_dim (bias, and the store of k), and v
  const int tail_vecs = (d - rot_dim) / VEC;
  for (int w = tl; w < (nh + nkv) * tail_vecs; w += ROPE_GROUP) {
    const int h = w / tail_vecs, i0 = rot_dim + (w - h * tail_vecs) * VEC;
    T* x = row + (size_t)h * d + i0;
    Vec a = *reinterpret_cast<const Vec*>(x);
    if (bias) {
      const FVec bv = *reinterpret_cast<const FVec*>(bias + h * d + i0);
#pragma unroll
      for (int i = 0; i < VEC; ++i) a.v[i] = from_float<T>(to_float(a.v[i]) + bv.v[i]);
      *reinterpret_cast<Vec*>(x) = a;
    }
    if (h >= nh && slot >= 0)
      *reinterpret_cast<Vec*>(k_pages + (((size_t)page * nkv + (h - nh)) * page_size + off) * d + i0) = a;
  }
  const int v_vecs = d / VEC;
  for (int w = tl; w < nkv * v_vecs; w += ROPE_GROUP) {
    const int h = w / v_vecs, i0 = (w - h * v_vecs) * VEC;
    T* x = row + (size_t)(nh + nkv + h) * d + i0;
    Vec a = *reinterpret_cast<const Vec*>(x);
    if (bias) {
      const FVec bv = *reinterpret_cast<const FVec*>(bias + (nh + nkv + h) * d + i0);
#pragma unroll
      for (int i = 0; i < VEC; ++i) a.v[i] = from_float<T>(to_float(a.v[i]) + bv.v[i]);
      *reinterpret_cast<Vec*>(x) = a;
    }
    if (slot < 0) continue;
    if (v_transposed) {   // [page][kv head][dim][page_size]: one element to each dim's row
      T* dst = v_pages + (((size_t)page * nkv + h) * d + i0) * page_size + off;
#pragma unroll
      for (int i = 0; i < VEC; ++i) dst[(size_t)i * page_size] = a.v[i];
    } else {
      *reinterpret_cast<Vec*>(v_pages + (((size_t)page * nkv + h) * page_size + off) * d + i0) = a;
    }
  }
}

// table[n][j] = (cos, sin) of float(positions[n]) * inv_freq[j], by the short routine that the rotation kernels for
// bfloat16 use: worked out once a step, the same for every layer.
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float2* __restrict__ table, int n_tokens, int half) {
  const int id = blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= n_tokens * half) return;
  const int n = id / half, j = id - n * half;
  float sn, cs;
  ms_sincos_rot((float)positions[n] * inv_freq[j], &sn, &cs);
  table[id] = make_float2(cs, sn);
}

extern "C" int ms_rope_table(const int* positions, const float* inv_freq, float* table, int n_tokens, int half,
                             hipStream_t stream) {
  if (n_tokens <= 0 || half <= 0) return MS_OK;
  if (!positions || !inv_freq || !table || (uintptr_t)table % 8) return MS_BAD_ARG;
  const long long total = (long long)n_tokens * half;
  if (total > 0x7fffffffLL) return MS_UNSUPPORTED;
  rope_table_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(positions, inv_freq, (float2*)table,
                                                                                   n_tokens, half);
  return ms_launch_status();
}

extern "C" int ms_rope_store(void* qkv, const float* bias, const int* positions, const float* inv_freq, const int* slot_mapping,
                             void* k_pages, void* v_pages, int n_tokens, int num_heads, int num_kv_heads,
                             int head_dim, int rot_dim, int page_size, int v_transposed, int dtype,
                             hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (num_heads < 0 || num_kv_heads < 0 || head_dim <= 0 || rot_dim < 0 || rot_dim > head_dim || (rot_dim & 1))
    return MS_BAD_ARG;
  if ((k_pages == nullptr) != (v_pages == nullptr)) return MS_BAD_ARG;
  if (k_pages && (page_size <= 0 || slot_mapping == nullptr)) return MS_BAD_ARG;
  if (rot_dim > 0 && (positions == nullptr || inv_freq == nullptr)) return MS_BAD_ARG;
  {  // 16 bytes at a time where the sizes allow
    const int vec = dtype == MS_BF16 ? 8 : 4;
    const bool aligned = ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)k_pages % 16) == 0 &&
                         ((uintptr_t)v_pages % 16) == 0 && ((uintptr_t)bias % 16) == 0;
    if ((dtype == MS_BF16 || dtype == MS_F32) && aligned && head_dim % vec == 0 && (rot_dim / 2) % vec == 0 &&
        rot_dim / 2 <= ROPE_MAX_HALF) {
      dim3 vgrid((n_tokens + ROPE_TOKENS - 1) / ROPE_TOKENS), vblock(ROPE_TOKENS * ROPE_GROUP);
#define LAUNCH_VEC(T, VEC) rope_store_vec_kernel<T, VEC><<<vgrid, vblock, 0, stream>>>((T*)qkv, bias, positions, inv_freq, slot_mapping, (T*)k_pages, (T*)v_pages, n_tokens, num_heads, num_kv_heads, head_dim, rot_dim, page_size, v_transposed)
      if (dtype == MS_BF16) LAUNCH_VEC(bf16, 8); else LAUNCH_VEC(float, 4);
#undef LAUNCH_VEC
      return ms_launch_status();
    }
  }
  dim3 grid(n_tokens), block(256);
#define LAUNCH(T) rope_store_kernel<T><<<grid, block, 0, stream>>>((T*)qkv, bias, positions, inv_freq, slot_mapping, (T*)k_pages, (T*)v_pages, num_heads, num_kv_heads, head_dim, rot_dim, page_size, v_transposed)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Between two decode steps that run back to back on the device: every live request (row < *n_live) moves one
// position on, takes the token the step before chose as its input, counts its draws on (draw_index, may be
// null) and gets the slots its new key and value go to, from its block tables.  One thread per row; up to MS_MAX_GROUPS cache groups.
struct AdvanceArgs {
  const int* prev_tokens;
  int* token_ids;
  int* positions;
  int* context_lens;
  const int* n_live;
  const int* table_rows;
  int* draw_index;
  const int* tables[MS_MAX_GROUPS];
  int* slots[MS_MAX_GROUPS];
  int n_groups, table_stride, page_size, n_rows;
};

__global__ void decode_advance_kernel(AdvanceArgs a) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= a.n_rows || r >= *a.n_live) return;
  const int pos = a.positions[r] + 1;
  a.positions[r] = pos;
  a.context_lens[r] = pos + 1;
  a.token_ids[r] = a.prev_tokens[r];
  if (a.draw_index) a.draw_index[r] += 1;     // the next draw of a request that samples is its next
  const size_t row = a.table_rows ? a.table_rows[r] : r;
  for (int g = 0; g < a.n_groups; ++g)
    a.slots[g][r] = a.tables[g][row * a.table_stride + pos / a.page_size] * a.page_size + pos % a.page_size;
}

extern "C" int ms_max_cache_groups() { return MS_MAX_GROUPS; }

extern "C" int ms_decode_advance(const int* prev_tokens, int* token_ids, int* positions, int* context_lens,
                                 const int* n_live, const int* table_rows, int* draw_index,
                                 const int* const* tables, int* const* slots, int n_groups, int table_stride,
                                 int page_size, int n_rows, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (n_groups < 0 || n_groups > MS_MAX_GROUPS || table_stride <= 0 || page_size <= 0) return MS_BAD_ARG;
  AdvanceArgs a;
  a.prev_tokens = prev_tokens; a.token_ids = token_ids; a.positions = positions; a.context_lens = context_lens;
  a.n_live = n_live; a.table_rows = table_rows; a.draw_index = draw_index; a.n_groups = n_groups; a.table_stride = table_stride;
  a.page_size = page_size; a.n_rows = n_rows;
  for (int g = 0; g < MS_MAX_GROUPS; ++g) { a.tables[g] = g < n_groups ? tables[g] : nullptr; a.slots[g] = g < n_groups ? slots[g] : nullptr; }
  decode_advance_kernel<<<dim3((n_rows + 63) / 64), dim3(64), 0, stream>>>(a);
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// The block tables live on the device for as long as the cache does; a step brings only the entries that
// changed since the last one (pages granted, pages a window has passed, rows given back).
struct TableUpdateArgs {
  int* tables[MS_MAX_GROUPS];
  const int* index[MS_MAX_GROUPS];
  const int* value[MS_MAX_GROUPS];
  const int* counts;
  long long table_elems;
};

__global__ void table_update_kernel(TableUpdateArgs a) {
  const int g = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= a.counts[g]) return;
  const long long at = a.index[g][i];
  if (at >= 0 && at < a.table_elems) a.tables[g][at] = a.value[g][i];
}

extern "C" int ms_table_update(int* const* tables, const int* const* index, const int* const* value,
                               const int* counts, int n_groups, int max_updates, long long table_elems,
                               hipStream_t stream) {
  if (n_groups <= 0 || max_updates <= 0) return MS_OK;
  if (n_groups > MS_MAX_GROUPS || table_elems <= 0 || counts == nullptr) return MS_BAD_ARG;
  TableUpdateArgs a;
  for (int g = 0; g < MS_MAX_GROUPS; ++g) {
    a.tables[g] = g < n_groups ? tables[g] : nullptr;
    a.index[g] = g < n_groups ? index[g] : nullptr;
    a.value[g] = g < n_groups ? value[g] : nullptr;
  }
  a.counts = counts; a.table_elems = table_elems;
  table_update_kernel<<<dim3((max_updates + 255) / 256, n_groups), dim3(256), 0, stream>>>(a);
  return ms_launch_status();
}

// Rows of a tensor set to zero: the state slots of requests whose first portion runs in this step.
__global__ void zero_rows_kernel(unsigned* __restrict__ base, size_t row_words, const int* __restrict__ rows,
                                 const int* __restrict__ count) {
  const int i = blockIdx.y;
  if (count && i >= *count) return;
  unsigned* p = base + (size_t)rows[i] * row_words;
  for (size_t w = (size_t)blockIdx.x * blockDim.x + threadIdx.x; w < row_words; w += (size_t)gridDim.x * blockDim.x)
    p[w] = 0u;
}

extern "C" int ms_zero_rows(void* base, long long row_bytes, const int* rows, const int* count, int n_rows,
                            hipStream_t stream) {
  if (n_rows <= 0 || row_bytes <= 0) return MS_OK;
  if (row_bytes % 4 || ((uintptr_t)base % 4) || n_rows > 65535) return MS_BAD_ARG;
  const size_t words = (size_t)row_bytes / 4;
  const unsigned bx = (unsigned)std::min<size_t>((words + 255) / 256, 64);
  zero_rows_kernel<<<dim3(bx, n_rows), dim3(256), 0, stream>>>((unsigned*)base, words, rows, count);
  return ms_launch_status();
}

// ------------------------------------------------------------------------------------------------
// A plain streaming read of `bytes` (a multiple of 16, 16-byte aligned), for measuring what bandwidth this
// device gives a kernel that does nothing else: every wave asks for 1 KB at a time, four requests in flight,
// the blocks dealt contiguous shares.  The exclusive-or of everything read goes to sink[block] so that the
// loads cannot be dropped.
__global__ void __launch_bounds__(1024)
read_probe_kernel(const uint4* __restrict__ base, size_t n16, unsigned* __restrict__ sink) {
  const size_t per_block = (n16 + gridDim.x - 1) / gridDim.x;
  const size_t begin = (size_t)blockIdx.x * per_block, end = begin + per_block < n16 ? begin + per_block : n16;
  uint4 acc = {0u, 0u, 0u, 0u};
  for (size_t i = begin + threadIdx.x; i < end; i += (size_t)4 * blockDim.x) {
    uint4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const size_t k = i + (size_t)j * blockDim.x;
      v[j] = k < end ? base[k] : uint4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) { acc.x ^= v[j].x; acc.y ^= v[j].y; acc.z ^= v[j].z; acc.w ^= v[j].w; }
  }
  unsigned r = acc.x ^ acc.y ^ acc.z ^ acc.w;
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) r ^= __shfl_xor(r, o, MS_WAVE);
  if ((threadIdx.x & (MS_WAVE - 1)) == 0) atomicXor(&sink[blockIdx.x], r);
}

// sink: unsigned [n_blocks], n_blocks = 8 blocks per compute unit (ms_read_probe_blocks).
extern "C" int ms_read_probe_blocks() { return 8 * ms_compute_units(); }

extern "C" int ms_read_probe(const void* base, long long bytes, unsigned* sink, hipStream_t stream) {
  if (bytes <= 0) return MS_OK;
  if (bytes % 16 || (uintptr_t)base % 16) return MS_BAD_ARG;
  read_probe_kernel<<<dim3(ms_read_probe_blocks()), dim3(1024), 0, stream>>>((const uint4*)base, (size_t)bytes / 16, sink);
  return ms_launch_status();
}
