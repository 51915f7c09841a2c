// Paged causal attention with grouped heads, any head size that is a multiple of 4 up to 256, for any mix
// of prompt portions and single decoded tokens.  One wave per (token, query head): scores, running
// maximum, exponentials, their sum and the weighted sum of values are all float.  It reads keys and
// values in place through the request's block table and never reads a key beyond the token's own
// position, so what a reused page still holds from an earlier request cannot reach the result.
// block_table int32 [rows, table_stride]; request r of the step has row table_rows[r] (null: row r).
// n_live_tokens (null: all): a device int; tokens from that index on belong to no request and are skipped.
// This is the attention of the 32-bit path and the any-shape fallback of the bfloat16 path.
#include "common.h"
#include "api.h"

namespace {

constexpr int WAVES = 4;
constexpr int MAX_D = 256;

template <typename T>
__global__ void __launch_bounds__(WAVES * MS_WAVE)
paged_attention_generic_kernel(const T* __restrict__ q, size_t q_stride, const T* __restrict__ k_pages,
                               const T* __restrict__ v_pages, const int* __restrict__ block_table, int table_stride,
                               const int* __restrict__ table_rows, const int* __restrict__ n_live_tokens,
                               const int* __restrict__ token_req, const int* __restrict__ positions,
                               T* __restrict__ out, size_t out_stride, int n_tokens, int nh, int nkv, int d,
                               int page_size, float scale, int window, int v_transposed) {
  __shared__ float qs[WAVES][MAX_D];
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const long long item = (long long)blockIdx.x * WAVES + wave;
  if (item >= (long long)n_tokens * nh) return;  // whole wave leaves; no block-wide barrier below
  const int n = (int)(item / nh), h = (int)(item - (long long)n * nh);
  if (n_live_tokens && n >= *n_live_tokens) return;   // a token that pads a captured batch belongs to no request
  const int kvh = h / (nh / nkv);
  const int pos = positions[n];
  const int req = token_req[n];
  const int* table = block_table + (size_t)(table_rows ? table_rows[req] : req) * table_stride;

  const T* qp = q + (size_t)n * q_stride + (size_t)h * d;
  for (int i = lane; i < d; i += MS_WAVE) qs[wave][i] = to_float(qp[i]) * scale;
  // the wave reads qs[wave] only after its own writes: a wave executes in lockstep, but make the
  // ordering explicit for the compiler
  __builtin_amdgcn_wave_barrier();

  int start = 0;
  if (window > 0 && pos - window + 1 > 0) start = pos - window + 1;

  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / MS_WAVE];
#pragma unroll
  for (int c = 0; c < MAX_D / MS_WAVE; ++c) acc[c] = 0.f;

  for (int base = start; base <= pos; base += MS_WAVE) {
    const int j = base + lane;
    const bool valid = j <= pos;
    int row = 0;
    float s = -INFINITY;
    if (valid) {
      const int page = table[j / page_size];
      row = (page * nkv + kvh) * page_size + (j % page_size);
      const T* kp = k_pages + (size_t)row * d;
      float dot = 0.f;
      for (int i = 0; i < d; i += 4) {
        dot = fmaf(qs[wave][i], to_float(kp[i]), dot);
        dot = fmaf(qs[wave][i + 1], to_float(kp[i + 1]), dot);
        dot = fmaf(qs[wave][i + 2], to_float(kp[i + 2]), dot);
        dot = fmaf(qs[wave][i + 3], to_float(kp[i + 3]), dot);
      }
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // 0 on the first chunk (m = -inf, m_new finite)
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < MAX_D / MS_WAVE; ++c) acc[c] *= corr;
    const int count = min(MS_WAVE, pos - base + 1);
    for (int jj = 0; jj < count; ++jj) {
      const float pj = __shfl(p, jj, MS_WAVE);
      const int vrow = __shfl(row, jj, MS_WAVE);
      // value pages are [page][kv head][slot][dim], or transposed [page][kv head][dim][slot]
      const T* vp = v_transposed ? v_pages + (size_t)(vrow / page_size) * page_size * d + vrow % page_size
                                 : v_pages + (size_t)vrow * d;
      const int vs = v_transposed ? page_size : 1;
#pragma unroll
      for (int c = 0; c < MAX_D / MS_WAVE; ++c) {
        const int i = lane + c * MS_WAVE;
        if (i < d) acc[c] = fmaf(pj, to_float(vp[(size_t)i * vs]), acc[c]);
      }
    }
  }
  T* op = out + (size_t)n * out_stride + (size_t)h * d;
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < MAX_D / MS_WAVE; ++c) {
    const int i = lane + c * MS_WAVE;
    if (i < d) op[i] = from_float<T>(acc[c] * inv);
  }
}

}  // namespace

extern "C" int ms_paged_attention_generic(const void* q, long long q_stride, const void* k_pages, const void* v_pages,
                                          const int* block_table, int table_stride, const int* table_rows,
                                          const int* n_live_tokens, const int* token_req,
                                          const int* positions, void* out, long long out_stride, int n_tokens,
                                          int num_heads, int num_kv_heads, int head_dim, int page_size,
                                          long long num_pages, float scale, int window, int v_transposed,
                                          int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || page_size <= 0 || table_stride <= 0)
    return MS_BAD_ARG;
  if (head_dim <= 0 || head_dim % 4 || head_dim > MAX_D) return MS_UNSUPPORTED;
  if (num_pages * num_kv_heads * page_size >= (1ll << 31)) return MS_UNSUPPORTED;  // row index is an int
  const long long items = (long long)n_tokens * num_heads;
  dim3 grid((unsigned)((items + WAVES - 1) / WAVES)), block(WAVES * MS_WAVE);
#define LAUNCH(T) paged_attention_generic_kernel<T><<<grid, block, 0, stream>>>((const T*)q, (size_t)q_stride, (const T*)k_pages, (const T*)v_pages, block_table, table_stride, table_rows, n_live_tokens, token_req, positions, (T*)out, (size_t)out_stride, n_tokens, num_heads, num_kv_heads, head_dim, page_size, scale, window, v_transposed)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
