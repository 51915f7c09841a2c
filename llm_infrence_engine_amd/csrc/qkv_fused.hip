// One kernel for the front of an attention layer on few rows (a decode step's tokens):
//   RMS norm (folded in as in gemm_skinny.hip) -> q, k, v projection with bias -> rotary encoding of q and k
//   (half-split pairing, float angles) -> q to its buffer, k and v straight into their cache pages.
// A block owns two 16-row tiles of the packed [q heads | k heads | v heads] weight that lie half a head
// apart, so a lane ends up holding both members (j, j + d/2) of four rotary pairs of one token and can
// rotate them in registers; or, for few tokens, one tile of 8 + 8 such rows (see PAIR8).  Requires the rotary
// dimension to be the whole head and d/2 a multiple of 16.
#include "common.h"
#include "api.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// PAIR8: a block owns one 16-row tile made of 8 rows from the lower half of a head and the 8 rows half a head
// above them, so a rotary pair (j, j + d/2) lies in two lanes of one token, 32 lanes apart, and is rotated after
// one exchange between them.  Twice as many blocks as with two whole tiles, each streaming half the weights: for
// few tokens, where a block's time is what its CU can draw and there are fewer blocks than CUs.
template <int MT, int WAVES, bool PAIR8>
__global__ void __launch_bounds__(WAVES * MS_WAVE)
qkv_rope_store_kernel(const float* __restrict__ X, size_t ldx, const float* __restrict__ norm_w, float eps,
                      const bf16* __restrict__ W, const float* __restrict__ bias, const int* __restrict__ positions,
                      const float* __restrict__ inv_freq, const int* __restrict__ slot_mapping,
                      bf16* __restrict__ q_out, bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int M, int K,
                      int nh, int nkv, int d, int page_size, int v_transposed) {
  constexpr int NACC = PAIR8 ? 1 : 2;
  __shared__ f32x4 red[WAVES - 1][NACC][MT][MS_WAVE];
  __shared__ float red_ss[WAVES][MT][16];
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int col = lane & 15, kq = lane >> 4;
  const int m0 = blockIdx.z * 16 * MT;                    // token groups beyond MT per block: further blocks along z
  const int head = blockIdx.y;                           // 0..nh-1: q, then nkv k heads, then nkv v heads
  const int half = d / 2;
  const int j0 = blockIdx.x * (PAIR8 ? 8 : 16);           // first feature of the block's lower rows within the head
  const int total_steps = (K + 31) / 32;

  // PAIR8: row `col` of the tile is lower feature j0 + col (col < 8) or upper feature j0 + col - 8 + d/2
  const int row_lo = PAIR8 ? (col < 8 ? j0 + col : j0 + col - 8 + half) : j0 + col;
  const bf16* w_lo = W + ((size_t)head * d + row_lo) * K + kq * 8;
  const bf16* w_hi = w_lo + (size_t)half * K;            // not PAIR8: the tile half a head above
  size_t xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xrow[t] = (size_t)min(m0 + t * 16 + col, M - 1) * ldx + kq * 8;

  // what the epilogue will need from memory is asked for now, so that it arrives under the main loop.
  // A lane ends up with four features of one token: not PAIR8, j0 + kq*4 + r of the lower tile and the same of the
  // upper; PAIR8, lanes kq = 0, 1 the lower features j0 + kq*4 + r, lanes kq = 2, 3 their partners half a head up.
  const int jl = PAIR8 ? j0 + (kq & 1) * 4 : j0 + kq * 4;   // the lower feature of this lane's first pair
  const bool upper = PAIR8 && kq >= 2;
  float b_lo[4], b_hi[4], freq[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    b_lo[r] = bias ? bias[head * d + jl + r + (upper ? half : 0)] : 0.f;
    b_hi[r] = (bias && !PAIR8) ? bias[head * d + jl + half + r] : 0.f;
    freq[r] = head < nh + nkv ? inv_freq[jl + r] : 0.f;
  }
  int pos_m[MT], slot_m[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = min(m0 + t * 16 + col, M - 1);
    pos_m[t] = positions[m];
    slot_m[t] = slot_mapping[m];
  }

  f32x4 lo[MT], hi[MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) { lo[t] = hi[t] = f32x4{0.f, 0.f, 0.f, 0.f}; ss[t] = 0.f; }

  for (int s = wave; s < total_steps; s += WAVES) {
    const int k = s * 32;
    const bool in = k + kq * 8 < K;
    bf16x8 wl = {0, 0, 0, 0, 0, 0, 0, 0}, wh = {0, 0, 0, 0, 0, 0, 0, 0};
    f32x4 nw0 = {0.f, 0.f, 0.f, 0.f}, nw1 = {0.f, 0.f, 0.f, 0.f};
    if (in) {
      wl = *reinterpret_cast<const bf16x8*>(w_lo + k);
      if (!PAIR8) wh = *reinterpret_cast<const bf16x8*>(w_hi + k);
      nw0 = *reinterpret_cast<const f32x4*>(norm_w + k + kq * 8);
      nw1 = *reinterpret_cast<const f32x4*>(norm_w + k + kq * 8 + 4);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      bf16x8 av = {0, 0, 0, 0, 0, 0, 0, 0};
      if (in) {
        const f32x4 x0 = *reinterpret_cast<const f32x4*>(X + xrow[t] + k);
        const f32x4 x1 = *reinterpret_cast<const f32x4*>(X + xrow[t] + k + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ss[t] = fmaf(x0[i], x0[i], ss[t]);
          ss[t] = fmaf(x1[i], x1[i], ss[t]);
          av[i] = (__bf16)(x0[i] * nw0[i]);
          av[4 + i] = (__bf16)(x1[i] * nw1[i]);
        }
      }
      lo[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wl, av, lo[t], 0, 0, 0);
      if (!PAIR8) hi[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wh, av, hi[t], 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] += __shfl_xor(ss[t], 16, MS_WAVE);
    ss[t] += __shfl_xor(ss[t], 32, MS_WAVE);
    if (kq == 0) red_ss[wave][t][col] = ss[t];
    const int owner = t % WAVES;  // token group t is finished by wave t; the others leave their share in LDS
    if (wave != owner) {
      red[wave < owner ? wave : wave - 1][0][t][lane] = lo[t];
      if (!PAIR8) red[wave < owner ? wave : wave - 1][NACC - 1][t][lane] = hi[t];
    }
  }
  __syncthreads();

#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = m0 + t * 16 + col;
    const int owner = t % WAVES;
    if (wave != owner) continue;       // the same for the whole wave (the exchange below needs all its lanes)
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += red_ss[w][t][col];
    const float inv = 1.0f / sqrtf(total / (float)K + eps);
    float a[4], b[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float va = 0.f, vb = 0.f;
      for (int w = 0; w < WAVES; ++w) {  // in wave order
        va += w == owner ? lo[t][r] : red[w < owner ? w : w - 1][0][t][lane][r];
        if (!PAIR8) vb += w == owner ? hi[t][r] : red[w < owner ? w : w - 1][NACC - 1][t][lane][r];
      }
      a[r] = va * inv + b_lo[r];
      b[r] = vb * inv + b_hi[r];
    }
    if (PAIR8) {
      // the partner of this lane's feature sits 32 lanes away: a lower lane takes (x1, x2) = (own, partner), an
      // upper lane (partner, own)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float other = __shfl_xor(a[r], 32, MS_WAVE);
        b[r] = upper ? a[r] : other;
        a[r] = upper ? other : a[r];
      }
    }
    if (head < nh + nkv) {  // q and k heads turn by position * inv_freq[j]
      const float pos = (float)pos_m[t];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float sn, cs;
        ms_sincos_rot(pos * freq[r], &sn, &cs);
        const float x1 = a[r], x2 = b[r];
        a[r] = x1 * cs - x2 * sn;
        b[r] = x2 * cs + x1 * sn;
      }
    }
    if (m >= M) continue;
    // what this lane stores: not PAIR8 both members (a at j, b at j + d/2); PAIR8 its own member only
    const int j = jl;
    const int row_a = head * d + j;
    bf16x4 pa, pb;
#pragma unroll
    for (int r = 0; r < 4; ++r) { pa[r] = (__bf16)a[r]; pb[r] = (__bf16)b[r]; }
    const bool store_a = !PAIR8 || !upper, store_b = !PAIR8 || upper;
    if (head < nh) {
      bf16* qp = q_out + (size_t)m * nh * d + row_a;
      if (store_a) *reinterpret_cast<bf16x4*>(qp) = pa;
      if (store_b) *reinterpret_cast<bf16x4*>(qp + half) = pb;
      continue;
    }
    const long long slot = slot_m[t];
    if (slot < 0) continue;
    // a page of a power of two (the usual case) needs no division
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    const long long page = pow2 ? slot >> (31 - __builtin_clz(page_size)) : slot / page_size;
    const int off = pow2 ? (int)(slot & (page_size - 1)) : (int)(slot % page_size);
    if (head < nh + nkv) {
      bf16* kp = k_pages + (((size_t)page * nkv + (head - nh)) * page_size + off) * d + j;
      if (store_a) *reinterpret_cast<bf16x4*>(kp) = pa;
      if (store_b) *reinterpret_cast<bf16x4*>(kp + half) = pb;
    } else if (v_transposed) {
      bf16* vp = v_pages + (((size_t)page * nkv + (head - nh - nkv)) * d + j) * page_size + off;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (store_a) vp[(size_t)r * page_size] = __float2bfloat16(a[r]);
        if (store_b) vp[(size_t)(half + r) * page_size] = __float2bfloat16(b[r]);
      }
    } else {
      bf16* vp = v_pages + (((size_t)page * nkv + (head - nh - nkv)) * page_size + off) * d + j;
      if (store_a) *reinterpret_cast<bf16x4*>(vp) = pa;
      if (store_b) *reinterpret_cast<bf16x4*>(vp + half) = pb;
    }
  }
}

int g_qkv_pair8 = -1;   // measurements: 0 / 1 force whole tiles / tiles of 8 + 8 rows, -1 leaves the choice

template <int MT>
int launch(const float* X, size_t ldx, const float* norm_w, float eps, const bf16* W, const float* bias,
           const int* positions, const float* inv_freq, const int* slot_mapping, bf16* q_out, bf16* k_pages,
           bf16* v_pages, int M, int K, int nh, int nkv, int d, int page_size, int v_transposed, hipStream_t stream) {
  const int steps = (K + 31) / 32;
  const int token_groups = (M + 16 * MT - 1) / (16 * MT);
  // Tiles of 8 + 8 rows (twice the blocks, half the weights each) while there are no more of them than CUs: a block's
  // time is what its CU can draw.  With more blocks than CUs every block reading all the activations costs
  // more than the shorter stream of weights saves.
  const int pair_blocks = (nh + 2 * nkv) * (d / 16) * token_groups;
  const bool pair8 = g_qkv_pair8 >= 0 ? g_qkv_pair8 != 0 : pair_blocks <= ms_compute_units();
  const int blocks = pair8 ? pair_blocks : pair_blocks / 2;
  // LDS holds (waves - 1) * 2 * MT KB.  (Measured at the 0.5B and 7B shapes: 8 waves are 0.4 to 1 us faster than
  // 16; tiles of 8 or 4 rows on more CUs are slower, by up to 2x, because every block reads all activations.)
  int waves = 4;
  while (waves < 8 && blocks * waves < 1024 && steps >= waves * 2) waves *= 2;
#define GO(WV, P8) qkv_rope_store_kernel<MT, WV, P8><<<dim3(d / (P8 ? 16 : 32), nh + 2 * nkv, token_groups), dim3(WV * MS_WAVE), 0, stream>>>(X, ldx, norm_w, eps, W, bias, positions, inv_freq, slot_mapping, q_out, k_pages, v_pages, M, K, nh, nkv, d, page_size, v_transposed)
  if (pair8) { if (waves == 4) GO(4, true); else GO(8, true); }
  else { if (waves == 4) GO(4, false); else GO(8, false); }
#undef GO
  return ms_launch_status();
}

}  // namespace

extern "C" void ms_qkv_rope_store_force(int pair8) { g_qkv_pair8 = pair8; }

// x float [M, K] (M <= 64), W bfloat16 [(nh + 2 nkv) d, K] packed q | k | v, bias float or null,
// q_out bfloat16 [M, nh d], pages bfloat16 as in ms_rope_store, inv_freq float [d / 2].
extern "C" int ms_qkv_rope_store(const float* x, long long ldx, const float* norm_w, float eps, const void* W,
                                 const float* bias, const int* positions, const float* inv_freq,
                                 const int* slot_mapping, void* q_out, void* k_pages, void* v_pages, int M, int K,
                                 int num_heads, int num_kv_heads, int head_dim, int page_size, int v_transposed,
                                 hipStream_t stream) {
  if (M <= 0) return MS_OK;
  if (M > 64 || head_dim % 32 || head_dim <= 0) return MS_UNSUPPORTED;
  if (K <= 0 || K % 8 || ldx % 4 || ldx < K) return MS_UNSUPPORTED;
  if (((uintptr_t)x | (uintptr_t)W | (uintptr_t)norm_w | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages) % 16)
    return MS_UNSUPPORTED;
  if (num_heads <= 0 || num_kv_heads <= 0 || page_size <= 0 || !positions || !inv_freq || !slot_mapping || !q_out ||
      !k_pages || !v_pages)
    return MS_BAD_ARG;
#define GO(MT) return launch<MT>(x, ldx, norm_w, eps, (const bf16*)W, bias, positions, inv_freq, slot_mapping, (bf16*)q_out, (bf16*)k_pages, (bf16*)v_pages, M, K, num_heads, num_kv_heads, head_dim, page_size, v_transposed, stream)
  // the packed projection is narrow (few tile pairs): every 16-token group gets blocks of its own
  GO(1);
#undef GO
}
