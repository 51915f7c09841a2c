// out[M,N] = A[M,K] . W[N,K]^T for few rows (M <= 64, a decode step's tokens), bfloat16 in, float accumulation
// on the matrix cores (v_mfma_f32_16x16x32_bf16).  The product is bound by reading W once from HBM, so
// the kernel is shaped for memory parallelism: a block owns NTILE tiles of 16 output features; its WAVES
// waves take interleaved 32-wide k-steps, each lane streaming 16 bytes of one weight row per tile and step,
// and the waves' accumulators are added through LDS in a fixed order (so a result does not depend on what
// else is in the batch).  The weight tile is the MFMA's A operand and the activation tile its B operand:
// a lane ends up with 4 consecutive output features of one token.  One activation load serves the NTILE
// weight tiles of the block, which matters as M grows and the activations are read once per block.
// (tile, 16-token group) pairs are spread over the waves for the final sum and the epilogue.
//
// Epilogues: plain (+ bias) to bfloat16 or float; gated activation over interleaved rows (2j: gate j,
// 2j+1: up j) writing silu(gate) * up; the residual sum out[m, n] += product (+ bias) on a float matrix, each
// element owned by one lane: no atomics.
//
// With NORM the activations are the float residual stream and the RMS norm before the product is folded
// in: the operand is bfloat16(x[m,k] * norm_weight[k]), the sum of squares of every row is gathered on the
// way (every block sees all of K), and the accumulators are scaled by rsqrt(mean(x^2) + eps) before the
// epilogue: norm(x) . W^T = rsqrt(..) * ((x * w) . W^T).
#include "common.h"
#include "api.h"
#include <algorithm>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 3 };

constexpr int UNIT = 2;   // rows of W are dealt out in units of two (a gate/up pair)

// The rows of W are dealt out evenly in units of two (a gate/up pair): the first `rem` blocks take q + 1 units,
// the others q, at most NTILE tiles of 16 rows either way, the last of them filled in part.  A CU
// draws from memory at a rate of its own, so a product is as slow as its block with the most rows: whole tiles
// would leave 3 against 2 of them (0.5B gate/up, 608 tiles for 256 CUs) or 2 against 1 (32B o, 320 tiles).
template <int MT, int NTILE, int WAVES, int EPI, typename TO, bool NORM>
__global__ void __launch_bounds__(WAVES * MS_WAVE)
gemm_skinny_kernel(const void* __restrict__ Av, size_t lda, const bf16* __restrict__ W, size_t ldw,
                   const float* __restrict__ bias, TO* __restrict__ out, size_t ldo, int M, int N, int K,
                   const float* __restrict__ norm_w, float eps, const int* __restrict__ rows, int q, int rem) {
  constexpr int ITEMS = NTILE * MT;
  __shared__ f32x4 red[WAVES - 1][ITEMS][MS_WAVE];
  __shared__ float red_ss[NORM ? WAVES : 1][MT][16];
  const bf16* A = (const bf16*)Av;
  const float* X = (const float*)Av;
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int col = lane & 15, kq = lane >> 4;
  const int n0 = ((int)blockIdx.x * q + min((int)blockIdx.x, rem)) * UNIT;
  const int n1 = min(N, n0 + (q + ((int)blockIdx.x < rem ? 1 : 0)) * UNIT);   // this block's rows: n0 .. n1 - 1
  const int nt = (n1 - n0 + 15) / 16;                                      // in tiles, at most NTILE
  const int m0 = blockIdx.y * 16 * MT;   // token groups beyond MT per block go to further blocks along y
  const int total_steps = (K + 31) / 32;

  const bf16* wrow[NTILE];
  bool mine[NTILE];                // rows past the block's last are not loaded (their products are zero and not stored)
#pragma unroll
  for (int u = 0; u < NTILE; ++u) {
    mine[u] = n0 + u * 16 + col < n1;
    wrow[u] = W + (size_t)min(n0 + u * 16 + col, N - 1) * ldw + kq * 8;
  }
  size_t arow[MT];  // element offset of this lane's activation row and k slice
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = min(m0 + t * 16 + col, M - 1);
    arow[t] = (size_t)(rows ? rows[m] : m) * lda + kq * 8;  // rows: the activations are gathered rows of A
  }

  f32x4 acc[NTILE][MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] = 0.f;
#pragma unroll
    for (int u = 0; u < NTILE; ++u) acc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // What the epilogue will need from memory is asked for now, so that it arrives under the main loop (after
  // the row addresses above, which may themselves wait for a load: these must not wait behind it).
  f32x4 pre[NTILE][MT];   // the residual values this wave will add to (EPI_RESIDUAL)
  f32x4 bv[NTILE];        // bias of this lane's 4 features per tile
#pragma unroll
  for (int u = 0; u < NTILE; ++u) {
    const int nb = n0 + u * 16 + kq * 4;
    bv[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (bias && EPI != EPI_SWIGLU) {
#pragma unroll
      for (int r = 0; r < 4; ++r) if (nb + r < n1) bv[u][r] = bias[nb + r];
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      pre[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (EPI == EPI_RESIDUAL && wave == (u * MT + t) % WAVES && m0 + t * 16 + col < M) {
        const float* o = reinterpret_cast<const float*>(out) + (size_t)(m0 + t * 16 + col) * ldo + nb;
#pragma unroll
        for (int r = 0; r < 4; ++r) if (nb + r < n1) pre[u][t][r] = o[r];
      }
    }
  }

  // A wave has one step's loads in flight; the memory parallelism comes from the 8 or 16 waves of a block.
  // (Issuing the loads of several steps before the first is used was measured and did not help: a CU pulls
  // 25 to 43 GB/s however many loads it has in flight.)
  for (int s = wave; s < total_steps; s += WAVES) {
    const int k = s * 32;
    const bool in = k + kq * 8 < K;  // K is a multiple of 8: a lane's 8 values are all inside or all outside
    bf16x8 wv[NTILE];
#pragma unroll
    for (int u = 0; u < NTILE; ++u) {
      wv[u] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (in && mine[u]) wv[u] = *reinterpret_cast<const bf16x8*>(wrow[u] + k);
    }
    f32x4 nw0 = {0.f, 0.f, 0.f, 0.f}, nw1 = {0.f, 0.f, 0.f, 0.f};
    if (NORM && in) {
      nw0 = *reinterpret_cast<const f32x4*>(norm_w + k + kq * 8);
      nw1 = *reinterpret_cast<const f32x4*>(norm_w + k + kq * 8 + 4);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      bf16x8 av = {0, 0, 0, 0, 0, 0, 0, 0};
      if (NORM) {
        if (in) {
          const f32x4 x0 = *reinterpret_cast<const f32x4*>(X + arow[t] + k);
          const f32x4 x1 = *reinterpret_cast<const f32x4*>(X + arow[t] + k + 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ss[t] = fmaf(x0[i], x0[i], ss[t]);
            ss[t] = fmaf(x1[i], x1[i], ss[t]);
            av[i] = (__bf16)(x0[i] * nw0[i]);
            av[4 + i] = (__bf16)(x1[i] * nw1[i]);
          }
        }
      } else {
        if (in) av = *reinterpret_cast<const bf16x8*>(A + arow[t] + k);
      }
#pragma unroll
      for (int u = 0; u < NTILE; ++u)
        if (u < nt) acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[u], av, acc[u][t], 0, 0, 0);
    }
  }

  if (NORM) {  // a row's squares are spread over the four lane groups and over the waves
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      ss[t] += __shfl_xor(ss[t], 16, MS_WAVE);
      ss[t] += __shfl_xor(ss[t], 32, MS_WAVE);
      if (kq == 0) red_ss[wave][t][col] = ss[t];
    }
  }
  // item (u, t) is finished by wave (u * MT + t) % WAVES; every other wave leaves its share in LDS
#pragma unroll
  for (int u = 0; u < NTILE; ++u)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int item = u * MT + t, owner = item % WAVES;
      if (wave != owner && u < nt) red[wave < owner ? wave : wave - 1][item][lane] = acc[u][t];
    }
  __syncthreads();

#pragma unroll
  for (int u = 0; u < NTILE; ++u)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int item = u * MT + t, owner = item % WAVES;
      if (wave != owner || u >= nt) continue;
      // sum in wave order: the waves below the owner, the owner itself, the waves above
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < WAVES; ++w) sum += w == owner ? acc[u][t] : red[w < owner ? w : w - 1][item][lane];
      if (NORM) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) total += red_ss[w][t][col];
        sum *= 1.0f / sqrtf(total / (float)K + eps);
      }
      // lane holds out[m = t*16 + col][n = nb + r], r = 0..3
      const int m = m0 + t * 16 + col;
      const int nb = n0 + u * 16 + kq * 4;
      if (m >= M) continue;
      if (EPI == EPI_SWIGLU) {
        // rows nb, nb+1 are (gate, up) of feature nb/2; rows nb+2, nb+3 of feature nb/2 + 1
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          if (nb + 2 * p + 1 < n1) {
            const float g = sum[2 * p], up = sum[2 * p + 1];
            out[(size_t)m * ldo + nb / 2 + p] = from_float<TO>(fast_silu(g) * up);
          }
        }
      } else {
        TO* o = out + (size_t)m * ldo + nb;
        // (one 16-byte store per lane instead of four of 4 bytes was measured on the head product: 75 us
        // against 64 us)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (nb + r < n1) o[r] = from_float<TO>(sum[r] + bv[u][r] + pre[u][t][r]);
        }
      }
    }
}

// Tuning knob: force (tiles per block, waves) for every launch; 0 leaves the choice to the heuristic below.
int g_force_ntile = 0, g_force_waves = 0, g_force_mt = 0;

// The shapes of block on offer: (tiles per block, waves).  LDS holds (waves - 1) * tiles * MT KB.
// (Splitting K over blocks as well, with the last block to arrive adding the partial sums, was measured and
// dropped: the device-scope fences it needs cost several microseconds per block on this chip.)
inline bool forced() { return g_force_ntile || g_force_waves || g_force_mt; }

template <int MT, int EPI, typename TO, bool NORM>
int launch_cfg(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M,
               int N, int K, hipStream_t stream, const float* norm_w, float eps, const int* rows) {
  const int tiles = (N + 15) / 16;
  const int steps = (K + 31) / 32;
  const int groups = (M + 16 * MT - 1) / (16 * MT);
  const int cus = ms_compute_units();
  // Every CU should stream an equal share of the matrix: the rows are dealt out in units of two over a whole
  // number of blocks per CU, of up to four tiles each (no last round that only some CUs take part in); with
  // several token groups four tiles go to a block.  An output with fewer tiles than CUs has a block per tile,
  // or, with up to 16 tokens, blocks of at least 8 rows on as many CUs as that gives (every block reads all the
  // activations, which is little then; with 32 tokens and more it costs more than the spread saves.  At 8
  // tokens: o of the 1.5B and 3B shapes 5.1 -> 4.8 and 5.9 -> 5.4 us, down of 3B and 7B 20.2 -> 18.8 and
  // 36.9 -> 35.5; the 0.5B shapes the same).
  const int units = (N + UNIT - 1) / UNIT;
  int blocks;
  if (tiles <= cus) blocks = M <= 16 ? std::max(tiles, std::min(cus, N / 8)) : tiles;
  else if (groups == 1 && tiles <= 16 * cus) blocks = cus * ((tiles + 4 * cus - 1) / (4 * cus));
  else blocks = (tiles + 3) / 4;      // many rounds: the last one matters little (measured: the head)
  if (g_force_ntile) blocks = (tiles + g_force_ntile - 1) / g_force_ntile;
  const int q = units / blocks, rem = units % blocks;   // blocks * q + rem units
  int ntile = ((q + (rem ? 1 : 0)) * UNIT + 15) / 16;   // tiles of the block with the most rows
  if (g_force_ntile && ntile <= g_force_ntile) ntile = g_force_ntile;
  int waves = ntile >= 3 ? (MT <= 2 && (MT == 1 || tiles < 1024) ? 8 : 4) : ((steps >= 32 || MT > 1) ? 16 : 8);
  if (g_force_ntile) waves = g_force_waves;
  if (ntile > 4 || (waves - 1) * ntile * MT > 60) return MS_UNSUPPORTED;  // LDS
#define GO(NT, WV) if (ntile == NT && waves == WV) { if constexpr ((WV - 1) * NT * MT <= 60) { gemm_skinny_kernel<MT, NT, WV, EPI, TO, NORM><<<dim3(blocks, groups), dim3(WV * MS_WAVE), 0, stream>>>(A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, q, rem); return ms_launch_status(); } }
  GO(4, 4) GO(4, 8) GO(3, 4) GO(3, 8) GO(2, 8) GO(2, 16) GO(1, 8) GO(1, 16)
#undef GO
  return MS_UNSUPPORTED;
}

template <int EPI, typename TO, bool NORM>
int launch_mt(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M,
              int N, int K, hipStream_t stream, const float* norm_w = nullptr, float eps = 0.f,
              const int* rows = nullptr) {
  // Several token groups per block share the weight loads; a narrow output has too few tiles to fill the chip
  // that way, so there every group gets blocks of its own (the weight tile is then re-read from L2).
  const int tiles = (N + 15) / 16;
  const int mt = g_force_mt ? g_force_mt : ((M <= 16 || tiles <= 128) ? 1 : ((M <= 32 || tiles < 1024) ? 2 : 4));
  if (mt == 1) return launch_cfg<1, EPI, TO, NORM>(A, lda, W, ldw, bias, out, ldo, M, N, K, stream, norm_w, eps, rows);
  if (mt == 2) return launch_cfg<2, EPI, TO, NORM>(A, lda, W, ldw, bias, out, ldo, M, N, K, stream, norm_w, eps, rows);
  return launch_cfg<4, EPI, TO, NORM>(A, lda, W, ldw, bias, out, ldo, M, N, K, stream, norm_w, eps, rows);
}

}  // namespace

// Tuning knob for measurements: force the block shape (tiles per block, waves) out of (4,4) (4,8) (3,4) (3,8) (2,8)
// (2,16) (1,8) (1,16), and the 16-token groups per block (1, 2 or 4; further groups go to further blocks), for
// every later ms_gemm_skinny* launch; zeros give the choice back to the heuristic.  While anything is forced,
// products of up to 16 rows stay in this kernel instead of going to ms_gemm_stream.
extern "C" void ms_gemm_skinny_force(int ntile, int waves, int token_groups) {
  g_force_ntile = ntile;
  g_force_waves = waves;
  g_force_mt = token_groups;
}

// epilogue 0: out[M,N] (out_dtype float or bfloat16) = product + bias
// epilogue 1: out[M,N/2] bfloat16 = silu(gate) * up over interleaved rows of W (no bias)
// epilogue 3: out[M,N] float += product + bias
extern "C" int ms_gemm_skinny(const void* A, long long lda, const void* W, long long ldw, const float* bias, void* out,
                              long long ldo, int M, int N, int K, int epilogue, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (M > 64) return MS_UNSUPPORTED;
  if (M <= 16 && !forced()) {   // one token group: the streaming kernel, where it takes the shape
    const int rc = ms_gemm_stream(A, lda, nullptr, nullptr, 0.f, W, ldw, bias, out, ldo, M, N, K, epilogue, out_dtype, 0, 0, stream);
    if (rc != MS_UNSUPPORTED) return rc;
  }
  if (!forced()) {    // the kernel that holds the activations in LDS, where it takes the shape
    const int rc = ms_gemm_panel(A, lda, nullptr, nullptr, 0.f, W, ldw, bias, out, ldo, M, N, K, epilogue, out_dtype, 0, 0, stream);
    if (rc != MS_UNSUPPORTED) return rc;
  }
  if (K <= 0 || K % 8 || lda % 8 || ldw % 8 || lda < K || ldw < K) return MS_UNSUPPORTED;
  if (((uintptr_t)A | (uintptr_t)W) % 16) return MS_UNSUPPORTED;
  const bf16* w = (const bf16*)W;
  if (epilogue == EPI_STORE) {
    if (ldo < N) return MS_BAD_ARG;
    if (out_dtype == MS_BF16) return launch_mt<EPI_STORE, bf16, false>(A, lda, w, ldw, bias, (bf16*)out, ldo, M, N, K, stream);
    if (out_dtype == MS_F32) return launch_mt<EPI_STORE, float, false>(A, lda, w, ldw, bias, (float*)out, ldo, M, N, K, stream);
    return MS_BAD_ARG;
  }
  if (epilogue == EPI_SWIGLU) {
    if (N % 2 || ldo < N / 2 || out_dtype != MS_BF16 || bias) return MS_BAD_ARG;
    return launch_mt<EPI_SWIGLU, bf16, false>(A, lda, w, ldw, nullptr, (bf16*)out, ldo, M, N, K, stream);
  }
  if (epilogue == EPI_RESIDUAL) {
    if (ldo < N || out_dtype != MS_F32) return MS_BAD_ARG;
    return launch_mt<EPI_RESIDUAL, float, false>(A, lda, w, ldw, bias, (float*)out, ldo, M, N, K, stream);
  }
  return MS_BAD_ARG;
}

// As ms_gemm_skinny with epilogue 0 or 1, but the activations are rows of the float residual stream x[M,K]
// and the RMS norm (weight norm_w[K], eps) that precedes the product is folded into the kernel.  With `rows`
// (int32 [M]) row m of the product comes from x[rows[m]].
extern "C" int ms_gemm_skinny_norm(const float* x, long long ldx, const int* rows, const float* norm_w, float eps,
                                   const void* W, long long ldw, const float* bias, void* out, long long ldo, int M,
                                   int N, int K, int epilogue, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (M > 64) return MS_UNSUPPORTED;
  if (M <= 16 && !forced()) {
    const int rc = ms_gemm_stream(x, ldx, rows, norm_w, eps, W, ldw, bias, out, ldo, M, N, K, epilogue, out_dtype, 1, 0, stream);
    if (rc != MS_UNSUPPORTED) return rc;
  }
  if (!forced()) {
    const int rc = ms_gemm_panel(x, ldx, rows, norm_w, eps, W, ldw, bias, out, ldo, M, N, K, epilogue, out_dtype, 1, 0, stream);
    if (rc != MS_UNSUPPORTED) return rc;
  }
  if (K <= 0 || K % 8 || ldx % 4 || ldw % 8 || ldx < K || ldw < K) return MS_UNSUPPORTED;
  if (((uintptr_t)x | (uintptr_t)W | (uintptr_t)norm_w) % 16) return MS_UNSUPPORTED;
  const bf16* w = (const bf16*)W;
  if (epilogue == EPI_STORE) {
    if (ldo < N) return MS_BAD_ARG;
    if (out_dtype == MS_BF16) return launch_mt<EPI_STORE, bf16, true>(x, ldx, w, ldw, bias, (bf16*)out, ldo, M, N, K, stream, norm_w, eps, rows);
    if (out_dtype == MS_F32) return launch_mt<EPI_STORE, float, true>(x, ldx, w, ldw, bias, (float*)out, ldo, M, N, K, stream, norm_w, eps, rows);
    return MS_BAD_ARG;
  }
  if (epilogue == EPI_SWIGLU) {
    if (N % 2 || ldo < N / 2 || out_dtype != MS_BF16 || bias) return MS_BAD_ARG;
    return launch_mt<EPI_SWIGLU, bf16, true>(x, ldx, w, ldw, nullptr, (bf16*)out, ldo, M, N, K, stream, norm_w, eps, rows);
  }
  return MS_BAD_ARG;
}
