// out[M,N] = A[M,K] . W[N,K]^T for up to 64 tokens (a decode step; mostly of a larger batch) and a W of many
// rows, bfloat16 in, float accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16).
//
// With this many tokens the activations, not the weights, are most of what a block has to load when it reads
// them as MFMA operands k-step by k-step: every 16-row tile of W needs all of A again, and what a CU can pull
// through its load path (from L2 as from memory) is about 1/256 of what the chip can.  So here every block
// loads A once, whole, into LDS (the panel: bfloat16, K padded to a multiple of 32 with zeros, rows an odd
// number of 32 bytes apart, where 16-byte fragment reads run at the full LDS rate; an odd number of 16 bytes
// gives half of it), and then streams its share of W against it: the 16-row tiles of W are dealt
// out evenly over as many blocks as the chip has CUs, and inside a block
//   * rounds of 16 tiles go to the 16 waves whole (no sum across waves);
//   * the tiles left over (all of them, for a block with fewer than 16) are shared, each among floor(16 / left)
//     waves that take the tile's k-steps in turn; their accumulators are added through LDS (over the panel,
//     which is no longer needed) in wave order.
// Either way an element's sum runs in an order that depends on the shape of the product alone.
//
// The weight tile is the A operand and the panel the B operand of the MFMA: a lane ends up with 4 consecutive
// output features of one token.  Epilogues and the folded RMS norm as in gemm_skinny: plain (+ bias) to bfloat16
// or float; gated activation over interleaved rows (2j: gate j, 2j+1: up j); the residual sum out += product
// (+ bias) on a float matrix.  With NORM the activations are the float residual stream: the panel holds
// bfloat16(x * norm_weight), the squares are summed on the way in a fixed order, and the accumulators are
// scaled by rsqrt(mean(x^2) + eps) before the epilogue.
#include "common.h"
#include "api.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;   // a 16-byte piece: 8 bfloat16

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 3 };

constexpr int WAVES = 16;       // waves of a block
constexpr int BATCH = 4;        // panel loads a wave has in flight
constexpr int MAX_TOKENS = 64;
constexpr int MAX_PARTS = 4;    // 64-piece (512-column) loads per row of A at most: K <= 2048

// id / parts for the small numbers that occur here (id < 4096, parts <= 16) by a multiplication
__device__ __forceinline__ int small_inverse(int parts) { return (65536 + parts - 1) / parts; }
__device__ __forceinline__ int small_div(int id, int inverse) { return (id * inverse) >> 16; }

// One chunk of the panel: columns k0 .. k0 + 8 * Kc8 of the M rows of A go to LDS as bfloat16 pieces
// xst[token * pitch + piece], the S * 4 - Kc8 pieces that a last k-step lacks as zeros.  A wave keeps to one
// 512-column part of the chunk (so it loads that part of the norm weights once) and takes every
// (16 / parts2)-th token, PB of them in flight.  With NORM the rows are float and are multiplied by the norm
// weights on the way; their squares are summed per (token, part): the lanes of a load in the fixed tree of
// wave_sum, a (token, part)'s chunks in order (the same wave has it in every chunk).
template <bool NORM, int PB>
__device__ __forceinline__ void load_panel(const void* __restrict__ Av, size_t lda, const float* __restrict__ norm_w,
                                           const int* __restrict__ rows, int M, int k0, int Kc8, int S, int parts,
                                           int pitch, bool first_chunk, u32x4* xst, float* ss_part, int wave, int lane) {
  const bf16* A = (const bf16*)Av;
  const float* X = (const float*)Av;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const int parts2 = parts <= 1 ? 1 : (parts <= 2 ? 2 : 4);
  const int part = wave & (parts2 - 1);
  const int tok_step = WAVES / parts2;
  const int c = part * 64 + lane;
  const bool in = c < Kc8;   // lanes past the chunk's end (and whole waves, when parts is 3) load nothing new
  const int cc = k0 + min(c, Kc8 - 1) * 8;
  f32x4 nwf[2];
  if (NORM) {
    nwf[0] = *reinterpret_cast<const f32x4*>(norm_w + cc);
    nwf[1] = *reinterpret_cast<const f32x4*>(norm_w + cc + 4);
  }
  if (part < parts) {
    for (int base = wave / parts2; base < M; base += tok_step * PB) {
      u32x4 piece[NORM ? 1 : PB];
      f32x4 xf[NORM ? PB : 1][2];
#pragma unroll
      for (int i = 0; i < PB; ++i) {
        const int tok = base + i * tok_step;
        if (tok >= M) break;   // the same for the whole wave
        const size_t at = (size_t)(rows ? rows[tok] : tok) * lda + cc;
        if (NORM) {
          xf[i][0] = *reinterpret_cast<const f32x4*>(X + at);
          xf[i][1] = *reinterpret_cast<const f32x4*>(X + at + 4);
        } else {
          piece[i] = *reinterpret_cast<const u32x4*>(A + at);
        }
      }
#pragma unroll
      for (int i = 0; i < PB; ++i) {
        const int tok = base + i * tok_step;
        if (tok >= M) break;
        u32x4 pc;
        if (NORM) {
          bf16x8 h;
          float ss = 0.f;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float x0 = in ? xf[i][0][e] : 0.f, x1 = in ? xf[i][1][e] : 0.f;
            ss = fmaf(x0, x0, ss);
            ss = fmaf(x1, x1, ss);
            h[e] = (__bf16)(x0 * nwf[0][e]);
            h[4 + e] = (__bf16)(x1 * nwf[1][e]);
          }
          pc = __builtin_bit_cast(u32x4, h);
          ss = wave_sum(ss);
          if (lane == 0) ss_part[tok * parts + part] = (first_chunk ? 0.f : ss_part[tok * parts + part]) + ss;
        } else {
          pc = piece[i];
        }
        if (in) xst[tok * pitch + c] = pc;
      }
    }
  }
  const int padn = S * 4 - Kc8;   // 0..3
  for (int t = threadIdx.x; t < M * padn; t += WAVES * MS_WAVE) {
    const int rr = t / padn;
    xst[rr * pitch + Kc8 + t - rr * padn] = zero;
  }
}

// After the last chunk: every token's rsqrt(mean(x^2) + eps) from its parts' sums, in part order.
__device__ __forceinline__ void finish_norm(const float* ss_part, float* inv_rms, int M, int K, int parts, float eps) {
  if (threadIdx.x < M) {
    float total = 0.f;
    for (int p = 0; p < parts; ++p) total += ss_part[threadIdx.x * parts + p];
    inv_rms[threadIdx.x] = 1.0f / sqrtf(total / (float)K + eps);
  }
  __syncthreads();
}

// A finished tile: lane (col, kq) holds out[token tt * 16 + col][n0 + kq * 4 + (0..3)] of the 16 features from n0.
template <int TT, int EPI, typename TO, bool NORM>
__device__ __forceinline__ void finish_tile(const f32x4* sum, int n0, int M, int N, const float* __restrict__ bias,
                                            TO* __restrict__ out, size_t ldo, const float* inv_rms, int col, int kq) {
  const int nb = n0 + kq * 4;
  f32x4 bv = {0.f, 0.f, 0.f, 0.f};
  if (bias && EPI != EPI_SWIGLU) {
#pragma unroll
    for (int r = 0; r < 4; ++r) if (nb + r < N) bv[r] = bias[nb + r];
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int m = tt * 16 + col;
    if (m >= M) continue;
    f32x4 v = sum[tt];
    if (NORM) v *= inv_rms[m];
    if (EPI == EPI_SWIGLU) {
      // rows nb, nb+1 are (gate, up) of feature nb/2; rows nb+2, nb+3 of feature nb/2 + 1
#pragma unroll
      for (int p = 0; p < 2; ++p)
        if (nb + 2 * p + 1 < N) out[(size_t)m * ldo + nb / 2 + p] = from_float<TO>(fast_silu(v[2 * p]) * v[2 * p + 1]);
    } else {
      TO* o = out + (size_t)m * ldo + nb;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (nb + r >= N) continue;
        if (EPI == EPI_RESIDUAL) o[r] = from_float<TO>(to_float(o[r]) + v[r] + bv[r]);
        else o[r] = from_float<TO>(v[r] + bv[r]);
      }
    }
  }
}

template <int TT, int EPI, typename TO, bool NORM>
__global__ void __launch_bounds__(WAVES * MS_WAVE)
gemm_panel_kernel(const void* __restrict__ Av, size_t lda, const bf16* __restrict__ W, size_t ldw,
                  const float* __restrict__ bias, TO* __restrict__ out, size_t ldo, int M, int N, int K,
                  const float* __restrict__ norm_w, float eps, const int* __restrict__ rows, int q, int rem) {
  // weight fragments a wave asks for before it multiplies them (with four token tiles the registers, 128 to a
  // lane with 16 waves on the CU, hold fewer)
  constexpr int DEPTH = TT >= 4 ? 7 : 8;
  extern __shared__ u32x4 smem[];   // the panel [tokens][pitch]; afterwards the waves' partial sums
  __shared__ float ss_part[MAX_TOKENS * MAX_PARTS];
  __shared__ float inv_rms[MAX_TOKENS];
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);   // the same for the whole wave
  const int col = lane & 15, kq = lane >> 4;
  const int K8 = K / 8, S = (K + 31) / 32;
  const int pitch = S * 4 + 2;   // rows an odd number of 32 bytes apart: 16-byte fragment reads at the full LDS rate
  const int parts = (K8 + 63) / 64;         // loads of 64 lanes x 8 columns per row of A
  u32x4* xst = smem;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  // ---- this block's tiles of W: dealt out evenly (the first `rem` blocks take one more).  Rounds of 16 tiles go
  // to the 16 waves whole; the tiles left over are shared, each among g waves that take its k-steps in turn.
  const int b = blockIdx.x;
  const int T = q + (b < rem ? 1 : 0);
  const int t0 = b * q + min(b, rem);
  const int T_whole = T & ~(WAVES - 1), T_left = T - T_whole;
  const int g = T_left ? WAVES / T_left : 1;
  int left_tile = 0, j = 0;     // this wave's shared tile (if below T_left) and its place among that tile's waves
  if (T_left) {
    left_tile = small_div(wave, small_inverse(g));
    j = wave - left_tile * g;
  }
  const bool shares = T_left && left_tile < T_left;

  bf16x8 wa[DEPTH];
  // fragments of DEPTH k-steps (s0, s0 + step, ...) of a tile: lane (col, kq) holds row col, columns kq * 8 ..
  auto fetch = [&](int tile, int s0, int step) {
    const bf16* wrow = W + (size_t)min((t0 + tile) * 16 + col, N - 1) * ldw;   // rows past N repeat the last
#pragma unroll
    for (int p = 0; p < DEPTH; ++p) {
      const int s = s0 + p * step;
      if (s >= S) break;   // the same for the whole wave
      const int k = s * 32 + kq * 8;
      wa[p] = *reinterpret_cast<const bf16x8*>(wrow + min(k, K - 8));   // K is a multiple of 8: a piece is in or out
      if (k >= K) wa[p] = __builtin_bit_cast(bf16x8, zero);
    }
  };
  // the wave's first fragments are asked for before the panel is built: they come from memory, the panel
  // from L2, and neither waits for the other
  if (T_whole) fetch(wave, 0, 1);
  else if (shares) fetch(left_tile, j, g);

  load_panel<NORM, BATCH>(Av, lda, norm_w, rows, M, 0, K8, S, parts, pitch, true, xst, ss_part, wave, lane);
  __syncthreads();
  if (NORM) finish_norm(ss_part, inv_rms, M, K, parts, eps);

  int xrow[TT];   // idle columns repeat the last token; their results are not stored
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) xrow[tt] = min(tt * 16 + col, M - 1) * pitch + kq;

  auto finish = [&](int tl, f32x4* sum) {
    finish_tile<TT, EPI, TO, NORM>(sum, (t0 + tl) * 16, M, N, bias, out, ldo, inv_rms, col, kq);
  };

  f32x4 acc[TT];
  // the fetched fragments of k-steps s0, s0 + step, ... times the panel
  auto multiply = [&](int s0, int step) {
#pragma unroll
    for (int p = 0; p < DEPTH; ++p) {
      const int s = s0 + p * step;
      if (s >= S) break;
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        const bf16x8 xb = __builtin_bit_cast(bf16x8, xst[xrow[tt] + 4 * s]);
        acc[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[p], xb, acc[tt], 0, 0, 0);
      }
    }
  };

  for (int tile = wave; tile < T_whole; tile += WAVES) {   // whole tiles: no sum across waves
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) acc[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < S; s0 += DEPTH) {
      if (tile != wave || s0 != 0) fetch(tile, s0, 1);   // the first were fetched above
      multiply(s0, 1);
    }
    finish(tile, acc);
  }
  if (!T_left) return;   // the same for the whole block

  if (shares) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) acc[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = j; s0 < S; s0 += g * DEPTH) {
      if (T_whole || s0 != j) fetch(T_whole + left_tile, s0, g);
      multiply(s0, g);
    }
  }
  // the first wave of a shared tile adds the others' accumulators in wave order
  __syncthreads();   // nobody reads the panel any more
  f32x4* red = reinterpret_cast<f32x4*>(smem);   // [WAVES][TT][64]
  if (shares && j > 0) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) red[(wave * TT + tt) * MS_WAVE + lane] = acc[tt];
  }
  __syncthreads();
  if (shares && j == 0) {
    for (int w = 1; w < g; ++w) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) acc[tt] += red[((wave + w) * TT + tt) * MS_WAVE + lane];
    }
    finish(T_whole + left_tile, acc);
  }
}

// The same for rows of A that do not fit LDS whole: the panel holds KC columns at a time, and a wave keeps the
// accumulators of all its tiles (up to NACC whole tiles and one shared tile) across the chunks.  Between two
// chunks the block waits twice: for the panel to be complete, and for everybody to be done with it.
template <int TT, int NACC, int EPI, typename TO, bool NORM>
__global__ void __launch_bounds__(WAVES * MS_WAVE)
gemm_panel_chunked_kernel(const void* __restrict__ Av, size_t lda, const bf16* __restrict__ W, size_t ldw,
                          const float* __restrict__ bias, TO* __restrict__ out, size_t ldo, int M, int N, int K,
                          const float* __restrict__ norm_w, float eps, const int* __restrict__ rows, int q, int rem,
                          int KC, int row_blocks, int k_per) {
  // weight fragments a wave asks for before it multiplies them: what the 128 registers of a lane (16 waves on
  // the CU) leave beside the accumulators, each fragment with its TT operands from the panel
  constexpr int FREE = (NACC >= 3 ? 88 : 96) - (NACC + 1) * TT * 4;
  constexpr int PB = (NACC + 1) * TT * 4 >= 48 ? 2 : BATCH;   // panel loads in flight, by the same budget
  constexpr int DEPTH = FREE / (4 * (1 + TT)) > 8 ? 8 : (FREE / (4 * (1 + TT)) < 1 ? 1 : FREE / (4 * (1 + TT)));
  extern __shared__ u32x4 smem[];   // the panel [tokens][pitch] of one chunk; afterwards the waves' partial sums
  __shared__ float ss_part[MAX_TOKENS * MAX_PARTS];
  __shared__ float inv_rms[MAX_TOKENS];
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);   // the same for the whole wave
  const int col = lane & 15, kq = lane >> 4;
  const int C8 = KC / 8;                    // pieces per row of a full chunk (KC is a multiple of 32)
  const int pitch = C8 + 2;      // rows an odd number of 32 bytes apart: 16-byte fragment reads at the full LDS rate
  const int parts = (C8 + 63) / 64;         // loads of 64 lanes x 8 columns per row and chunk
  u32x4* xst = smem;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  // this block's tiles of W, as in the kernel above.  When the columns are split as well (k_per < K: block ids
  // beyond row_blocks take the next k_per columns of the same tiles), a block's result is a partial sum that
  // goes to its own [M, ldo] slice of `out`, to be added up by splitk_reduce_kernel.
  const int k_part = blockIdx.x / row_blocks;
  const int b = blockIdx.x - k_part * row_blocks;
  const int k_begin = k_part * k_per, k_end = min(K, k_begin + k_per);
  out += (size_t)k_part * M * ldo;
  const int T = q + (b < rem ? 1 : 0);
  const int t0 = b * q + min(b, rem);
  const int T_whole = T & ~(WAVES - 1), T_left = T - T_whole;
  const int n_whole = T_whole / WAVES;      // whole tiles of every wave: wave, wave + 16, ...; at most NACC
  const int g = T_left ? WAVES / T_left : 1;
  int left_tile = 0, j = 0;
  if (T_left) {
    left_tile = small_div(wave, small_inverse(g));
    j = wave - left_tile * g;
  }
  const bool shares = T_left && left_tile < T_left;

  int xrow[TT];   // idle columns repeat the last token; their results are not stored
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) xrow[tt] = min(tt * 16 + col, M - 1) * pitch + kq;

  f32x4 acc[NACC][TT], acc_left[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    acc_left[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  for (int k0 = k_begin; k0 < k_end; k0 += KC) {
    const int Kc8 = min(KC, k_end - k0) / 8;  // pieces per row of this chunk
    const int S = (Kc8 + 3) / 4;              // its k-steps
    load_panel<NORM, PB>(Av, lda, norm_w, rows, M, k0, Kc8, S, parts, pitch, k0 == k_begin, xst, ss_part, wave, lane);
    __syncthreads();

    // ---- this chunk's k-steps of the wave's tiles
    auto run = [&](int tile, int s_first, int step, f32x4* a) {
      const bf16* wrow = W + (size_t)min((t0 + tile) * 16 + col, N - 1) * ldw + k0;   // rows past N repeat the last
      for (int s0 = s_first; s0 < S; s0 += step * DEPTH) {
        bf16x8 wa[DEPTH];
#pragma unroll
        for (int p = 0; p < DEPTH; ++p) {
          const int s = s0 + p * step;
          if (s >= S) break;   // the same for the whole wave
          const int k = s * 32 + kq * 8;
          wa[p] = *reinterpret_cast<const bf16x8*>(wrow + min(k, k_end - k0 - 8));   // a piece is in or out
          if (k0 + k >= k_end) wa[p] = __builtin_bit_cast(bf16x8, zero);
        }
#pragma unroll
        for (int p = 0; p < DEPTH; ++p) {
          const int s = s0 + p * step;
          if (s >= S) break;
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            const bf16x8 xb = __builtin_bit_cast(bf16x8, xst[xrow[tt] + 4 * s]);
            a[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[p], xb, a[tt], 0, 0, 0);
          }
        }
      }
    };
#pragma unroll
    for (int i = 0; i < NACC; ++i) {
      if (i >= n_whole) break;
      run(wave + i * WAVES, 0, 1, acc[i]);
    }
    if (shares) run(T_whole + left_tile, j, g, acc_left);
    __syncthreads();   // the next chunk overwrites the panel
  }

  if (NORM) finish_norm(ss_part, inv_rms, M, K, parts, eps);

  auto finish = [&](int tl, f32x4* sum) {
    finish_tile<TT, EPI, TO, NORM>(sum, (t0 + tl) * 16, M, N, bias, out, ldo, inv_rms, col, kq);
  };
#pragma unroll
  for (int i = 0; i < NACC; ++i) {
    if (i >= n_whole) break;
    finish(wave + i * WAVES, acc[i]);
  }
  if (!T_left) return;   // the same for the whole block

  // the first wave of a shared tile adds the others' accumulators in wave order (the panel is free: the loop
  // ended with a wait)
  f32x4* red = reinterpret_cast<f32x4*>(smem);   // [WAVES][TT][64]
  if (shares && j > 0) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) red[(wave * TT + tt) * MS_WAVE + lane] = acc_left[tt];
  }
  __syncthreads();
  if (shares && j == 0) {
    for (int w = 1; w < g; ++w) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) acc_left[tt] += red[((wave + w) * TT + tt) * MS_WAVE + lane];
    }
    finish(T_whole + left_tile, acc_left);
  }
}

// out[m, n] (=, +=) sum over the column parts of partial[part][m][n], in part order, + bias.
template <int EPI, typename TO>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float* __restrict__ partial, int parts, const float* __restrict__ bias, TO* __restrict__ out,
                     size_t ldo, int M, int N) {
  const int quads = (N + 3) / 4;
  const int id = blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= M * quads) return;
  const int m = id / quads, n = (id - m * quads) * 4;
  float sum[4] = {0.f, 0.f, 0.f, 0.f};
  const size_t slice = (size_t)M * N;
  const bool whole = n + 3 < N && N % 4 == 0;   // rows of the partial sums are 16-byte aligned then
  for (int p = 0; p < parts; ++p) {
    const float* src = partial + p * slice + (size_t)m * N + n;
    if (whole) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] += v[r];
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) sum[r] += src[r];
    }
  }
  TO* o = out + (size_t)m * ldo + n;
  for (int r = 0; r < 4 && n + r < N; ++r) {
    const float v = sum[r] + (bias ? bias[n + r] : 0.f);
    if (EPI == EPI_RESIDUAL) o[r] = from_float<TO>(to_float(o[r]) + v);
    else o[r] = from_float<TO>(v);
  }
}

constexpr int LDS_BUDGET = 144 * 1024;   // of the CU's 160 KB, for the panel

template <int TT, int EPI, typename TO, bool NORM>
int launch(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M, int N,
           int K, const float* norm_w, float eps, const int* rows, int blocks, int q, int rem, size_t lds,
           hipStream_t stream) {
  static bool raised = false;   // once per instantiation: allow more dynamic LDS than the default 64 KB
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_panel_kernel<TT, EPI, TO, NORM>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BUDGET) != hipSuccess)
      return MS_LAUNCH_FAILED;
    raised = true;
  }
  gemm_panel_kernel<TT, EPI, TO, NORM><<<dim3(blocks), dim3(WAVES * MS_WAVE), lds, stream>>>(
      A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, q, rem);
  return ms_launch_status();
}

template <int TT, int NACC, int EPI, typename TO, bool NORM>
int launch_chunked(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M,
                   int N, int K, const float* norm_w, float eps, const int* rows, int blocks, int q, int rem, int KC,
                   size_t lds, hipStream_t stream, int k_parts = 1, int k_per = 0) {
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_panel_chunked_kernel<TT, NACC, EPI, TO, NORM>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BUDGET) != hipSuccess)
      return MS_LAUNCH_FAILED;
    raised = true;
  }
  gemm_panel_chunked_kernel<TT, NACC, EPI, TO, NORM><<<dim3(blocks * k_parts), dim3(WAVES * MS_WAVE), lds, stream>>>(
      A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, q, rem, KC, blocks, k_parts > 1 ? k_per : K);
  return ms_launch_status();
}

template <int EPI, typename TO, bool NORM>
int plan(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M, int N,
         int K, const float* norm_w, float eps, const int* rows, bool any_shape, hipStream_t stream) {
  const int cus = ms_compute_units();
  const int tiles = (N + 15) / 16;
  // Where this kernel wins over ms_gemm_skinny, by measurement.  More than 16 tokens: from 7/8 of a tile of W
  // for every CU on (the 7B shape's down projection, 224 tiles: 81 against 101 us at 64 tokens; with 96 or 128
  // tiles the panel, which every block loads whole, costs more than it saves).  Up to 16 tokens: a W of at least
  // four tiles per CU with long rows (gate/up and head of the 7B shape at 8 tokens: 54 against 66 us, 212 against
  // 248; at the 0.5B shape the two kernels are equal or this one slower).
  if (!any_shape && (M > 16 ? tiles * 8 < cus * 7 : (tiles < 4 * cus || K < 2048))) return MS_UNSUPPORTED;
  const int tt = (M + 15) / 16;
  const int S = (K + 31) / 32;
  const int blocks = tiles < cus ? tiles : cus;
  const int q = tiles / blocks, rem = tiles % blocks;
  const size_t red = (size_t)WAVES * tt * MS_WAVE * 16;
  size_t lds = (size_t)M * (S * 4 + 2) * 16;
  if (lds <= (size_t)LDS_BUDGET && (K / 8 + 63) / 64 <= MAX_PARTS) {   // the rows fit whole
    if (lds < red) lds = red;
#define GO(TTV) if (tt == TTV) return launch<TTV, EPI, TO, NORM>(A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, blocks, q, rem, lds, stream)
    GO(1); GO(2); GO(3); GO(4);
#undef GO
    return MS_UNSUPPORTED;
  }
  // in chunks of KC columns: the widest of 2048, 1536, 1024, 512 that fits
  int KC = 0;
  for (int kc = 2048; kc >= 512; kc -= 512) {
    if ((size_t)M * (kc / 8 + 2) * 16 <= (size_t)LDS_BUDGET) { KC = kc; break; }
  }
  if (!KC) return MS_UNSUPPORTED;
  lds = (size_t)M * (KC / 8 + 2) * 16;
  if (lds < red) lds = red;
  const int nacc = (q + (rem ? 1 : 0)) / WAVES;   // whole tiles a wave keeps accumulators for
  if (nacc > 3 || (tt == 4 && nacc > 2)) return MS_UNSUPPORTED;   // what a lane's registers hold
#define GO(TTV, NA) if (tt == TTV && (nacc < 1 ? 1 : nacc) == NA) return launch_chunked<TTV, NA, EPI, TO, NORM>(A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, blocks, q, rem, KC, lds, stream)
  GO(1, 1); GO(2, 1); GO(3, 1); GO(4, 1);
  GO(1, 2); GO(2, 2); GO(3, 2); GO(4, 2);
  GO(1, 3); GO(2, 3); GO(3, 3);
#undef GO
  return MS_UNSUPPORTED;
}

// Columns split over blocks as well, for a W with long rows and too few tiles to give every CU a share of
// whole rows that is worth its loads of the activations (down projections): the number of column parts, 0 if
// the shape is not one for it.  Every block then takes at most 16 tiles (one round of its waves).
int splitk_parts(int M, int N, int K) {
  const int cus = ms_compute_units();
  const int tiles = (N + 15) / 16;
  if (M <= 0 || M > MAX_TOKENS || K % 8 || tiles > 2 * cus) return 0;
  // Rows of 8,192 columns or more (down projections) always; with more than 32 tokens also rows from 3,072
  // columns on against a W of about a tile per CU (the o and q/k/v products of the 7B and 32B shapes), where an
  // unsplit block reads all activations, four times its weights, for a single tile (64 tokens, 3,584 x 3,584:
  // 21.5 -> 16.9 us in four parts; 4,608 x 3,584: 23.8 -> 18.3; 5,120 x 5,120: 31.7 -> 24.1; with 32 tokens, or
  // rows of 2,048 columns, splitting is no faster or slower)
  const bool long_rows = K >= 8192;
  if (!long_rows && !(M > 32 && K >= 3072 && tiles * 4 >= cus * 3)) return 0;
  // up to 16 tokens a W with a tile for (nearly) every CU and no more is served as well unsplit (7B shape's down
  // projection, 224 tiles, at 8 tokens: 34 us unsplit, 39 split; 320 tiles of the 14B and 32B shapes: 47 -> 39
  // and 93 -> 64 us split, for the second round of blocks that unsplit they need)
  if (M <= 16 && tiles <= cus) return 0;
  int best = 0;
  for (int parts = 2; parts <= 16; parts *= 2) {
    const int row_blocks = cus / parts;
    if (row_blocks < 1 || (tiles + row_blocks - 1) / row_blocks > WAVES) continue;
    if (K / parts < (long_rows ? 1024 : 768)) break;
    best = parts;
  }
  return best;
}

template <int EPI, typename TO>
int run_splitk(const bf16* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M, int N,
               int K, float* partial, int parts, hipStream_t stream) {
  const int cus = ms_compute_units();
  const int tiles = (N + 15) / 16;
  const int row_blocks = tiles < cus / parts ? tiles : cus / parts;
  const int q = tiles / row_blocks, rem = tiles % row_blocks;
  const int k_per = ((K + parts - 1) / parts + 31) / 32 * 32;
  const int tt = (M + 15) / 16;
  int KC = 0;
  for (int kc = 2048; kc >= 512; kc -= 512) {
    if ((size_t)M * (kc / 8 + 2) * 16 <= (size_t)LDS_BUDGET) { KC = kc; break; }
  }
  if (!KC) return MS_UNSUPPORTED;
  size_t lds = (size_t)M * (KC / 8 + 2) * 16;
  const size_t red = (size_t)WAVES * tt * MS_WAVE * 16;
  if (lds < red) lds = red;
  int rc = MS_UNSUPPORTED;
#define GO(TTV) if (tt == TTV) rc = launch_chunked<TTV, 1, EPI_STORE, float, false>(A, lda, W, ldw, nullptr, partial, (size_t)N, M, N, K, nullptr, 0.f, nullptr, row_blocks, q, rem, KC, lds, stream, parts, k_per)
  GO(1); GO(2); GO(3); GO(4);
#undef GO
  if (rc != MS_OK) return rc;
  const int threads = M * ((N + 3) / 4);
  splitk_reduce_kernel<EPI, TO><<<dim3((threads + 255) / 256), dim3(256), 0, stream>>>(partial, parts, bias, out, ldo, M, N);
  return ms_launch_status();
}

}  // namespace

// The product of up to 64 rows with W[N,K]^T, the rows held whole in LDS.  norm = 0: A is bfloat16 [M, lda];
// norm = 1: A is the float residual stream and the RMS norm (norm_w[K], eps) is folded in; rows (int32 [M], may
// be null) gathers the rows of A.
// epilogue 0: out[M,N] (out_dtype float or bfloat16) = product + bias
// epilogue 1: out[M,N/2] bfloat16 = silu(gate) * up over interleaved rows of W (no bias)
// epilogue 3: out[M,N] float += product + bias (not with norm)
// MS_UNSUPPORTED for shapes it does not take (the caller then uses ms_gemm_skinny): with any_shape = 0 all but
// those it is the faster kernel for; with any_shape = 1 (tests, measurements) only those it cannot compute
// (more than 63 tiles of W to a block, 47 with more than 48 rows, when the rows have to go through LDS in chunks).
extern "C" int ms_gemm_panel(const void* A, long long lda, const int* rows, const float* norm_w, float eps,
                             const void* W, long long ldw, const float* bias, void* out, long long ldo, int M, int N,
                             int K, int epilogue, int out_dtype, int norm, int any_shape, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (M > MAX_TOKENS) return MS_UNSUPPORTED;
  if (K <= 0 || K % 8 || ldw % 8 || lda < K || ldw < K || lda % (norm ? 4 : 8)) return MS_UNSUPPORTED;
  if (((uintptr_t)A | (uintptr_t)W) % 16 || (norm && ((uintptr_t)norm_w % 16))) return MS_UNSUPPORTED;
  if (norm && !norm_w) return MS_BAD_ARG;
  const bf16* w = (const bf16*)W;
#define RUN(EPI, TO, NORMV) return plan<EPI, TO, NORMV>(A, lda, w, ldw, bias, (TO*)out, ldo, M, N, K, norm_w, eps, rows, any_shape != 0, stream)
  if (epilogue == EPI_STORE) {
    if (ldo < N) return MS_BAD_ARG;
    if (out_dtype == MS_BF16) { if (norm) RUN(EPI_STORE, bf16, true); else RUN(EPI_STORE, bf16, false); }
    if (out_dtype == MS_F32) { if (norm) RUN(EPI_STORE, float, true); else RUN(EPI_STORE, float, false); }
    return MS_BAD_ARG;
  }
  if (epilogue == EPI_SWIGLU) {
    if (N % 2 || ldo < N / 2 || out_dtype != MS_BF16 || bias) return MS_BAD_ARG;
    if (norm) RUN(EPI_SWIGLU, bf16, true); else RUN(EPI_SWIGLU, bf16, false);
  }
  if (epilogue == EPI_RESIDUAL) {
    if (ldo < N || out_dtype != MS_F32 || norm) return MS_BAD_ARG;
    RUN(EPI_RESIDUAL, float, false);
  }
#undef RUN
  return MS_BAD_ARG;
}

// Column parts that ms_gemm_panel_splitk uses for this shape (the caller sizes `partial` by it); 0: not a
// shape for it.
extern "C" int ms_gemm_panel_splitk_parts(int M, int N, int K) { return splitk_parts(M, N, K); }

// The product with the columns of W split over blocks too: partial sums float [parts, M, N] in `partial`, then
// added up in part order into out with epilogue 0 (out_dtype float or bfloat16, + bias) or 3 (out float += ).
// A bfloat16 [M, lda], no folded norm.
extern "C" int ms_gemm_panel_splitk(const void* A, long long lda, const void* W, long long ldw, const float* bias,
                                    void* out, long long ldo, int M, int N, int K, int epilogue, int out_dtype,
                                    void* partial, int parts, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (parts <= 1 || parts != splitk_parts(M, N, K) || !partial) return MS_BAD_ARG;
  if (ldw % 8 || lda < K || ldw < K || lda % 8 || ldo < N) return MS_UNSUPPORTED;
  if (((uintptr_t)A | (uintptr_t)W | (uintptr_t)partial) % 16) return MS_UNSUPPORTED;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  if (epilogue == EPI_STORE && out_dtype == MS_BF16)
    return run_splitk<EPI_STORE, bf16>(a, lda, w, ldw, bias, (bf16*)out, ldo, M, N, K, (float*)partial, parts, stream);
  if (epilogue == EPI_STORE && out_dtype == MS_F32)
    return run_splitk<EPI_STORE, float>(a, lda, w, ldw, bias, (float*)out, ldo, M, N, K, (float*)partial, parts, stream);
  if (epilogue == EPI_RESIDUAL && out_dtype == MS_F32)
    return run_splitk<EPI_RESIDUAL, float>(a, lda, w, ldw, bias, (float*)out, ldo, M, N, K, (float*)partial, parts, stream);
  return MS_BAD_ARG;
}
