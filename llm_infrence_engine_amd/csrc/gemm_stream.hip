// out[M,N] = A[M,K] . W[N,K]^T for one group of tokens (M <= 16: a decode step of a small batch), bfloat16 in,
// float accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16), shaped by two measurements of this chip:
//
//   * what one CU can pull from memory is about 1/256 of what the chip can, so a product is only fast if every
//     CU streams an equal share of W: the rows of W are dealt out in units of four over as many blocks as
//     there are CUs (more for a wide W);
//   * a CU's time goes by the number of load instructions it issues (some 60 to 90 cycles each), not by the
//     bytes: every load here is 64 lanes reading 1 KB of one row in a piece, and the activations, which every
//     block needs whole, are read once per block in the same way instead of once per k-step as MFMA operands.
//
// So weights and activations go global -> registers -> LDS in 16-byte pieces, in stages of up to KC columns,
// and the waves read their MFMA operands from LDS (rows padded by one piece: conflict-free).  The loads of the
// next stage are in flight while the current one is multiplied.  The 16 waves take the 32-wide k-steps of a
// stage in turn and their accumulators are added through LDS in wave order, so a result does not depend on
// what else is in the batch.  The weight tile is the A operand and the activations the B operand: a lane ends
// up with 4 consecutive output features of one token.
//
// Epilogues and the folded RMS norm as in gemm_skinny: plain (+ bias) to bfloat16 or float; gated activation
// over interleaved rows (2j: gate j, 2j+1: up j); the residual sum out[m, n] += product (+ bias) on a float
// matrix, each element owned by one lane.  With NORM the activations are the float residual stream: the
// piece that goes to LDS is bfloat16(x * norm_weight), the squares are summed on the way in a fixed order, and
// the accumulators are scaled by rsqrt(mean(x^2) + eps) before the epilogue.
#include "common.h"
#include "api.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;   // a 16-byte piece: 8 bfloat16

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 3 };

// id / parts for the small numbers that occur here (id < 4096, parts <= 16) by a multiplication: dividing by a
// run-time value costs some twenty instructions even when both are the same for the whole wave, and the item
// arithmetic below would do it two dozen times before the first load is issued.
__device__ __forceinline__ int small_inverse(int parts) { return (65536 + parts - 1) / parts; }
__device__ __forceinline__ int small_div(int id, int inverse) { return (id * inverse) >> 16; }

constexpr int WAVES = 16;     // waves of a block
constexpr int WI_MAX = 6;     // weight loads a wave has in flight per stage (WAVES * WI_MAX KB of W per stage)
constexpr int XI_BF16 = 6;    // activation loads a wave has in flight per stage: bfloat16 rows (16 bytes a lane),
constexpr int XI_F32 = 2;     // float rows with their norm weights (64 bytes a lane)
constexpr int KC_MAX = 8192;  // columns of a stage at most

template <int NT, int EPI, typename TO, bool NORM>
__global__ void __launch_bounds__(WAVES * MS_WAVE)
gemm_stream_kernel(const void* __restrict__ Av, size_t lda, const bf16* __restrict__ W, size_t ldw,
                   const float* __restrict__ bias, TO* __restrict__ out, size_t ldo, int M, int N, int K,
                   const float* __restrict__ norm_w, float eps, const int* __restrict__ rows, int q, int rem,
                   int KC, int rcap) {
  constexpr int XI_MAX = NORM ? XI_F32 : XI_BF16;
  extern __shared__ u32x4 smem[];
  __shared__ float red_ss[XI_MAX * WAVES];
  const bf16* A = (const bf16*)Av;
  const float* X = (const float*)Av;
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);   // the same for the whole wave
  const int col = lane & 15, kq = lane >> 4;
  // this block's rows of W: units of four, dealt out evenly (the first `rem` blocks take one unit more)
  const int b = blockIdx.x;
  const int r0 = 4 * (b * q + min(b, rem));
  const int R = 4 * (q + (b < rem ? 1 : 0));   // at most 16 * NT and at most rcap; may run past N in the last block
  const int C8cap = min(KC, (K + 31) / 32 * 32) / 8;   // pieces per row of a full stage
  const int pitch = C8cap + 2;   // rows an odd number of 32 bytes apart: 16-byte fragment reads at the full LDS rate
  const int parts = (C8cap + 63) / 64;                  // loads per row and stage
  const int parts_inv = small_inverse(parts);
  u32x4* wst = smem;
  u32x4* xst = smem + (size_t)rcap * pitch;

  // what the epilogue will need from memory is asked for now, so that it arrives under the main loop:
  // tile u is finished by wave u
  f32x4 pre = {0.f, 0.f, 0.f, 0.f}, bv = {0.f, 0.f, 0.f, 0.f};
  if (wave < NT) {
    const int f = wave * 16 + kq * 4;   // first of this lane's four features within the block
    const int nb = r0 + f;
    if (f < R && col < M) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (nb + r >= N) continue;
        if (bias && EPI != EPI_SWIGLU) bv[r] = bias[nb + r];
        if (EPI == EPI_RESIDUAL) pre[r] = reinterpret_cast<const float*>(out)[(size_t)col * ldo + nb + r];
      }
    }
  }

  // the activation loads of this wave: item id = wave + j * WAVES is (token, part), the same in every stage
  size_t xoff[XI_MAX];
  int xtok[XI_MAX], xpart[XI_MAX];
  float ss[XI_MAX];
#pragma unroll
  for (int j = 0; j < XI_MAX; ++j) {
    const int id = wave + j * WAVES;
    xtok[j] = small_div(id, parts_inv);
    xpart[j] = id - xtok[j] * parts;
    if (xtok[j] >= M) xtok[j] = -1;
    xoff[j] = xtok[j] < 0 ? 0 : (size_t)(rows ? rows[xtok[j]] : xtok[j]) * lda;
    ss[j] = 0.f;
  }

  u32x4 wreg[WI_MAX];
  u32x4 xreg[NORM ? 1 : XI_MAX];
  f32x4 xf[NORM ? XI_MAX : 1][2], nwf[NORM ? XI_MAX : 1][2];
  const u32x4 zero = {0u, 0u, 0u, 0u};

  // global -> registers for the stage that starts at column k0 and has S8 pieces per row
  auto issue = [&](int k0, int S8) {
    const int parts_s = (S8 + 63) / 64;
    const int inv_s = parts_s == parts ? parts_inv : small_inverse(parts_s);
    // the weights first: they come from HBM, the activations from L2
#pragma unroll
    for (int j = 0; j < WI_MAX; ++j) {
      const int id = wave + j * WAVES;
      if (id >= R * parts_s) break;   // the same for the whole wave
      const int row = small_div(id, inv_s), c = (id - row * parts_s) * 64 + lane;
      wreg[j] = *reinterpret_cast<const u32x4*>(W + (size_t)min(r0 + row, N - 1) * ldw + k0 + (size_t)min(c, S8 - 1) * 8);
    }
#pragma unroll
    for (int j = 0; j < XI_MAX; ++j) {
      const int c = xpart[j] * 64 + lane;
      if (xtok[j] < 0 || xpart[j] >= parts_s) continue;   // the same for the whole wave
      const bool in = c < S8;
      const size_t at = xoff[j] + k0 + (size_t)min(c, S8 - 1) * 8;
      if (NORM) {
        xf[j][0] = *reinterpret_cast<const f32x4*>(X + at);
        xf[j][1] = *reinterpret_cast<const f32x4*>(X + at + 4);
        nwf[j][0] = *reinterpret_cast<const f32x4*>(norm_w + k0 + min(c, S8 - 1) * 8);
        nwf[j][1] = *reinterpret_cast<const f32x4*>(norm_w + k0 + min(c, S8 - 1) * 8 + 4);
        if (!in) xf[j][0] = xf[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
      } else {
        xreg[j] = *reinterpret_cast<const u32x4*>(A + at);
      }
    }
  };
  // registers -> LDS
  auto commit = [&](int S8) {
    const int parts_s = (S8 + 63) / 64;
    const int inv_s = parts_s == parts ? parts_inv : small_inverse(parts_s);
#pragma unroll
    for (int j = 0; j < XI_MAX; ++j) {
      const int c = xpart[j] * 64 + lane;
      if (xtok[j] < 0 || xpart[j] >= parts_s) continue;
      u32x4 piece;
      if (NORM) {
        bf16x8 h;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float x0 = xf[j][0][i], x1 = xf[j][1][i];
          ss[j] = fmaf(x0, x0, ss[j]);
          ss[j] = fmaf(x1, x1, ss[j]);
          h[i] = (__bf16)(x0 * nwf[j][0][i]);
          h[4 + i] = (__bf16)(x1 * nwf[j][1][i]);
        }
        piece = __builtin_bit_cast(u32x4, h);
      } else {
        piece = xreg[j];
      }
      if (c < S8) xst[xtok[j] * pitch + c] = piece;
    }
#pragma unroll
    for (int j = 0; j < WI_MAX; ++j) {
      const int id = wave + j * WAVES;
      if (id >= R * parts_s) break;
      const int row = small_div(id, inv_s), c = (id - row * parts_s) * 64 + lane;
      if (c < S8) wst[row * pitch + c] = wreg[j];
    }
    // a last k-step that K fills only in part reads zeros for the rest
    const int padn = (4 - (S8 & 3)) & 3;
    for (int t = threadIdx.x; t < (R + M) * padn; t += WAVES * MS_WAVE) {
      const int rr = t / padn, cc = S8 + t - rr * padn;
      if (rr < R) wst[rr * pitch + cc] = zero; else xst[(rr - R) * pitch + cc] = zero;
    }
  };

  f32x4 acc[NT];
#pragma unroll
  for (int u = 0; u < NT; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int K8 = K / 8;
  const int xrow = min(col, M - 1) * pitch;   // idle columns repeat the last token; their results are not stored
  int arow[NT];
#pragma unroll
  for (int u = 0; u < NT; ++u) arow[u] = min(u * 16 + col, R - 1) * pitch;   // rows past the block's repeat its last

  issue(0, min(C8cap, K8));
  for (int k0 = 0; k0 < K; k0 += C8cap * 8) {
    const int S8 = min(C8cap, K8 - k0 / 8);
    commit(S8);
    __syncthreads();
    const int k1 = k0 + C8cap * 8;
    if (k1 < K) issue(k1, min(C8cap, K8 - k1 / 8));   // in flight while this stage is multiplied
    const int steps = (S8 + 3) / 4;
    for (int s = wave; s < steps; s += WAVES) {
      const bf16x8 xb = __builtin_bit_cast(bf16x8, xst[xrow + 4 * s + kq]);
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        if (u * 16 >= R) break;   // the same for the whole block
        const bf16x8 wa = __builtin_bit_cast(bf16x8, wst[arow[u] + 4 * s + kq]);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb, acc[u], 0, 0, 0);
      }
    }
    __syncthreads();   // the stage's buffers are free again
  }

  if (NORM) {   // a token's squares: lanes of a load in a fixed tree, then its loads in order
#pragma unroll
    for (int j = 0; j < XI_MAX; ++j) {
      const float v = wave_sum(ss[j]);
      if (lane == 0) red_ss[wave + j * WAVES] = v;
    }
  }
  // tile u is finished by wave u; every other wave leaves its share in LDS (the stage buffers are free)
  f32x4* red = reinterpret_cast<f32x4*>(smem);   // [WAVES - 1][NT][64]
#pragma unroll
  for (int u = 0; u < NT; ++u) {
    if (u * 16 >= R) break;
    if (wave != u) red[((wave < u ? wave : wave - 1) * NT + u) * MS_WAVE + lane] = acc[u];
  }
  __syncthreads();

#pragma unroll
  for (int u = 0; u < NT; ++u) {
    if (wave != u || u * 16 >= R) continue;
    // sum in wave order: the waves below the owner, the owner itself, the waves above
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < WAVES; ++w) sum += w == u ? acc[u] : red[((w < u ? w : w - 1) * NT + u) * MS_WAVE + lane];
    if (NORM) {
      float total = 0.f;
      const int tok = min(col, M - 1);
      for (int p = 0; p < parts; ++p) total += red_ss[tok * parts + p];
      sum *= 1.0f / sqrtf(total / (float)K + eps);
    }
    // lane holds out[m = col][n = nb + r], r = 0..3
    const int f = u * 16 + kq * 4;
    const int nb = r0 + f;
    if (col >= M || f >= R) continue;
    if (EPI == EPI_SWIGLU) {
      // rows nb, nb+1 are (gate, up) of feature nb/2; rows nb+2, nb+3 of feature nb/2 + 1
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        if (nb + 2 * p + 1 < N) {
          const float g = sum[2 * p], up = sum[2 * p + 1];
          out[(size_t)col * ldo + nb / 2 + p] = from_float<TO>(fast_silu(g) * up);
        }
      }
    } else {
      TO* o = out + (size_t)col * ldo + nb;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (nb + r < N) o[r] = from_float<TO>(sum[r] + bv[r] + pre[r]);
      }
    }
  }
}

constexpr int LDS_BUDGET = 120 * 1024;   // of the CU's 160 KB, for the stage buffers

template <int NT, int EPI, typename TO, bool NORM>
int launch(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M, int N,
           int K, const float* norm_w, float eps, const int* rows, int blocks, int q, int rem, int KC, int rcap,
           size_t lds, hipStream_t stream) {
  static bool raised = false;   // once per instantiation: allow more dynamic LDS than the default 64 KB
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_stream_kernel<NT, EPI, TO, NORM>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BUDGET) != hipSuccess)
      return MS_LAUNCH_FAILED;
    raised = true;
  }
  gemm_stream_kernel<NT, EPI, TO, NORM><<<dim3(blocks), dim3(WAVES * MS_WAVE), lds, stream>>>(
      A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, q, rem, KC, rcap);
  return ms_launch_status();
}

template <int EPI, typename TO, bool NORM>
int plan(const void* A, size_t lda, const bf16* W, size_t ldw, const float* bias, TO* out, size_t ldo, int M, int N,
         int K, const float* norm_w, float eps, const int* rows, bool any_shape, hipStream_t stream) {
  const int cus = ms_compute_units();
  const int units = (N + 3) / 4;
  // Where this kernel wins, by measurement against ms_gemm_skinny (which costs less to set up and has no LDS
  // stage between the loads and the matrix cores): few rows of W per CU and many columns: the down projection
  // of the 0.5B shape, 896 x 4864: 6.2 us against 8.0 at one token, 7.1 against 9.5 at 8, 10.0 against 11.0 at
  // 16.  There a block of the other kernel spends its time on the activations, which it reads as MFMA operands,
  // one load a k-step.  Wider or shorter matrices were slower here by 5 to 30 %.
  if (!any_shape && (units > cus || K < 2048)) return MS_UNSUPPORTED;
  if (units > 16 * cus) return MS_UNSUPPORTED;   // more than 64 rows to a block
  const int blocks = units < cus ? units : cus;
  const int q = units / blocks, rem = units % blocks;
  const int rcap = 4 * (q + (rem ? 1 : 0));
  const int nt = (rcap + 15) / 16;
  if (nt > 4) return MS_UNSUPPORTED;
  // the widest stage whose loads fit the registers and whose pieces fit LDS
  const int k32 = (K + 31) / 32 * 32;
  int KC = 0;
  size_t lds = 0;
  for (int kc = KC_MAX; kc >= 256; kc /= 2) {
    const int c8 = (kc < k32 ? kc : k32) / 8, parts = (c8 + 63) / 64;
    lds = (size_t)(rcap + M) * (c8 + 2) * 16;
    if (rcap * parts <= WI_MAX * WAVES && M * parts <= (NORM ? XI_F32 : XI_BF16) * WAVES && lds <= (size_t)LDS_BUDGET) {
      KC = kc;
      break;
    }
  }
  if (!KC) return MS_UNSUPPORTED;
  const size_t red = (size_t)(WAVES - 1) * nt * MS_WAVE * 16;
  if (lds < red) lds = red;
#define GO(NTV) if (nt == NTV) return launch<NTV, EPI, TO, NORM>(A, lda, W, ldw, bias, out, ldo, M, N, K, norm_w, eps, rows, blocks, q, rem, KC, rcap, lds, stream)
  GO(1); GO(2); GO(3); GO(4);
#undef GO
  return MS_UNSUPPORTED;
}

}  // namespace

// The product of up to 16 rows with W[N,K]^T.  norm = 0: A is bfloat16 [M, lda]; norm = 1: A is the float residual
// stream and the RMS norm (norm_w[K], eps) is folded in; rows (int32 [M], may be null) gathers the rows of A.
// epilogue 0: out[M,N] (out_dtype float or bfloat16) = product + bias
// epilogue 1: out[M,N/2] bfloat16 = silu(gate) * up over interleaved rows of W (no bias)
// epilogue 3: out[M,N] float += product + bias (not with norm)
// MS_UNSUPPORTED for shapes it does not take (the caller then uses ms_gemm_skinny): with any_shape = 0 all but
// those it is the faster kernel for; with any_shape = 1 (tests, measurements) only those it cannot compute.
extern "C" int ms_gemm_stream(const void* A, long long lda, const int* rows, const float* norm_w, float eps,
                              const void* W, long long ldw, const float* bias, void* out, long long ldo, int M, int N,
                              int K, int epilogue, int out_dtype, int norm, int any_shape, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (M > 16) return MS_UNSUPPORTED;
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
