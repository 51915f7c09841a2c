// C[M,N] (+)= A[M,K] . W[N,K]^T (+ bias[N]) with float accumulation on the vector ALUs.
// This is the true 32-bit matrix product of the float path (no reduced-precision matrix mode) and the
// any-shape fallback of the bfloat16 path.  Every output element sums its K products in the same
// order whatever M is, so a token's result does not depend on what else is in the batch.
#include "common.h"
#include "api.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;

template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float4 type; };
template <> struct Vec4<bf16> { typedef uint2 type; };

__device__ __forceinline__ void unpack4(const float4& v, float* o) { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
__device__ __forceinline__ void unpack4(const uint2& v, float* o) {
  o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
  o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
}

// Loads 4 consecutive k values of one row into o (zeros outside the matrix).
template <typename T, bool VEC>
__device__ __forceinline__ void load4(const T* __restrict__ base, int row, int n_rows, size_t ld, int k, int K, float* o) {
  if (row >= n_rows || k >= K) { o[0] = o[1] = o[2] = o[3] = 0.f; return; }
  const T* p = base + (size_t)row * ld + k;
  if (VEC) {
    unpack4(*reinterpret_cast<const typename Vec4<T>::type*>(p), o);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (k + i < K) ? to_float(p[i]) : 0.f;
  }
}

template <typename TA, typename TC, bool VEC>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const TA* __restrict__ A, const TA* __restrict__ W, const float* __restrict__ bias,
                    TC* __restrict__ C, int M, int N, int K, size_t lda, size_t ldw, size_t ldc, int accumulate) {
  __shared__ float As[BK][BM + PAD];
  __shared__ float Ws[BK][BN + PAD];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int lrow = tid >> 2, lk = (tid & 3) * 4;  // this thread stages row lrow, k offset lk of both tiles

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    float a4[4], w4[4];
    load4<TA, VEC>(A, m0 + lrow, M, lda, k0 + lk, K, a4);
    load4<TA, VEC>(W, n0 + lrow, N, ldw, k0 + lk, K, w4);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) { As[lk + i][lrow] = a4[i]; Ws[lk + i][lrow] = w4[i]; }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      const float4 a = *reinterpret_cast<const float4*>(&As[k][ty * 4]);
      const float4 w = *reinterpret_cast<const float4*>(&Ws[k][tx * 4]);
      const float av[4] = {a.x, a.y, a.z, a.w}, wv[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      TC* c = C + (size_t)m * ldc + n;
      if (accumulate) v += to_float(*c);
      *c = from_float<TC>(v);
    }
  }
}

template <typename TA, typename TC>
int launch(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, size_t lda, size_t ldw,
           size_t ldc, int accumulate, hipStream_t stream) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM), block(256);
  const size_t vec_bytes = 4 * sizeof(TA);
  const bool vec = (K % 4 == 0) && (lda % 4 == 0) && (ldw % 4 == 0) && ((uintptr_t)A % vec_bytes == 0) &&
                   ((uintptr_t)W % vec_bytes == 0);
  if (vec)
    gemm_generic_kernel<TA, TC, true><<<grid, block, 0, stream>>>((const TA*)A, (const TA*)W, bias, (TC*)C, M, N, K, lda, ldw, ldc, accumulate);
  else
    gemm_generic_kernel<TA, TC, false><<<grid, block, 0, stream>>>((const TA*)A, (const TA*)W, bias, (TC*)C, M, N, K, lda, ldw, ldc, accumulate);
  return ms_launch_status();
}

}  // namespace

extern "C" int ms_gemm_generic(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                               long long lda, long long ldw, long long ldc, int in_dtype, int out_dtype,
                               int accumulate, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return MS_BAD_ARG;
  if ((long long)((M + BM - 1) / BM) > 65535) return MS_UNSUPPORTED;
  if (in_dtype == MS_F32 && out_dtype == MS_F32) return launch<float, float>(A, W, bias, C, M, N, K, lda, ldw, ldc, accumulate, stream);
  if (in_dtype == MS_BF16 && out_dtype == MS_BF16) return launch<bf16, bf16>(A, W, bias, C, M, N, K, lda, ldw, ldc, accumulate, stream);
  if (in_dtype == MS_BF16 && out_dtype == MS_F32) return launch<bf16, float>(A, W, bias, C, M, N, K, lda, ldw, ldc, accumulate, stream);
  return MS_BAD_ARG;
}
