// Shared helpers of the gfx950 kernels: element types, conversions, wave/block reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define MS_WAVE 64
#define MS_MAX_GROUPS 8   // cache groups one ms_decode_advance / ms_table_update call serves

// Element type codes of the C entry points.
enum { MS_F32 = 0, MS_BF16 = 1 };

// Error codes returned by the C entry points (0 = launched).
enum { MS_OK = 0, MS_BAD_ARG = 1, MS_UNSUPPORTED = 2, MS_LAUNCH_FAILED = 3 };

typedef __hip_bfloat16 bf16;

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return __bfloat162float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return __float2bfloat16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, MS_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = MS_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MS_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` holds 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int nwaves = (blockDim.x + MS_WAVE - 1) / MS_WAVE;
  v = wave_sum(v);
  __syncthreads();  // `red` may still be read from a previous call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += red[i];
  return t;
}

// g * sigmoid(g) through the hardware's exp2 and reciprocal (each good to about one unit in the last place of
// a float; the callers round the result to bfloat16)
__device__ __forceinline__ float fast_silu(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

// sin and cos of a rotation angle for bfloat16 results: three-part Cody-Waite reduction by pi/2 (the first
// two parts have 11 bits, so n * part is exact for |x| < 2^13 * pi/2) and short polynomials on [-pi/4, pi/4];
// absolute error ~2e-7.  Larger angles take the library routine.
__device__ __forceinline__ void ms_sincos_rot(float x, float* sn, float* cs) {
  if (fabsf(x) > 12000.f) { sincosf(x, sn, cs); return; }
  const float n = rintf(x * 0.636619772367581343f);
  float r = fmaf(-n, 1.5703125f, x);
  r = fmaf(-n, 4.837512969970703e-4f, r);
  r = fmaf(-n, 7.549790126404332e-08f, r);
  const float r2 = r * r;
  const float sp = fmaf(r2, fmaf(r2, fmaf(r2, 2.7557314297e-6f, -1.9841270114e-4f), 8.3333337680e-3f), -1.6666667163e-1f);
  const float s0 = fmaf(r * r2, sp, r);
  const float cp = fmaf(r2, fmaf(r2, fmaf(r2, 2.4801587642e-5f, -1.3888889225e-3f), 4.1666667908e-2f), -0.5f);
  const float c0 = fmaf(r2, cp, 1.0f);
  const int q = (int)n & 3;
  const float s1 = (q & 1) ? c0 : s0, c1 = (q & 1) ? s0 : c0;
  *sn = (q & 2) ? -s1 : s1;
  *cs = ((q + 1) & 2) ? -c1 : c1;
}

// Compute units of the current device (256 on an MI355X); asked once.
static inline int ms_compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) n = v;
    else n = 256;
  }
  return n;
}

static inline int ms_launch_status() {
  return hipGetLastError() == hipSuccess ? MS_OK : MS_LAUNCH_FAILED;
}
