// out[M,N] = A[M,K] . W[N,K]^T for many tokens (prompt portions), bfloat16 in, float accumulation on the
// matrix cores (v_mfma_f32_16x16x32_bf16), with the gated activation as an epilogue: the product of the
// interleaved gate/up weight never goes to memory, which saves the write of [M, 2I], its read and a kernel.
//
// A block of 8 waves owns a tile of BN features by BM tokens, as large as registers allow (256 x 256: a byte
// loaded does 128 multiply-adds; a CU draws some 80 GB/s from L2).  Per step of 64 columns the tile's rows of W
// and A go from memory straight to LDS (global_load_lds, 16 bytes a lane: no registers, no LDS write
// instructions) into one of two buffers, a step before they are multiplied.  LDS rows are 128 bytes with their
// eight 16-byte pieces permuted by the row number (piece c at place c ^ (row & 7)): fragment reads then run at
// the full LDS rate (measured 237 bytes a clock; rows 144 bytes apart give 116).  A step has one barrier, in
// its middle, and the matrix pipe has work on both sides of it (see the main loop).
//
// W is the A operand of the MFMA and the tokens the B operand, so a lane ends up with 4 output features of one
// token per tile.  Which 16 features make up a tile is free: tile i of a wave takes, for q = 0..3, the four
// features q * 4 FT + i * 4 .. + 3 of the wave's FT * 16, so that the lane with quarter q holds 4 FT consecutive
// features of its token over its FT tiles and stores them as one run.
#include "common.h"
#include "api.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum { EPI_STORE = 0, EPI_SWIGLU = 1 };

constexpr int BK = 64;                  // columns a step
constexpr int PITCH = BK;               // LDS rows of 128 bytes; piece c of row l lies at place c ^ (l & 7)

// LDS row l of the block's W rows (l < WF * FT * 16) holds this feature of the tile
template <int FT>
__device__ __forceinline__ int feature_of_row(int l) {
  const int wf = l / (FT * 16), rem = l - wf * (FT * 16);
  const int i = rem >> 4, rr = rem & 15;
  return wf * (FT * 16) + (rr >> 2) * (4 * FT) + i * 4 + (rr & 3);
}

// The instruction order of a step's first half, told to the scheduler: before the TT products of tile I the reads
// that the source has there (the next tile of W but for the last, tile I of the second half, token fragment I
// of the second half while there are any).  0x100: reads from LDS, 0x008: matrix instructions.
template <int I, int FT, int TT>
struct FirstHalfOrder {
  static __device__ __forceinline__ void apply() {
    __builtin_amdgcn_sched_group_barrier(0x100, (I + 1 < FT ? 1 : 0) + 1 + (I < TT ? 1 : 0), 0);
    __builtin_amdgcn_sched_group_barrier(0x008, TT, 0);
    FirstHalfOrder<I + 1, FT, TT>::apply();
  }
};
template <int FT, int TT>
struct FirstHalfOrder<FT, FT, TT> {
  static __device__ __forceinline__ void apply() {}
};

// WF x WT waves along features and tokens, each with FT x TT tiles of 16 x 16.  K is a multiple of 64.
template <int WF, int WT, int FT, int TT, int EPI, typename TO>
__global__ void __launch_bounds__(WF * WT * MS_WAVE)
gemm_tiled_kernel(const bf16* __restrict__ A, size_t lda, const bf16* __restrict__ W, size_t ldw,
                  TO* __restrict__ out, size_t ldo, int M, int N, int K, int m_tiles, int n_tiles) {
  constexpr int NWAVES = WF * WT, THREADS = NWAVES * MS_WAVE;
  constexpr int BN = WF * FT * 16, BM = WT * TT * 16, ROWS = BN + BM;
  constexpr int LOADS = ROWS / 8 / NWAVES;   // loads of 8 rows (1 KB) a wave makes per step
  static_assert(ROWS % (8 * NWAVES) == 0, "the tile's rows are dealt out evenly");
  static_assert(TT < FT, "the main loop reads the token fragments beside the first TT + 1 tiles of W");
  extern __shared__ __align__(16) unsigned char lds_raw[];
  bf16* lds = reinterpret_cast<bf16*>(lds_raw);          // two buffers of ROWS x PITCH

  // Blocks with consecutive ids go to consecutive XCDs, each with an L2 of its own: an XCD takes every eighth
  // tile of W with all token tiles (those fastest), so a tile of W is read from memory by one XCD only.  The
  // host launches 8 * ceil(n_tiles / 8) * m_tiles blocks; one without a tile leaves.
  const int nt = ((int)(blockIdx.x >> 3) / m_tiles) * 8 + (blockIdx.x & 7);
  const int mt = (int)(blockIdx.x >> 3) % m_tiles;
  if (nt >= n_tiles) return;
  const int n0 = nt * BN, m0 = mt * BM;
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int wf = wave % WF, wt = wave / WF;
  const int col = lane & 15, kq = lane >> 4;

  // Load p of a wave fills LDS rows (wave + p * NWAVES) * 8 .. + 7: lane l's 16 bytes land at l * 16 of that 1 KB,
  // which is place l & 7 of row l >> 3, so the lane asks memory for the piece that belongs there.  Rows past the
  // end of W or A repeat the last row (their results are not stored).
  const bf16* src[LOADS];
#pragma unroll
  for (int p = 0; p < LOADS; ++p) {
    const int l = (wave + p * NWAVES) * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ (l & 7);
    if (l < BN) src[p] = W + (size_t)min(n0 + feature_of_row<FT>(l), N - 1) * ldw + piece * 8;
    else src[p] = A + (size_t)min(m0 + l - BN, M - 1) * lda + piece * 8;
  }
  typedef __attribute__((address_space(3))) void lds_void;
  typedef const __attribute__((address_space(1))) void global_void;
  auto load_rows = [&](int k, int buffer) {
#pragma unroll
    for (int p = 0; p < LOADS; ++p)
      __builtin_amdgcn_global_load_lds((global_void*)(src[p] + k),
                                       (lds_void*)(lds + buffer + (wave + p * NWAVES) * 8 * PITCH), 16, 0, 0);
  };

  f32x4 acc[FT][TT];
#pragma unroll
  for (int i = 0; i < FT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // a lane's fragment pieces: columns kq * 8 of the first 32 columns of a step at place kq ^ (row & 7), of the
  // second 32 at that place ^ 4 (rows of a tile start at a multiple of 16, so row & 7 is col & 7)
  static_assert(BK == 64, "a step is two products of 32 columns deep");
  const int place0 = (kq ^ (col & 7)) * 8, place1 = ((kq + 4) ^ (col & 7)) * 8;
  const bf16* w_frag = lds + (wf * FT * 16 + col) * PITCH;
  const bf16* a_frag = lds + (BN + wt * TT * 16 + col) * PITCH;

  // A step has one barrier, in its middle.  First half: the products of the first 32 columns, whose token
  // fragments are in registers already and whose tiles of W are read one ahead; meanwhile every fragment of the
  // second 32 columns is read too.  Then nothing of this step is left in its buffer: the wave waits for the rows
  // of the next step (asked for a step ago), the barrier makes them visible to all and says that all are done
  // with this buffer, and the rows of the step after next are asked for into it.  Second half: the products of
  // the second 32 columns from registers, meanwhile the first fragments of the next step are read.  So no read
  // from LDS and no load from memory is waited for with the matrix pipe idle, except at the barrier itself.
  const int steps = K / BK;
  load_rows(0, 0);
  if (steps > 1) load_rows(BK, ROWS * PITCH);
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the loads to LDS have landed
  __syncthreads();
  bf16x8 a0[TT], a1[TT], w1[FT];
#pragma unroll
  for (int j = 0; j < TT; ++j) a0[j] = *reinterpret_cast<const bf16x8*>(a_frag + j * 16 * PITCH + place0);
  bf16x8 w_next = *reinterpret_cast<const bf16x8*>(w_frag + place0);
  for (int s = 0; s < steps; ++s) {
    const int buf = (s & 1) * ROWS * PITCH, other = ((s + 1) & 1) * ROWS * PITCH;
#pragma unroll
    for (int i = 0; i < FT; ++i) {
      const bf16x8 w_cur = w_next;
      if (i + 1 < FT) w_next = *reinterpret_cast<const bf16x8*>(w_frag + buf + (i + 1) * 16 * PITCH + place0);
      w1[i] = *reinterpret_cast<const bf16x8*>(w_frag + buf + i * 16 * PITCH + place1);
      if (i < TT) a1[i] = *reinterpret_cast<const bf16x8*>(a_frag + buf + i * 16 * PITCH + place1);
#pragma unroll
      for (int j = 0; j < TT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur, a0[j], acc[i][j], 0, 0, 0);
    }
    // the order of the instructions (left to itself the compiler reads a fragment right before its products and
    // waits for it): the reads written before each group of TT products stay there
    FirstHalfOrder<0, FT, TT>::apply();
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) and lgkmcnt(0): the next step's rows have landed, this step's are read
    __syncthreads();
    if (s + 2 < steps) load_rows((s + 2) * BK, buf);
    // (after the last step these reads bring what nobody uses)
#pragma unroll
    for (int i = 0; i < FT; ++i) {
      if (i < TT) a0[i] = *reinterpret_cast<const bf16x8*>(a_frag + other + i * 16 * PITCH + place0);
      if (i == TT) w_next = *reinterpret_cast<const bf16x8*>(w_frag + other + place0);
#pragma unroll
      for (int j = 0; j < TT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[i], a1[j], acc[i][j], 0, 0, 0);
    }
  }

  // the lane's run of 4 FT features of token m (tile j): acc[i][j][r] is feature f0 + i * 4 + r
  const int f0 = n0 + wf * (FT * 16) + kq * (4 * FT);
#pragma unroll
  for (int j = 0; j < TT; ++j) {
    const int m = m0 + wt * TT * 16 + j * 16 + col;
    if (m >= M) continue;
    if (EPI == EPI_SWIGLU) {   // features 2g, 2g + 1 are gate g and up g: 2 FT outputs from o0 on
      const int o0 = f0 / 2, n_out = N / 2;
      TO* o = out + (size_t)m * ldo + o0;
      float v[2 * FT];
#pragma unroll
      for (int i = 0; i < FT; ++i) {
        v[2 * i] = fast_silu(acc[i][j][0]) * acc[i][j][1];
        v[2 * i + 1] = fast_silu(acc[i][j][2]) * acc[i][j][3];
      }
      if (o0 + 2 * FT <= n_out && ((uintptr_t)o & 15) == 0 && sizeof(TO) == 2) {
#pragma unroll
        for (int g = 0; g < 2 * FT; g += 8) {
          bf16x8 pk;
#pragma unroll
          for (int e = 0; e < 8; ++e) pk[e] = (__bf16)v[g + e];
          *reinterpret_cast<bf16x8*>(reinterpret_cast<bf16*>(o) + g) = pk;
        }
      } else {
#pragma unroll
        for (int g = 0; g < 2 * FT; ++g)
          if (o0 + g < n_out) o[g] = from_float<TO>(v[g]);
      }
    } else {
      TO* o = out + (size_t)m * ldo + f0;
      if (f0 + 4 * FT <= N && ((uintptr_t)o & 15) == 0 && sizeof(TO) == 2) {
#pragma unroll
        for (int g = 0; g < 4 * FT; g += 8) {
          bf16x8 pk;
#pragma unroll
          for (int e = 0; e < 8; ++e) pk[e] = (__bf16)acc[(g + e) >> 2][j][(g + e) & 3];
          *reinterpret_cast<bf16x8*>(reinterpret_cast<bf16*>(o) + g) = pk;
        }
      } else {
#pragma unroll
        for (int g = 0; g < 4 * FT; ++g)
          if (f0 + g < N) o[g] = from_float<TO>(acc[g >> 2][j][g & 3]);
      }
    }
  }
}

template <int WF, int WT, int FT, int TT, int EPI, typename TO>
int launch(const bf16* A, size_t lda, const bf16* W, size_t ldw, TO* out, size_t ldo, int M, int N, int K,
           hipStream_t stream) {
  constexpr int BN = WF * FT * 16, BM = WT * TT * 16;
  constexpr size_t lds = 2 * (size_t)(BN + BM) * PITCH * sizeof(bf16);
  static bool raised = false;   // once per instantiation: allow more dynamic LDS than the default 64 KB
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiled_kernel<WF, WT, FT, TT, EPI, TO>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return MS_LAUNCH_FAILED;
    raised = true;
  }
  const int n_tiles = (N + BN - 1) / BN, m_tiles = (M + BM - 1) / BM;
  const long long blocks = (long long)((n_tiles + 7) / 8) * 8 * m_tiles;
  if (blocks > 0x7fffffffLL) return MS_UNSUPPORTED;
  gemm_tiled_kernel<WF, WT, FT, TT, EPI, TO><<<dim3((unsigned)blocks), dim3(WF * WT * MS_WAVE), lds, stream>>>(
      A, lda, W, ldw, out, ldo, M, N, K, m_tiles, n_tiles);
  return ms_launch_status();
}

int g_tile = 0;   // measurements: 0 leaves the choice of tile, 1, 2 and 3 force one

// Tiles of 256 x 256 (a byte loaded does 128 multiply-adds; one block to a CU, 1.7 us a step of 64 columns, in
// whole rounds over the CUs) or of 128 x 128 (two blocks to a CU, 1.26 us a step each; they end at different
// times, so their rounds are counted as they come, plus 0.3 for the last): the one that takes less.  Agrees
// with the measured choice at 65 to 8,192 tokens of the 0.5B to 32B gate/up shapes but for near ties.
int choose_tile(int M, int N) {
  const long long cus = ms_compute_units();
  const long long big = (long long)((N + 255) / 256) * ((M + 255) / 256);
  const long long small = (long long)((N + 127) / 128) * ((M + 127) / 128);
  // fewer tiles of 128 x 128 than CUs: tiles of 64 x 64 (four waves) put four times as many CUs to work, and a
  // tile's time is the time its CU needs to draw its rows (q/k/v of the 0.5B shape, 512 tokens: 11.3 -> 8.7 us;
  // gate/up at 128 tokens 16.6 -> 12.9, at 256 tokens 16.0 -> 14.9; from 512 tokens on 20.4 against 25.5)
  if (small < cus) return 3;
  const double t_big = (double)((big + cus - 1) / cus) * 1.70;
  const double t_small = ((double)small / (double)(2 * cus) + 0.3) * 1.26;
  return t_big <= t_small ? 1 : 2;
}

}  // namespace

extern "C" void ms_gemm_tiled_force(int tile) { g_tile = tile; }

// Whether the gated product of M tokens is faster here than as the library's product and an activation kernel
// (measured with a different W every call, 65 to 8,192 tokens): up to 1,536 columns always (0.5 to 0.98 of the
// library's time); beyond that the two are within 15 % of each other either way, and this kernel is taken where it
// won throughout: up to 2,048 tokens whose 256 x 256 tiles fill at least 9/10 of their last round over the CUs.
extern "C" int ms_gemm_tiled_pays(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % BK) return 0;
  if (K <= 1536) return 1;
  if (M > 2048) return 0;
  const long long cus = ms_compute_units();
  const long long big = (long long)((N + 255) / 256) * ((M + 255) / 256);
  return big * 10 >= ((big + cus - 1) / cus) * cus * 9;
}

// A bfloat16 [M, lda], W bfloat16 [N, ldw] (rows of K, K a multiple of 64), out bfloat16.
// epilogue 0: out[M, N] = product;  epilogue 1: out[M, N / 2] = silu(gate) * up over interleaved rows of W.
extern "C" int ms_gemm_tiled(const void* A, long long lda, const void* W, long long ldw, void* out, long long ldo, int M,
                             int N, int K, int epilogue, hipStream_t stream) {
  if (M <= 0 || N <= 0) return MS_OK;
  if (K <= 0 || K % BK || lda % 8 || ldw % 8 || lda < K || ldw < K) return MS_UNSUPPORTED;
  if (((uintptr_t)A | (uintptr_t)W) % 16) return MS_UNSUPPORTED;
  if (epilogue == EPI_SWIGLU ? (N % 2 || ldo < N / 2) : (epilogue != EPI_STORE || ldo < N)) return MS_BAD_ARG;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  bf16* o = (bf16*)out;
  int tile = g_tile;
  if (tile == 0) tile = choose_tile(M, N);
#define GO(WF, WT, FT, TT) return epilogue == EPI_SWIGLU ? launch<WF, WT, FT, TT, EPI_SWIGLU, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream) \
                                                        : launch<WF, WT, FT, TT, EPI_STORE, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream)
  if (tile == 1) GO(2, 4, 8, 4);   // 256 x 256
  if (tile == 3) GO(1, 4, 4, 1);   // 64 x 64, four waves
  GO(2, 4, 4, 2);                  // 128 x 128
#undef GO
}

// Whether a plain product of M tokens should run here rather than in the library.  On the GPU the library's
// kernels are as fast or faster; but a call into the library costs the host 19 us and a call here 5, and a
// portion of up to about a thousand tokens of a narrow model is over on the GPU before the host has enqueued
// its 200 launches.  Measured at the 0.5B shape with the q/k/v and o products here: a prompt of up to 512 tokens
// 3.3 -> 2.7 ms, of 1,024 tokens 3.3 -> 3.15, of 1,536 tokens 3.4 -> 3.5 (so not beyond 1,024); the down projection's
// long rows take this kernel three times as long as the library and stay there.
extern "C" int ms_gemm_tiled_plain_pays(int M, int N, int K) {
  return M > 0 && M <= 1024 && N > 0 && N <= 2048 && K > 0 && K <= 1024 && K % BK == 0;
}

