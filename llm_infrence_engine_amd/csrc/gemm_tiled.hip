// out[M,N] = A[M,K] . W[N,K]^T for many tokens (prompt portions), bfloat16 in, float accumulation on the
// matrix cores (v_mfma_f32_16x16x32_bf16), with the gated activation as an epilogue: the product of the
// interleaved gate/up weight never goes to memory, which saves the write of [M, 2I], its read and a kernel.
//
// A block of 8 waves owns a tile of BN features by BM tokens, as large as registers allow (256 x 256: a byte
// loaded does 128 multiply-adds; a CU draws 100 GB/s and more from its XCD's L2 but 27 GB/s from beyond it, some
// 40 GB/s in this kernel, where a fifth of the requests miss).  Per step of 64 columns the tile's rows of W
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

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_QKV = 2 };

// What the q/k/v epilogue needs beside the product: W's rows are [q heads | k heads | v heads] of FT * 16 features.
struct QkvEpilogue {
  const float* bias;        // [(nh + 2 nkv) d] or null
  const float2* table;      // [M, d / 2]: (cos, sin) of each token's rotation angles
  const int* slots;         // [M], < 0: the token's k and v are not stored
  bf16* k_pages;            // [pages, nkv, page_size, d]
  bf16* v_pages;            // the same, or [pages, nkv, d, page_size] with v_transposed
  int nh, nkv, page_size, v_transposed;
};

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

// A lane's run of RUN consecutive results goes to memory in the widest pieces that RUN allows (16 bytes for a
// multiple of 8 bfloat16, else 8 or 4), when the row starts at such an address.
template <int RUN>
__device__ __forceinline__ void store_run(bf16* o, const float* v, int valid) {
  constexpr int PIECE = RUN % 8 == 0 ? 8 : (RUN % 4 == 0 ? 4 : (RUN % 2 == 0 ? 2 : 1));
  typedef __attribute__((ext_vector_type(PIECE))) __bf16 piece_t;
  if (PIECE > 1 && valid >= RUN && ((uintptr_t)o % (PIECE * 2)) == 0) {
#pragma unroll
    for (int g = 0; g < RUN; g += PIECE) {
      piece_t pk;
#pragma unroll
      for (int e = 0; e < PIECE; ++e) pk[e] = (__bf16)v[g + e];
      *reinterpret_cast<piece_t*>(o + g) = pk;
    }
  } else {
#pragma unroll
    for (int g = 0; g < RUN; ++g)
      if (g < valid) o[g] = from_float<bf16>(v[g]);
  }
}

// WF x WT waves along features and tokens, each with FT x TT tiles of 16 x 16.  K is a multiple of 64.
template <int WF, int WT, int FT, int TT, int EPI, typename TO>
__global__ void __launch_bounds__(WF * WT * MS_WAVE)
gemm_tiled_kernel(const bf16* __restrict__ A, size_t lda, const bf16* __restrict__ W, size_t ldw,
                  TO* __restrict__ out, size_t ldo, int M, int N, int K, int m_tiles, int n_tiles, int xm, QkvEpilogue qkv) {
  constexpr int NWAVES = WF * WT, THREADS = NWAVES * MS_WAVE;
  constexpr int BN = WF * FT * 16, BM = WT * TT * 16, ROWS = BN + BM;
  constexpr int LOADS = (ROWS / 8 + NWAVES - 1) / NWAVES;   // loads of 8 rows (1 KB) a wave makes per step at most
  static_assert(ROWS % 8 == 0, "a load brings eight rows");
  static_assert(TT < FT, "the main loop reads the token fragments beside the first TT + 1 tiles of W");
  extern __shared__ __align__(16) unsigned char lds_raw[];
  bf16* lds = reinterpret_cast<bf16*>(lds_raw);          // two buffers of ROWS x PITCH

  // Blocks with consecutive ids go to consecutive XCDs, each with an L2 of its own.  The 8 XCDs are laid over the
  // tiles as xm x (8 / xm): an XCD takes every xm-th token tile and every (8 / xm)-th tile of W, its token tiles
  // running fastest (they share a tile of W at the same time).  With xm = 1 a tile of W is read from memory by
  // one XCD only and every XCD reads all of A; a larger xm leaves an XCD 1 / xm of A to keep in its L2.  The host
  // launches 8 * ceil(m_tiles / xm) * ceil(n_tiles / (8 / xm)) blocks; one without a tile leaves.
  const int xcd = blockIdx.x & 7, local = (int)(blockIdx.x >> 3);
  const int xn = 8 / xm, mi = (m_tiles + xm - 1) / xm;
  const int nt = (local / mi) * xn + xcd / xm;
  const int mt = (local % mi) * xm + xcd % xm;
  if (nt >= n_tiles || mt >= m_tiles) return;
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
    const int l = min((wave + p * NWAVES) * 8 + (lane >> 3), ROWS - 1);   // (past the tile's rows: not loaded)
    const int piece = (lane & 7) ^ (l & 7);
    if (l < BN) src[p] = W + (size_t)min(n0 + feature_of_row<FT>(l), N - 1) * ldw + piece * 8;
    else src[p] = A + (size_t)min(m0 + l - BN, M - 1) * lda + piece * 8;
  }
  typedef __attribute__((address_space(3))) void lds_void;
  typedef const __attribute__((address_space(1))) void global_void;
  auto load_rows = [&](int k, int buffer) {
#pragma unroll
    for (int p = 0; p < LOADS; ++p)
      if ((p + 1) * NWAVES * 8 <= ROWS || (wave + p * NWAVES) * 8 < ROWS)   // the last round may be for some waves only
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
  if (EPI == EPI_QKV) {
    // A wave's FT * 16 features are one head, and a lane holds a quarter of it: quarters 0 and 1 are the first
    // half of the head, 2 and 3 the second, so the value that a rotation pairs with lies at the same place in the
    // lane 32 further.  q heads go to out [M, nh d] rotated, k heads rotated and v heads as they are into the pages.
    constexpr int D = FT * 16, RUN = 4 * FT;
    const int head = (n0 + wf * D) / D;
    if (head >= qkv.nh + 2 * qkv.nkv) return;
    const bool rotated = head < qkv.nh + qkv.nkv;
    const int e0 = kq * RUN;
    const bool is_v = !rotated;
    const int kvh = head - qkv.nh - (is_v ? qkv.nkv : 0);
    const float* bias = qkv.bias ? qkv.bias + (size_t)head * D + e0 : nullptr;
#pragma unroll
    for (int j = 0; j < TT; ++j) {
      const int m = m0 + wt * TT * 16 + j * 16 + col;
      const int mm = min(m, M - 1);       // lanes past the last token take part in the exchange and store nothing
      const float2* turn = qkv.table + (size_t)mm * (D / 2) + (kq & 1) * RUN;
      bf16* dst = nullptr;                // a run of the lane's values, or (values transposed) a column of the page
      size_t step = 1;
      if (m < M) {
        if (head < qkv.nh) {
          dst = reinterpret_cast<bf16*>(out) + (size_t)m * ldo + (size_t)head * D + e0;
        } else {
          const long long slot = qkv.slots[m];
          if (slot >= 0) {
            const long long page = slot / qkv.page_size;
            const int off = (int)(slot - page * qkv.page_size);
            if (is_v && qkv.v_transposed) {
              dst = qkv.v_pages + (((size_t)page * qkv.nkv + kvh) * D + e0) * qkv.page_size + off;
              step = (size_t)qkv.page_size;
            } else {
              dst = (is_v ? qkv.v_pages : qkv.k_pages) + (((size_t)page * qkv.nkv + kvh) * qkv.page_size + off) * D + e0;
            }
          }
        }
      }
#pragma unroll
      for (int g0 = 0; g0 < RUN; g0 += 8) {     // eight values at a time: few registers live beside the sums
        bf16x8 pk;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int g = g0 + e;
          float v = acc[g >> 2][j][g & 3] + (bias ? bias[g] : 0.f);
          if (rotated) {
            const float2 cs = turn[g];
            const float other = __shfl_xor(v, 32);
            v = kq < 2 ? v * cs.x - other * cs.y : v * cs.x + other * cs.y;
          }
          pk[e] = (__bf16)v;
        }
        if (!dst) continue;
        if (step == 1) {
          *reinterpret_cast<bf16x8*>(dst + g0) = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) reinterpret_cast<__bf16*>(dst)[(size_t)(g0 + e) * step] = pk[e];
        }
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < TT; ++j) {
    const int m = m0 + wt * TT * 16 + j * 16 + col;
    if (m >= M) continue;
    if (EPI == EPI_SWIGLU) {   // features 2g, 2g + 1 are gate g and up g: 2 FT outputs from o0 on
      const int o0 = f0 / 2, n_out = N / 2;
      float v[2 * FT];
#pragma unroll
      for (int i = 0; i < FT; ++i) {
        v[2 * i] = fast_silu(acc[i][j][0]) * acc[i][j][1];
        v[2 * i + 1] = fast_silu(acc[i][j][2]) * acc[i][j][3];
      }
      store_run<2 * FT>(reinterpret_cast<bf16*>(out) + (size_t)m * ldo + o0, v, n_out - o0);
    } else {
      float v[4 * FT];
#pragma unroll
      for (int g = 0; g < 4 * FT; ++g) v[g] = acc[g >> 2][j][g & 3];
      store_run<4 * FT>(reinterpret_cast<bf16*>(out) + (size_t)m * ldo + f0, v, N - f0);
    }
  }
}

int g_xcd_split = 0;   // measurements: 0 leaves the choice, 1, 2, 4, 8 force the number of XCD rows

// Over how many XCDs the token tiles are spread (see the kernel).  Measured at the gate/up shapes of 0.5B to 32B:
// no difference up to 4,096 tokens; at 8,192 tokens of the 0.5B and 1.5B shapes four rows of XCDs take 143 against
// 155 us and 406 against 425 (an XCD then keeps a quarter of A in its L2 instead of fetching all of it again and
// again), two rows lie between.
int choose_xcd_split(int M) {
  if (g_xcd_split) return g_xcd_split;
  return M >= 6144 ? 4 : (M >= 4096 ? 2 : 1);
}

template <int WF, int WT, int FT, int TT, int EPI, typename TO>
int launch(const bf16* A, size_t lda, const bf16* W, size_t ldw, TO* out, size_t ldo, int M, int N, int K,
           hipStream_t stream, const QkvEpilogue& qkv = QkvEpilogue{}) {
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
  const int xm = choose_xcd_split(M);
  const long long blocks = 8LL * ((m_tiles + xm - 1) / xm) * ((n_tiles + 8 / xm - 1) / (8 / xm));
  if (blocks > 0x7fffffffLL) return MS_UNSUPPORTED;
  gemm_tiled_kernel<WF, WT, FT, TT, EPI, TO><<<dim3((unsigned)blocks), dim3(WF * WT * MS_WAVE), lds, stream>>>(
      A, lda, W, ldw, out, ldo, M, N, K, m_tiles, n_tiles, xm, qkv);
  return ms_launch_status();
}

int g_tile = 0;   // measurements: 0 leaves the choice of tile; 1 to 5 force one (256, 128, 64, 192, 160 features wide)

// The tile that takes the least time by a model of the measurements.  A block of 256 tokens by 256, 192 or 160
// features has a CU to itself; its time is what the CU needs to draw its rows (some 40 GB/s whatever the tile), so
// a step of 64 columns takes 1.70, 1.44 or 1.32 us, a tile 3 us more for its start and end, and the tiles run in
// whole rounds over the CUs: the narrower tiles pay where they fill the rounds better (2,048 tokens of the 0.5B
// gate/up shape: 304 tiles of 256 features take two rounds, 51.7 us; 488 of 160 take two shorter ones, 45.0;
// 1,024 tokens: 28.2 -> 22.6 in one round).  Tiles of 128 x 128 go two to a CU, 1.26 us a step each; they end at
// different times, so their rounds are counted as they come, plus 0.3 for the last.  Within 5 % of the measured
// times at 256 to 4,096 tokens of the 0.5B and 1.5B gate/up shapes.
struct TileChoice { int tile; double us; long long tiles, slots; };

TileChoice choose_tile(int M, int N, int K) {
  const long long cus = ms_compute_units();
  const double steps = (double)((K + BK - 1) / BK);
  const long long small = (long long)((N + 127) / 128) * ((M + 127) / 128);
  // fewer tiles of 128 x 128 than CUs: tiles of 64 x 64 (four waves) put four times as many CUs to work, and a
  // tile's time is the time its CU needs to draw its rows (q/k/v of the 0.5B shape, 512 tokens: 11.3 -> 8.7 us;
  // gate/up at 128 tokens 16.6 -> 12.9, at 256 tokens 16.0 -> 14.9; from 512 tokens on 20.4 against 25.5)
  if (small < cus) {
    const long long tiny = (long long)((N + 63) / 64) * ((M + 63) / 64);
    return {3, 0.0, tiny, (tiny + 5 * cus - 1) / (5 * cus) * 5 * cus};
  }
  TileChoice best{2, ((double)small / (double)(2 * cus) + 0.3) * 1.26 * steps, small, (small + 2 * cus - 1) / (2 * cus) * 2 * cus};
  const struct { int tile, features; double step_us; } wide[] = {{1, 256, 1.70}, {4, 192, 1.44}, {5, 160, 1.32}};
  for (const auto& w : wide) {
    const long long tiles = (long long)((N + w.features - 1) / w.features) * ((M + 255) / 256);
    const long long rounds = (tiles + cus - 1) / cus;
    const double us = (double)rounds * (3.0 + steps * w.step_us);
    if (us < best.us) best = {w.tile, us, tiles, rounds * cus};
  }
  return best;
}

}  // namespace

extern "C" void ms_gemm_tiled_force(int tile) { g_tile = tile; }
extern "C" void ms_gemm_tiled_force_xcd_split(int xm) { g_xcd_split = xm; }

// Whether the gated product of M tokens is faster here than as the library's product and an activation kernel
// (measured with a different W every call, 65 to 8,192 tokens): up to 1,536 columns always (0.5 to 0.98 of the
// library's time); beyond that the two are within 15 % of each other either way, and this kernel is taken where it
// won throughout: up to 2,048 tokens whose tiles fill at least 9/10 of their rounds over the CUs.
extern "C" int ms_gemm_tiled_pays(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % BK) return 0;
  if (K <= 1536) return 1;
  if (M > 2048) return 0;
  const TileChoice c = choose_tile(M, N, K);
  return c.tiles * 10 >= c.slots * 9;
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
  if (tile == 0) tile = choose_tile(M, N, K).tile;
#define GO(WF, WT, FT, TT) return epilogue == EPI_SWIGLU ? launch<WF, WT, FT, TT, EPI_SWIGLU, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream) \
                                                        : launch<WF, WT, FT, TT, EPI_STORE, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream)
  if (tile == 1) GO(2, 4, 8, 4);   // 256 x 256
  if (tile == 3) GO(1, 4, 4, 1);   // 64 x 64, four waves
  if (tile == 4) GO(2, 4, 6, 4);   // 192 features x 256 tokens
  if (tile == 5) GO(2, 4, 5, 4);   // 160 features x 256 tokens
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


// The q/k/v product of a prompt portion with what follows it as the epilogue: bias, rotation of the q and k heads
// (pairs (j, j + d/2) turned by the angle whose cosine and sine rope_table[token][j] holds: ms_rope_table makes
// them once a step for all layers) and the store of k and v into the cache pages, so the projection of k and v
// never goes to memory as a matrix and q is written once.
// A [M, lda] bfloat16, W [(nh + 2 nkv) d, ldw], q_out [M, nh d]; head_dim 64 or 128 (a wave's features are one
// head), rotation over the whole head.  Pays where the plain product here keeps up with the library's: narrow
// models (ms_gemm_tiled_qkv_pays).
extern "C" int ms_gemm_tiled_qkv_pays(int M, int N, int K, int head_dim) {
  return M > 0 && N > 0 && K > 0 && K % BK == 0 && K <= 1024 && N <= 2048 && (head_dim == 64 || head_dim == 128);
}

extern "C" int ms_gemm_tiled_qkv(const void* A, long long lda, const void* W, long long ldw, const float* bias,
                                 const float* rope_table, const int* slot_mapping, void* q_out,
                                 void* k_pages, void* v_pages, int M, int K, int nh, int nkv, int head_dim, int page_size,
                                 int v_transposed, hipStream_t stream) {
  if (M <= 0) return MS_OK;
  if (nh <= 0 || nkv <= 0 || page_size <= 0 || !rope_table || !slot_mapping || !q_out || !k_pages || !v_pages)
    return MS_BAD_ARG;
  if (head_dim != 64 && head_dim != 128) return MS_UNSUPPORTED;
  if (K <= 0 || K % BK || lda % 8 || ldw % 8 || lda < K || ldw < K) return MS_UNSUPPORTED;
  if (((uintptr_t)A | (uintptr_t)W | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages | (uintptr_t)rope_table) % 16) return MS_UNSUPPORTED;
  const int N = (nh + 2 * nkv) * head_dim;
  const QkvEpilogue e{bias, (const float2*)rope_table, slot_mapping, (bf16*)k_pages, (bf16*)v_pages, nh, nkv, page_size,
                      v_transposed};
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  bf16* o = (bf16*)q_out;
  const size_t ldo = (size_t)nh * head_dim;
  // heads of 128: tiles of 256 features by 128 tokens (with 256 tokens the epilogue no longer fits the registers)
  if (head_dim == 128) return launch<2, 4, 8, 2, EPI_QKV, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream, e);
  int tile = g_tile;
  if (tile == 0) tile = choose_tile(M, N, K).tile;
  if (tile == 3) return launch<1, 4, 4, 1, EPI_QKV, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream, e);
  return launch<2, 4, 4, 2, EPI_QKV, bf16>(a, lda, w, ldw, o, ldo, M, N, K, stream, e);
}
