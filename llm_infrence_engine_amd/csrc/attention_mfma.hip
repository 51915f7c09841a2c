// Paged causal attention on the matrix cores (v_mfma_f32_16x16x32_bf16), bfloat16 in, float softmax.
//
// One wave owns NT*16 *columns* of one (request, key/value head): a column is a (token, query head of the
// group) pair, so every key and value that is loaded serves all query heads that share it, and in a prompt
// portion also NT*16/group consecutive tokens.  Keys are walked in blocks of 32:
//
//   S^T[key, col]  = K[key, :] . Q^T[:, col]        A operand: 16 keys x 32 dims, read in place from the
//                                                   page (a lane reads 16 contiguous bytes of one key);
//                                                   B operand: the query, kept in registers
//   online softmax per column in float, in log2 units (scale * log2(e) is folded into the exponent's
//   multiply-add); the running reference follows the maximum in steps, so rescaling is rare
//   O^T[dim, col] += V^T[dim, key] . P^T[key, col]  B operand: P^T straight from the S^T accumulators (a lane
//                                                   holds 4+4 keys of its own column: no transpose);
//                                                   A operand: V^T, which is why value pages are stored
//                                                   transposed, [page][kv head][dim][page_size]: a lane reads
//                                                   8 contiguous bytes (4 keys) of one dim from each page.
//
// The WAVES waves of a block share a column tile and take its key blocks in turn (wave w: blocks w, w + WAVES,
// ...), each with its own running maximum, sum and accumulators; at the end they are merged through LDS by
// wave 0 in a fixed order.  That shortens the chain of dependent key blocks (a late prompt tile, a long
// context) by WAVES and puts several waves on every SIMD to hide the latency of the page reads.  The next
// block's keys and values are loaded while the current one is multiplied.  Keys beyond a column's own
// position are masked, values beyond the last visible key are zeroed before use, and pages past the
// context are never dereferenced, so what a reused page still holds cannot reach the result.
//
// Two launch shapes: general (any mix of portions and single tokens; grid = column tiles x kv heads x
// requests, surplus tiles leave at once; a decode-only batch is the case of one tile per request) and
// split (every request has one token and a long context: the keys are also split over several blocks which
// write unnormalised partial results, and a second kernel combines them).
#include "common.h"
#include "api.h"
#include <algorithm>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr float REF_SLACK = 8.0f;   // log2 units by which a column's maximum may run ahead of its reference

template <int D>
struct KeyBlock {          // one block of 32 keys as this lane sees it
  bf16x8 k[2][D / 32];     // [16-key subtile][32-dim step]
};
template <int CT>
struct ValueBlock {        // and its values, for the CT tiles of 16 dims that this block works out
  bf16x4 v[CT][2];         // [16-dim tile][subtile]: 4 keys of one dim; the two subtiles are one MFMA operand
};

// Page arithmetic: pages of a power of two (page_shift >= 0) need no division.
struct PageGeom {
  int size, shift;
  __device__ __forceinline__ int index(int key) const { return shift >= 0 ? key >> shift : key / size; }
  __device__ __forceinline__ int offset(int key) const { return shift >= 0 ? key & (size - 1) : key % size; }
};

// The pages of the two 16-key halves of the block at `base` (the same for every lane, so they are kept in
// scalar registers and so is all address arithmetic that follows from them); past the context: the null page.
__device__ __forceinline__ void pages_of(const int* __restrict__ table, int base, int key_hi, PageGeom pg,
                                         int* pages) {
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int kb = base + u * 16;
    pages[u] = kb <= key_hi ? __builtin_amdgcn_readfirstlane(table[pg.index(kb)]) : 0;
  }
}

// Where the two 16-key halves of a block start inside their page's part of one kv head: uniform values.
struct BlockPlace {
  size_t head[2];   // element offset of (page, kv head) in either pool
  int off[2];       // first key inside the page
};

__device__ __forceinline__ BlockPlace place_of(const int* pages, int base, int g, int nkv, PageGeom pg, int D) {
  BlockPlace bp;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    bp.head[u] = ((size_t)pages[u] * nkv + g) * pg.size * D;
    bp.off[u] = pg.offset(base + u * 16);
  }
  return bp;
}

template <int D>
__device__ __forceinline__ void load_keys(KeyBlock<D>& b, const bf16* __restrict__ k_pages, const BlockPlace& bp,
                                          int lane) {
  const int k_lane = (lane & 15) * D + (lane >> 4) * 8;   // this lane's key and dims inside a 16-key half
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const bf16* kp = k_pages + bp.head[u] + bp.off[u] * D;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) b.k[u][s] = *reinterpret_cast<const bf16x8*>(kp + k_lane + s * 32);
  }
}

template <int CT>
__device__ __forceinline__ void load_values(ValueBlock<CT>& b, const bf16* __restrict__ vt_pages,
                                            const BlockPlace& bp, PageGeom pg, int dim0, int lane) {
  const int v_lane = (dim0 + (lane & 15)) * pg.size + (lane >> 4) * 4;   // this lane's dim and keys inside a tile
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const bf16* vp = vt_pages + bp.head[u] + bp.off[u];
#pragma unroll
    for (int c = 0; c < CT; ++c) b.v[c][u] = *reinterpret_cast<const bf16x4*>((vp + c * 16 * pg.size) + v_lane);
  }
}

// Two waves of a wide tile on every SIMD (256 registers each) hide each other's waits; narrow tiles fit anyway.
//
// VS > 1 (narrow tiles only) shares one tile among VS blocks: each works out all scores and the whole softmax
// but only D / VS of the output's dims, so it reads all keys and 1 / VS of the values.  A compute unit draws
// its data at a small fraction of the chip's rate, so when a step has fewer tiles than the chip has units this
// shortens the longest chain without a second kernel; the blocks write disjoint dims and share nothing.
template <int D, int NT, int WAVES, bool SPLIT, int VS>
__global__ void __launch_bounds__(WAVES * MS_WAVE, (NT > 1 ? 2 : 1))
attention_mfma_kernel(const bf16* __restrict__ q, size_t q_stride, const bf16* __restrict__ k_pages,
                      const bf16* __restrict__ vt_pages, const int* __restrict__ block_table, int table_stride,
                      const int* __restrict__ table_rows, const int* __restrict__ q_start,
                      const int* __restrict__ context_lens, bf16* __restrict__ out, size_t out_stride,
                      float* __restrict__ part_o, float* __restrict__ part_ml, int nh, int nkv, int page_size,
                      int page_shift, float scale_log2e, int window, int min_blocks, int n_splits) {
  // SPLIT: min_blocks and n_splits say how a request's key blocks are spread.  Else min_blocks != 0 asks for
  // the order of tiles in which a long tile's companion on its CU is a short one (see below), and n_splits is
  // the number of requests whose tiles the grid's second dimension runs over (0: one tile to a request)
  __shared__ float sm_m[WAVES][NT][16], sm_l[WAVES][NT][16];
  static_assert(VS == 1 || (NT == 1 && !SPLIT), "only narrow tiles of the general shape share their dims out");
  static_assert((D / 16) % VS == 0, "whole tiles of 16 dims to a block");
  constexpr int CT = D / 16 / VS;
  __shared__ f32x4 sm_o[WAVES > 1 ? WAVES - 1 : 1][CT][NT][MS_WAVE];
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);   // the same for the whole wave
  const int col16 = lane & 15, kq = lane >> 4;
  // general shape: grid (kv heads, column tiles of the whole step, blocks that share a tile's dims): blocks are
  // handed out with the kv head running fastest; split shape: grid (splits, kv heads, requests)
  const int g = SPLIT ? blockIdx.y : blockIdx.x;
  const int bx = SPLIT ? blockIdx.x : blockIdx.z;
  const int rep = nh / nkv;
  const PageGeom pg = {page_size, page_shift};
  // Which request, and which of its tiles.  A request owns ceil(columns / tile width) tiles, requests in order,
  // so the launch needs to know only how many tokens and requests a step has, not how the tokens are dealt out
  // (a captured graph serves every mix).  The waves of a block find their place alike: a lane per request
  // works out its tiles, a prefix sum over the wave and a vote say where this block's tile falls.
  int r, rank, n_tiles;
  if (SPLIT) {
    r = blockIdx.z; rank = 0; n_tiles = 1;
  } else if (n_splits == 0) {
    r = blockIdx.y; rank = 0; n_tiles = 1;
  } else if (n_splits == 1) {
    r = 0; rank = blockIdx.y;
    n_tiles = ((q_start[1] - q_start[0]) * rep + 16 * NT - 1) / (16 * NT);
    if (rank >= n_tiles) return;
  } else {
    const int flat = blockIdx.y;
    int before = 0;
    r = -1; rank = 0; n_tiles = 0;
    for (int base = 0; base < n_splits; base += MS_WAVE) {
      const int i = base + lane;
      int mine = 0;
      if (i < n_splits) mine = ((q_start[i + 1] - q_start[i]) * rep + 16 * NT - 1) / (16 * NT);
      int upto = mine;   // tiles of the requests base..i
#pragma unroll
      for (int o = 1; o < MS_WAVE; o <<= 1) {
        const int v = __shfl_up(upto, o, MS_WAVE);
        if (lane >= o) upto += v;
      }
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(flat < before + upto);
      if (hit) {
        const int first = __builtin_ctzll(hit);
        r = base + first;
        n_tiles = __shfl(mine, first, MS_WAVE);
        rank = flat - before - (__shfl(upto, first, MS_WAVE) - n_tiles);
        break;
      }
      before += __shfl(upto, MS_WAVE - 1, MS_WAVE);
    }
    if (r < 0) return;   // the grid has room for a partial tile of every request; this block is surplus
    r = __builtin_amdgcn_readfirstlane(r);
    rank = __builtin_amdgcn_readfirstlane(rank);
    n_tiles = __builtin_amdgcn_readfirstlane(n_tiles);
  }
  const int row = table_rows ? table_rows[r] : r;
  const int* table = block_table + (size_t)row * table_stride;
  // Without a window a wave's first key block is known before the request's lengths are: ask for its page
  // ids at once, so that they travel together with the lengths instead of after them.
  int first_pages[2] = {0, 0};
  const bool early = !SPLIT && window <= 0;
  if (early) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
      first_pages[u] = __builtin_amdgcn_readfirstlane(table[min(pg.index(wave * 32 + u * 16), table_stride - 1)]);
  }
  const int q0 = q_start[r];
  const int qlen = q_start[r + 1] - q0;
  const int start_pos = context_lens[r] - qlen;
  const int ncols = qlen * rep;
  // Late tiles of a prompt see the most keys: they go first, so that the long ones do not finish last.  When
  // all blocks fit on the chip at once (two to a CU), only the later half goes first, latest tile first, and
  // then the earlier half, earliest first: blocks that start one round of the chip apart tend to share a CU, and
  // so a long tile's companion is a short one that soon leaves the SIMDs to it (2,048 tokens: 34.0 -> 29.4 us).
  const int dim0 = VS > 1 ? bx * CT * 16 : 0;   // the first of this block's output dims
  const int half = (!SPLIT && min_blocks) ? (n_tiles + 1) / 2 : n_tiles;
  const int tile = rank < half ? n_tiles - 1 - rank : rank - half;
  const int c0 = SPLIT ? 0 : tile * 16 * NT;
  if (c0 >= ncols) return;

  // key range of the tile: from the first column's window start to the last column's own position
  const int last_col = min(ncols, c0 + 16 * NT) - 1;
  int key_hi = start_pos + last_col / rep;
  int key_lo = 0;
  if (window > 0) key_lo = max(0, start_pos + c0 / rep - window + 1);
  int blk_begin = key_lo / 32, blk_end = key_hi / 32 + 1;
  // a block whose keys every column of the tile sees needs no mask: all keys at or before the first column's
  // position (and, with a window, after the last column's window start); tiles with idle columns always mask
  const int first_pos = start_pos + c0 / rep;
  const bool full_tile = c0 + 16 * NT <= ncols;
  if (SPLIT) {
    // every request spreads its own key blocks evenly over the splits (at least min_blocks each)
    const int per = max(min_blocks, (blk_end - blk_begin + n_splits - 1) / n_splits);
    blk_begin += bx * per;
    blk_end = min(blk_end, blk_begin + per);
    if (blk_begin >= blk_end) return;
  }

  // this lane's columns
  int pos[NT];   // -1: an idle column (sees no key; its result is not written)
  bf16x8 qv[NT][D / 32];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int c = c0 + t * 16 + col16;
    const int cc = min(c, ncols - 1);
    const int tok = q0 + cc / rep, head = g * rep + cc % rep;
    pos[t] = c < ncols ? start_pos + cc / rep : -1;
    const bf16* qp = q + (size_t)tok * q_stride + (size_t)head * D + kq * 8;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) qv[t][s] = *reinterpret_cast<const bf16x8*>(qp + s * 32);
  }

  // The sums of the exponentials come from the matrix cores too: one more product per column tile, of P^T with
  // a V^T of ones, gives every lane its columns' sums over all 32 keys of the block (of the same bfloat16 values
  // that the weighted sum of the values uses), where adding them up lane by lane took 32 additions and, at the
  // end, two exchanges between lanes; the matrix pipe has the time.
  // (The widest tile at head size 64 has no registers left for it and adds its exponentials up on the vector
  // pipe, a lane's share at a time, with two exchanges between lanes at the end.)
  constexpr bool SUMS_BY_MATRIX = !(D == 64 && NT == 4);
  float m[NT], lvec[NT];
  f32x4 o[CT][NT], lsum[SUMS_BY_MATRIX ? NT : 1];
  bf16x8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    m[t] = -INFINITY;
    lvec[t] = 0.f;
    if (SUMS_BY_MATRIX) lsum[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < CT; ++c) o[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // A narrow tile (decode) has registers to spare and few waves to hide a wait behind: it fetches the next
  // block's values early, together with its keys.  A wide tile fetches values at the top of the pass that
  // uses them (the score products and the softmax run meanwhile, and so does the SIMD's other wave).
  constexpr bool VALUES_EARLY = NT == 1;
  KeyBlock<D> buf_k[2];
  ValueBlock<CT> buf_v[2];
  BlockPlace buf_at[2];
  if (blk_begin + wave < blk_end) {
    KeyBlock<D>& cur_k = buf_k[0];
    ValueBlock<CT>& cur_v = buf_v[0];
    BlockPlace& cur_at = buf_at[0];
    const int base = (blk_begin + wave) * 32;
    int pages[2];
    if (early) {  // blk_begin is 0 here; halves past the last key fall back to the null page
#pragma unroll
      for (int u = 0; u < 2; ++u) pages[u] = base + u * 16 <= key_hi ? first_pages[u] : 0;
    } else {
      pages_of(table, base, key_hi, pg, pages);
    }
    cur_at = place_of(pages, base, g, nkv, pg, D);
    load_keys<D>(cur_k, k_pages, cur_at, lane);
    if (VALUES_EARLY) load_values<CT>(cur_v, vt_pages, cur_at, pg, dim0, lane);
  }
  // The page ids of a block are asked for one block before its keys are: the keys' loads then go out at the top of
  // an iteration instead of behind a table lookup (8,192 tokens of the 0.5B shape: 235 -> 232 us; 2,048 tokens at
  // head size 128: 99.9 -> 96.7 us).  (Keeping the loads of two blocks in flight for narrow tiles was measured and
  // dropped: a decode tile's time is what its CU can draw, 102 KB at about 43 GB/s at 640 keys, not its waits.)
  int ahead_pages[2] = {0, 0};
  if (blk_begin + wave + WAVES < blk_end) pages_of(table, (blk_begin + wave + WAVES) * 32, key_hi, pg, ahead_pages);
  // One block of 32 keys: the step works on the buffers it is handed as current and fills those it is handed
  // as next; the loop below calls it with the two sets of buffers in turn, so nothing is copied between them.
  auto step = [&](int blk, KeyBlock<D>& cur_k, ValueBlock<CT>& cur_v, BlockPlace& cur_at, KeyBlock<D>& nxt_k,
                  ValueBlock<CT>& nxt_v, BlockPlace& nxt_at) __attribute__((always_inline)) {
    const int base = blk * 32;
    if (!VALUES_EARLY) load_values<CT>(cur_v, vt_pages, cur_at, pg, dim0, lane);
    if (blk + WAVES < blk_end) {
      nxt_at = place_of(ahead_pages, base + WAVES * 32, g, nkv, pg, D);
      load_keys<D>(nxt_k, k_pages, nxt_at, lane);
      if (VALUES_EARLY) load_values<CT>(nxt_v, vt_pages, nxt_at, pg, dim0, lane);
      if (blk + 2 * WAVES < blk_end) pages_of(table, base + 2 * WAVES * 32, key_hi, pg, ahead_pages);
    }

    // scores: s[u][t] holds keys base + u*16 + kq*4 + (0..3) of column t*16 + col16
    f32x4 s[2][NT];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur_k.k[u][ks], qv[t][ks], acc, 0, 0, 0);
        s[u][t] = acc;
      }

    // values past the last visible key may be anything a reused page still holds: make them zero
    if (base + 31 > key_hi) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (base + u * 16 + kq * 4 + i > key_hi) {
#pragma unroll
            for (int c = 0; c < CT; ++c) cur_v.v[c][u][i] = (__bf16)0.0f;
          }
    }

    const bool unmasked = full_tile && base + 31 <= first_pos && (window <= 0 || base > key_hi - window);
    bf16x8 p[NT];
    float corr[NT], bmax[NT];
    bool moved = false;
    // the block's maxima of the raw scores (the scale is positive, so they are the maxima of the scaled ones
    // too); one branch for the whole tile, so that what follows is straight-line code for all its columns
    if (unmasked) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float bm = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) bm = fmaxf(bm, s[u][t][i]);
        bmax[t] = bm;
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float bm = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = base + u * 16 + kq * 4 + i;
            const bool see = key <= pos[t] && (window <= 0 || key > pos[t] - window);
            const float v = see ? s[u][t][i] : -INFINITY;
            s[u][t][i] = v;
            bm = fmaxf(bm, v);
          }
        bmax[t] = bm;
      }
    }
    float m_safe[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float bm = bmax[t];
      bm = fmaxf(bm, __shfl_xor(bm, 16, MS_WAVE));
      bm = fmaxf(bm, __shfl_xor(bm, 32, MS_WAVE));
      bm *= scale_log2e;
      // m is the reference that the exponents are taken against, not necessarily the maximum: it follows the
      // maximum only when that has run ahead by more than REF_SLACK (a factor 2^REF_SLACK in the terms, far
      // inside float's range), so that the accumulators are rescaled rarely.  Any reference gives the same
      // softmax; all lanes of a column decide alike because bm is the same in all of them.
      const bool step = bm > m[t] + REF_SLACK;
      const float m_new = step ? bm : m[t];
      corr[t] = step ? fast_exp2(m[t] - m_new) : 1.0f;   // m = -inf: 0
      moved |= step;
      m[t] = m_new;
      m_safe[t] = m_new == -INFINITY ? 0.f : m_new;
    }
    if (NT == 1 || __builtin_amdgcn_ballot_w64(moved) != 0) {   // the same branch for the whole wave
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (SUMS_BY_MATRIX) lsum[t] *= corr[t]; else lvec[t] *= corr[t];
#pragma unroll
        for (int c = 0; c < CT; ++c) o[c][t] *= corr[t];
      }
    }
    // column by column, so that the products of one column run on the matrix cores while the next column's
    // exponentials are taken
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = fast_exp2(fmaf(s[u][t][i], scale_log2e, -m_safe[t]));
          if (!SUMS_BY_MATRIX) lvec[t] += e;
          p[t][u * 4 + i] = (__bf16)e;
        }
      if (SUMS_BY_MATRIX) lsum[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p[t], lsum[t], 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        bf16x8 vv;
#pragma unroll
        for (int i = 0; i < 4; ++i) { vv[i] = cur_v.v[c][0][i]; vv[4 + i] = cur_v.v[c][1][i]; }
        o[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, p[t], o[c][t], 0, 0, 0);
      }
    }
  };
  for (int blk = blk_begin + wave; blk < blk_end; blk += 2 * WAVES) {
    step(blk, buf_k[0], buf_v[0], buf_at[0], buf_k[1], buf_v[1], buf_at[1]);
    if (blk + WAVES < blk_end) step(blk + WAVES, buf_k[1], buf_v[1], buf_at[1], buf_k[0], buf_v[0], buf_at[0]);
  }

  float l[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (SUMS_BY_MATRIX) {
      l[t] = lsum[t][0];   // every row of the product of ones is the column's sum
    } else {               // a column's sum is spread over the four lane groups
      l[t] = lvec[t] + __shfl_xor(lvec[t], 16, MS_WAVE);
      l[t] += __shfl_xor(l[t], 32, MS_WAVE);
    }
  }
  if (WAVES > 1) {
    // merge the waves' partial results (each relative to its own maximum) in wave order
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (kq == 0) { sm_m[wave][t][col16] = m[t]; sm_l[wave][t][col16] = l[t]; }
      if (wave > 0) {
#pragma unroll
        for (int c = 0; c < CT; ++c) sm_o[wave - 1][c][t][lane] = o[c][t];
      }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float big = m[t];
      for (int w = 1; w < WAVES; ++w) big = fmaxf(big, sm_m[w][t][col16]);
      const float safe = big == -INFINITY ? 0.f : big;
      const float f0 = fast_exp2(m[t] - safe);
      float lsum = l[t] * f0;
#pragma unroll
      for (int c = 0; c < CT; ++c) o[c][t] *= f0;
      for (int w = 1; w < WAVES; ++w) {
        const float f = fast_exp2(sm_m[w][t][col16] - safe);
        lsum += f * sm_l[w][t][col16];
#pragma unroll
        for (int c = 0; c < CT; ++c) o[c][t] += sm_o[w - 1][c][t][lane] * f;
      }
      m[t] = big;
      l[t] = lsum;
    }
  }

#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const float lt = l[t];
    if (pos[t] < 0) continue;
    const int c = c0 + t * 16 + col16;   // worked out again rather than kept through the loop
    const int tok = q0 + c / rep, head = g * rep + c % rep;
    if (SPLIT) {
      // unnormalised: O, the running maximum (log2 units) and the sum; the combine kernel weighs the splits
      const size_t slot = ((size_t)r * nh + head) * n_splits + bx;
      float* po = part_o + slot * D + kq * 4;
#pragma unroll
      for (int c = 0; c < CT; ++c) *reinterpret_cast<f32x4*>(po + c * 16) = o[c][t];
      if (kq == 0) { part_ml[slot * 2] = m[t]; part_ml[slot * 2 + 1] = lt; }
    } else {
      const float inv = 1.0f / lt;
      bf16* op = out + (size_t)tok * out_stride + (size_t)head * D + dim0 + kq * 4;
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = (__bf16)(o[c][t][i] * inv);
        *reinterpret_cast<bf16x4*>(op + c * 16) = w;
      }
    }
  }
}

// out[r, h, :] = sum_s 2^(m_s - M) O_s / sum_s 2^(m_s - M) l_s over the splits that request r used.
// One block per (request, head): the splits' maxima and sums are fetched side by side, the
// weights are worked out once into LDS, then a thread per dim adds the weighted partial results in split order.
constexpr int COMBINE_MAX_SPLITS = 128;

template <int D>
__global__ void __launch_bounds__(D < 64 ? 64 : D)
attention_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                         const int* __restrict__ q_start, const int* __restrict__ context_lens,
                         bf16* __restrict__ out, size_t out_stride, int nh, int window, int min_blocks,
                         int n_splits) {
  __shared__ float sm_m[COMBINE_MAX_SPLITS], sm_w[COMBINE_MAX_SPLITS];
  const int r = blockIdx.x / nh, h = blockIdx.x % nh;
  if (q_start[r + 1] == q_start[r]) return;   // a row that pads a captured batch: no token, nothing to write
  const int key_hi = context_lens[r] - 1;
  const int key_lo = window > 0 ? max(0, key_hi - window + 1) : 0;
  const int blocks = key_hi / 32 + 1 - key_lo / 32;
  const int per = max(min_blocks, (blocks + n_splits - 1) / n_splits);
  const int used = (blocks + per - 1) / per;
  const size_t slot0 = ((size_t)r * nh + h) * n_splits;
  const int t = threadIdx.x;
  for (int s = t; s < used; s += blockDim.x) sm_m[s] = part_ml[(slot0 + s) * 2];
  __syncthreads();
  float big = -INFINITY;
  for (int s = 0; s < used; ++s) big = fmaxf(big, sm_m[s]);
  __syncthreads();
  // the weights, and in sm_m (no longer needed) the splits' weighted sums for the denominator in split order
  for (int s = t; s < used; s += blockDim.x) {
    const float w = fast_exp2(sm_m[s] - big);
    sm_w[s] = w;
    sm_m[s] = w * part_ml[(slot0 + s) * 2 + 1];
  }
  __syncthreads();
  float den = 0.f;
  for (int s = 0; s < used; ++s) den += sm_m[s];
  const float inv = 1.0f / den;
  bf16* op = out + (size_t)q_start[r] * out_stride + (size_t)h * D;
  for (int d = t; d < D; d += blockDim.x) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < used; ++s) acc += sm_w[s] * part_o[(slot0 + s) * D + d];
    op[d] = __float2bfloat16(acc * inv);
  }
}

int g_force_nt = 0, g_force_waves = 0, g_force_vs = 0;

inline int page_shift_of(int page_size) {   // log2 of a power of two, else -1
  if (page_size & (page_size - 1)) return -1;
  int sh = 0;
  while ((1 << sh) < page_size) ++sh;
  return sh;
}

template <int D, int NT, int WAVES, int VS>
int launch_general(const bf16* q, size_t q_stride, const bf16* k, const bf16* vt, const int* table, int table_stride,
                   const int* table_rows, const int* q_start, const int* ctx, bf16* out, size_t out_stride,
                   int n_requests, int n_tokens, int max_q_len, int nh, int nkv, int page_size, float scale,
                   int window, hipStream_t stream) {
  const int rep = nh / nkv;
  const long long per_request = ((long long)max_q_len * rep + 16 * NT - 1) / (16 * NT);
  // every request may end in a partial tile; no step has more tiles than if each request were the longest
  long long tiles = (long long)n_tokens * rep / (16 * NT) + n_requests;
  if (tiles > per_request * n_requests) tiles = per_request * n_requests;
  if (tiles > 65535) return MS_UNSUPPORTED;   // grid.y
  const int pair_order = tiles * VS * nkv <= 2LL * ms_compute_units() ? 1 : 0;
  const int scan = per_request == 1 ? 0 : n_requests;   // one tile to a request: the tile's index is the request's
  dim3 grid(nkv, (unsigned)tiles, VS), block(WAVES * MS_WAVE);
  attention_mfma_kernel<D, NT, WAVES, false, VS><<<grid, block, 0, stream>>>(q, q_stride, k, vt, table, table_stride, table_rows, q_start, ctx, out, out_stride, nullptr, nullptr, nh, nkv, page_size, page_shift_of(page_size), scale * 1.4426950408889634f, window, pair_order, scan);
  return ms_launch_status();
}

template <int D>
int launch_split(const bf16* q, size_t q_stride, const bf16* k, const bf16* vt, const int* table, int table_stride,
                 const int* table_rows, const int* q_start, const int* ctx, bf16* out, size_t out_stride, float* part_o, float* part_ml,
                 int n_requests, int nh, int nkv, int page_size, float scale, int window, int min_blocks,
                 int n_splits, hipStream_t stream) {
  dim3 grid(n_splits, nkv, n_requests), block(4 * MS_WAVE);
  attention_mfma_kernel<D, 1, 4, true, 1><<<grid, block, 0, stream>>>(q, q_stride, k, vt, table, table_stride, table_rows, q_start, ctx, out, out_stride, part_o, part_ml, nh, nkv, page_size, page_shift_of(page_size), scale * 1.4426950408889634f, window, min_blocks, n_splits);
  attention_combine_kernel<D><<<dim3(n_requests * nh), dim3(D < 64 ? 64 : D), 0, stream>>>(part_o, part_ml, q_start, ctx, out, out_stride, nh, window, min_blocks, n_splits);
  return ms_launch_status();
}

}  // namespace

// Tuning knob: force the general shape's tile width (16 * nt columns), waves per tile and (narrow tiles) the
// number of blocks that share a tile's dims; 0 restores the choice by size.  Shapes outside the menu are
// refused at the call.
extern "C" void ms_attention_mfma_force(int nt, int waves, int dim_shares) {
  g_force_nt = nt;
  g_force_waves = waves;
  g_force_vs = dim_shares;
}

// Whether the matrix-core kernels take this geometry (else the caller uses the generic kernel).
extern "C" int ms_attention_mfma_supported(int head_dim, int page_size) {
  return (head_dim == 32 || head_dim == 64 || head_dim == 128) && page_size > 0 && page_size % 16 == 0;
}

// General shape.  q [N, >= nh*d] bfloat16 (row stride q_stride), k_pages [P, nkv, page_size, d],
// vt_pages [P, nkv, d, page_size], block_table int32 [rows, table_stride], table_rows int32 [R] (the table's row
// of each request; null: request r has row r), q_start int32 [R + 1], context_lens int32 [R] (keys held after
// this step), out [N, nh*d] (row stride out_stride).  n_tokens = q_start[R] or more, max_q_len the longest
// portion or more: the launch is sized by these two and n_requests alone, so tokens beyond q_start[R] and
// requests without tokens cost a block that leaves at once.
extern "C" int ms_paged_attention_mfma(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                                       const int* block_table, int table_stride, const int* table_rows,
                                       const int* q_start, const int* context_lens, void* out, long long out_stride,
                                       int n_requests, int n_tokens, int max_q_len, int num_heads, int num_kv_heads,
                                       int head_dim, int page_size, float scale, int window, hipStream_t stream) {
  if (n_requests <= 0 || max_q_len <= 0 || n_tokens <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || table_stride <= 0) return MS_BAD_ARG;
  if (!(scale > 0.f)) return MS_BAD_ARG;   // maxima are taken of the raw scores
  if (!ms_attention_mfma_supported(head_dim, page_size)) return MS_UNSUPPORTED;
  if (q_stride % 8 || out_stride % 4 || ((uintptr_t)q % 16) || ((uintptr_t)out % 8)) return MS_UNSUPPORTED;
  if (n_requests > 65535 || num_kv_heads > 65535) return MS_UNSUPPORTED;
#define GO(D, NT, WV, VS) return launch_general<D, NT, WV, VS>((const bf16*)q, q_stride, (const bf16*)k_pages, (const bf16*)vt_pages, block_table, table_stride, table_rows, q_start, context_lens, (bf16*)out, out_stride, n_requests, n_tokens, max_q_len, num_heads, num_kv_heads, page_size, scale, window, stream)
  // Tile width (NT * 16 columns) and waves over a tile's keys.  Few columns (a decode step): one narrow tile
  // per request and many waves over its keys.
  const int cols = max_q_len * (num_heads / num_kv_heads);
  int nt = cols > 16 ? (head_dim == 128 ? 2 : 4) : 1;
  int waves = nt > 1 ? 4 : (head_dim == 128 ? 8 : 16);
  // narrow tiles, fewer of them than compute units: blocks share a tile's dims as far as there is a unit for
  // every block (measured at 200, 640 and 1,000 keys, head sizes 64 and 128: up to 64 tiles four ways, up to 128
  // two ways, e.g. 128 tiles at 640 keys 8.0 -> 7.0 us; with more blocks than units the keys' repeated reading
  // costs more than the shorter streams save).  Very many tiles of the large head size: four waves to a tile
  // (512 tiles at 640 keys: 32.2 -> 29.3 us).
  int vs = 1;
  if (nt == 1) {
    const long long per_request = (cols + 15) / 16;
    const long long tiles = num_kv_heads * std::min(per_request * n_requests, (long long)n_tokens * (num_heads / num_kv_heads) / 16 + n_requests);
    const int cus = ms_compute_units();
    while (vs < 4 && (head_dim / 16) % (vs * 2) == 0 && tiles * vs * 2 <= cus) vs *= 2;
    if (head_dim == 128 && tiles >= 2LL * cus) waves = 4;
  }
  if (g_force_nt) { nt = g_force_nt; waves = g_force_waves; }
  if (g_force_vs) vs = g_force_vs;
  if (nt > 1) vs = 1;
#define PICK(D, NT, WV) if (head_dim == D && nt == NT && waves == WV && vs == 1) GO(D, NT, WV, 1)
#define PICK_SHARED(D, WV, VS) if (head_dim == D && nt == 1 && waves == WV && vs == VS) GO(D, 1, WV, VS)
  PICK(32, 4, 4); PICK(32, 2, 4); PICK(32, 2, 8); PICK(32, 1, 8); PICK(32, 1, 16);
  PICK(64, 4, 4); PICK(64, 2, 4); PICK(64, 2, 8); PICK(64, 1, 4); PICK(64, 1, 8); PICK(64, 1, 16);
  PICK(128, 2, 4); PICK(128, 1, 4); PICK(128, 1, 8);
  PICK_SHARED(32, 16, 2);
  PICK_SHARED(64, 16, 2); PICK_SHARED(64, 16, 4); PICK_SHARED(64, 8, 2); PICK_SHARED(64, 8, 4);
  PICK_SHARED(128, 8, 2); PICK_SHARED(128, 8, 4);
#undef PICK_SHARED
#undef PICK
  return MS_UNSUPPORTED;
#undef GO
}

// Split shape, for long contexts in small batches: every request has exactly one token and the group
// (num_heads / num_kv_heads) is at most 16; the keys are spread over n_splits blocks and combined.
// part_o: float [R, nh, n_splits, d], part_ml: float [R, nh, n_splits, 2].  Each request spreads its blocks of
// 32 keys evenly over the n_splits waves, at least min_blocks to a wave, so the launch does not depend on
// how long the contexts are.
extern "C" int ms_paged_attention_mfma_decode(const void* q, long long q_stride, const void* k_pages,
                                              const void* vt_pages, const int* block_table, int table_stride,
                                              const int* table_rows, const int* q_start, const int* context_lens, void* out,
                                              long long out_stride, void* part_o, void* part_ml, int n_requests,
                                              int num_heads, int num_kv_heads, int head_dim, int page_size,
                                              float scale, int window, int min_blocks, int n_splits,
                                              hipStream_t stream) {
  if (n_requests <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || table_stride <= 0) return MS_BAD_ARG;
  if (num_heads / num_kv_heads > 16) return MS_UNSUPPORTED;
  if (!(scale > 0.f)) return MS_BAD_ARG;
  if (!ms_attention_mfma_supported(head_dim, page_size)) return MS_UNSUPPORTED;
  if (min_blocks <= 0 || n_splits <= 0 || n_splits > COMBINE_MAX_SPLITS) return MS_BAD_ARG;
  if (q_stride % 8 || out_stride % 4 || ((uintptr_t)q % 16) || ((uintptr_t)out % 8) || ((uintptr_t)part_o % 16)) return MS_UNSUPPORTED;
  if (n_requests > 65535 || num_kv_heads > 65535) return MS_UNSUPPORTED;
#define GO(D) return launch_split<D>((const bf16*)q, q_stride, (const bf16*)k_pages, (const bf16*)vt_pages, block_table, table_stride, table_rows, q_start, context_lens, (bf16*)out, out_stride, (float*)part_o, (float*)part_ml, n_requests, num_heads, num_kv_heads, page_size, scale, window, min_blocks, n_splits, stream)
  if (head_dim == 32) GO(32);
  if (head_dim == 64) GO(64);
  GO(128);
#undef GO
}
