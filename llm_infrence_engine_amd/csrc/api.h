// C entry points of the gfx950 kernel library.  Every function enqueues work on `stream` and returns
// 0, or a non-zero code (see common.h) without launching when it refuses its arguments.  Pointers are
// device pointers; matrices are row-major.  `dtype` is 0 for float and 1 for bfloat16.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

int ms_embed(const int* ids, const void* table, float* out, int n_tokens, int hidden, int dtype, hipStream_t stream);

int ms_rms_norm(float* x, const void* delta, int delta_dtype, int n_partials, long long partial_stride,
                const float* weight, const int* rows, void* out, int n_rows, int hidden, float eps, int write_back,
                int dtype, hipStream_t stream);

int ms_bias_add(void* x, const float* bias, int n_rows, int width, int dtype, hipStream_t stream);

// tables / slots: host arrays of n_groups device pointers (block table int32 [table rows, table_stride], slot
// mapping int32 [n_rows]); table_rows int32 [n_rows]: the table's row of each row of the batch; draw_index int32
// [n_rows] (may be null): counted up by one for every live row.  At most ms_max_cache_groups() groups.
int ms_max_cache_groups();
int ms_decode_advance(const int* prev_tokens, int* token_ids, int* positions, int* context_lens, const int* n_live,
                      const int* table_rows, int* draw_index, const int* const* tables, int* const* slots,
                      int n_groups, int table_stride, int page_size, int n_rows, hipStream_t stream);

// Block tables kept on the device: tables[g][index[g][i]] = value[g][i] for i < counts[g] (counts: device ints),
// every index at most once per group; max_updates bounds counts, table_elems bounds the indices.
int ms_table_update(int* const* tables, const int* const* index, const int* const* value, const int* counts,
                    int n_groups, int max_updates, long long table_elems, hipStream_t stream);

// rows[i] of a [n, row_bytes] tensor become zero (row_bytes a multiple of 4), i < n_rows; `count` (null: n_rows)
// is a device int that may ask for fewer.
int ms_zero_rows(void* base, long long row_bytes, const int* rows, const int* count, int n_rows, hipStream_t stream);

// A plain streaming read of `bytes` for bandwidth measurements; sink: unsigned [ms_read_probe_blocks()].
int ms_read_probe_blocks();
int ms_read_probe(const void* base, long long bytes, unsigned* sink, hipStream_t stream);

int ms_residual_add(float* x, const void* delta, long long total, int dtype, hipStream_t stream);

int ms_silu_mul(const void* gate_up, void* out, int n_tokens, int intermediate, int dtype, hipStream_t stream);

int ms_rope_store(void* qkv, const float* bias, const int* positions, const float* inv_freq, const int* slot_mapping, void* k_pages,
                  void* v_pages, int n_tokens, int num_heads, int num_kv_heads, int head_dim, int rot_dim,
                  int page_size, int v_transposed, int dtype, hipStream_t stream);

// table float [n_tokens, half, 2] = (cos, sin) of float(positions[n]) * inv_freq[j]
int ms_rope_table(const int* positions, const float* inv_freq, float* table, int n_tokens, int half, hipStream_t stream);

int ms_gemm_generic(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, long long lda,
                    long long ldw, long long ldc, int in_dtype, int out_dtype, int accumulate, hipStream_t stream);

int ms_gemm_skinny(const void* A, long long lda, const void* W, long long ldw, const float* bias, void* out,
                   long long ldo, int M, int N, int K, int epilogue, int out_dtype, hipStream_t stream);

void ms_gemm_skinny_force(int ntile, int waves, int token_groups);
void ms_attention_mfma_force(int nt, int waves, int dim_shares);

int ms_gemm_stream(const void* A, long long lda, const int* rows, const float* norm_w, float eps, const void* W,
                   long long ldw, const float* bias, void* out, long long ldo, int M, int N, int K, int epilogue,
                   int out_dtype, int norm, int any_shape, hipStream_t stream);

int ms_gemm_panel(const void* A, long long lda, const int* rows, const float* norm_w, float eps, const void* W,
                   long long ldw, const float* bias, void* out, long long ldo, int M, int N, int K, int epilogue,
                   int out_dtype, int norm, int any_shape, hipStream_t stream);

int ms_gemm_panel_splitk_parts(int M, int N, int K);
int ms_gemm_panel_splitk(const void* A, long long lda, const void* W, long long ldw, const float* bias, void* out,
                         long long ldo, int M, int N, int K, int epilogue, int out_dtype, void* partial, int parts,
                         hipStream_t stream);

// Many rows (prompt portions): the tiled matrix-core product, bfloat16 in and out, with the gated activation
// as epilogue 1; K a multiple of 64 (ms_gemm_tiled_force: measurements, 0 leaves the choice of tile, 1 to 5 force one;
// ms_gemm_tiled_pays: whether the gated product is faster here than as library product and activation kernel).
int ms_gemm_tiled(const void* A, long long lda, const void* W, long long ldw, void* out, long long ldo, int M, int N,
                  int K, int epilogue, hipStream_t stream);
void ms_gemm_tiled_force(int tile);
void ms_gemm_tiled_force_xcd_split(int xm);   // measurements: rows of XCDs over the tiles (1, 2, 4, 8); 0 leaves the choice
int ms_gemm_tiled_pays(int M, int N, int K);
int ms_gemm_tiled_plain_pays(int M, int N, int K);   // the same question for a plain product (epilogue 0)

// The q/k/v product of many tokens with bias, rotation (whole heads, pairs (j, j + d/2)) and the store of k and v
// into the cache pages as its epilogue: A [M, lda] bfloat16, W [(nh + 2 nkv) d, ldw], q_out [M, nh d] bfloat16;
// head_dim 64 or 128; rope_table float [M, d / 2, 2] from ms_rope_table.  Pages as in ms_rope_store.  ms_gemm_tiled_qkv_pays: where it beats product + rotation kernel.
int ms_gemm_tiled_qkv(const void* A, long long lda, const void* W, long long ldw, const float* bias,
                      const float* rope_table, const int* slot_mapping, void* q_out, void* k_pages, void* v_pages, int M,
                      int K, int nh, int nkv, int head_dim, int page_size, int v_transposed, hipStream_t stream);
int ms_gemm_tiled_qkv_pays(int M, int N, int K, int head_dim);

int ms_gemm_skinny_norm(const float* x, long long ldx, const int* rows, const float* norm_w, float eps, const void* W,
                        long long ldw, const float* bias, void* out, long long ldo, int M, int N, int K, int epilogue,
                        int out_dtype, hipStream_t stream);

void ms_qkv_rope_store_force(int pair8);

int ms_qkv_rope_store(const float* x, long long ldx, const float* norm_w, float eps, const void* W, const float* bias,
                      const int* positions, const float* inv_freq, const int* slot_mapping, void* q_out,
                      void* k_pages, void* v_pages, int M, int K, int num_heads, int num_kv_heads, int head_dim,
                      int page_size, int v_transposed, hipStream_t stream);

int ms_paged_attention_generic(const void* q, long long q_stride, const void* k_pages, const void* v_pages,
                               const int* block_table, int table_stride, const int* table_rows,
                               const int* n_live_tokens, const int* token_req, const int* positions,
                               void* out, long long out_stride, int n_tokens, int num_heads, int num_kv_heads,
                               int head_dim, int page_size, long long num_pages, float scale, int window,
                               int v_transposed, int dtype, hipStream_t stream);

int ms_attention_mfma_supported(int head_dim, int page_size);

int ms_paged_attention_mfma(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                            const int* block_table, int table_stride, const int* table_rows, const int* q_start,
                            const int* context_lens, void* out, long long out_stride, int n_requests, int n_tokens,
                            int max_q_len, int num_heads, int num_kv_heads, int head_dim, int page_size, float scale,
                            int window, hipStream_t stream);

int ms_paged_attention_mfma_decode(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                                   const int* block_table, int table_stride, const int* table_rows,
                                   const int* q_start, const int* context_lens, void* out, long long out_stride,
                                   void* part_o,
                                   void* part_ml, int n_requests, int num_heads, int num_kv_heads, int head_dim,
                                   int page_size, float scale, int window, int min_blocks, int n_splits,
                                   hipStream_t stream);

int ms_argmax(const float* logits, long long ld, int n_rows, int vocab, float* scratch_val, int* scratch_idx,
              int n_chunks, int* out, hipStream_t stream);

// The one entry point that allocates nothing.  It has no counterpart in the reference; it is for callers that
// cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  Same result as ms_argmax, but the stage-1 results live in a static device array of the library
// (256 KB on every GPU the library runs on, held until the process ends) instead of scratch_val / scratch_idx.
// The caller still passes logits and out; `stream` must belong to the current device.  Limits: n_rows <= 256
// and n_chunks <= 128 (ms_argmax_static_limits reports them); beyond them the call returns MS_UNSUPPORTED (2)
// and launches nothing.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (different
// streams or threads) race; calls on one stream, or ordered by events, do not.  Nothing in the array needs
// clearing between calls.  The array's address is looked up once per device, at the first call there or by
// ms_argmax_static_init() with that device current (call it before a stream capture starts).
int ms_argmax_static_init();
void ms_argmax_static_limits(int* max_rows, int* max_chunks);
int ms_argmax_static(const float* logits, long long ld, int n_rows, int vocab, int n_chunks, int* out,
                     hipStream_t stream);

// workspace: ms_sample_workspace_bytes(n_rows) bytes of device memory (any contents); use_top_k / use_top_p: 0 if
// no row has a top_k in (0, vocab) / a top_p below 1.
long long ms_sample_workspace_bytes(int n_rows);
int ms_sample(const float* logits, long long ld, int n_rows, int vocab, const float* temperature, const int* top_k,
              const float* top_p, const unsigned long long* seeds, const int* draw_index, int* out, void* workspace,
              int use_top_k, int use_top_p, hipStream_t stream);

}  // extern "C"
