// The C interface of the kernel libraries: what `ops/kernels.py` binds through ctypes, and what a
// C or C++ program may link against.  One shared library per source file (libti_<name>.<hash>.so,
// built by build.py); each also exports `const char* ti_last_error()`.
//
// Conventions.  Every pointer is device memory of the GPU that `stream` belongs to.  Every function
// returns 0 on success, 3 for sizes its kernels do not serve (nothing was launched; use the more
// general function) and another non-zero value for an error; `ti_last_error()` of the same library
// then holds the message.  Nothing here allocates: scratch comes in through arguments.
// dtype codes: 0 = float32, 1 = bfloat16.  Epilogue codes `epi`: 0 store f32, 1 add into f32,
// 2 store in the operand dtype, 3 SwiGLU over stacked [gate; up] rows.
//
// Shapes: M tokens (rows) of a step; H residual width; a cache pool of one layer is
// [pages][2][n_kv][P][hd] with keys as [row][hd] and values transposed as [hd][row]; `table` is
// int32 [requests][table_stride] of page ids (-1: none), `slot[m]` the table row of token m, `pos[m]`
// its position.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// ---- libti_core: embedding, norms, rotation, cache write (templated on the storage dtype)
int ti_embed(int dtype, const void* table, const int* tok, float* x, int M, int H, int V, hipStream_t stream);
// the same; a token below zero stands for fed[-1 - token], an id an earlier kernel on the stream left (fed may be null)
int ti_embed_fed(int dtype, const void* table, const int* tok, const int* fed, int n_fed, float* x, int M, int H, int V,
                 hipStream_t stream);
// out[r] = rmsnorm(x[rows ? rows[r] : r]) * w, in `out_dtype`
int ti_rmsnorm(int out_dtype, const float* x, const float* w, const int* rows, void* out, int n_rows, int H, float eps,
               hipStream_t stream);
// x[r] += partial[0][r] + ... + partial[KS - 1][r] (partial: [KS][n_rows][H], what a product with a
// split K left), written back, then the same norm of the new x.  Returns 3 for what it does not serve.
int ti_rmsnorm_add_partials(int out_dtype, float* x, const float* partial, int KS, const float* w, void* out,
                            int n_rows, int H, float eps, hipStream_t stream);
// half-split rotation in place on f32 [M, heads, hd] (rows `row_stride` floats apart)
int ti_rope_neox(float* x, const int* pos, const float* inv_freq, int M, int heads, int hd, long row_stride,
                 hipStream_t stream);
// table[p][k] = (cos, sin)(p * inv_freq[k]) for p < n_pos
int ti_rope_table(float* table, const float* inv_freq, int half, int n_pos, hipStream_t stream);
// qkv f32 [M, (n_head + 2 n_kv) hd]: per-head norm (weights may be null), rotation (inv_freq may be
// null; rope_table [table_len][hd/2][2] may be null), q to q_out, k and v into the cache pages
int ti_qk_norm_rope_kv_write(int dtype, const float* qkv, const float* q_w, const float* k_w, const float* inv_freq,
                             const float* rope_table, int table_len, const int* pos, const int* slot, const int* table,
                             int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int hd,
                             int page_size, float eps, hipStream_t stream);
// the per-head norm alone, in place
int ti_qk_norm_inplace(float* qkv, int row_width, const float* q_w, const float* k_w, int M, int n_head, int n_kv, int hd,
                       float eps, hipStream_t stream);
// zero `bytes` bytes (whole four-byte words) with a kernel
int ti_fill_zero(void* p, long bytes, hipStream_t stream);
// random values, element i a pure function of (seed, i).  dtype 0 / 1: kind 0 normal(a, b), 1 uniform
// [a, b), 2 constant a; dtype 2 (int32): uniform integers in [a, b)
int ti_fill_random(int dtype, void* p, long n, int kind, float a, float b, unsigned long seed, hipStream_t stream);

// ---- libti_gemm_generic: out (op)= A W^T for any sizes, float32 or bfloat16, fixed summation order
int ti_gemm_generic(int dtype, const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                    hipStream_t stream);

// ---- libti_gemm_bf16: the same on the matrix cores (K a multiple of 8)
int ti_gemm_bf16(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi, hipStream_t stream);
// The adding product for 17..64 rows and a weight of few rows: MFMAs fed straight from memory, K
// split over workgroups whose sums go through `partial` (workspace of partial_bytes).  defer = 0:
// they are added to out here (served: products large enough to gain even so); defer = 1: they stay
// in partial [*splits][M][N] and the caller adds them (ti_gemm_bf16_partials_add, or
// ti_rmsnorm_add_partials on the way to the next norm); defer = 2: as 1, but added here.
// Returns 3 for what it does not serve.
int ti_gemm_bf16_add_split(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                         void* partial, long partial_bytes, int defer, int* splits, hipStream_t stream);
int ti_gemm_bf16_partials_add(float* out, const float* partial, int KS, long count, hipStream_t stream);
// out = A W^T stored in 32-bit for 17..64 rows times a large weight of few tiles: K split over workgroups
// (partial: workspace of partial_bytes), the shares added up by a kernel of its own; 3: not served
int ti_gemm_bf16_store_split(const void* A, const void* W, void* out, int M, int N, int K, long lda, void* partial,
                             long partial_bytes, hipStream_t stream);
// the kernel of ti_gemm_bf16_add_split alone, for tests: any epilogue, 1..64 rows, K split ks ways
int ti_gemm_bf16_mblocks_any(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                             void* partial, int ks, hipStream_t stream);
// the kernel for up to 16 rows that takes the token rows through LDS in pieces, alone, for tests: any
// epilogue, K a multiple of 64 split ks ways (adding epilogue only; partial f32 [ks][M][N])
int ti_gemm_bf16_pieces_any(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                            void* partial, int ks, hipStream_t stream);
// out (op)= rmsnorm(x; nw, eps) W^T for M <= 16, K a multiple of 64
int ti_gemm_bf16_normed(const float* x, const float* nw, float eps, const void* W, void* out, int M, int N, int K, int epi,
                        hipStream_t stream);
// the q/k/v product of a step (M > 16) that finishes its heads itself: see ti_qk_norm_rope_kv_write
int ti_gemm_bf16_qkv_prep(const void* A, const void* W, int M, int K, long lda, const float* q_w, const float* k_w,
                          float eps, const float* inv_freq, const float* rope_table, int table_len, const int* pos,
                          const int* slot, const int* table, int table_stride, void* pool, void* q_out, int n_head,
                          int n_kv, int hd, int page_size, hipStream_t stream);

// ---- libti_attention_generic: paged causal attention of every row, any head size in steps of 16
int ti_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                      const int* slot, void* out, int M, int n_head, int n_kv, int hd, int page_size, float scale,
                      int window, hipStream_t stream);

// ---- libti_attention_bf16: the same on the matrix cores (head sizes 32, 64, 128; pages of 16 n rows)
// rows of single tokens; n_splits > 1 needs part_o f32 [n_rows, n_head, n_splits, hd] and part_ml f32
// [n_rows, n_head, n_splits, 2]
int ti_attention_decode_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                             const int* slot, const int* rows, void* out, float* part_o, float* part_ml, int n_rows,
                             int n_head, int n_kv, int hd, int page_size, float scale, int window, int n_splits,
                             hipStream_t stream);
// the same from the 32-bit projections: norm, rotation and the cache write of the row's own key and
// value happen inside (head sizes 64 and 128, at most 16 q heads per kv head).  slot may be null
// (both entry points) where row m of the step is row m of the block tables and a table row has at
// most 1,024 entries: the page ids are then fetched beside the position, not behind it
int ti_attention_decode_prepared_bf16(const float* qkv, int row_width, const float* q_w, const float* k_w, float eps,
                                      const float* inv_freq, const float* rope_table, int table_len, void* pool,
                                      int write_kv, const int* table, int table_stride, const int* pos,
                                      const int* slot, void* out, float* part_o, float* part_ml, int n_rows,
                                      int n_head, int n_kv, int hd, int page_size, float scale, int window,
                                      int n_splits, hipStream_t stream);
// portions of prompts: tiles int32 [n_tiles][2] = (entry, first row) of 128 rows each, entries int32
// [n_entries][4] = (row0, n_tokens, start_pos, -)
int ti_attention_prefill_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* tiles,
                              const int* entries, void* out, int n_tiles, int n_head, int n_kv, int hd, int page_size,
                              float scale, int window, hipStream_t stream);
// the same for launches of few tiles (head sizes 64, 128): tiles of 64 rows ordered from the most visible
// keys to the fewest; a workgroup takes tile b and tile n_tiles - 1 - b, so that all have about the same work
// n_splits > 1 (up to 8): the keys of every tile are cut into that many runs, each with a workgroup of its
// own, for launches of few tiles against a long context; their results go through part_o [n_rows][n_head]
// [n_splits][hd] and part_ml [n_rows][n_head][n_splits][2] and are merged into out for all n_rows rows of the
// step (rows of no tile get what lies in the buffers: whoever owns them writes them afterwards).
// paired = 0: the same kernel with a workgroup per tile, for launches that fit the chip in one round.
int ti_attention_prefill_paired_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                     const int* tiles, const int* entries, void* out, int n_tiles, int n_head,
                                     int n_kv, int hd, int page_size, float scale, int window, int n_rows,
                                     float* part_o, float* part_ml, int n_splits, int paired, hipStream_t stream);

// ---- libti_sampling
// out[r] = lowest index of the largest logit; scratch: 2 * 64 * n_rows four-byte words (two stages:
// 64 workgroups per row, then one) or null (one workgroup reads a whole row)
int ti_argmax(const float* logits, int* out, void* scratch, int n_rows, int V, hipStream_t stream);
// ti_argmax for callers that cannot allocate (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc): the same two-stage kernels with their partial results in a
// device array of the library itself (128 KiB on each GPU it runs on, kept until the process ends)
// instead of a workspace argument.  At most 256 rows, else an error.  It calls no hipMalloc, hipFree or
// allocating routine; calls that overlap on one GPU share the array and race.  It has no counterpart in
// the reference: it is there for callers that cannot allocate.
int ti_argmax_static(const float* logits, int* out, int n_rows, int V, hipStream_t stream);
// temperature, top-k (0: all), top-p and one uniform number per row.  scratch: ti_sample_scratch_bytes(n_rows)
// bytes, zero before the first call and touched by nothing else since (the kernels leave them at zero; calls
// that overlap on one workspace race), or null: then one workgroup walks a whole row, as it does for the rows
// that have no top-k cut.
long ti_sample_scratch_bytes(int n_rows);
int ti_sample(const float* logits, const float* temp, const int* top_k, const float* top_p, const float* uni, int* out,
              void* scratch, int n_rows, int V, hipStream_t stream);


// ---- libti_measure: what the GPU delivers, for the bench tool's fractions
// reads `bytes` bytes (a multiple of 16) once with `blocks` workgroups of 256 threads; sink: `blocks` words
int ti_measure_read(const void* p, long bytes, void* sink, int blocks, hipStream_t stream);
// `blocks` workgroups of four wavefronts, each wavefront `iters` rounds of four 32x32x16 bfloat16 MFMAs on
// registers: blocks * 4 * iters * 4 * 32,768 flops
int ti_measure_mfma(int blocks, int iters, void* sink, hipStream_t stream);
// `blocks` workgroups of one wavefront each read one word every `stride` bytes of [p, p + bytes)
int ti_measure_touch(const void* p, long bytes, long stride, void* sink, int blocks, hipStream_t stream);

#ifdef __cplusplus
}
#endif
