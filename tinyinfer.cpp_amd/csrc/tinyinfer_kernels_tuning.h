// Switches of the kernel libraries for tests and measurements only: each forces a choice that the
// libraries otherwise make by the shape (0 restores that).  They are process-wide and no part of the
// product's interface: nothing in the engine calls them.
#pragma once
#ifdef __cplusplus
extern "C" {
#endif
void ti_gemm_bf16_force_tile(int which);      // 1: 256 x 128, 3: 128 x 64, 5: 64 x 128 (SwiGLU only), 6: 64 x 64, 8: 128 x 160, 9: 256 x 160
void ti_gemm_bf16_normed_weight_below(long elements);  // weights of fewer elements keep the norm inside the product (0: the default)
void ti_gemm_bf16_tiles_160(int on);          // 0: no tiles of 160 columns
void ti_gemm_bf16_two_ranges(int on);         // 0: never split a product's columns between 256 x 128 and 128 x 64 tiles
void ti_gemm_bf16_skinny_waves(int waves);    // 4 or 8 wavefronts in the kernel for M <= 64
void ti_gemm_bf16_qkv_prep_min_rows(int rows); // the fewest rows ti_gemm_bf16_qkv_prep serves (17)
void ti_gemm_bf16_qkv_prep_rows(int rows);    // 128 / 256: the rows of ti_gemm_bf16_qkv_prep's tile; 0: by the shape
void ti_gemm_bf16_wide_rows_on(int on);       // 0: 17..64 rows times a weight of 16,384 rows or more take the other kernels
void ti_gemm_bf16_tiled_from(long rows_times_elems); // 17..64 rows x weight elements from which they take the tiled kernels
void ti_gemm_bf16_add_split_on(int on);         // 0: ti_gemm_bf16_add_split serves nothing
void ti_gemm_bf16_use_pipelined(int on);      // 0: the plain tiled kernel for every K
void ti_gemm_bf16_row_per_wave(int on);        // 0: few tokens and a weight of few rows take the 16-row kernels too
void ti_gemm_bf16_skinny_copy(int on);        // 0: up to 16 tokens, fragments of the token rows straight from memory
void ti_gemm_bf16_pieces_on(int on);          // 0: up to 16 rows never take the kernel with the token rows in pieces
void ti_gemm_bf16_skinny_deep(int on);        // 0: four chunks of K in flight per wavefront also for a long K
void ti_attention_decode_shared_query(int on);   // 0: every wavefront of a decode workgroup prepares the query itself
void ti_attention_prefill_groups(int groups);  // 1 or 2 groups of wavefronts per workgroup, 0: by the launch
void ti_attention_prefill_use_lds(int on);     // 0: the kernel without LDS for every head size
#ifdef __cplusplus
}
#endif
