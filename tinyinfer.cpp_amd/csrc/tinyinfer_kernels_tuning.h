// Switches of the bfloat16 kernel libraries for tests and measurements only: each forces a choice that a
// library otherwise makes by the shape.  They are no part of the product's interface: nothing in the engine
// sets one.  Each of libti_gemm_bf16 and libti_attention_bf16 exports the two functions below; the state is
// the library's (process-wide), and the host library's Ops applies an object's own overrides around its calls
// (Ops::tune) and resets them afterwards.
//
// libti_gemm_bf16:
//   force_tile           1: 256 x 128, 3: 128 x 64, 5: 64 x 128 (SwiGLU only), 6: 64 x 64, 8: 128 x 160, 9: 256 x 160, 10: 256 x 256; 0: by the shape
//   normed_weight_below  weights of fewer elements keep the norm inside the product (0: the default)
//   tiles_160            0: no tiles of 160 columns
//   tiles_256            0: no tiles of 256 x 256
//   two_ranges           0: never split a product's columns between 256 x 128 and 128 x 64 tiles
//   xcd_rows             row tiles per block of the order in which a die takes the tiles of a tiled product (-1: the grid's order,
//                        0: by the weight's size)
//   skinny_waves         4 or 8 wavefronts in the kernel for M <= 64 (0: by the shape)
//   qkv_prep_min_rows    the fewest rows ti_gemm_bf16_qkv_prep serves (17)
//   qkv_prep_rows        128 / 256: the rows of ti_gemm_bf16_qkv_prep's tile; 0: by the shape
//   wide_rows            0: 17..64 rows times a weight of 16,384 rows or more take the other kernels
//   tiled_from           17..64 rows x weight elements from which they take the tiled kernels (280 Mi)
//   add_split            0: ti_gemm_bf16_add_split serves nothing
//   use_pipelined        0: the plain tiled kernel for every K
//   row_per_wave         0: few tokens and a weight of few rows take the 16-row kernels too
//   skinny_copy          0: up to 16 tokens, fragments of the token rows straight from memory
//   pieces               0: up to 16 rows never take the kernel with the token rows in pieces
//   skinny_deep          0: four chunks of K in flight per wavefront also for a long K
//   rows_direct          0: the kernel with a weight row per wavefront takes its token rows through LDS for every K
//   wide_rows_min_n      the fewest weight rows from which 17..64 rows take the kernel that keeps them in registers (16,384)
//   wide_rows_grid       its number of workgroups (0: a tile of 16 weight rows each, at most one per compute unit)
// libti_attention_bf16:
//   decode_shared_query  0: every wavefront of a decode workgroup prepares the query itself
//   prefill_groups       1 or 2 groups of wavefronts per workgroup, 0: by the launch
//   prefill_use_lds      0: the kernel without LDS for every head size
#pragma once
#ifdef __cplusplus
extern "C" {
#endif
int ti_tuning_set(const char* name, long value);     // 0, or 1 for a name the library does not know
void ti_tuning_reset();                              // every choice back to the library's own
#ifdef __cplusplus
}
#endif
