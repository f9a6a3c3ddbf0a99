// Paged causal grouped-query attention in bfloat16 on the matrix cores of gfx950,
// for decode rows (flash decoding: the context of a row is split over several
// workgroups and merged) and for portions of prompts (flash attention over the
// pages, earlier portions included).
//
// Both walk the cache in blocks of 16 positions.  A page holds keys as
// [row][head_dim] and values transposed as [head_dim][row], so both products
// read their operands along the dimension they reduce over, straight from memory:
//   S^T (16 keys x 16 columns)  = K (16 x hd) . Q^T          v_mfma_f32_16x16x32_bf16
//   O^T (hd x 16 columns)      += V^T (hd x 16 keys) . P^T   v_mfma_f32_16x16x16_bf16
// The transposed score tile leaves each lane with four keys of one column, which
// is exactly the operand layout the second product wants for P^T: no shuffles,
// no LDS between the two.  The softmax statistics of a column are one scalar per
// lane; scores, statistics and outputs are 32-bit.
//
// What the 16 columns are differs:
//   decode   the q heads that share one kv head, for one token: the kv head's
//            keys and values are read once for all of them.  Four wavefronts take
//            the blocks of the split in turn and merge through LDS.
//   prefill  16 consecutive tokens of one q head; a workgroup's four wavefronts
//            take four such tiles of the same head, so they walk the same pages
//            together and share them in the cache.
// (The reference scans positions with 16-lane groups and FMA for both cases:
// /root/reference/src/cuda/attention.cu:107-198.)
#include "common.h"

TI_ERROR_API

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short short4v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Frag8 {
  uint4 u;
  bf16x8 v;
};
union Frag4 {
  uint2 u;
  short4v v;
  bf16_t h[4];
};

struct PagedKV {
  const bf16_t* pool;   // [pages][2][n_kv][P * hd]
  const int* table;     // block-table row of the request
  int P;                // rows per page (multiple of 16)
  int n_kv;
  int kvh;
};

// One block of 16 keys [key0, key0 + 16) for this wavefront's 16 columns.
//   qf       Q^T fragments: column lane % 16, dims 32 * step + 8 * (lane / 16) .. + 7
//   lo, hi   the keys this lane's column may see: lo <= key <= hi
//   kv_last  last position of the request that has been written (rows after it hold rubbish)
//   check    false if every key of the block is visible to every column and written
template <int HD>
__device__ __forceinline__ void attend_block(const PagedKV& kv, const Frag8* qf, int key0, int lo, int hi,
                                             int kv_last, bool check, float scale, float& m, float& l,
                                             floatx4* o) {
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int page = kv.table[key0 / kv.P];
  if (page < 0) return;   // given back or never taken: nothing visible lies there
  const int prow = key0 % kv.P;
  const size_t page_elems = (size_t)2 * kv.n_kv * kv.P * HD;
  const bf16_t* kbase = kv.pool + (size_t)page * page_elems + (size_t)kv.kvh * kv.P * HD + (size_t)prow * HD;
  const bf16_t* vbase = kv.pool + (size_t)page * page_elems + (size_t)(kv.n_kv + kv.kvh) * kv.P * HD + prow;

  // S^T = K . Q^T
  Frag8 kf[HD / 32];
#pragma unroll
  for (int s = 0; s < HD / 32; ++s)
    kf[s].u = *reinterpret_cast<const uint4*>(kbase + (size_t)r16 * HD + s * 32 + quad * 8);
  // the value fragments do not depend on the scores: issue their loads now
  Frag4 vf[HD / 16];
#pragma unroll
  for (int d = 0; d < HD / 16; ++d)
    vf[d].u = *reinterpret_cast<const uint2*>(vbase + (size_t)(d * 16 + r16) * kv.P + quad * 4);
  floatx4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < HD / 32; ++s) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[s].v, qf[s].v, sc, 0, 0, 0);

  // this lane: keys key0 + 4 quad + i of column r16
  float sv[4];
  float bm = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int key = key0 + quad * 4 + i;
    sv[i] = (!check || (key >= lo && key <= hi)) ? sc[i] * scale : -INFINITY;
    bm = fmaxf(bm, sv[i]);
  }
  bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
  bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
  const float m_new = fmaxf(m, bm);
  const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
  const float alpha = __expf(m - m_safe);
  Frag4 pf;
  float ps = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float p = __expf(sv[i] - m_safe);
    ps += p;
    pf.h[i] = f2bf(p);
  }
  l = l * alpha + ps;
  m = m_new;
  if (check) {
    // rows never written may hold anything, NaN included, and 0 * NaN is NaN
#pragma unroll
    for (int d = 0; d < HD / 16; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (key0 + quad * 4 + i > kv_last) vf[d].h[i] = 0;
  }
#pragma unroll
  for (int d = 0; d < HD / 16; ++d) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[d][i] *= alpha;
    o[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[d].v, pf.v, o[d], 0, 0, 0);
  }
}

// =================================================================== decode
// grid (rows, n_kv * head_parts, splits), 256 threads.  Partials (splits > 1):
//   part_o [row][head][split][hd], part_ml [row][head][split][2] = (max, sum)
template <int HD>
__global__ void __launch_bounds__(256)
attn_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool, const int* __restrict__ table,
                   int table_stride, const int* __restrict__ pos, const int* __restrict__ slot,
                   const int* __restrict__ rows, bf16_t* __restrict__ out, float* __restrict__ part_o,
                   float* __restrict__ part_ml, int n_head, int n_kv, int P, float scale, int window,
                   int n_splits) {
  __shared__ float s_o[4][HD / 16][4][64];
  __shared__ float s_m[4][16], s_l[4][16];
  const int ridx = blockIdx.x;
  const int m_row = rows ? rows[ridx] : ridx;
  const int G = n_head / n_kv;
  const int parts = (G + 15) / 16;   // q heads per kv head, in sets of up to 16 columns
  const int kvh = blockIdx.y / parts, part = blockIdx.y % parts;
  const int split = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int n_cols = min(16, G - part * 16);
  const int head = kvh * G + part * 16 + r16;   // valid if r16 < n_cols

  const int p_q = pos[m_row];
  const int lo = (window > 0 && p_q - window + 1 > 0) ? p_q - window + 1 : 0;
  const int blk_lo = lo / 16, blk_hi = p_q / 16;
  const int n_blk = blk_hi - blk_lo + 1;
  const int per = (n_blk + n_splits - 1) / n_splits;
  const int b0 = blk_lo + split * per;
  const int b1 = min(blk_hi + 1, b0 + per);

  PagedKV kv{pool, table + (size_t)slot[m_row] * table_stride, P, n_kv, kvh};
  Frag8 qf[HD / 32];
#pragma unroll
  for (int s = 0; s < HD / 32; ++s) {
    qf[s].u = make_uint4(0, 0, 0, 0);
    if (r16 < n_cols)
      qf[s].u = *reinterpret_cast<const uint4*>(q + ((size_t)m_row * n_head + head) * HD + s * 32 + quad * 8);
  }
  float mx = -INFINITY, l = 0.f;
  floatx4 o[HD / 16];
#pragma unroll
  for (int d = 0; d < HD / 16; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int b = b0 + wave; b < b1; b += 4) {
    const bool check = (b == blk_lo) || (b == blk_hi);
    attend_block<HD>(kv, qf, b * 16, lo, p_q, p_q, check, scale, mx, l, o);
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // merge the four wavefronts: lane keeps its (column, dims) in all of them
#pragma unroll
  for (int d = 0; d < HD / 16; ++d)
#pragma unroll
    for (int i = 0; i < 4; ++i) s_o[wave][d][i][lane] = o[d][i];
  if (quad == 0) {
    s_m[wave][r16] = mx;
    s_l[wave][r16] = l;
  }
  __syncthreads();
  float mm = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) mm = fmaxf(mm, s_m[w][r16]);
  float wgt[4], lt = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    wgt[w] = (s_m[w][r16] == -INFINITY) ? 0.f : __expf(s_m[w][r16] - mm);
    lt += s_l[w][r16] * wgt[w];
  }
  if (r16 >= n_cols) return;
  // wavefront w finishes dim blocks w, w + 4, ...
  for (int d = wave; d < HD / 16; d += 4) {
    float acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[i] = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) acc[i] += s_o[w][d][i][lane] * wgt[w];
    }
    const int dim = d * 16 + quad * 4;
    if (n_splits == 1) {
      const float inv = 1.0f / lt;
      Frag4 r;
#pragma unroll
      for (int i = 0; i < 4; ++i) r.h[i] = f2bf(acc[i] * inv);
      *reinterpret_cast<uint2*>(out + ((size_t)m_row * n_head + head) * HD + dim) = r.u;
    } else {
      float* po = part_o + (((size_t)ridx * n_head + head) * n_splits + split) * HD + dim;
      *reinterpret_cast<float4*>(po) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    }
  }
  if (n_splits > 1 && wave == 0 && quad == 0) {
    float* pm = part_ml + (((size_t)ridx * n_head + head) * n_splits + split) * 2;
    pm[0] = mm;
    pm[1] = lt;
  }
}

// grid (rows, n_head), HD threads: out = sum_s w_s o_s / sum_s w_s l_s, w_s = exp(m_s - max m)
template <int HD>
__global__ void __launch_bounds__(HD)
attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                  const int* __restrict__ rows, bf16_t* __restrict__ out, int n_head, int n_splits) {
  const int ridx = blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  const int m_row = rows ? rows[ridx] : ridx;
  const float* pm = part_ml + ((size_t)ridx * n_head + head) * n_splits * 2;
  const float* po = part_o + ((size_t)ridx * n_head + head) * n_splits * HD;
  float mm = -INFINITY;
  for (int s = 0; s < n_splits; ++s) mm = fmaxf(mm, pm[2 * s]);
  float lt = 0.f, acc = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float w = (pm[2 * s] == -INFINITY) ? 0.f : __expf(pm[2 * s] - mm);
    lt += pm[2 * s + 1] * w;
    acc += po[(size_t)s * HD + d] * w;
  }
  out[((size_t)m_row * n_head + head) * HD + d] = f2bf(acc / lt);
}

// ================================================================== prefill
// grid (tiles, n_head), 256 threads.  tiles[t] = (entry, first row); entries[e] =
// (row0, n_tokens, start_pos, -).  A tile is 64 rows; wavefront w takes rows
// first + 16 w .. + 15 as its columns.
template <int HD>
__global__ void __launch_bounds__(256)
attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool, const int* __restrict__ table,
                    int table_stride, const int* __restrict__ tiles, const int* __restrict__ entries,
                    bf16_t* __restrict__ out, int n_head, int n_kv, int P, float scale, int window) {
  const int entry = tiles[2 * blockIdx.x], first = tiles[2 * blockIdx.x + 1];
  const int row0 = entries[4 * entry], n_tok = entries[4 * entry + 1], start = entries[4 * entry + 2];
  const int head = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int w_first = first + wave * 16;            // first row of this wavefront's tile
  const int row_end = row0 + n_tok;
  if (w_first >= row_end) return;
  const int w_rows = min(16, row_end - w_first);
  const int my_row = w_first + r16;
  const bool col_ok = r16 < w_rows;
  const int my_pos = start + (my_row - row0);       // position of this lane's column
  const int kv_last = start + n_tok - 1;
  const int pos_first = start + (w_first - row0), pos_last = pos_first + w_rows - 1;
  const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
  const int tile_lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;

  PagedKV kv{pool, table + (size_t)entry * table_stride, P, n_kv, head / (n_head / n_kv)};
  Frag8 qf[HD / 32];
#pragma unroll
  for (int s = 0; s < HD / 32; ++s) {
    qf[s].u = make_uint4(0, 0, 0, 0);
    if (col_ok) qf[s].u = *reinterpret_cast<const uint4*>(q + ((size_t)my_row * n_head + head) * HD + s * 32 + quad * 8);
  }
  float mx = -INFINITY, l = 0.f;
  floatx4 o[HD / 16];
#pragma unroll
  for (int d = 0; d < HD / 16; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int blk_lo = tile_lo / 16, blk_hi = pos_last / 16;
  // a block is free of checks if every column sees all of it: it ends at or before the
  // tile's first position and (with a window) starts inside the last column's window
  const int hi_col = col_ok ? my_pos : -1;          // columns beyond the portion see nothing
  for (int b = blk_lo; b <= blk_hi; ++b) {
    const int key0 = b * 16;
    const bool inside = (key0 + 15 <= pos_first) && (w_rows == 16) &&
                        (window <= 0 || key0 >= pos_last - window + 1) && (key0 >= tile_lo);
    attend_block<HD>(kv, qf, key0, my_lo, hi_col, kv_last, !inside, scale, mx, l, o);
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!col_ok) return;
  const float inv = 1.0f / l;
#pragma unroll
  for (int d = 0; d < HD / 16; ++d) {
    Frag4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.h[i] = f2bf(o[d][i] * inv);
    *reinterpret_cast<uint2*>(out + ((size_t)my_row * n_head + head) * HD + d * 16 + quad * 4) = r.u;
  }
}

// ------------------------------------------------------------------ dispatch
static int check_common(const char* what, int n_head, int n_kv, int hd, int P, int table_stride) {
  if (!(hd == 32 || hd == 64 || hd == 128)) {
    ti_set_error("%s: head_dim %d is not served by the matrix-core kernels (32, 64, 128)", what, hd);
    return 3;
  }
  if (P % 16 != 0) {
    ti_set_error("%s: page size %d is not a multiple of 16", what, P);
    return 3;
  }
  if (n_head <= 0 || n_kv <= 0 || n_head % n_kv != 0 || table_stride <= 0) {
    ti_set_error("%s: heads %d / kv_heads %d / table_stride %d", what, n_head, n_kv, table_stride);
    return 1;
  }
  return 0;
}

// Decode rows.  rows: which rows of the step (nullptr: rows 0..n_rows-1).  n_splits > 1 needs
// part_o (float [n_rows, n_head, n_splits, hd]) and part_ml (float [n_rows, n_head, n_splits, 2]).
// Returns 3 for sizes these kernels do not serve.
extern "C" int ti_attention_decode_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                        const int* pos, const int* slot, const int* rows, void* out,
                                        float* part_o, float* part_ml, int n_rows, int n_head, int n_kv, int hd,
                                        int page_size, float scale, int window, int n_splits,
                                        hipStream_t stream) {
  int rc = check_common("attention_decode", n_head, n_kv, hd, page_size, table_stride);
  if (rc) return rc;
  TI_REQUIRE(n_splits >= 1 && n_splits <= 65535, "attention_decode: bad split count %d", n_splits);
  TI_REQUIRE(n_splits == 1 || (part_o && part_ml), "attention_decode: splits need partial buffers");
  if (n_rows == 0) return 0;
  const int parts = (n_head / n_kv + 15) / 16;
  TI_REQUIRE(n_kv * parts <= 65535, "attention_decode: too many heads");
  dim3 grid(n_rows, n_kv * parts, n_splits);
#define TI_DEC(H)                                                                                          \
  case H:                                                                                                  \
    attn_decode_kernel<H><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table,           \
                                                    table_stride, pos, slot, rows, (bf16_t*)out, part_o,    \
                                                    part_ml, n_head, n_kv, page_size, scale, window,        \
                                                    n_splits);                                              \
    if (n_splits > 1)                                                                                       \
      attn_merge_kernel<H><<<dim3(n_rows, n_head), H, 0, stream>>>(part_o, part_ml, rows, (bf16_t*)out,     \
                                                                   n_head, n_splits);                       \
    break;
  switch (hd) {
    TI_DEC(32) TI_DEC(64) TI_DEC(128)
  }
#undef TI_DEC
  TI_LAUNCH_CHECK();
  return 0;
}

// Portions of prompts.  tiles: int [n_tiles, 2] = (entry, first row), each tile 64 rows;
// entries: int [n_entries, 4] = (row0, n_tokens, start_pos, -); table row e belongs to entry e.
extern "C" int ti_attention_prefill_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                         const int* tiles, const int* entries, void* out, int n_tiles,
                                         int n_head, int n_kv, int hd, int page_size, float scale, int window,
                                         hipStream_t stream) {
  int rc = check_common("attention_prefill", n_head, n_kv, hd, page_size, table_stride);
  if (rc) return rc;
  TI_REQUIRE(n_head <= 65535, "attention_prefill: too many heads");
  if (n_tiles == 0) return 0;
  dim3 grid(n_tiles, n_head);
#define TI_PRE(H)                                                                                          \
  case H:                                                                                                  \
    attn_prefill_kernel<H><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table,          \
                                                     table_stride, tiles, entries, (bf16_t*)out, n_head,    \
                                                     n_kv, page_size, scale, window);                       \
    break;
  switch (hd) {
    TI_PRE(32) TI_PRE(64) TI_PRE(128)
  }
#undef TI_PRE
  TI_LAUNCH_CHECK();
  return 0;
}
