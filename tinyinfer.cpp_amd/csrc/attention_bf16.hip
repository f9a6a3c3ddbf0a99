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
#include <string>
#include <type_traits>
#include <utility>
#include "common.h"
#include "tinyinfer_kernels.h"
#include "tinyinfer_kernels_tuning.h"
#include "qk_prep.h"

TI_ERROR_API

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short short4v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define TI_LOG2E 1.4426950408889634f

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

// The fragments of two blocks of 16 keys each, [keyA, keyA + 16) and [keyB, keyB + 16),
// for the two products.  The pair is what one turn of the walk handles: one softmax
// update and one rescaling of the output for 32 keys, and the second product as
// v_mfma_f32_16x16x32_bf16 over both blocks at once.
template <int HD>
struct KVPair {
  Frag8 k[2][HD / 32];   // K:   row lane % 16, dims 32 s + 8 (lane / 16) .. + 7
  Frag8 v[HD / 16];      // V^T: row (dim) 16 d + lane % 16; elements 0..3: keys 4 (lane / 16) .. + 3 of
                         //      block A, elements 4..7: the same keys of block B
};

// Issue the loads of a pair.  They are unconditional (the caller passes pages that
// exist, whatever they hold) so that the compiler can count them and let the
// arithmetic of the pair before run while they are in flight.
template <int HD>
__device__ __forceinline__ void load_pair(const PagedKV& kv, int pageA, int keyA, int pageB, int keyB,
                                          KVPair<HD>& f) {
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  // where a block's keys and values start is the same in every lane (scalar registers); a lane
  // adds one offset of its own, and the steps are constants in the load instructions
  const size_t page_elems = (size_t)2 * kv.n_kv * kv.P * HD;
  const int rowA = keyA % kv.P, rowB = keyB % kv.P;
  const bf16_t* ka = kv.pool + (size_t)pageA * page_elems + (size_t)kv.kvh * kv.P * HD + (size_t)rowA * HD;
  const bf16_t* kb = kv.pool + (size_t)pageB * page_elems + (size_t)kv.kvh * kv.P * HD + (size_t)rowB * HD;
  const bf16_t* va = kv.pool + (size_t)pageA * page_elems + (size_t)(kv.n_kv + kv.kvh) * kv.P * HD + rowA;
  const bf16_t* vb = kv.pool + (size_t)pageB * page_elems + (size_t)(kv.n_kv + kv.kvh) * kv.P * HD + rowB;
  const unsigned k_lane = (unsigned)(r16 * HD + quad * 8);          // elements
  const unsigned v_lane = (unsigned)(r16 * kv.P + quad * 4);
#pragma unroll
  for (int s = 0; s < HD / 32; ++s) {
    f.k[0][s].u = *reinterpret_cast<const uint4*>(ka + k_lane + s * 32);
    f.k[1][s].u = *reinterpret_cast<const uint4*>(kb + k_lane + s * 32);
  }
  const unsigned v_step = 16u * kv.P;                                // elements between blocks of 16 dims
#pragma unroll
  for (int d = 0; d < HD / 16; ++d) {
    const uint2 a = *reinterpret_cast<const uint2*>(va + v_lane + d * v_step);
    const uint2 b = *reinterpret_cast<const uint2*>(vb + v_lane + d * v_step);
    f.v[d].u = make_uint4(a.x, a.y, b.x, b.y);
  }
}

// What the walk knows of one block.
struct BlockInfo {
  int key0;     // first key
  bool valid;   // false: the block does not count (a stand-in loaded to keep the loads
                // unconditional, or a page that was given back)
  bool check;   // true: some key of it may be hidden from some column, or not written yet
};

// One pair of blocks for this wavefront's 16 columns.
//   qf       Q^T fragments: column lane % 16, dims 32 * step + 8 * (lane / 16) .. + 7
//   scale    softmax scale times log2(e): scores, maxima and partial maxima are in units of log 2,
//            so that the weights are bare exp2
//   lo, hi   the keys this lane's column may see: lo <= key <= hi
//   kv_last  last position of the request that has been written (rows after it hold rubbish)
template <int HD>
__device__ __forceinline__ void attend_pair(KVPair<HD>& f, const Frag8* qf, BlockInfo A, BlockInfo B, int lo,
                                            int hi, int kv_last, float scale, float& m, float& l, floatx4* o) {
  const int lane = threadIdx.x & 63;
  const int quad = lane >> 4;
  // S^T = K . Q^T, both blocks
  floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < HD / 32; ++s) {
    sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[0][s].v, qf[s].v, sa, 0, 0, 0);
    sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[1][s].v, qf[s].v, sb, 0, 0, 0);
  }
  // this lane: keys key0 + 4 quad + i of column lane % 16, in each block
  float sv[8];
  const bool plain = A.valid && B.valid && !A.check && !B.check;   // the same in every lane
  if (plain) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sv[i] = sa[i] * scale;
      sv[4 + i] = sb[i] * scale;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ka = A.key0 + quad * 4 + i, kb = B.key0 + quad * 4 + i;
      const bool see_a = A.valid & (!A.check | ((ka >= lo) & (ka <= hi)));   // bitwise: selects, no branches
      const bool see_b = B.valid & (!B.check | ((kb >= lo) & (kb <= hi)));
      sv[i] = see_a ? sa[i] * scale : -INFINITY;
      sv[4 + i] = see_b ? sb[i] * scale : -INFINITY;
      // rows never written may hold anything, NaN included, and 0 * NaN is NaN
      const bool zero_a = !A.valid | (ka > kv_last), zero_b = !B.valid | (kb > kv_last);
      const unsigned keep_a = zero_a ? ((i & 1) ? 0x0000FFFFu : 0xFFFF0000u) : 0xFFFFFFFFu;
      const unsigned keep_b = zero_b ? ((i & 1) ? 0x0000FFFFu : 0xFFFF0000u) : 0xFFFFFFFFu;
#pragma unroll
      for (int d = 0; d < HD / 16; ++d) {
        unsigned* wv = reinterpret_cast<unsigned*>(&f.v[d].u);
        wv[i >> 1] &= keep_a;             // element i of block A
        wv[2 + (i >> 1)] &= keep_b;       // element 4 + i: block B
      }
    }
  }
  float bm = sv[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) bm = fmaxf(bm, sv[i]);
  bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
  bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
  const float m_new = fmaxf(m, bm);
  const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
  Frag8 pf;
  float pv[8], ps = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    pv[i] = __builtin_amdgcn_exp2f(sv[i] - m_safe);      // scores are in units of log 2
    ps += pv[i];
  }
  pf.u = make_uint4(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]), pack_bf16x2(pv[4], pv[5]),
                    pack_bf16x2(pv[6], pv[7]));
  // the running maximum settles after a few blocks; then nothing needs rescaling
  if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
    const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
    l *= alpha;
#pragma unroll
    for (int d = 0; d < HD / 16; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[d][i] *= alpha;
    m = m_new;
  }
  l += ps;
#pragma unroll
  for (int d = 0; d < HD / 16; ++d)
    o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[d].v, pf.v, o[d], 0, 0, 0);
}

// Walk blocks first, first + stride, ... (n of them) of one request, two at a time.
// The page ids of 64 blocks are fetched at once, one per lane, so that the walk waits
// for the block table once per 1024 positions and not once per block; within such a
// run the loads of the next pair are in flight while a pair is computed (two fragment
// sets take turns; loads past the end repeat the last block and are not used).
// `check(block)` tells whether a block needs masks.
struct NoHook {
  __device__ __forceinline__ void operator()() const {}
};

// `after_table` runs once, right after the first load of page ids has been issued, and
// `before_attend` once, after the loads of the first pair have been issued and before the
// first pair is computed (both also when there is no block to walk; every wavefront of a
// workgroup runs each exactly once, so they may hold a barrier).  Loads come back in the
// order they were issued: what a caller asks for in `after_table` arrives before the keys
// and values, and what it computes in `before_attend` runs while those are in flight.
template <int HD, typename Check, typename AfterTable = NoHook, typename BeforeAttend = NoHook>
__device__ __forceinline__ void walk_blocks(const PagedKV& kv, const Frag8* qf, int first, int stride, int n,
                                            int lo, int hi, int kv_last, float scale, Check check, float& m,
                                            float& l, floatx4* o, AfterTable after_table = NoHook{},
                                            BeforeAttend before_attend = NoHook{}) {
  const int lane = threadIdx.x & 63;
  bool hooks_due = true;
  for (int c0 = 0; c0 < n; c0 += 64) {
    const int nc = min(64, n - c0);
    const int mine = (lane < nc) ? kv.table[((first + (c0 + lane) * stride) * 16) / kv.P] : -1;
    if (hooks_due) {
      __builtin_amdgcn_sched_barrier(0);
      after_table();
      __builtin_amdgcn_sched_barrier(0);
    }
    KVPair<HD> f0, f1;
    BlockInfo a0, b0, a1, b1;
    // block j of this run, clamped to the run's last block
    auto info = [&](int j, int& page) {
      const int jc = min(j, nc - 1);
      const int blk = first + (c0 + jc) * stride;
      page = __builtin_amdgcn_readlane(mine, jc);
      return BlockInfo{blk * 16, j < nc && page >= 0, check(blk)};
    };
    auto issue = [&](int j, KVPair<HD>& f, BlockInfo& A, BlockInfo& B) {
      int pa, pb;
      A = info(j, pa);
      B = info(j + 1, pb);
      load_pair<HD>(kv, max(pa, 0), A.key0, max(pb, 0), B.key0, f);
    };
    issue(0, f0, a0, b0);
    if (hooks_due) {
      __builtin_amdgcn_sched_barrier(0);
      before_attend();
      __builtin_amdgcn_sched_barrier(0);
      hooks_due = false;
    }
    for (int i = 0; i < nc; i += 4) {
      issue(i + 2, f1, a1, b1);
      attend_pair<HD>(f0, qf, a0, b0, lo, hi, kv_last, scale, m, l, o);
      issue(i + 4, f0, a0, b0);
      if (i + 2 < nc) attend_pair<HD>(f1, qf, a1, b1, lo, hi, kv_last, scale, m, l, o);
    }
  }
  if (hooks_due) {
    after_table();
    before_attend();
  }
}

// ------------------------------------------- queries and the new key prepared in place
// What the decode kernel needs to start from the 32-bit projections instead of prepared
// queries: it norms and rotates its own query heads, and the workgroup whose blocks hold the
// row's own position writes that position's key and value into the cache before it walks.
struct QKPrep {
  const float* qkv;          // [rows, row_width]: q heads, then (if keys are written) k heads, v heads
  int row_width;
  const float* q_w;          // per-head norm weights or nullptr
  const float* k_w;
  float eps;
  const float* inv_freq;     // nullptr: no rotation
  const float2* rope_table;  // (cos, sin) [table_len][hd / 2] or nullptr
  int table_len;
  bf16_t* pool_w;            // the cache to write the new key and value into; nullptr: nothing is written
};

template <int HD>
struct QueryLoads {
  static_assert(HD == 64 || HD == 128, "a lane holds whole rotation pairs for these head sizes only");
  static constexpr int NS = HD / 32, NP = NS / 2, HALF = HD / 2;
  float x[NS][8];
  float wl[NP][8], wh[NP][8];
  float2 cs[NP][8];
  bool from_table;

  // everything the preparation reads, asked for in one go (the table case and the computed case
  // of the angles are told apart once, not per element, so that the loads go out together)
  __device__ __forceinline__ void load(const QKPrep& pr, const float* __restrict__ src, int p) {
    const int lane = threadIdx.x & 63, quad = lane >> 4;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const float4 a = *reinterpret_cast<const float4*>(src + s * 32 + quad * 8);
      const float4 b = *reinterpret_cast<const float4*>(src + s * 32 + quad * 8 + 4);
      x[s][0] = a.x; x[s][1] = a.y; x[s][2] = a.z; x[s][3] = a.w;
      x[s][4] = b.x; x[s][5] = b.y; x[s][6] = b.z; x[s][7] = b.w;
    }
    from_table = pr.inv_freq && pr.rope_table && p < pr.table_len;   // the same in every lane
#pragma unroll
    for (int sp = 0; sp < NP; ++sp) {
      const int i0 = sp * 32 + quad * 8;
      if (pr.q_w) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float4 a = *reinterpret_cast<const float4*>(pr.q_w + i0 + 4 * h);
          const float4 b = *reinterpret_cast<const float4*>(pr.q_w + i0 + HALF + 4 * h);
          wl[sp][4 * h] = a.x; wl[sp][4 * h + 1] = a.y; wl[sp][4 * h + 2] = a.z; wl[sp][4 * h + 3] = a.w;
          wh[sp][4 * h] = b.x; wh[sp][4 * h + 1] = b.y; wh[sp][4 * h + 2] = b.z; wh[sp][4 * h + 3] = b.w;
        }
      }
      if (from_table) {
        const float4* t = reinterpret_cast<const float4*>(pr.rope_table + (size_t)p * HALF + i0);
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          const float4 v = t[h];
          cs[sp][2 * h] = make_float2(v.x, v.y);
          cs[sp][2 * h + 1] = make_float2(v.z, v.w);
        }
      }
    }
  }

  // Q^T fragments of this lane's column (one q head): the same arithmetic as qk_head_wave, in
  // the layout of the first product.  A lane holds the dims 32 s + 8 quad + j (s < HD / 32,
  // j < 8), which are both halves of its rotation pairs; the sum of squares goes up the same
  // tree as the butterfly of a wavefront with one pair per lane.
  __device__ __forceinline__ void finish(const QKPrep& pr, int p, bool valid, Frag8* qf) {
    const int lane = threadIdx.x & 63, quad = lane >> 4;
    float scale = 1.f;
    if (pr.q_w) {
      float u[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        u[j] = qk_pair_square(x[0][j], x[NP][j]);
        if (NP == 2) u[j] += qk_pair_square(x[1][j], x[1 + NP][j]);   // pairs i and i + 32
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) u[j] += __shfl_xor(u[j], 32, 64);   // pairs i and i ^ 16
#pragma unroll
      for (int j = 0; j < 8; ++j) u[j] += __shfl_xor(u[j], 16, 64);   // i ^ 8
#pragma unroll
      for (int j = 0; j < 4; ++j) u[j] += u[j + 4];                   // i ^ 4
      u[0] += u[2];                                                   // i ^ 2
      u[1] += u[3];
      scale = qk_norm_scale(u[0] + u[1], HD, pr.eps);                 // i ^ 1
    }
    if (pr.inv_freq && !from_table) {
#pragma unroll
      for (int sp = 0; sp < NP; ++sp)
#pragma unroll
        for (int j = 0; j < 8; ++j) cs[sp][j] = qk_cos_sin(sp * 32 + quad * 8 + j, HALF, p, pr.inv_freq, nullptr, 0);
    }
#pragma unroll
    for (int sp = 0; sp < NP; ++sp) {
      bf16_t* lo_h = reinterpret_cast<bf16_t*>(&qf[sp].u);
      bf16_t* hi_h = reinterpret_cast<bf16_t*>(&qf[sp + NP].u);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float lo = x[sp][j] * scale, hi = x[sp + NP][j] * scale;
        if (pr.q_w) {
          lo *= wl[sp][j];
          hi *= wh[sp][j];
        }
        if (pr.inv_freq) qk_rotate(lo, hi, cs[sp][j]);
        lo_h[j] = f2bf(valid ? lo : 0.f);
        hi_h[j] = f2bf(valid ? hi : 0.f);
      }
    }
  }
};

// =================================================================== decode
// grid (rows, n_kv * head_parts, splits), 256 threads.  Partials (splits > 1):
//   part_o [row][head][split][hd], part_ml [row][head][split][2] = (max, sum)
// PREP: the queries come from the 32-bit projections (see QKPrep); needs parts == 1.
// SHARED (with PREP): the four wavefronts need the same query; one prepares it, after the
// first keys and values have been asked for by all four, and hands it over through LDS.  The
// others' load units are then free for keys and values from the start, and the preparation
// runs while those are on their way.  It costs registers (one wavefront per SIMD): for launches
// of at most one workgroup per compute unit, where the start of the kernel is most of its time.
#define DEC_TABLE_LDS 1024     // entries of a block-table row that the decode kernel can hold in LDS
template <int HD, bool PREP, bool SHARED = false>
__global__ void __launch_bounds__(256)
attn_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool, const int* __restrict__ table,
                   int table_stride, const int* __restrict__ pos, const int* __restrict__ slot,
                   const int* __restrict__ rows, bf16_t* __restrict__ out, float* __restrict__ part_o,
                   float* __restrict__ part_ml, int n_head, int n_kv, int P, float scale, int window,
                   int n_splits, QKPrep prep) {
  __shared__ float s_o[4][HD / 16][4][64];
  __shared__ float s_m[4][16], s_l[4][16];
  __shared__ __attribute__((aligned(16))) bf16_t s_kv[PREP ? 2 * HD : 2];   // the row's own key, then its value
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

  // slot == nullptr: row m of the step is row m of the block tables (a step of single tokens, where the
  // host knows it), and a table row has at most DEC_TABLE_LDS entries.  The row's page ids are then asked
  // for at once, all of them, beside the position instead of behind it (which pages the workgroup walks
  // depends on the position), and looked up in LDS afterwards: one round trip to memory less before the
  // first keys can be asked for (0.15 us of the kernel's 19 at batch 8 of Qwen3-0.6B's sizes).
  __shared__ int s_table[DEC_TABLE_LDS];
  const bool early = slot == nullptr;
  int ids[DEC_TABLE_LDS / 256];
  if (early) {
    const int* table_row = table + (size_t)m_row * table_stride;
#pragma unroll
    for (int j = 0; j < DEC_TABLE_LDS / 256; ++j) {
      const int i = threadIdx.x + 256 * j;
      ids[j] = i < table_stride ? table_row[i] : -1;
    }
  }
  const int p_q = pos[m_row];
  const int lo = (window > 0 && p_q - window + 1 > 0) ? p_q - window + 1 : 0;
  const int blk_lo = lo / 16, blk_hi = p_q / 16;
  const int n_blk = blk_hi - blk_lo + 1;
  const int per = (n_blk + n_splits - 1) / n_splits;
  const int b0 = blk_lo + split * per;
  const int b1 = min(blk_hi + 1, b0 + per);
  if (early) {
#pragma unroll
    for (int j = 0; j < DEC_TABLE_LDS / 256; ++j) s_table[threadIdx.x + 256 * j] = ids[j];
    __syncthreads();
  }

  PagedKV kv{pool, early ? s_table : table + (size_t)slot[m_row] * table_stride, P, n_kv, kvh};
  Frag8 qf[HD / 32];
  float mx = -INFINITY, l = 0.f;
  floatx4 o[HD / 16];
#pragma unroll
  for (int d = 0; d < HD / 16; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int mine = (b1 - (b0 + wave) + 3) / 4;   // blocks b0 + wave, + 4, ... below b1
  auto edge = [=](int b) { return b == blk_lo || b == blk_hi; };
  bool own_key = false;   // PREP: this workgroup takes the row's own key and value from LDS, not from the cache
  if constexpr (PREP) {
    const float* row = prep.qkv + (size_t)m_row * prep.row_width;
    own_key = prep.pool_w && blk_hi >= b0 && blk_hi < b1;
    const int last = own_key ? p_q - 1 : p_q;      // what the cache holds for this workgroup
    const float* q_src = row + (size_t)(r16 < n_cols ? head : kvh * G) * HD;
    // this workgroup walks the block of the row's own position: the position's key and value
    // are computed here (by the code that prepares whole steps) into LDS; from there they go
    // into the cache for later steps, and into this step's attention as a block of their own,
    // so nothing waits for the cache to hold them.
    auto own_key_to_lds = [&]() {
      if (wave == (SHARED ? 1 : 0))
        qk_head_wave<bf16_t>(row + (size_t)(n_head + kvh) * HD, s_kv, 1, prep.k_w, prep.eps, prep.inv_freq,
                             prep.rope_table, prep.table_len, p_q, HD);
      if (wave == (SHARED ? 2 : 1)) v_head_wave<bf16_t>(row + (size_t)(n_head + n_kv + kvh) * HD, s_kv + HD, 1, HD);
    };
    auto own_key_to_cache = [&]() {          // after a barrier
      const int page = kv.table[p_q / P];
      if (page >= 0) {    // the host reserves pages first; never write astray
        bf16_t* kd = kv_page_slot<bf16_t>(prep.pool_w, page, 0, kvh, p_q % P, n_kv, P, HD);
        bf16_t* vd = kv_page_slot<bf16_t>(prep.pool_w, page, 1, kvh, p_q % P, n_kv, P, HD);
        for (int i = threadIdx.x; i < HD; i += 256) {
          kd[i] = s_kv[i];
          vd[(size_t)i * P] = s_kv[HD + i];
        }
      }
    };
    if constexpr (SHARED) {
      __shared__ uint4 s_q[HD / 32][64];
      QueryLoads<HD> ql;
      walk_blocks<HD>(
          kv, qf, b0 + wave, 4, mine, lo, last, last, scale * TI_LOG2E, edge, mx, l, o,
          [&]() {
            if (wave == 0) ql.load(prep, q_src, p_q);   // the same for every lane of the wavefront
          },
          [&]() {
            if (own_key) own_key_to_lds();
            if (wave == 0) {
              ql.finish(prep, p_q, r16 < n_cols, qf);
#pragma unroll
              for (int s = 0; s < HD / 32; ++s) s_q[s][lane] = qf[s].u;
            }
            __syncthreads();
            if (wave != 0) {
#pragma unroll
              for (int s = 0; s < HD / 32; ++s) qf[s].u = s_q[s][lane];
            }
            if (own_key) own_key_to_cache();
          });
    } else {
      if (own_key) own_key_to_lds();
      QueryLoads<HD> ql;
      ql.load(prep, q_src, p_q);
      ql.finish(prep, p_q, r16 < n_cols, qf);
      if (own_key) {
        __syncthreads();
        own_key_to_cache();
      }
      walk_blocks<HD>(kv, qf, b0 + wave, 4, mine, lo, last, last, scale * TI_LOG2E, edge, mx, l, o);
    }
  } else {
#pragma unroll
    for (int s = 0; s < HD / 32; ++s) {
      qf[s].u = make_uint4(0, 0, 0, 0);
      if (r16 < n_cols)
        qf[s].u = *reinterpret_cast<const uint4*>(q + ((size_t)m_row * n_head + head) * HD + s * 32 + quad * 8);
    }
    walk_blocks<HD>(kv, qf, b0 + wave, 4, mine, lo, p_q, p_q, scale * TI_LOG2E, edge, mx, l, o);
  }
  if (PREP && own_key && wave == 0) {
    // the row's own key and value: a block whose first key is the only one that counts
    KVPair<HD> f;
#pragma unroll
    for (int s = 0; s < HD / 32; ++s) {
      f.k[0][s].u = (r16 == 0) ? *reinterpret_cast<const uint4*>(s_kv + s * 32 + quad * 8) : make_uint4(0, 0, 0, 0);
      f.k[1][s].u = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int d = 0; d < HD / 16; ++d)
      f.v[d].u = make_uint4(quad == 0 ? (unsigned)s_kv[HD + d * 16 + r16] : 0u, 0, 0, 0);
    attend_pair<HD>(f, qf, BlockInfo{p_q, true, true}, BlockInfo{p_q, false, false}, p_q, p_q, p_q, scale * TI_LOG2E,
                    mx, l, o);
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
    wgt[w] = (s_m[w][r16] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s_m[w][r16] - mm);
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

// grid (rows, n_head), max(HD, 64) threads: out = sum_s w_s o_s / sum_s w_s l_s, w_s = 2^(m_s - max m).
// The partial outputs are fetched in batches of eight independent loads: the kernel waits for
// memory a few times, not once per split.
#define MERGE_MAX_SPLITS 64
template <int HD>
__global__ void __launch_bounds__(HD < 64 ? 64 : HD)
attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                  const int* __restrict__ rows, bf16_t* __restrict__ out, int n_head, int n_splits) {
  const int ridx = blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  if (d >= HD) return;
  const int m_row = rows ? rows[ridx] : ridx;
  const float2* pm = reinterpret_cast<const float2*>(part_ml) + ((size_t)ridx * n_head + head) * n_splits;
  const float* po = part_o + ((size_t)ridx * n_head + head) * n_splits * HD + d;
  // every thread works the weights of the splits out for itself: they are few, and no thread waits
  // for another.  Up to 16 splits: everything asked for at once, one round trip to memory (splits
  // beyond the last repeat it and count for nothing).
  auto at_once = [&](auto cap_tag) {
    constexpr int CAP = decltype(cap_tag)::value;
    float v[CAP];
    float2 ml[CAP];
#pragma unroll
    for (int j = 0; j < CAP; ++j) {
      const int sj = j < n_splits ? j : n_splits - 1;
      ml[j] = pm[sj];
      v[j] = po[(size_t)sj * HD];
    }
    float mm = -INFINITY;
#pragma unroll
    for (int j = 0; j < CAP; ++j)
      if (j < n_splits) mm = fmaxf(mm, ml[j].x);
    float acc = 0.f, lt = 0.f;
#pragma unroll
    for (int j = 0; j < CAP; ++j)
      if (j < n_splits) {
        const float w = split_weight(ml[j].x, mm);
        lt = fmaf(ml[j].y, w, lt);
        acc = split_accumulate(acc, v[j], w);
      }
    out[((size_t)m_row * n_head + head) * HD + d] = f2bf(acc * (1.0f / lt));
  };
  if (n_splits <= 8) {
    at_once(std::integral_constant<int, 8>{});
    return;
  }
  if (n_splits <= 16) {
    at_once(std::integral_constant<int, 16>{});
    return;
  }
  float mm = -INFINITY;
  for (int s = 0; s < n_splits; ++s) mm = fmaxf(mm, pm[s].x);
  float acc = 0.f, lt = 0.f;
  int s = 0;
  for (; s + 8 <= n_splits; s += 8) {
    float v[8];
    float2 ml[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v[j] = po[(size_t)(s + j) * HD];
      ml[j] = pm[s + j];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float w = split_weight(ml[j].x, mm);
      lt = fmaf(ml[j].y, w, lt);
      acc = split_accumulate(acc, v[j], w);
    }
  }
  for (; s < n_splits; ++s) {
    const float2 ml = pm[s];
    const float w = split_weight(ml.x, mm);
    lt = fmaf(ml.y, w, lt);
    acc = split_accumulate(acc, po[(size_t)s * HD], w);
  }
  out[((size_t)m_row * n_head + head) * HD + d] = f2bf(acc * (1.0f / lt));
}

// ================================================================== prefill
// grid (tiles, n_head), 512 threads.  tiles[t] = (entry, first row); entries[e] =
// (row0, n_tokens, start_pos, -).  A tile is 128 rows; wavefront w takes rows
// first + 16 w .. + 15 as its columns.
template <int HD>
__global__ void __launch_bounds__(512)
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
  walk_blocks<HD>(kv, qf, blk_lo, 1, blk_hi - blk_lo + 1, my_lo, hi_col, kv_last, scale * TI_LOG2E,
                  [=](int b) {
                    const int key0 = b * 16;
                    const bool inside = (key0 + 15 <= pos_first) && (w_rows == 16) &&
                                        (window <= 0 || key0 >= pos_last - window + 1) && (key0 >= tile_lo);
                    return !inside;
                  },
                  mx, l, o);
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

// ======================================================= prefill, through LDS
// The prefill kernel for head sizes 64 and 128.  A workgroup takes 128 consecutive
// tokens of one q head; a wavefront's tokens are column blocks of 32 of
// v_mfma_f32_32x32x16_bf16 (one block each for four wavefronts, or two each for two).  Keys and values come in turns of 32 keys by direct
// global-to-LDS loads, several turns deep, and are shared by the wavefronts.
//
//   S^T (32 keys x 32 tokens) = K (32 x hd) . Q^T          8 (hd=128) MFMAs per column block
//   O^T (hd x 32 tokens)     += V^T (hd x 32 keys) . P^T   hd/32 x 2 MFMAs per column block
//
// LDS rows of K are not in key order: row r of a 16-row group holds the key whose
// bits 2 and 3 are those of r swapped.  The score tile then leaves a lane with eight
// keys that are contiguous in memory (8h .. 8h+7 of each 16), so that the matching
// V^T fragment is one 16-byte read.  Pieces are XOR-swizzled against bank conflicts.
#define PF_ROWS 128
#define PF_KEYS 32
#define PF_STAGES 4      // LDS stages: PF_STAGES - 1 turns are in flight while one is computed

typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

__device__ __forceinline__ void lgkm_wait(int n) {
  switch (n) {
#define TI_LGKM(N) case N: asm volatile("s_waitcnt lgkmcnt(" #N ")" ::: "memory"); break;
    TI_LGKM(1) TI_LGKM(2) TI_LGKM(3) TI_LGKM(4) TI_LGKM(5) TI_LGKM(6) TI_LGKM(7) TI_LGKM(8)
    TI_LGKM(9) TI_LGKM(10) TI_LGKM(11) TI_LGKM(12) TI_LGKM(13) TI_LGKM(14) TI_LGKM(15)
#undef TI_LGKM
    default: asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); break;
  }
}
// wait until at most k * LOADS vector-memory operations are outstanding
// (s_waitcnt with only vmcnt set: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
template <int LOADS, int STAGES>
__device__ __forceinline__ void vm_wait_turns(int k) {
#define TI_VM(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | ((((N) >> 4) & 3) << 14))
  static_assert(LOADS * (STAGES - 2) <= 63, "vmcnt has six bits");
  switch (k) {
    case 0: TI_VM(0); break;
    case 1: TI_VM(LOADS); break;
    case 2: TI_VM(2 * LOADS); break;
    case 3: TI_VM(3 * LOADS); break;
    case 4: TI_VM(4 * LOADS); break;
    case 5: TI_VM(5 * LOADS); break;
    case 6: TI_VM(6 * LOADS); break;
    default: TI_VM(0); break;
  }
#undef TI_VM
}

// f(integral_constant<int, 0>), f(<1>), ... f(<N - 1>), until one returns false
template <typename F, int... Is>
__device__ __forceinline__ void unrolled_while_impl(F&& f, std::integer_sequence<int, Is...>) {
  (void)(f(std::integral_constant<int, Is>{}) && ...);
}
template <int N, typename F>
__device__ __forceinline__ void unrolled_while(F&& f) {
  unrolled_while_impl(f, std::make_integer_sequence<int, N>{});
}

// NG groups of NW wavefronts in the workgroup.  A tile is 32 NW rows: a column block of 32
// tokens per wavefront of a group, and every group takes all of the tile's rows.  With more
// than one group the turns (32 keys) go to the groups in rotation (each group loads and walks
// its own turns through its own ST LDS stages) and their partial results are merged through
// LDS at the end.  More groups put two wavefronts on every SIMD when a launch has only one
// workgroup per compute unit, so that one's loads, LDS reads and vector work hide behind the
// other's matrix products.
// CB: column blocks of 32 tokens per wavefront.  (Two, for groups of one wavefront that need no barrier
// and read every K fragment once for 64 tokens, do not fit the registers: the accumulators and the
// queries alone are 192, and the compiler moves them through the other register file all the time.)
// PAIRED: a workgroup takes two tiles, one after the other: tiles[blockIdx.x] and
// tiles[n_tiles - 1 - blockIdx.x] of a list ordered from the most keys to the fewest, so that
// under a causal mask every workgroup of a launch has about the same work.
template <int HD, int NG, int NW = 4, int ST = PF_STAGES, bool PAIRED = false, int CB = 1>
__global__ void __launch_bounds__(64 * NW * NG)
attn_prefill_lds_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool,
                        const int* __restrict__ table, int table_stride, const int* __restrict__ tiles,
                        int n_tiles, const int* __restrict__ entries, bf16_t* __restrict__ out, int n_head,
                        int n_kv, int P, float scale, int window, float* __restrict__ part_o = nullptr,
                        float* __restrict__ part_ml = nullptr) {
  // gridDim.z > 1: the keys a tile sees are cut into gridDim.z runs of whole turns, workgroup z takes
  // run z and leaves its maxima, sums and unscaled outputs in part_ml [row][head][z] = (m, l) and
  // part_o [row][head][z][HD] for the kernel that merges them
  const int n_splits = gridDim.z, split = blockIdx.z;
  constexpr int WROWS = 32 * CB;                      // tokens per wavefront
  constexpr int TROWS = NW * WROWS;                   // tokens per tile
  constexpr int NP = HD / 8;                          // 16-byte pieces per K row
  constexpr int K_BYTES = PF_KEYS * HD * 2;
  constexpr int STAGE = 2 * K_BYTES;                  // K tile + V^T tile
  constexpr int K_ROWS = 1024 / (HD * 2);             // K rows per wavefront load
  constexpr int K_LOADS = PF_KEYS / K_ROWS;
  constexpr int V_LOADS = HD / 16;                    // 16 dims (64 bytes each) per wavefront load
  static_assert(K_LOADS % NW == 0 && V_LOADS % NW == 0, "every wavefront takes the same kinds of loads");
  constexpr int MY_K = K_LOADS / NW, MY_LOADS = (K_LOADS + V_LOADS) / NW;   // per wavefront and turn
  constexpr int KS = HD / 16;                         // k-steps of the first product
  constexpr int DB = HD / 32;                         // 32-dim blocks of the output
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  // Which (tile, head) this workgroup takes.  Workgroups go to the eight XCDs in turn (linear id
  // mod 8) and each XCD has an L2 of its own: with a multiple of eight kv heads, an XCD is given
  // whole kv heads, so that the keys and values of a head are read into one L2 only.
  int head = blockIdx.y, bx = blockIdx.x;
  if (n_kv % 8 == 0) {
    const int id = blockIdx.y * gridDim.x + blockIdx.x;
    const int xcd = id & 7, local = id >> 3;
    const int per_kv = (n_head / n_kv) * gridDim.x;       // workgroups of one kv head
    const int rest = local % per_kv;
    head = (xcd + 8 * (local / per_kv)) * (n_head / n_kv) + rest / gridDim.x;
    bx = rest % gridDim.x;
  }
  // the wavefront's number in scalar registers: what follows from it (which turns it loads, where they
  // go, which rows are its own) is then worked out once per wavefront, not once per lane
  const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = wid / NW, wave = wid % NW, lane = threadIdx.x & 63;
  const int r32 = lane & 31, h = lane >> 5;
  const int kvh = head / (n_head / n_kv);
  const size_t page_elems = (size_t)2 * n_kv * P * HD;
  const bf16_t* kpool = pool + (size_t)kvh * P * HD;
  const bf16_t* vpool = pool + (size_t)(n_kv + kvh) * P * HD;

  // scores are kept in units of log 2: softmax weights are then bare exp2
  const float scale2 = scale * 1.4426950408889634f;

  // what this lane fetches in each of its loads of a turn
  //  K load g: LDS rows K_ROWS g .. + K_ROWS - 1; lane i -> row r = K_ROWS g + i / NP, slot c = i % NP,
  //            holds piece c ^ (r & (NP - 1)) of key 16 (r / 16) + swap23(r % 16)
  //  V load g: dims 16 g .. 16 g + 15, 64 bytes each; lane i -> dim d = 16 g + i / 4, slot c = i % 4,
  //            holds piece c ^ ((d >> 2) & 3): keys 16 (piece / 2) + 8 (piece % 2) .. + 7
  // In bytes from a block's first K row, K load g takes for lane i (lr = i / NP < K_ROWS, c = i % NP)
  //   (k_lane ^ X(g)) + C(g),  k_lane = swap23(lr) * HD * 2 + (c ^ lr) * 16,
  //   X(g) = ((K_ROWS g) & (NP - 1)) * 16,  C(g) = swap23((K_ROWS g) & 15) * HD * 2
  // (the row number K_ROWS g + lr has g's bits and the lane's bits apart, and so have its pieces), from the
  // first block of the turn if (K_ROWS g) & 16 is clear, else from the second; and V load g takes, from
  // the V^T row of a block's first key, v_lane + 32 g P, v_lane = ((i / 4) P + 8 (piece & 1)) * 2, from the
  // second block in the lanes whose piece is 2 or 3.  One register a kind instead of one a load.
  static_assert(K_ROWS <= 16 && (K_ROWS & (K_ROWS - 1)) == 0, "rows of a K load lie in one block of 16");
  auto swap23 = [](int r16) __attribute__((always_inline)) { return ((r16 & 4) << 1) | ((r16 & 8) >> 1) | (r16 & 3); };
  const unsigned k_lane = (unsigned)(swap23(lane / NP) * HD * 2 + (((lane % NP) ^ (lane / NP)) << 4));
  const int v_piece = (lane & 3) ^ ((lane >> 4) & 3);
  const unsigned v_lane = (unsigned)((((lane >> 2) * P) + (v_piece & 1) * 8) * 2);
  const bool v_second = (v_piece >> 1) != 0;

  const unsigned lds0 = (unsigned)(size_t)smem + grp * (ST * STAGE);   // this group's stages
  // the wavefronts of a group wait for each other at the workgroup's barrier (a handshake of a group's
  // two wavefronts through a word of LDS, which lets the groups drift apart, was slower: 4.72 ms against
  // 4.59 ms for a prompt of 2,048 tokens at Qwen3-0.6B's sizes)
  auto group_sync = [&]() __attribute__((always_inline)) {
    if constexpr (NW > 1) __builtin_amdgcn_s_barrier();
  };
  // LDS addresses of this lane's fragments; the stage, and the dim block of a V^T fragment, are
  // constants in the read instructions
  unsigned k_addr[KS], v_addr[2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_addr[ks] = lds0 + r32 * (HD * 2) + (((ks * 2 + h) ^ (r32 & (NP - 1))) << 4);
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) v_addr[tt] = lds0 + K_BYTES + r32 * 64 + (((tt * 2 + h) ^ ((r32 >> 2) & 3)) << 4);

  for (int slot = 0; slot < (PAIRED ? 2 : 1); ++slot) {
  // ---- this slot's tile
  const int tile = (slot == 0) ? bx : n_tiles - 1 - bx;
  if (PAIRED && slot == 1 && tile <= bx) break;                     // an odd count: the middle tile came first
  const int entry = tiles[2 * tile], first = tiles[2 * tile + 1];
  const int row0 = entries[4 * entry], n_tok = entries[4 * entry + 1], start = entries[4 * entry + 2];
  const int row_end = row0 + n_tok;
  const int kv_last = start + n_tok - 1;
  const int* tab = table + (size_t)entry * table_stride;

  // this wavefront: rows w_first .. w_first + WROWS - 1, in column blocks of 32
  const int w_first = first + wave * WROWS;
  const int w_rows = max(0, min(WROWS, row_end - w_first));
  const int w_pos_first = start + (w_first - row0), w_pos_last = w_pos_first + w_rows - 1;
  const int w_lo = (window > 0 && w_pos_first - window + 1 > 0) ? w_pos_first - window + 1 : 0;
  // the workgroup: rows first .. first + TROWS - 1
  const int g_rows = min(TROWS, row_end - first);
  const int g_pos_first = start + (first - row0), g_pos_last = g_pos_first + g_rows - 1;
  const int g_lo = (window > 0 && g_pos_first - window + 1 > 0) ? g_pos_first - window + 1 : 0;

  int blk_lo = (g_lo / PF_KEYS) * 2, blk_hi = g_pos_last / 16;         // 16-key blocks, starting on a turn
  const int v_limit = min(kv_last, blk_hi * 16 + 15);               // last key whose value row is real
  if (n_splits > 1) {
    const int per = (((blk_hi + 1 - blk_lo) + n_splits - 1) / n_splits + 1) & ~1;   // whole turns
    blk_lo += split * per;
    blk_hi = min(blk_hi, blk_lo + per - 1);                         // a run past the end is empty
  }

  // A run is up to 64 blocks.  Lane i keeps where block c0 + i starts in the pool (in elements: the V^T
  // row of its first key; its first K row lies prow * (HD - 1) further) and the row of its first key in
  // its page, so that the walk waits for the block table once per run and divides by the page size once
  // per run.  Blocks past the end stand on page 0, and so do blocks whose page was given back (all their
  // keys are masked).
  long base = 0;
  int prow = 0;
  auto run_blocks = [&](int c0, int nblk) __attribute__((always_inline)) {
    const int key = (c0 + lane) * 16, pidx = key / P;
    prow = key - pidx * P;
    int page = (lane < nblk) ? tab[pidx] : 0;
    if (page < 0) page = 0;
    base = (long)page * (long)page_elems + prow;
  };
  // The loads of this group's turn i of the run into a stage (stage_off: its offset, a constant where
  // the loop is unrolled).  Which blocks, which pages and where in LDS is the same in every lane and
  // worked out in scalar registers; a lane adds the offset of its piece.  (Asking for a turn in portions
  // between the steps of the turn before, so that the unit that takes the addresses (64 bytes a cycle
  // for the whole compute unit) works beside the matrix cores, gained nothing.)
  auto issue = [&](int i, unsigned stage_off) __attribute__((always_inline)) {
    const int t = i * NG + grp;
    const int ja = min(2 * t, 63), jb = min(2 * t + 1, 63);
    const unsigned lo_a = __builtin_amdgcn_readlane((int)(unsigned)base, ja), hi_a = __builtin_amdgcn_readlane((int)(base >> 32), ja);
    const unsigned lo_b = __builtin_amdgcn_readlane((int)(unsigned)base, jb), hi_b = __builtin_amdgcn_readlane((int)(base >> 32), jb);
    const long v_a = (long)(((unsigned long)hi_a << 32) | lo_a), v_b = (long)(((unsigned long)hi_b << 32) | lo_b);
    const long k_a = v_a + (long)__builtin_amdgcn_readlane(prow, ja) * (HD - 1);
    const long k_b = v_b + (long)__builtin_amdgcn_readlane(prow, jb) * (HD - 1);
#pragma unroll
    for (int j = 0; j < MY_LOADS; ++j) {
      const char* src;
      unsigned dst;
      if (j < MY_K) {
        const int g = wave + NW * j;                              // the same in every lane
        const int rows = K_ROWS * g;
        const char* from = reinterpret_cast<const char*>(kpool + ((rows & 16) ? k_b : k_a)) +
                           swap23(rows & 15) * HD * 2;
        src = from + (k_lane ^ (unsigned)((rows & (NP - 1)) << 4));
        dst = g * 1024;
      } else {
        const int gv = wave + NW * (j - MY_K);
        const char* from = reinterpret_cast<const char*>(vpool + (v_second ? v_b : v_a));
        src = from + v_lane + (size_t)gv * 32 * P;
        dst = K_BYTES + gv * 1024;
      }
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(size_t)(lds0 + stage_off + dst), 16, 0, 0);
    }
  };
  constexpr int AHEAD = ST - 1;
  // the first run's blocks and first turns are asked for before the queries: those arrive meanwhile
  // (a workgroup whose run of keys is empty walks nothing, and nothing may be on its way into LDS
  // when it goes on to the merge)
  if (blk_lo <= blk_hi) {
    const int nblk = min(64, blk_hi + 1 - blk_lo);
    run_blocks(blk_lo, nblk);
    const int my_turns = ((nblk + 1) / 2 - grp + NG - 1) / NG;
#pragma unroll
    for (int i = 0; i < AHEAD; ++i)
      if (i < my_turns) issue(i, i * STAGE);
  }

  v4u qf[CB][KS];
  int my_pos[CB];
  bool col_ok[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    const int row = w_first + cb * 32 + r32;
    col_ok[cb] = row < row_end;
    my_pos[cb] = start + (row - row0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[cb][ks] = v4u{0, 0, 0, 0};
      if (col_ok[cb]) {
        const uint4 t = *reinterpret_cast<const uint4*>(q + ((size_t)row * n_head + head) * HD + ks * 16 + h * 8);
        qf[cb][ks] = v4u{t.x, t.y, t.z, t.w};
      }
    }
  }
  float mx[CB], l[CB];
  floatx16 o[CB][DB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    mx[cb] = -INFINITY;
    l[cb] = 0.f;
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[cb][d][i] = 0.f;
  }

  // One turn of 32 keys from a stage for this wavefront's columns, in two steps: the scores, then the
  // softmax and the second product.  plain (the same in every lane): every key of the turn is visible
  // to every column and written: no compare at all.
  auto turn_scores = [&](auto stage_tag, floatx16* sc) __attribute__((always_inline)) {
    constexpr unsigned SOFF = decltype(stage_tag)::value * STAGE;
    // ---- the fragments: keys now, values right behind them
    v4u kf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[ks]) : "v"(k_addr[ks]), "n"(SOFF));
    // ---- S^T = K . Q^T
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) sc[cb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (cb == 0) {
          lgkm_wait(KS - 1 - ks);        // the first ks + 1 of the KS reads have arrived
          asm volatile("" : "+v"(kf[ks]));
        }
        sc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[ks]),
                                                         __builtin_bit_cast(bf16x8, qf[cb][ks]), sc[cb], 0, 0, 0);
      }
    }
  };
  auto turn_rest = [&](auto stage_tag, int key0, bool plain, const floatx16* sc) __attribute__((always_inline)) {
    constexpr unsigned SOFF = decltype(stage_tag)::value * STAGE;
    // the value fragments are asked for now and waited for after the softmax
    v4u vf[DB][2];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(vf[d][tt]) : "v"(v_addr[tt]), "n"(SOFF + d * 32 * 64));

    // ---- masks, the online softmax and O^T += V^T . P^T, column block by column block: the matrix
    // core works on one block's second product while the next block's softmax runs.  The scores stay
    // as the first product left them: the maximum is taken over them and scaled once (the scale is
    // positive), and the scale goes into the multiply-add of the exponent.
    // element i of a lane: key key0 + 16 (i / 8) + 8 h + 4 ((i / 4) % 2) + i % 4
    // (the keys' numbers are worked out behind the branches that need them, not before the loop and kept
    // in registers: the compiler takes `hm` for something the branch has made)
    int hm = h;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      float sv[16];
      if (plain) {
#pragma unroll
        for (int i = 0; i < 16; ++i) sv[i] = sc[cb][i];
      } else {
        asm volatile("" : "+v"(hm));
        const int hi = col_ok[cb] ? my_pos[cb] : -1;
        const int lo = (window > 0) ? my_pos[cb] - window + 1 : 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = key0 + 16 * (i >> 3) + 8 * hm + 4 * ((i >> 2) & 1) + (i & 3);
          const bool see = (key <= hi) & (key >= lo);      // bitwise on purpose: selects, no branches
          sv[i] = see ? sc[cb][i] : -INFINITY;
        }
      }
      float bm = sv[0];
#pragma unroll
      for (int i = 1; i < 16; ++i) bm = fmaxf(bm, sv[i]);
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(mx[cb], bm * scale2);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      float ps = 0.f;
      float pv[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        pv[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], scale2, -m_safe));
        ps += pv[i];
      }
      v4u pf[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
        pf[tt] = v4u{pack_bf16x2(pv[8 * tt], pv[8 * tt + 1]), pack_bf16x2(pv[8 * tt + 2], pv[8 * tt + 3]),
                     pack_bf16x2(pv[8 * tt + 4], pv[8 * tt + 5]), pack_bf16x2(pv[8 * tt + 6], pv[8 * tt + 7])};
      // the running maximum settles after a few turns; then nothing needs rescaling
      if (__builtin_amdgcn_ballot_w64(m_new != mx[cb]) != 0) {
        const float alpha = __builtin_amdgcn_exp2f(mx[cb] - m_safe);
        l[cb] *= alpha;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[cb][d][i] *= alpha;
        mx[cb] = m_new;
      }
      l[cb] += ps;

      if (cb == 0) {
        // the value fragments have had the first block's softmax to arrive
        lgkm_wait(0);
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int tt = 0; tt < 2; ++tt) asm volatile("" : "+v"(vf[d][tt]));
        if (!plain) {
          if (key0 + PF_KEYS - 1 > v_limit || key0 < g_lo) {
            // rows never written, and the stand-in page read for a block that was given back or
            // lies past the end, may hold anything, NaN included, and 0 * NaN is NaN
            asm volatile("" : "+v"(hm));
#pragma unroll
            for (int d = 0; d < DB; ++d)
#pragma unroll
              for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                  const int key = key0 + 16 * tt + 8 * hm + e;
                  const bool drop = (key > v_limit) | (key < g_lo);
                  const unsigned keep = drop ? ((e & 1) ? 0x0000FFFFu : 0xFFFF0000u) : 0xFFFFFFFFu;
                  vf[d][tt][e >> 1] &= keep;
                }
          }
        }
      }
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
          o[cb][d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[d][tt]),
                                                             __builtin_bit_cast(bf16x8, pf[tt]), o[cb][d], 0, 0, 0);
    }
  };

  for (int c0 = blk_lo; c0 <= blk_hi; c0 += 64) {
    const int nblk = min(64, blk_hi + 1 - c0);
    const int n_turns = (nblk + 1) / 2;
    // this group's turns are turns grp, grp + NG, ... of the run; i counts them, and turn i of a run
    // goes through stage i % ST
    const int my_turns = (n_turns - grp + NG - 1) / NG;
    const int n_iter = (n_turns + NG - 1) / NG;                      // the first group's count: the most
    if (c0 != blk_lo) {
      run_blocks(c0, nblk);
#pragma unroll
      for (int i = 0; i < AHEAD; ++i)
        if (i < my_turns) issue(i, i * STAGE);
    }
    for (int i0 = 0; i0 < n_iter; i0 += ST) {
      // ST turns, each with its stage as a constant; ends with the run
      unrolled_while<ST>([&](auto si_tag) __attribute__((always_inline)) {
        constexpr int si = decltype(si_tag)::value;
        const int i = i0 + si;
        if (i >= n_iter) return false;
        // this wavefront's part of the group's turn i has landed: only its turns issued after it (at
        // most AHEAD - 1) may be outstanding.  Then the group's wavefronts wait for each other: the
        // whole turn has landed, and everyone is done with the turn before, whose stage turn
        // i + AHEAD goes into.
        vm_wait_turns<MY_LOADS, ST>(max(0, min(AHEAD - 1, my_turns - 1 - i)));
        group_sync();
        // turn i + AHEAD goes into the stage that turn i - 1 has left
        if (i + AHEAD < my_turns) issue(i + AHEAD, ((si + AHEAD) % ST) * STAGE);
        if (i >= my_turns) return true;
        const int key0 = (c0 + 2 * (i * NG + grp)) * 16;
        // nothing of this turn is visible to this wavefront: it only helps loading
        if (w_rows == 0 || key0 > w_pos_last || key0 + PF_KEYS - 1 < w_lo) return true;
        const bool plain = (key0 + PF_KEYS - 1 <= w_pos_first) && (w_rows == WROWS) &&
                           (window <= 0 || key0 >= w_pos_last - window + 1);
        floatx16 sc[CB];
        turn_scores(si_tag, sc);
        turn_rest(si_tag, key0, plain, sc);
        return true;
      });
    }
    // every wavefront of the group is done with this run's stages before the next run (or the merge)
    // writes into them
    group_sync();
  }

  // ---- the result: o[cb][d][i] is dim 32 d + 8 (i / 4) + 4 h + i % 4 of token (column) r32 of block cb.
  // `first_val`, `count_tag`: which of a lane's DB * 16 values of a block (value v = 16 d + i) these are; a
  // lane's values come in fours of consecutive dims.
  auto write_out = [&](int cb, const float* val, int first_val, auto count_tag, float m_all, float lt) __attribute__((always_inline)) {
    constexpr int n_val = decltype(count_tag)::value;
    if (!col_ok[cb]) return;
    const int row = w_first + cb * 32 + r32;
    if (n_splits > 1) {
      const size_t at = ((size_t)row * n_head + head) * n_splits + split;
      float* po = part_o + at * HD;
#pragma unroll
      for (int j = 0; j < n_val; j += 4) {
        const int v = first_val + j;
        *reinterpret_cast<float4*>(po + 32 * (v >> 4) + 8 * ((v & 15) >> 2) + 4 * h) =
            make_float4(val[j], val[j + 1], val[j + 2], val[j + 3]);
      }
      if (h == 0 && first_val == 0) reinterpret_cast<float2*>(part_ml)[at] = make_float2(m_all, lt);
      return;
    }
    const float inv = 1.0f / lt;
    bf16_t* dst = out + ((size_t)row * n_head + head) * HD;
#pragma unroll
    for (int j = 0; j < n_val; j += 4) {
      const int v = first_val + j;
      *reinterpret_cast<uint2*>(dst + 32 * (v >> 4) + 8 * ((v & 15) >> 2) + 4 * h) =
          make_uint2(pack_bf16x2(val[j] * inv, val[j + 1] * inv), pack_bf16x2(val[j + 2] * inv, val[j + 3] * inv));
    }
  };
  if constexpr (NG == 1) {
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      float val[DB * 16];
#pragma unroll
      for (int v = 0; v < DB * 16; ++v) val[v] = o[cb][v >> 4][v & 15];
      write_out(cb, val, 0, std::integral_constant<int, DB * 16>{}, mx[cb], l[cb] + __shfl_xor(l[cb], 32, 64));
    }
  } else {
    // The groups merge their partial results through LDS (the stages are free now), each group the
    // values it owns: values VPG g .. VPG (g + 1) - 1 of every lane are group g's.  A group leaves the
    // values it does not own (in their order), its maximum and its sum in its part of LDS; after a
    // barrier it reads the others' contributions to its own values, merges them with its own and
    // writes them out.  Which registers a group takes its values from is a choice between registers by
    // the group's number, which every lane of a wavefront shares: the accumulators stay in registers.
    constexpr int VALS = DB * 16, VPG = VALS / NG, ML = VALS - VPG, SLOTS = ML + 2;
    static_assert(VALS % NG == 0 && VPG % 4 == 0, "a group owns whole fours of values");
    static_assert(NG * NW * SLOTS * 64 * 4 <= NG * ST * STAGE, "the partial results fit into the stages");
    typedef __attribute__((address_space(3))) float lds_float;
    auto part_of = [&](int g) __attribute__((always_inline)) {
      return (lds_float*)(size_t)((unsigned)(size_t)smem + (unsigned)(((g * NW + wave) * SLOTS * 64 + lane) * 4));
    };
    // only the workgroup's barrier tells that every group is done with its stages
    if constexpr (NW == 1) __syncthreads();
    const int first = grp * VPG;                     // this group's first value
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      if (cb > 0) __syncthreads();                   // the block before has been read
      lds_float* mine = part_of(grp);
#pragma unroll
      for (int sl = 0; sl < ML; ++sl)                // slot sl: value sl below this group's own, sl + VPG above them
        mine[sl * 64] = (sl < first) ? o[cb][sl >> 4][sl & 15] : o[cb][(sl + VPG) >> 4][(sl + VPG) & 15];
      mine[ML * 64] = mx[cb];
      mine[(ML + 1) * 64] = l[cb];
      __syncthreads();
      float m_g[NG], l_g[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        m_g[g] = part_of(g)[ML * 64];
        l_g[g] = part_of(g)[(ML + 1) * 64];
      }
      float m_all = m_g[0];
#pragma unroll
      for (int g = 1; g < NG; ++g) m_all = fmaxf(m_all, m_g[g]);
      const float m_safe = (m_all == -INFINITY) ? 0.f : m_all;
      float a_g[NG], l_all = 0.f;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        a_g[g] = __builtin_amdgcn_exp2f(m_g[g] - m_safe);
        l_all += l_g[g] * a_g[g];
      }
      const float a_own = __builtin_amdgcn_exp2f(mx[cb] - m_safe);
      float val[VPG];
#pragma unroll
      for (int j = 0; j < VPG; ++j) {
        float own = o[cb][j >> 4][j & 15];
#pragma unroll
        for (int g = 1; g < NG; ++g)
          if (grp == g) own = o[cb][(g * VPG + j) >> 4][(g * VPG + j) & 15];
        val[j] = own * a_own;
      }
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        if (g == grp) continue;                      // the same in every lane
        const lds_float* theirs = part_of(g) + (first + (grp > g ? -VPG : 0)) * 64;
#pragma unroll
        for (int j = 0; j < VPG; ++j) val[j] += theirs[j * 64] * a_g[g];
      }
      write_out(cb, val, first, std::integral_constant<int, VPG>{}, m_all, l_all + __shfl_xor(l_all, 32, 64));
    }
  }
  // the next tile's loads go into the LDS that the merge has just read
  if (PAIRED && NG > 1) __syncthreads();
  }   // slot
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

// compute units of the current device (asked once)
static int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      n = v;
    else
      n = 256;
  }
  return n;
}
// 1 (default): small decode launches from the projections let one wavefront prepare the query
static int g_decode_shared_query = 1;

// Decode rows.  rows: which rows of the step (nullptr: rows 0..n_rows-1).  n_splits > 1 needs
// part_o (float [n_rows, n_head, n_splits, hd]) and part_ml (float [n_rows, n_head, n_splits, 2]).
// Returns 3 for sizes these kernels do not serve.
template <bool PREP>
static int launch_decode(const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                         const int* slot, const int* rows, void* out, float* part_o, float* part_ml, int n_rows,
                         int n_head, int n_kv, int hd, int page_size, float scale, int window, int n_splits,
                         QKPrep prep, hipStream_t stream) {
  TI_REQUIRE(n_splits >= 1 && n_splits <= MERGE_MAX_SPLITS, "attention_decode: bad split count %d (1..%d)", n_splits, MERGE_MAX_SPLITS);
  TI_REQUIRE(n_splits == 1 || (part_o && part_ml), "attention_decode: splits need partial buffers");
  TI_REQUIRE(slot || table_stride <= DEC_TABLE_LDS, "attention_decode: without slots a table row has at most %d entries, not %d",
             DEC_TABLE_LDS, table_stride);
  if (n_rows == 0) return 0;
  const int parts = (n_head / n_kv + 15) / 16;
  TI_REQUIRE(n_kv * parts <= 65535, "attention_decode: too many heads");
  dim3 grid(n_rows, n_kv * parts, n_splits);
  // at most one workgroup per compute unit: one wavefront prepares the query for all four
  const bool shared = PREP && g_decode_shared_query && (long)n_rows * n_kv * parts * n_splits <= compute_units();
#define TI_DEC(H)                                                                                          \
  case H:                                                                                                  \
    if (shared)                                                                                            \
      attn_decode_kernel<H, PREP, PREP><<<grid, 256, 0, stream>>>(                                         \
          (const bf16_t*)q, (const bf16_t*)pool, table, table_stride, pos, slot, rows, (bf16_t*)out,        \
          part_o, part_ml, n_head, n_kv, page_size, scale, window, n_splits, prep);                         \
    else                                                                                                   \
      attn_decode_kernel<H, PREP><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table,   \
                                                            table_stride, pos, slot, rows, (bf16_t*)out,    \
                                                            part_o, part_ml, n_head, n_kv, page_size,       \
                                                            scale, window, n_splits, prep);                 \
    if (n_splits > 1)                                                                                       \
      attn_merge_kernel<H><<<dim3(n_rows, n_head), (H < 64 ? 64 : H), 0, stream>>>(part_o, part_ml, rows,   \
                                                                                  (bf16_t*)out, n_head,    \
                                                                                  n_splits);               \
    break;
  switch (hd) {
    TI_DEC(64) TI_DEC(128)
    case 32:
      if constexpr (!PREP) {
        attn_decode_kernel<32, false><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table,
                                                                table_stride, pos, slot, rows, (bf16_t*)out,
                                                                part_o, part_ml, n_head, n_kv, page_size, scale,
                                                                window, n_splits, prep);
        if (n_splits > 1)
          attn_merge_kernel<32><<<dim3(n_rows, n_head), 64, 0, stream>>>(part_o, part_ml, rows, (bf16_t*)out,
                                                                         n_head, n_splits);
      }
      break;
  }
#undef TI_DEC
  TI_LAUNCH_CHECK();
  return 0;
}

extern "C" int ti_attention_decode_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                        const int* pos, const int* slot, const int* rows, void* out,
                                        float* part_o, float* part_ml, int n_rows, int n_head, int n_kv, int hd,
                                        int page_size, float scale, int window, int n_splits,
                                        hipStream_t stream) {
  int rc = check_common("attention_decode", n_head, n_kv, hd, page_size, table_stride);
  if (rc) return rc;
  return launch_decode<false>(q, pool, table, table_stride, pos, slot, rows, out, part_o, part_ml, n_rows, n_head,
                              n_kv, hd, page_size, scale, window, n_splits, QKPrep{}, stream);
}

// The same for rows 0..n_rows-1 of a step, starting from the 32-bit projections: qkv is float
// [n_rows, row_width] with the q heads first and, if write_kv, the k heads and v heads after
// them.  Per-head norm (q_w, k_w: float [hd] or nullptr), rotation (inv_freq float [hd/2] or
// nullptr; rope_table float [table_len, hd/2, 2] or nullptr) and the write of each row's key
// and value at its own position happen inside the attention kernel.  Returns 3 for what it
// does not serve: head sizes other than 64 and 128, more than 16 q heads per kv head.
extern "C" int ti_attention_decode_prepared_bf16(const float* qkv, int row_width, const float* q_w,
                                                 const float* k_w, float eps, const float* inv_freq,
                                                 const float* rope_table, int table_len, void* pool, int write_kv,
                                                 const int* table, int table_stride, const int* pos,
                                                 const int* slot, void* out, float* part_o, float* part_ml,
                                                 int n_rows, int n_head, int n_kv, int hd, int page_size,
                                                 float scale, int window, int n_splits, hipStream_t stream) {
  int rc = check_common("attention_decode_prepared", n_head, n_kv, hd, page_size, table_stride);
  if (rc) return rc;
  if (hd == 32 || n_head / n_kv > 16 || ((uintptr_t)q_w & 15) || ((uintptr_t)rope_table & 15)) {
    ti_set_error("attention_decode_prepared: head_dim %d with %d q heads per kv head is not served (or a norm "
                 "weight or the sin/cos table is not 16-byte aligned)", hd, n_head / n_kv);
    return 3;
  }
  TI_REQUIRE(qkv && row_width >= (n_head + (write_kv ? 2 * n_kv : 0)) * hd && row_width % 4 == 0 &&
                 ((uintptr_t)qkv & 15) == 0,
             "attention_decode_prepared: the projections do not fit (row_width %d)", row_width);
  TI_REQUIRE(inv_freq || !rope_table, "attention_decode_prepared: a sin/cos table without inv_freq");
  QKPrep prep{qkv, row_width, q_w, k_w, eps, inv_freq, (const float2*)rope_table, table_len,
              write_kv ? (bf16_t*)pool : nullptr};
  return launch_decode<true>(nullptr, pool, table, table_stride, pos, slot, nullptr, out, part_o, part_ml, n_rows,
                             n_head, n_kv, hd, page_size, scale, window, n_splits, prep, stream);
}

static int g_prefill_groups = 0;   // for measurements: 1 or 2 wavefront groups per workgroup, 0 = by the launch
static int g_prefill_lds = 1;
// 1: head sizes 64 and 128 take the kernel that shares keys and values through LDS
// (default); 0: every head size takes the kernel that reads them per wavefront

// Portions of prompts.  tiles: int [n_tiles, 2] = (entry, first row), each tile 128 rows;
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
  if (g_prefill_lds && (hd == 64 || hd == 128)) {
    // two groups of wavefronts per workgroup when the launch would else leave a SIMD with one wavefront
    const int groups = g_prefill_groups ? g_prefill_groups : ((long)n_tiles * n_head < 512 ? 2 : 1);
    const int lds = groups * PF_STAGES * 2 * PF_KEYS * hd * 2;
    static bool ready = false;          // allow more than 64 KiB of dynamic LDS, once
    if (!ready) {
      const int most = 2 * PF_STAGES * 2 * PF_KEYS * 128 * 2;
      if (hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<128, 1>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, most / 2) != hipSuccess ||
          hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<128, 2>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess ||
          hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<64, 1>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, most / 4) != hipSuccess ||
          hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<64, 2>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, most / 2) != hipSuccess) {
        ti_set_error("attention_prefill: cannot reserve %d bytes of LDS", most);
        return 2;
      }
      ready = true;
    }
#define TI_PLDS(H, G)                                                                                          \
  attn_prefill_lds_kernel<H, G><<<grid, 256 * G, lds, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table,   \
                                                                table_stride, tiles, n_tiles, entries,          \
                                                                (bf16_t*)out, n_head, n_kv, page_size, scale,   \
                                                                window)
    if (hd == 128 && groups == 2) TI_PLDS(128, 2);
    else if (hd == 128) TI_PLDS(128, 1);
    else if (groups == 2) TI_PLDS(64, 2);
    else TI_PLDS(64, 1);
#undef TI_PLDS
    TI_LAUNCH_CHECK();
    return 0;
  }
#define TI_PRE(H)                                                                                          \
  case H:                                                                                                  \
    attn_prefill_kernel<H><<<grid, 512, 0, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table,          \
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

// The same for launches of few tiles, with the work evened out under a causal mask.  tiles: int
// [n_tiles, 2] = (entry, first row) of tiles of 64 rows, ordered from the tile that sees the most
// keys to the one that sees the fewest; a workgroup takes tile b and tile n_tiles - 1 - b, one
// after the other, with four groups of two wavefronts taking the turns of keys in rotation.
// Returns 3 for head sizes other than 64 and 128.
extern "C" int ti_attention_prefill_paired_bf16(const void* q, const void* pool, const int* table, int table_stride,
                                                const int* tiles, const int* entries, void* out, int n_tiles,
                                                int n_head, int n_kv, int hd, int page_size, float scale,
                                                int window, int n_rows, float* part_o, float* part_ml,
                                                int n_splits, int paired, hipStream_t stream) {
  int rc = check_common("attention_prefill_paired", n_head, n_kv, hd, page_size, table_stride);
  if (rc) return rc;
  if (hd == 32) {
    ti_set_error("attention_prefill_paired: head_dim 32 is not served (64, 128)");
    return 3;
  }
  TI_REQUIRE(n_head <= 65535, "attention_prefill_paired: too many heads");
  TI_REQUIRE(n_splits >= 1 && n_splits <= 8 && (n_splits == 1 || (part_o && part_ml && n_rows > 0)),
             "attention_prefill_paired: 1 to 8 runs of keys, more than one with buffers for their results");
  if (n_tiles == 0) return 0;
  constexpr int NG = 4, NW = 2, ST = 2, CB = 1;
  const int lds = NG * ST * 2 * PF_KEYS * hd * 2;
  static bool ready = false;          // allow more than 64 KiB of dynamic LDS, once
  if (!ready) {
    if (hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<128, NG, NW, ST, true, CB>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, NG * ST * 2 * PF_KEYS * 128 * 2) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<64, NG, NW, ST, true, CB>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, NG * ST * 2 * PF_KEYS * 64 * 2) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<128, NG, NW, ST, false, CB>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, NG * ST * 2 * PF_KEYS * 128 * 2) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<64, NG, NW, ST, false, CB>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, NG * ST * 2 * PF_KEYS * 64 * 2) != hipSuccess) {
      ti_set_error("attention_prefill_paired: cannot reserve the LDS");
      return 2;
    }
    ready = true;
  }
  // paired = 0: a workgroup per tile (a launch that fits the chip in one round lasts as long as its
  // heaviest tile then, not as the heaviest and the lightest together)
  dim3 grid(paired ? (n_tiles + 1) / 2 : n_tiles, n_head, n_splits);
#define TI_GO(H, PAIRED)                                                                                          \
  attn_prefill_lds_kernel<H, NG, NW, ST, PAIRED, CB><<<grid, 64 * NW * NG, lds, stream>>>(                            \
      (const bf16_t*)q, (const bf16_t*)pool, table, table_stride, tiles, n_tiles, entries, (bf16_t*)out, n_head, \
      n_kv, page_size, scale, window, part_o, part_ml)
  if (hd == 128 && paired) TI_GO(128, true);
  else if (hd == 128) TI_GO(128, false);
  else if (paired) TI_GO(64, true);
  else TI_GO(64, false);
#undef TI_GO
  if (n_splits > 1) {
    // every row of the step has its runs (rows of single tokens too: theirs are not read by anyone)
    if (hd == 128)
      attn_merge_kernel<128><<<dim3(n_rows, n_head), 128, 0, stream>>>(part_o, part_ml, nullptr, (bf16_t*)out, n_head,
                                                                     n_splits);
    else
      attn_merge_kernel<64><<<dim3(n_rows, n_head), 64, 0, stream>>>(part_o, part_ml, nullptr, (bf16_t*)out, n_head,
                                                                   n_splits);
  }
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------- tests and measurements
// One entry for every choice above that a test or a measurement may want to force (names as in
// tinyinfer_kernels_tuning.h); process-wide in the library, applied and reset around its calls by the
// host library's Ops.  Returns 0, or 1 for an unknown name.
extern "C" void ti_tuning_reset() {
  g_decode_shared_query = 1;
  g_prefill_groups = 0;
  g_prefill_lds = 1;
}
extern "C" int ti_tuning_set(const char* name, long value) {
  const std::string n = name ? name : "";
  if (n == "decode_shared_query") g_decode_shared_query = (int)value;
  else if (n == "prefill_groups") g_prefill_groups = (int)value;
  else if (n == "prefill_use_lds") g_prefill_lds = (int)value;
  else return 1;
  return 0;
}
