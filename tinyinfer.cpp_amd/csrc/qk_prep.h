// Per-head preparation of queries and keys: RMS-norm over head_dim, then the half-split
// rotation (/root/reference/src/cuda/rope.cu:31-52: q_norm/k_norm are applied before the
// rotation, pairs are (i, i + head_dim / 2)).  The kernel that prepares a whole step's rows
// and the decode attention kernel that prepares its own query both go through these
// functions, with the products and sums spelled out, so that they produce the same bits.
#pragma once
#include "common.h"

// x_lo^2 + x_hi^2 of one rotation pair
__device__ __forceinline__ float qk_pair_square(float lo, float hi) { return fmaf(hi, hi, lo * lo); }

__device__ __forceinline__ float qk_norm_scale(float sum_squares, int hd, float eps) {
  return 1.0f / sqrtf(sum_squares / (float)hd + eps);
}

// (cos, sin) of pair i at position p: from the table for positions it holds, else computed
__device__ __forceinline__ float2 qk_cos_sin(int i, int half, int p, const float* inv_freq, const float2* rope_table,
                                             int table_len) {
  if (rope_table && p < table_len) return rope_table[(size_t)p * half + i];
  float s, c;
  sincosf((float)p * inv_freq[i], &s, &c);
  return make_float2(c, s);
}

// (lo, hi) of a pair -> rotated by the angle whose (cos, sin) is cs
__device__ __forceinline__ void qk_rotate(float& lo, float& hi, float2 cs) {
  const float a = fmaf(lo, cs.x, -(hi * cs.y));
  const float b = fmaf(lo, cs.y, hi * cs.x);
  lo = a;
  hi = b;
}

// One head (hd floats at src) by one wavefront: lane i takes the pairs i, i + 64, ...
// w: norm weight or nullptr; inv_freq: nullptr = no rotation.  Element d of the result goes
// to dst[d * dst_stride].
template <typename T>
__device__ __forceinline__ void qk_head_wave(const float* __restrict__ src, T* __restrict__ dst, size_t dst_stride,
                                             const float* __restrict__ w, float eps,
                                             const float* __restrict__ inv_freq,
                                             const float2* __restrict__ rope_table, int table_len, int p, int hd) {
  const int lane = threadIdx.x % TI_WAVE;
  const int half = hd / 2;
  float scale = 1.f;
  if (w) {
    float ss = 0.f;
    for (int i = lane; i < half; i += TI_WAVE) ss += qk_pair_square(src[i], src[i + half]);
    scale = qk_norm_scale(group_sum<TI_WAVE>(ss), hd, eps);
  }
  for (int i = lane; i < half; i += TI_WAVE) {
    float lo = src[i] * scale, hi = src[i + half] * scale;
    if (w) {
      lo *= w[i];
      hi *= w[i + half];
    }
    if (inv_freq) qk_rotate(lo, hi, qk_cos_sin(i, half, p, inv_freq, rope_table, table_len));
    st<T>(dst + (size_t)i * dst_stride, lo);
    st<T>(dst + (size_t)(i + half) * dst_stride, hi);
  }
}

// A value head: copied (rounded to T), element d to dst[d * dst_stride]
template <typename T>
__device__ __forceinline__ void v_head_wave(const float* __restrict__ src, T* __restrict__ dst, size_t dst_stride,
                                            int hd) {
  const int lane = threadIdx.x % TI_WAVE;
  for (int i = lane; i < hd; i += TI_WAVE) st<T>(dst + (size_t)i * dst_stride, src[i]);
}

// Where keys (which = 0) and values (which = 1) of kv head `kvh` at row `prow` of a page
// start: keys [row][d] (stride 1 over d), values [d][row] (stride P over d).
template <typename T>
__device__ __forceinline__ T* kv_page_slot(T* pool, int page, int which, int kvh, int prow, int n_kv, int P, int hd) {
  return pool + (size_t)page * 2 * n_kv * P * hd + ((size_t)which * n_kv + kvh) * P * hd +
         (which ? (size_t)prow : (size_t)prow * hd);
}
