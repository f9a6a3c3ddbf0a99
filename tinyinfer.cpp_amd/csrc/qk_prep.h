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

// One head by one thread, from hd floats at `src` (LDS or memory) to hd contiguous bfloat16 at
// `dst` (16-byte aligned): the arithmetic of qk_head_wave with the sum of squares going up the
// same tree as its butterfly (partners at distance 32, 16, ..., 1), so the bits are the same.
// Eight pairs at a time: their angles come in as four 16-byte loads, their results leave as two.
template <int HD>
__device__ __forceinline__ void qk_head_thread(const float* src, bf16_t* dst, const float* w, float eps,
                                               const float* inv_freq, const float2* rope_table, int table_len,
                                               int p) {
  constexpr int HALF = HD / 2;
  static_assert(HALF == 32 || HALF == 64, "the tree below is that of a 64-lane butterfly with one pair a lane");
  float scale = 1.f;
  if (w) {
    float t[HALF];
#pragma unroll
    for (int i = 0; i < HALF; ++i) t[i] = qk_pair_square(src[i], src[i + HALF]);
#pragma unroll
    for (int o = HALF / 2; o >= 1; o >>= 1)
#pragma unroll
      for (int i = 0; i < o; ++i) t[i] += t[i + o];
    scale = qk_norm_scale(t[0], HD, eps);
  }
  auto run_of_eight = [&](int c, const float2* cs) {
    float lo[8], hi[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      lo[j] = src[c + j] * scale;
      hi[j] = src[c + j + HALF] * scale;
      if (w) {
        lo[j] *= w[c + j];
        hi[j] *= w[c + j + HALF];
      }
      if (inv_freq) qk_rotate(lo[j], hi[j], cs[j]);
    }
    *reinterpret_cast<uint4*>(dst + c) = make_uint4(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]),
                                                    pack_bf16x2(lo[4], lo[5]), pack_bf16x2(lo[6], lo[7]));
    *reinterpret_cast<uint4*>(dst + c + HALF) = make_uint4(pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]),
                                                           pack_bf16x2(hi[4], hi[5]), pack_bf16x2(hi[6], hi[7]));
  };
  if (inv_freq && rope_table && p < table_len) {
    // all angles of the row at once (sixteen-byte loads that do not wait for one another)
    float2 cs[HALF];
    const float4* tp = reinterpret_cast<const float4*>(rope_table + (size_t)p * HALF);
#pragma unroll
    for (int h = 0; h < HALF / 2; ++h) {
      const float4 v = tp[h];
      cs[2 * h] = make_float2(v.x, v.y);
      cs[2 * h + 1] = make_float2(v.z, v.w);
    }
#pragma unroll
    for (int c = 0; c < HALF; c += 8) run_of_eight(c, cs + c);
  } else {
    for (int c = 0; c < HALF; c += 8) {
      float2 cs[8];
      if (inv_freq) {
#pragma unroll
        for (int j = 0; j < 8; ++j) cs[j] = qk_cos_sin(c + j, HALF, p, inv_freq, nullptr, 0);
      }
      run_of_eight(c, cs);
    }
  }
}

// One head by eight adjacent lanes of a wavefront: lane j of the eight takes HD / 16 consecutive pairs,
// HD / 16 j .. HD / 16 (j + 1) - 1, of the row: what it reads (LDS, weights, angles) and what it writes
// are runs of consecutive bytes.  The three functions below give such a lane its norm weights, its
// angles, and the finished elements.  The loads of the first two do not wait for one another, and a
// caller with several rows asks for all their angles before it finishes the first.
template <int HD>
__device__ __forceinline__ void qk_lanes_weights(float (&wlo)[HD / 16], float (&whi)[HD / 16], const float* w) {
  constexpr int PPL = HD / 16;
  const int j = threadIdx.x & 7;
#pragma unroll
  for (int k = 0; k < PPL; ++k) {
    wlo[k] = w ? w[PPL * j + k] : 1.f;
    whi[k] = w ? w[HD / 2 + PPL * j + k] : 1.f;
  }
}

// (cos, sin) of this lane's pairs at position p; inv_freq must not be nullptr
template <int HD>
__device__ __forceinline__ void qk_lanes_angles(float2 (&cs)[HD / 16], int p, const float* inv_freq,
                                                const float2* rope_table, int table_len) {
  constexpr int HALF = HD / 2, PPL = HD / 16;
  const int j = threadIdx.x & 7;
  const bool held = rope_table && p < table_len;
  if (rope_table) {
    // every lane loads (a row beyond the table reads the last one and computes below)
    const float4* tp = reinterpret_cast<const float4*>(rope_table + (size_t)min(p, table_len - 1) * HALF + PPL * j);
#pragma unroll
    for (int k = 0; k < PPL; k += 2) {
      const float4 v = tp[k / 2];
      cs[k] = make_float2(v.x, v.y);
      cs[k + 1] = make_float2(v.z, v.w);
    }
  }
  if (!held) {
#pragma unroll
    for (int k = 0; k < PPL; ++k) cs[k] = qk_cos_sin(PPL * j + k, HALF, p, inv_freq, nullptr, 0);
  }
}

// From HD floats at `row` (LDS, 16-byte aligned) to this lane's finished elements as bfloat16 pairs:
// lo[k] holds elements HD / 16 j + 2 k, + 1, hi[k] the same of the second half (HD / 2 further on).  The
// sum of squares goes up the tree of qk_head_wave's butterfly, so the bits are the same: partners at
// pair distance HD / 4, HD / 8, HD / 16 sit in the lanes j ^ 4, j ^ 2, j ^ 1 with the same k (every
// lane's HD / 16 partial sums cross the lanes), the closer ones in the lane itself.  All lanes of the
// wavefront call it together.  NORMED: with the norm (weights wlo, whi); ROTATE: with the rotation by cs.
template <int HD, bool NORMED, bool ROTATE>
__device__ __forceinline__ void qk_head_lanes(const float* row, const float (&wlo)[HD / 16], const float (&whi)[HD / 16],
                                              float eps, const float2 (&cs)[HD / 16], unsigned (&lo_out)[HD / 32],
                                              unsigned (&hi_out)[HD / 32]) {
  constexpr int HALF = HD / 2, PPL = HD / 16;
  static_assert(PPL == 4 || PPL == 8, "the tree below is that of a 64-lane butterfly with one pair a lane");
  const int j = threadIdx.x & 7;
  float lo[PPL], hi[PPL];
#pragma unroll
  for (int k = 0; k < PPL; k += 4) {
    const float4 a = *reinterpret_cast<const float4*>(row + PPL * j + k);
    const float4 b = *reinterpret_cast<const float4*>(row + HALF + PPL * j + k);
    lo[k] = a.x; lo[k + 1] = a.y; lo[k + 2] = a.z; lo[k + 3] = a.w;
    hi[k] = b.x; hi[k + 1] = b.y; hi[k + 2] = b.z; hi[k + 3] = b.w;
  }
  float scale = 1.f;
  if (NORMED) {
    float t[PPL];
#pragma unroll
    for (int k = 0; k < PPL; ++k) t[k] = qk_pair_square(lo[k], hi[k]);
#pragma unroll
    for (int o = 4; o >= 1; o >>= 1)
#pragma unroll
      for (int k = 0; k < PPL; ++k) t[k] += __shfl_xor(t[k], o, TI_WAVE);
#pragma unroll
    for (int o = PPL / 2; o >= 1; o >>= 1)
#pragma unroll
      for (int k = 0; k < o; ++k) t[k] += t[k + o];
    scale = qk_norm_scale(t[0], HD, eps);
  }
#pragma unroll
  for (int k = 0; k < PPL; k += 2) {
    float a[2], b[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      a[e] = lo[k + e] * scale;
      b[e] = hi[k + e] * scale;
      if (NORMED) {
        a[e] *= wlo[k + e];
        b[e] *= whi[k + e];
      }
      if (ROTATE) qk_rotate(a[e], b[e], cs[k + e]);
    }
    lo_out[k / 2] = pack_bf16x2(a[0], a[1]);
    hi_out[k / 2] = pack_bf16x2(b[0], b[1]);
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
