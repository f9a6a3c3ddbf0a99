// Element-wise and per-row kernels of the step: embedding gather, RMSNorm (with
// an optional row gather), rotary encoding, and the fused per-head norm +
// rotation + paged cache write.  All arithmetic is 32-bit; T is the storage
// type of activations, weights and cache (float or bfloat16).
#include "common.h"
#include "tinyinfer_kernels.h"
#include "qk_prep.h"

TI_ERROR_API

// ------------------------------------------------------------------ embedding
// x[m, :] = float(E[t, :]) with t = tok[m], or, where tok[m] is below zero, t = fed[-1 - tok[m]]:
// an id that an earlier kernel on the stream (the sampler) left on the device, so that the host
// can launch a step before it has read the step before.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tok, const int* __restrict__ fed, int n_fed,
                             float* __restrict__ x, int H, int V) {
  const int m = blockIdx.x;
  int t = tok[m];
  if (t < 0 && fed && -1 - t < n_fed) t = fed[-1 - t];
  float* row = x + (size_t)m * H;
  if (t < 0 || t >= V) {   // the host refuses such ids; never read out of bounds
    for (int i = threadIdx.x; i < H; i += blockDim.x) row[i] = 0.f;
    return;
  }
  const T* src = table + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) row[i] = ld<T>(src + i);
}

extern "C" int ti_embed_fed(int dtype, const void* table, const int* tok, const int* fed, int n_fed, float* x, int M, int H,
                            int V, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0 && V > 0 && n_fed >= 0, "embed: bad sizes M=%d H=%d V=%d n_fed=%d", M, H, V, n_fed);
  if (M == 0) return 0;
  if (dtype == TI_F32)
    embed_kernel<float><<<M, 256, 0, stream>>>((const float*)table, tok, fed, n_fed, x, H, V);
  else if (dtype == TI_BF16)
    embed_kernel<bf16_t><<<M, 256, 0, stream>>>((const bf16_t*)table, tok, fed, n_fed, x, H, V);
  else
    TI_REQUIRE(false, "embed: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

extern "C" int ti_embed(int dtype, const void* table, const int* tok, float* x, int M, int H, int V,
                        hipStream_t stream) {
  return ti_embed_fed(dtype, table, tok, nullptr, 0, x, M, H, V, stream);
}

// -------------------------------------------------------------------- RMSNorm
// out[r, :] = x[src(r), :] * rsqrt(mean(x^2) + eps) * w ; src(r) = rows ? rows[r] : r
template <typename T>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               const int* __restrict__ rows, T* __restrict__ out, int H, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const float* src = x + (size_t)(rows ? rows[r] : r) * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float v = src[i];
    ss += v * v;
  }
  ss = block_sum<256>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)H + eps);
  T* dst = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += 256) st<T>(dst + i, src[i] * scale * w[i]);
}

// the same for widths that are multiples of four: a wavefront per row, four rows a workgroup
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_wave_kernel(const float* __restrict__ x, const float* __restrict__ w, const int* __restrict__ rows,
                    T* __restrict__ out, int n_rows, int H, float eps) {
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (r >= n_rows) return;
  const float* src = x + (size_t)(rows ? rows[r] : r) * H;
  float ss = 0.f;
#pragma unroll 8
  for (int k = lane * 4; k < H; k += 256) ss = rms_accumulate(ss, *reinterpret_cast<const float4*>(src + k));
  const float scale = rms_scale(ss, H, eps);
  T* dst = out + (size_t)r * H;
#pragma unroll 4
  for (int k = lane * 4; k < H; k += 256) {
    const float4 v = *reinterpret_cast<const float4*>(src + k);
    const float4 g = *reinterpret_cast<const float4*>(w + k);
    st<T>(dst + k, v.x * scale * g.x);
    st<T>(dst + k + 1, v.y * scale * g.y);
    st<T>(dst + k + 2, v.z * scale * g.z);
    st<T>(dst + k + 3, v.w * scale * g.w);
  }
}

// Rows wider than RMS_WIDE_FROM: a workgroup of 1,024 threads per row, thread t the 16-byte pieces
// t, t + 1024, ... (a wavefront per row would walk such a row in twenty round trips to memory).
// ADD: x[r] += partial[0][r] + ... + partial[KS - 1][r] first, in that order, written back (see
// rmsnorm_add_partials_kernel); the partial sums are asked for four at a time.  The sum of squares:
// each thread over its pieces in ascending order, then block_sum.  With and without ADD: the same
// bits for the same x.
#define RMS_WIDE_FROM 4096
#define RMS_WIDE_THREADS 1024
template <typename T, bool ADD>
__global__ void __launch_bounds__(RMS_WIDE_THREADS)
rmsnorm_wide_kernel(float* __restrict__ x, const float* __restrict__ partial, int KS, const float* __restrict__ w,
                    const int* __restrict__ rows, T* __restrict__ out, int n_rows, int H, float eps) {
  constexpr int NT = RMS_WIDE_THREADS, PER = 2, SPAN = NT * 4 * PER;   // floats a pass covers
  __shared__ float red[NT / 64];
  const int r = blockIdx.x;
  float* src = x + (size_t)(rows ? rows[r] : r) * H;
  const size_t count = (size_t)n_rows * H;
  const float* prow = partial + (size_t)r * H;
  T* dst = out + (size_t)r * H;
  float4 v[PER];
  auto fetch = [&](int base) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int k = base + threadIdx.x * 4 + i * NT * 4;
      v[i] = *reinterpret_cast<const float4*>(src + (k < H ? k : 0));
    }
    if (ADD) {
      for (int s0 = 0; s0 < KS; s0 += 4) {
        float4 q[4][PER];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < PER; ++i) {
            const int k = base + threadIdx.x * 4 + i * NT * 4;
            q[j][i] = *reinterpret_cast<const float4*>(prow + (size_t)(s0 + j < KS ? s0 + j : s0) * count + (k < H ? k : 0));
          }
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (s0 + j < KS) {
#pragma unroll
            for (int i = 0; i < PER; ++i) {
              v[i].x += q[j][i].x;
              v[i].y += q[j][i].y;
              v[i].z += q[j][i].z;
              v[i].w += q[j][i].w;
            }
          }
      }
    }
  };
  auto scaled = [&](int k, float4 val, float scale) {
    const float4 g = *reinterpret_cast<const float4*>(w + k);
    st<T>(dst + k, val.x * scale * g.x);
    st<T>(dst + k + 1, val.y * scale * g.y);
    st<T>(dst + k + 2, val.z * scale * g.z);
    st<T>(dst + k + 3, val.w * scale * g.w);
  };
  float ss = 0.f;
  for (int base = 0; base < H; base += SPAN) {
    fetch(base);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int k = base + threadIdx.x * 4 + i * NT * 4;
      if (k < H) {
        if (ADD) *reinterpret_cast<float4*>(src + k) = v[i];
        ss = rms_accumulate(ss, v[i]);
      }
    }
  }
  ss = block_sum<NT>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)H + eps);
  if (H <= SPAN) {   // the row is still in registers
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int k = threadIdx.x * 4 + i * NT * 4;
      if (k < H) scaled(k, v[i], scale);
    }
    return;
  }
  for (int base = 0; base < H; base += SPAN) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int k = base + threadIdx.x * 4 + i * NT * 4;
      if (k < H) scaled(k, *reinterpret_cast<const float4*>(src + k), scale);     // this thread's own store above
    }
  }
}

extern "C" int ti_rmsnorm(int out_dtype, const float* x, const float* w, const int* rows, void* out,
                          int n_rows, int H, float eps, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && H > 0, "rmsnorm: bad sizes rows=%d H=%d", n_rows, H);
  TI_REQUIRE(out_dtype == TI_F32 || out_dtype == TI_BF16, "rmsnorm: unknown dtype %d", out_dtype);
  if (n_rows == 0) return 0;
  if (H % 4 == 0 && H > RMS_WIDE_FROM && (((uintptr_t)x | (uintptr_t)w) & 15) == 0) {
    if (out_dtype == TI_F32)
      rmsnorm_wide_kernel<float, false><<<n_rows, RMS_WIDE_THREADS, 0, stream>>>((float*)x, nullptr, 0, w, rows, (float*)out, n_rows, H, eps);
    else
      rmsnorm_wide_kernel<bf16_t, false><<<n_rows, RMS_WIDE_THREADS, 0, stream>>>((float*)x, nullptr, 0, w, rows, (bf16_t*)out, n_rows, H, eps);
    TI_LAUNCH_CHECK();
    return 0;
  }
  if (H % 4 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0) {
    const int grid = (n_rows + 3) / 4;
    if (out_dtype == TI_F32)
      rmsnorm_wave_kernel<float><<<grid, 256, 0, stream>>>(x, w, rows, (float*)out, n_rows, H, eps);
    else
      rmsnorm_wave_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, w, rows, (bf16_t*)out, n_rows, H, eps);
    TI_LAUNCH_CHECK();
    return 0;
  }
  if (out_dtype == TI_F32)
    rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>(x, w, rows, (float*)out, H, eps);
  else if (out_dtype == TI_BF16)
    rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, w, rows, (bf16_t*)out, H, eps);
  else
    TI_REQUIRE(false, "rmsnorm: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// The norm of rows whose last product left its sums of a split K in `partial` [KS][n_rows][H]:
// x[r] += partial[0][r] + ... + partial[KS - 1][r] (in that order, written back), then the norm of
// rmsnorm_wave_kernel over the new x.  A wavefront per row, four rows a workgroup.
// KS_T: the number of partial sums if known when compiled (their loads then do not wait for one
// another), 0: KS.  PIECES: 16-byte pieces of a row a lane keeps in registers between the sum and
// the scaling (rows up to 256 PIECES floats wide; wider rows take the kernels below).
template <typename T, int KS_T, int PIECES>
__global__ void __launch_bounds__(256)
rmsnorm_add_partials_kernel(float* __restrict__ x, const float* __restrict__ partial, int KS,
                            const float* __restrict__ w, T* __restrict__ out, int n_rows, int H, float eps) {
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (r >= n_rows) return;
  float* src = x + (size_t)r * H;
  const size_t count = (size_t)n_rows * H;
  const float* prow = partial + (size_t)r * H;
  if (KS_T) KS = KS_T;
  auto summed = [&](int k) {   // KS_T partial sums, all asked for at once
    float4 v = *reinterpret_cast<const float4*>(src + k);
    float4 p[KS_T ? KS_T : 1];
#pragma unroll
    for (int s = 0; s < KS_T; ++s) p[s] = *reinterpret_cast<const float4*>(prow + s * count + k);
#pragma unroll
    for (int s = 0; s < KS_T; ++s) {
      v.x += p[s].x;
      v.y += p[s].y;
      v.z += p[s].z;
      v.w += p[s].w;
    }
    return v;
  };
  auto scaled = [&](int k, float4 v, float scale) {
    const float4 g = *reinterpret_cast<const float4*>(w + k);
    T* dst = out + (size_t)r * H;
    st<T>(dst + k, v.x * scale * g.x);
    st<T>(dst + k + 1, v.y * scale * g.y);
    st<T>(dst + k + 2, v.z * scale * g.z);
    st<T>(dst + k + 3, v.w * scale * g.w);
  };
  float ss = 0.f;
  {
    float4 v[PIECES];
    if (KS_T) {
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        const int k = lane * 4 + i * 256;
        if (k < H) v[i] = summed(k);
      }
    } else {
      // the row, then one partial sum after the other, each asked for as a whole: 1 + KS round trips
      // to memory, not one per piece
#pragma unroll
      for (int i = 0; i < PIECES; ++i) {
        const int k = lane * 4 + i * 256;
        v[i] = *reinterpret_cast<const float4*>(src + (k < H ? k : 0));
      }
      for (int s = 0; s < KS; ++s) {
        float4 q[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
          const int k = lane * 4 + i * 256;
          q[i] = *reinterpret_cast<const float4*>(prow + s * count + (k < H ? k : 0));
        }
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
          v[i].x += q[i].x;
          v[i].y += q[i].y;
          v[i].z += q[i].z;
          v[i].w += q[i].w;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int k = lane * 4 + i * 256;
      if (k < H) {
        *reinterpret_cast<float4*>(src + k) = v[i];
        ss = rms_accumulate(ss, v[i]);
      }
    }
    const float scale = rms_scale(ss, H, eps);
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int k = lane * 4 + i * 256;
      if (k < H) scaled(k, v[i], scale);
    }
  }
}

// The same for rows of 1,025 to 4,096 floats: a workgroup per row, so that four times as many loads
// are on their way as with a wavefront per row (64 rows of 4,096 with 8 partial sums: 26 -> ~7 us).
// Thread t adds up the 16-byte pieces t, t + 256, ... (the partial sums four at a time), writes them
// back and leaves them in LDS; wavefront 0 takes the sum of squares from there in the order of
// rmsnorm_wave_kernel (lane l the pieces l, l + 64, ...), so the bits are that kernel's.
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_add_partials_row_kernel(float* __restrict__ x, const float* __restrict__ partial, int KS,
                                const float* __restrict__ w, T* __restrict__ out, int n_rows, int H, float eps) {
  __shared__ __attribute__((aligned(16))) float row[4096];
  __shared__ float s_scale;
  const int r = blockIdx.x, lane = threadIdx.x & 63;
  float* src = x + (size_t)r * H;
  const size_t count = (size_t)n_rows * H;
  const float* prow = partial + (size_t)r * H;
  float4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = threadIdx.x * 4 + i * 1024;
    v[i] = *reinterpret_cast<const float4*>(src + (k < H ? k : 0));
  }
  for (int s0 = 0; s0 < KS; s0 += 4) {
    float4 q[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = threadIdx.x * 4 + i * 1024;
        q[j][i] = *reinterpret_cast<const float4*>(prow + (size_t)(s0 + j < KS ? s0 + j : s0) * count + (k < H ? k : 0));
      }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (s0 + j < KS) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[i].x += q[j][i].x;
          v[i].y += q[j][i].y;
          v[i].z += q[j][i].z;
          v[i].w += q[j][i].w;
        }
      }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = threadIdx.x * 4 + i * 1024;
    if (k < H) {
      *reinterpret_cast<float4*>(src + k) = v[i];
      *reinterpret_cast<float4*>(row + k) = v[i];
    }
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    float ss = 0.f;
    for (int k = lane * 4; k < H; k += 256) ss = rms_accumulate(ss, *reinterpret_cast<const float4*>(row + k));
    const float scale = rms_scale(ss, H, eps);
    if (lane == 0) s_scale = scale;
  }
  __syncthreads();
  const float scale = s_scale;
  T* dst = out + (size_t)r * H;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = threadIdx.x * 4 + i * 1024;
    if (k < H) {
      const float4 g = *reinterpret_cast<const float4*>(w + k);
      st<T>(dst + k, v[i].x * scale * g.x);
      st<T>(dst + k + 1, v[i].y * scale * g.y);
      st<T>(dst + k + 2, v[i].z * scale * g.z);
      st<T>(dst + k + 3, v[i].w * scale * g.w);
    }
  }
}

template <typename T>
static void launch_rmsnorm_add_partials(float* x, const float* partial, int KS, const float* w, T* out, int n_rows,
                                        int H, float eps, hipStream_t stream) {
  if (H > RMS_WIDE_FROM) {
    rmsnorm_wide_kernel<T, true><<<n_rows, RMS_WIDE_THREADS, 0, stream>>>(x, partial, KS, w, nullptr, out, n_rows, H, eps);
    return;
  }
  const int grid = (n_rows + 3) / 4;
#define TI_GO(KS_T, PIECES) \
  rmsnorm_add_partials_kernel<T, KS_T, PIECES><<<grid, 256, 0, stream>>>(x, partial, KS, w, out, n_rows, H, eps)
  if (H <= 1024 && KS == 4) TI_GO(4, 4);
  else if (H <= 1024 && KS == 2) TI_GO(2, 4);
  else if (H <= 1024 && KS == 8) TI_GO(8, 4);
  else if (H <= 1024) TI_GO(0, 4);
  else rmsnorm_add_partials_row_kernel<T><<<n_rows, 256, 0, stream>>>(x, partial, KS, w, out, n_rows, H, eps);
#undef TI_GO
}

// Returns 3 for a width or an alignment it does not serve (the caller adds the partial sums with
// their own kernel then, and norms with ti_rmsnorm).
extern "C" int ti_rmsnorm_add_partials(int out_dtype, float* x, const float* partial, int KS, const float* w,
                                       void* out, int n_rows, int H, float eps, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && H > 0 && KS >= 1, "rmsnorm_add_partials: bad sizes rows=%d H=%d KS=%d", n_rows, H, KS);
  TI_REQUIRE(out_dtype == TI_F32 || out_dtype == TI_BF16, "rmsnorm_add_partials: unknown dtype %d", out_dtype);
  if (H % 4 != 0 || (((uintptr_t)x | (uintptr_t)w | (uintptr_t)partial) & 15) != 0) {
    ti_set_error("rmsnorm_add_partials: serves widths that are multiples of 4 and 16-byte aligned operands");
    return 3;
  }
  if (n_rows == 0) return 0;
  if (out_dtype == TI_F32)
    launch_rmsnorm_add_partials<float>(x, partial, KS, w, (float*)out, n_rows, H, eps, stream);
  else
    launch_rmsnorm_add_partials<bf16_t>(x, partial, KS, w, (bf16_t*)out, n_rows, H, eps, stream);
  TI_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------- rotary, by itself
// In place on f32 x[m, h, :] with row stride `row_stride` floats: pair (k, k+hd/2)
// turns by pos[m] * inv_freq[k].
__global__ void rope_neox_kernel(float* __restrict__ x, const int* __restrict__ pos,
                                 const float* __restrict__ inv_freq, int heads, int hd, long row_stride) {
  const int m = blockIdx.x;
  const int half = hd / 2;
  const float p = (float)pos[m];
  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half, k = i % half;
    float* v = x + (size_t)m * row_stride + (size_t)h * hd;
    float s, c;
    sincosf(p * inv_freq[k], &s, &c);
    const float lo = v[k], hi = v[k + half];
    v[k] = lo * c - hi * s;
    v[k + half] = lo * s + hi * c;
  }
}

extern "C" int ti_rope_neox(float* x, const int* pos, const float* inv_freq, int M, int heads, int hd,
                            long row_stride, hipStream_t stream) {
  TI_REQUIRE(hd > 0 && hd % 2 == 0, "rope: head_dim %d must be even", hd);
  TI_REQUIRE(row_stride >= (long)heads * hd, "rope: row stride %ld shorter than heads*head_dim", row_stride);
  if (M == 0 || heads == 0) return 0;
  rope_neox_kernel<<<M, 256, 0, stream>>>(x, pos, inv_freq, heads, hd, row_stride);
  TI_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------- sin/cos table
// table[p][k] = (cos, sin)(float(p) * inv_freq[k]) for p < n_pos: the same 32-bit
// angle and the same precise sincosf the kernels would compute on the fly.
__global__ void rope_table_kernel(float2* __restrict__ table, const float* __restrict__ inv_freq, int half,
                                  int n_pos) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_pos * half) return;
  const int p = i / half, k = i % half;
  float s, c;
  sincosf((float)p * inv_freq[k], &s, &c);
  table[i] = make_float2(c, s);
}

extern "C" int ti_rope_table(float* table, const float* inv_freq, int half, int n_pos, hipStream_t stream) {
  TI_REQUIRE(half > 0 && n_pos > 0, "rope_table: bad sizes half=%d positions=%d", half, n_pos);
  const long n = (long)half * n_pos;
  rope_table_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((float2*)table, inv_freq, half, n_pos);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------- per-head norm + rotation + cache write
// One wavefront per (token, head): grid (M, ceil(units / 4)), units = q heads +
// k heads + v heads.  For q heads and k heads: RMS-norm over head_dim (if a weight
// is given), then the half-split rotation (if inv_freq is given; cos and sin come
// from `rope_table` for positions below `table_len`, else they are computed).  q
// goes to q_out (T), k and v into the cache page of the token's position,
// page = table[slot][pos / P]:
//   keys   pool[page][0][kv head][pos % P][d]   (a key's dims are contiguous: the
//                                                 score sums over d)
//   values pool[page][1][kv head][d][pos % P]   (transposed: the mix sums over
//                                                 positions, so these are contiguous)
// v is copied unchanged.  n_kv == 0: only q is handled (the layer reads another
// layer's keys and values).
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_kv_write_kernel(
    const float* __restrict__ qkv, const float* __restrict__ q_w, const float* __restrict__ k_w,
    const float* __restrict__ inv_freq, const float2* __restrict__ rope_table, int table_len,
    const int* __restrict__ pos, const int* __restrict__ slot,
    const int* __restrict__ table, int table_stride, T* __restrict__ pool, T* __restrict__ q_out,
    int n_head, int n_kv, int hd, int P, float eps) {
  const int m = blockIdx.x;
  const int wave = threadIdx.x / TI_WAVE, lane = threadIdx.x % TI_WAVE;
  const int u = blockIdx.y * (blockDim.x / TI_WAVE) + wave;
  if (u >= n_head + 2 * n_kv) return;
  const int nq = n_head * hd, nk = n_kv * hd;
  const float* row = qkv + (size_t)m * (nq + 2 * nk);
  const int p = pos[m];
  const bool is_q = u < n_head;
  const bool is_v = u >= n_head + n_kv;
  const float* src = row + (size_t)u * hd;
  if (is_q) {
    qk_head_wave<T>(src, q_out + (size_t)m * nq + (size_t)u * hd, 1, q_w, eps, inv_freq, rope_table, table_len, p,
                    hd);
    return;
  }
  const int page = table[(size_t)slot[m] * table_stride + p / P];
  if (page < 0) return;   // the host reserves pages first; never write astray
  const int kvh = is_v ? u - n_head - n_kv : u - n_head;
  T* dst = kv_page_slot<T>(pool, page, is_v ? 1 : 0, kvh, p % P, n_kv, P, hd);
  if (is_v)
    v_head_wave<T>(src, dst, (size_t)P, hd);
  else
    qk_head_wave<T>(src, dst, 1, k_w, eps, inv_freq, rope_table, table_len, p, hd);
}

extern "C" int ti_qk_norm_rope_kv_write(int dtype, const float* qkv, const float* q_w, const float* k_w,
                                        const float* inv_freq, const float* rope_table, int table_len,
                                        const int* pos, const int* slot,
                                        const int* table, int table_stride, void* pool, void* q_out,
                                        int M, int n_head, int n_kv, int hd, int page_size, float eps,
                                        hipStream_t stream) {
  TI_REQUIRE(hd > 0 && hd % 2 == 0, "qk_norm_rope_kv_write: head_dim %d must be even", hd);
  TI_REQUIRE(n_head > 0 && n_kv >= 0 && page_size > 0 && table_stride > 0,
             "qk_norm_rope_kv_write: bad sizes heads=%d kv_heads=%d page=%d table_stride=%d", n_head, n_kv,
             page_size, table_stride);
  if (M == 0) return 0;
  const int units = n_head + 2 * n_kv;
  TI_REQUIRE((units + 3) / 4 <= 65535, "qk_norm_rope_kv_write: too many heads");
  dim3 grid(M, (units + 3) / 4);
  if (dtype == TI_F32)
    qk_norm_rope_kv_write_kernel<float><<<grid, 256, 0, stream>>>(
        qkv, q_w, k_w, inv_freq, (const float2*)rope_table, table_len, pos, slot, table, table_stride,
        (float*)pool, (float*)q_out, n_head, n_kv, hd, page_size, eps);
  else if (dtype == TI_BF16)
    qk_norm_rope_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>(
        qkv, q_w, k_w, inv_freq, (const float2*)rope_table, table_len, pos, slot, table, table_stride,
        (bf16_t*)pool, (bf16_t*)q_out, n_head, n_kv, hd, page_size, eps);
  else
    TI_REQUIRE(false, "qk_norm_rope_kv_write: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// The per-head norm alone, in place on the 32-bit projections (rows of `row_width` floats: q heads,
// then k heads): for a position encoding that has no fused form and must see normed heads.
// Grid (M, ceil(units / 4)), a wavefront per (token, head); a weight that is nullptr leaves its
// heads as they are.
__global__ void __launch_bounds__(256)
qk_norm_inplace_kernel(float* qkv, int row_width, const float* __restrict__ q_w,
                       const float* __restrict__ k_w, int n_head, int n_kv, int hd, float eps) {
  const int m = blockIdx.x;
  const int u = blockIdx.y * (blockDim.x / TI_WAVE) + threadIdx.x / TI_WAVE;
  if (u >= n_head + n_kv) return;
  const float* w = u < n_head ? q_w : k_w;
  if (!w) return;
  float* head = qkv + (size_t)m * row_width + (size_t)u * hd;
  // the arithmetic of qk_head_wave without a rotation; each lane reads its own elements before it
  // writes them
  const int lane = threadIdx.x % TI_WAVE, half = hd / 2;
  float ss = 0.f;
  for (int i = lane; i < half; i += TI_WAVE) ss += qk_pair_square(head[i], head[i + half]);
  const float scale = qk_norm_scale(group_sum<TI_WAVE>(ss), hd, eps);
  for (int i = lane; i < half; i += TI_WAVE) {
    float lo = head[i] * scale, hi = head[i + half] * scale;
    lo *= w[i];
    hi *= w[i + half];
    head[i] = lo;
    head[i + half] = hi;
  }
}

extern "C" int ti_qk_norm_inplace(float* qkv, int row_width, const float* q_w, const float* k_w, int M, int n_head,
                                  int n_kv, int hd, float eps, hipStream_t stream) {
  TI_REQUIRE(hd > 0 && hd % 2 == 0 && n_head > 0 && n_kv >= 0 && row_width >= (n_head + n_kv) * hd,
             "qk_norm_inplace: bad sizes heads=%d kv_heads=%d head_dim=%d row_width=%d", n_head, n_kv, hd, row_width);
  if (M == 0) return 0;
  const int units = n_head + n_kv;
  TI_REQUIRE((units + 3) / 4 <= 65535, "qk_norm_inplace: too many heads");
  qk_norm_inplace_kernel<<<dim3(M, (units + 3) / 4), 256, 0, stream>>>(qkv, row_width, q_w, k_w, n_head, n_kv, hd, eps);
  TI_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------------- fills
// Zero `words` four-byte words (a kernel, not a memset node: a caller may be capturing a graph).
__global__ void fill_zero_kernel(uint32_t* __restrict__ p, long words) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (long)gridDim.x * blockDim.x) p[i] = 0u;
}

extern "C" int ti_fill_zero(void* p, long bytes, hipStream_t stream) {
  TI_REQUIRE(bytes >= 0 && bytes % 4 == 0 && ((uintptr_t)p & 3) == 0, "fill_zero: %ld bytes at %p are not whole words",
             bytes, p);
  if (bytes == 0) return 0;
  const long words = bytes / 4;
  const unsigned blocks = (unsigned)((words + 255) / 256 < 4096 ? (words + 255) / 256 : 4096);
  fill_zero_kernel<<<blocks, 256, 0, stream>>>((uint32_t*)p, words);
  TI_LAUNCH_CHECK();
  return 0;
}

// Random weights on the device.  Element i of a tensor is a pure function of (seed, i): two
// 24-bit uniforms from splitmix64's output function, then Box-Muller for a normal.  The host's
// generator (the one that writes model folders) is the same function.  The logarithm, root and
// cosine are taken in double precision and the value is rounded to 32-bit once at the end: the two
// libraries' double results differ far below a 32-bit step, so the device draws the bits the host
// draws (32-bit logf/cosf of two libraries differ in the last bit for a third of the values).
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
// kind 0: normal(a, b); 1: uniform [a, b); 2: constant a
template <typename T>
__global__ void fill_random_kernel(T* __restrict__ p, long n, int kind, float a, float b, uint64_t seed) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const uint64_t z = mix64(mix64(seed) ^ (uint64_t)i);
    const double u1 = ((double)((z >> 40) & 0xffffffu) + 1.0) * (1.0 / 16777216.0);   // (0, 1]
    const double u2 = (double)((z >> 16) & 0xffffffu) * (1.0 / 16777216.0);            // [0, 1)
    float v;
    if (kind == 0) v = (float)((double)a + (double)b * (sqrt(-2.0 * log(u1)) * cos(6.28318530717958647692 * u2)));
    else if (kind == 1) v = (float)((double)a + ((double)b - (double)a) * u2);
    else v = a;
    st<T>(p + i, v);
  }
}
__global__ void fill_random_int_kernel(int* __restrict__ p, long n, int lo, int hi, uint64_t seed) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const uint64_t z = mix64(mix64(seed) ^ (uint64_t)i);
    p[i] = lo + (int)((z >> 11) % (uint64_t)(hi > lo ? hi - lo : 1));
  }
}

extern "C" int ti_fill_random(int dtype, void* p, long n, int kind, float a, float b, unsigned long seed,
                              hipStream_t stream) {
  TI_REQUIRE(n >= 0 && kind >= 0 && kind <= 2, "fill_random: bad count %ld or kind %d", n, kind);
  TI_REQUIRE(dtype == TI_F32 || dtype == TI_BF16 || dtype == 2, "fill_random: unknown dtype %d", dtype);
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  if (dtype == TI_F32) fill_random_kernel<float><<<blocks, 256, 0, stream>>>((float*)p, n, kind, a, b, seed);
  else if (dtype == TI_BF16) fill_random_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)p, n, kind, a, b, seed);
  else fill_random_int_kernel<<<blocks, 256, 0, stream>>>((int*)p, n, (int)a, (int)b, seed);
  TI_LAUNCH_CHECK();
  return 0;
}
