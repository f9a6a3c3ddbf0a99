// Shared device helpers for the gfx950 kernels: storage types, bfloat16
// conversion, reductions over 64-lane wavefronts, host-side argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <math.h>

typedef uint16_t bf16_t;   // bfloat16 bits; arithmetic always happens in float

#define TI_WAVE 64

// dtype codes of the C ABI
#define TI_F32 0
#define TI_BF16 1

// epilogues of the matrix products
#define TI_EPI_STORE_F32 0   // out f32 [M,N] = A W^T
#define TI_EPI_ADD_F32 1     // out f32 [M,N] += A W^T        (residual sum in 32-bit)
#define TI_EPI_STORE_ACT 2   // out T   [M,N] = A W^T
#define TI_EPI_SWIGLU 3      // W = [gate; up] ([2F,K]); out T [M,F] = silu(g) * u
#define TI_EPI_QKV_PREP 4    // W = [q; k; v] heads: per-head norm, rotation, q out and cache write (own entry point)

__device__ __forceinline__ float bf2f(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// two floats -> two bfloat16 in one word (first in the low half), round to nearest even:
// gfx950 has an instruction for it (v_cvt_pk_bf16_f32)
typedef float ti_float2v __attribute__((ext_vector_type(2)));
typedef __bf16 ti_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const ti_float2v v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, ti_bf16x2));
}
// one float -> bfloat16, round to nearest even, NaN stays NaN (the same instruction)
__device__ __forceinline__ bf16_t f2bf(float f) { return (bf16_t)(pack_bf16x2(f, 0.f) & 0xffffu); }

template <typename T> __device__ __forceinline__ float ld(const T* p);
template <> __device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st(T* p, float v);
template <> __device__ __forceinline__ void st<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// sum over the `width` consecutive lanes a lane belongs to (width: power of two <= 64);
// every lane of the group ends with the total
template <int WIDTH> __device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = WIDTH / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TI_WAVE);
  return v;
}
template <int WIDTH> __device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int o = WIDTH / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TI_WAVE));
  return v;
}

// The RMSNorm of a row by one wavefront, in pieces of four floats: lane l holds the pieces
// l, l + 64, ...  Every kernel that norms a row this way goes through these two functions,
// so they all produce the same bits.
__device__ __forceinline__ float rms_accumulate(float acc, float4 v) {
  acc = fmaf(v.x, v.x, acc);
  acc = fmaf(v.y, v.y, acc);
  acc = fmaf(v.z, v.z, acc);
  return fmaf(v.w, v.w, acc);
}
__device__ __forceinline__ float rms_scale(float lane_acc, int width, float eps) {
  return 1.0f / sqrtf(group_sum<TI_WAVE>(lane_acc) / (float)width + eps);
}

// The merge of an attention that was split over the context.  Split s of a (row, head) left
// (m_s, l_s): its maximum in the exp2 domain and the sum of its weights, and o_s, its
// weighted values.  With mm = max_s m_s and w_s = 2^(m_s - mm), the merged row is
// (sum_s o_s w_s) / (sum_s l_s w_s), both sums taken in ascending order of s with fused
// multiply-adds.  Every kernel that merges goes through these functions: same bits.
__device__ __forceinline__ float split_weight(float m_s, float mm) {
  return (m_s == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_s - mm);
}
__device__ __forceinline__ float split_accumulate(float acc, float o_s, float w) { return fmaf(o_s, w, acc); }
__device__ __forceinline__ float4 split_accumulate(float4 acc, float4 o_s, float w) {
  return make_float4(fmaf(o_s.x, w, acc.x), fmaf(o_s.y, w, acc.y), fmaf(o_s.z, w, acc.z), fmaf(o_s.w, w, acc.w));
}

// sum over a workgroup of NT threads (NT multiple of 64, <= 1024); `red` holds
// NT/64 floats of LDS.  Every thread gets the total.  Fixed order: deterministic.
template <int NT> __device__ __forceinline__ float block_sum(float v, float* red) {
  v = group_sum<TI_WAVE>(v);
  const int w = threadIdx.x / TI_WAVE;
  __syncthreads();
  if ((threadIdx.x & (TI_WAVE - 1)) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / TI_WAVE; ++i) t += red[i];
  return t;
}
template <int NT> __device__ __forceinline__ float block_max(float v, float* red) {
  v = group_max<TI_WAVE>(v);
  const int w = threadIdx.x / TI_WAVE;
  __syncthreads();
  if ((threadIdx.x & (TI_WAVE - 1)) == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < NT / TI_WAVE; ++i) t = fmaxf(t, red[i]);
  return t;
}

// ---------------------------------------------------------------- host side
#include <stdarg.h>
// every kernel library keeps its own last-error text and exports ti_last_error()
static thread_local char ti_err_buf[512];
static inline void ti_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(ti_err_buf, sizeof(ti_err_buf), fmt, ap);
  va_end(ap);
}
#define TI_ERROR_API \
  extern "C" const char* ti_last_error() { return ti_err_buf; }

#define TI_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      ti_set_error(__VA_ARGS__);         \
      return 1;                          \
    }                                    \
  } while (0)

#define TI_LAUNCH_CHECK()                                                       \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) {                                                     \
      ti_set_error("%s:%d: launch failed: %s", __FILE__, __LINE__, hipGetErrorString(e_)); \
      return 2;                                                                 \
    }                                                                           \
  } while (0)
