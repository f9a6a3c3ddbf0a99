// Sampling on the device: greedy argmax (of equal logits the lowest index wins,
// as /root/reference/src/cuda/sample.cu:5-11) and temperature sampling with
// optional top-k and top-p cuts (/root/reference/src/main.cpp:40-83 does these
// on the host with a sort).  One workgroup per row of logits.
//
// Temperature sampling draws by inverse CDF over the index order from one
// uniform number per row, which the host derives from (seed, request, number of
// tokens generated), so a draw does not depend on what else is in the batch.
// The cuts are found without sorting: the k-th largest logit, and the logit at
// which the descending cumulative mass reaches top_p, each by 32 steps of
// bisection over the order-preserving integer image of the floats; every sum is
// reduced in a fixed order, so the result is reproducible.
#include <mutex>

#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define SNT 1024

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ int block_sum_int(int v, int* red) {
#pragma unroll
  for (int o = TI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TI_WAVE);
  __syncthreads();
  if ((threadIdx.x & (TI_WAVE - 1)) == 0) red[threadIdx.x / TI_WAVE] = v;
  __syncthreads();
  int t = 0;
#pragma unroll
  for (int i = 0; i < SNT / TI_WAVE; ++i) t += red[i];
  return t;
}

__device__ int row_argmax(const float* __restrict__ row, int V, float* s_val, int* s_idx) {
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += SNT) {
    const float v = row[i];
    if (v > bv || (bi == 0x7fffffff && v == v)) {   // first finite or -inf value, then strictly greater
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int o = TI_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, TI_WAVE);
    const int oi = __shfl_xor(bi, o, TI_WAVE);
    if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
      bv = ov;
      bi = oi;
    }
  }
  __syncthreads();
  if ((threadIdx.x & (TI_WAVE - 1)) == 0) {
    s_val[threadIdx.x / TI_WAVE] = bv;
    s_idx[threadIdx.x / TI_WAVE] = bi;
  }
  __syncthreads();
  float fv = s_val[0];
  int fi = s_idx[0];
  for (int i = 1; i < SNT / TI_WAVE; ++i) {
    const float ov = s_val[i];
    const int oi = s_idx[i];
    if (oi != 0x7fffffff && (fi == 0x7fffffff || ov > fv || (ov == fv && oi < fi))) {
      fv = ov;
      fi = oi;
    }
  }
  return fi == 0x7fffffff ? 0 : fi;
}

__global__ void __launch_bounds__(SNT)
argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V) {
  __shared__ float s_val[SNT / TI_WAVE];
  __shared__ int s_idx[SNT / TI_WAVE];
  const int r = blockIdx.x;
  const int best = row_argmax(logits + (size_t)r * V, V, s_val, s_idx);
  if (threadIdx.x == 0) out[r] = best;
}

// Greedy choice of a long row in two steps, so that a row is read by many
// workgroups at once: grid (rows, ARG_PARTS) finds the best of each slice, then
// one wavefront per row picks among the ARG_PARTS winners (lowest index on ties).
#define ARG_PARTS 64
__global__ void __launch_bounds__(256)
argmax_part_kernel(const float* __restrict__ logits, float* __restrict__ part_val, int* __restrict__ part_idx,
                   int V) {
  __shared__ float s_val[4];
  __shared__ int s_idx[4];
  const int r = blockIdx.x, c = blockIdx.y;
  const int chunk = (V + ARG_PARTS - 1) / ARG_PARTS;
  const int b = c * chunk, e = min(V, b + chunk);
  const float* row = logits + (size_t)r * V;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = b + threadIdx.x; i < e; i += 256) {
    const float v = row[i];
    if (v > bv || (bi == 0x7fffffff && v == v)) {
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int o = TI_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, TI_WAVE);
    const int oi = __shfl_xor(bi, o, TI_WAVE);
    if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
      bv = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    s_val[threadIdx.x >> 6] = bv;
    s_idx[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      const float ov = s_val[w];
      const int oi = s_idx[w];
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
        bv = ov;
        bi = oi;
      }
    }
    part_val[r * ARG_PARTS + c] = bv;
    part_idx[r * ARG_PARTS + c] = bi;
  }
}

__global__ void __launch_bounds__(64)
argmax_final_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx, int* __restrict__ out) {
  const int r = blockIdx.x;
  float bv = part_val[r * ARG_PARTS + threadIdx.x];
  int bi = part_idx[r * ARG_PARTS + threadIdx.x];
#pragma unroll
  for (int o = TI_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, TI_WAVE);
    const int oi = __shfl_xor(bi, o, TI_WAVE);
    if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
      bv = ov;
      bi = oi;
    }
  }
  if (threadIdx.x == 0) out[r] = bi == 0x7fffffff ? 0 : bi;
}

// temp[r] <= 0: greedy.  top_k[r] <= 0 or >= V: no top-k cut.  top_p[r] >= 1: no top-p cut.
__global__ void __launch_bounds__(SNT)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temp, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ uni, int* __restrict__ out, int V) {
  __shared__ float s_val[SNT / TI_WAVE];
  __shared__ int s_idx[SNT / TI_WAVE];
  __shared__ float s_chunk[SNT];
  __shared__ int s_pick;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * V;
  const float T = temp[r];
  const int best = row_argmax(row, V, s_val, s_idx);
  if (!(T > 0.f)) {
    if (threadIdx.x == 0) out[r] = best;
    return;
  }
  const float mx = row[best];
  const float inv_t = 1.0f / T;

  uint32_t cut = 0;   // keep keys >= cut
  const int k = top_k[r];
  if (k > 0 && k < V) {
    uint32_t prefix = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = prefix | (1u << bit);
      int c = 0;
      for (int i = threadIdx.x; i < V; i += SNT) c += (row[i] == row[i] && order_key(row[i]) >= cand) ? 1 : 0;
      c = block_sum_int(c, s_idx);
      if (c >= k) prefix = cand;
    }
    cut = prefix;
  }
  const float p_keep = top_p[r];
  if (p_keep < 1.0f) {
    float s = 0.f;
    for (int i = threadIdx.x; i < V; i += SNT) {
      const float v = row[i];
      if (v == v && order_key(v) >= cut) s += expf((v - mx) * inv_t);
    }
    const float total = block_sum<SNT>(s, s_val);
    const float need = p_keep * total;
    uint32_t prefix = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = prefix | (1u << bit);
      float ms = 0.f;
      for (int i = threadIdx.x; i < V; i += SNT) {
        const float v = row[i];
        if (v == v && order_key(v) >= cand && order_key(v) >= cut) ms += expf((v - mx) * inv_t);
      }
      ms = block_sum<SNT>(ms, s_val);
      if (ms >= need) prefix = cand;
    }
    if (prefix > cut) cut = prefix;
  }

  // inverse CDF over the index order; thread t owns indices [t*C, (t+1)*C)
  const int C = (V + SNT - 1) / SNT;
  const int b = threadIdx.x * C, e = min(V, b + C);
  float cs = 0.f;
  for (int i = b; i < e; ++i) {
    const float v = row[i];
    if (v == v && order_key(v) >= cut) cs += expf((v - mx) * inv_t);
  }
  s_chunk[threadIdx.x] = cs;
  if (threadIdx.x == 0) s_pick = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int i = 0; i < SNT; ++i) total += s_chunk[i];
    const float target = uni[r] * total;
    float acc = 0.f;
    int owner = -1, last_nonzero = 0;
    for (int i = 0; i < SNT; ++i) {
      if (s_chunk[i] > 0.f) last_nonzero = i;
      if (owner < 0 && s_chunk[i] > 0.f && target < acc + s_chunk[i]) {
        owner = i;
        break;
      }
      acc += s_chunk[i];
    }
    if (owner < 0) {   // rounding pushed the target past the end: the last kept entry
      owner = last_nonzero;
      acc = -1.f;      // marks "take the owner's last kept index"
    }
    // walk the owner's chunk
    const int ob = owner * C, oe = min(V, ob + C);
    int pick = -1, last = -1;
    float a = acc;
    for (int i = ob; i < oe; ++i) {
      const float v = row[i];
      if (!(v == v) || order_key(v) < cut) continue;
      last = i;
      if (acc < 0.f) continue;
      a += expf((v - mx) * inv_t);
      if (target < a) {
        pick = i;
        break;
      }
    }
    s_pick = pick >= 0 ? pick : (last >= 0 ? last : best);
  }
  __syncthreads();
  if (threadIdx.x == 0) out[r] = s_pick;
}

// scratch: 2 * n_rows * 64 four-byte words, or nullptr (then one workgroup reads a whole row)
extern "C" int ti_argmax(const float* logits, int* out, void* scratch, int n_rows, int V, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", n_rows, V);
  if (n_rows == 0) return 0;
  if (scratch && V >= 16384) {
    float* pv = (float*)scratch;
    int* pi = (int*)scratch + (size_t)n_rows * ARG_PARTS;
    argmax_part_kernel<<<dim3(n_rows, ARG_PARTS), 256, 0, stream>>>(logits, pv, pi, V);
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(pv, pi, out);
  } else {
    argmax_kernel<<<n_rows, SNT, 0, stream>>>(logits, out, V);
  }
  TI_LAUNCH_CHECK();
  return 0;
}

// The same greedy choice for callers that cannot allocate (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc): the two-stage kernels above, with their partial
// results in a file-scope device array instead of a workspace argument.  Each GPU holds its own
// copy of the array (128 KiB) until the process ends; its address on a device is asked for once,
// with that device current, and kept.  Nothing in the array has to start at zero: the first stage
// writes every slot of the rows it is given before the second stage reads them.  Every call on a
// GPU shares that GPU's array, so calls that overlap on one GPU (two streams, two threads) race.
#define ARGMAX_STATIC_MAX_ROWS 256
static __device__ __align__(256) unsigned int scratch[2 * ARG_PARTS * ARGMAX_STATIC_MAX_ROWS];
#define ARGMAX_STATIC_MAX_DEVICES 64
static void* g_scratch_ptr[ARGMAX_STATIC_MAX_DEVICES];     // per device: where `scratch` lies there
static std::mutex g_scratch_mutex;

extern "C" int ti_argmax_static(const float* logits, int* out, int n_rows, int V, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && V > 0, "argmax_static: bad sizes rows=%d V=%d", n_rows, V);
  TI_REQUIRE(n_rows <= ARGMAX_STATIC_MAX_ROWS,
             "argmax_static: %d rows are more than the %d its fixed scratch array serves (use ti_argmax with a workspace)",
             n_rows, ARGMAX_STATIC_MAX_ROWS);
  if (n_rows == 0) return 0;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  TI_REQUIRE(e == hipSuccess && dev >= 0 && dev < ARGMAX_STATIC_MAX_DEVICES, "argmax_static: no current device (%s)",
             hipGetErrorString(e));
  void* ptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      TI_REQUIRE(e == hipSuccess && p, "argmax_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      g_scratch_ptr[dev] = p;
    }
    ptr = g_scratch_ptr[dev];
  }
  float* pv = (float*)ptr;
  int* pi = (int*)ptr + (size_t)n_rows * ARG_PARTS;
  argmax_part_kernel<<<dim3(n_rows, ARG_PARTS), 256, 0, stream>>>(logits, pv, pi, V);
  argmax_final_kernel<<<n_rows, 64, 0, stream>>>(pv, pi, out);
  TI_LAUNCH_CHECK();
  return 0;
}

extern "C" int ti_sample(const float* logits, const float* temp, const int* top_k, const float* top_p,
                         const float* uni, int* out, int n_rows, int V, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && V > 0, "sample: bad sizes rows=%d V=%d", n_rows, V);
  if (n_rows == 0) return 0;
  sample_kernel<<<n_rows, SNT, 0, stream>>>(logits, temp, top_k, top_p, uni, out, V);
  TI_LAUNCH_CHECK();
  return 0;
}
