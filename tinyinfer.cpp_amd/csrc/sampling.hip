// Sampling on the device: greedy argmax (of equal logits the lowest index wins,
// as /root/reference/src/cuda/sample.cu:5-11) and temperature sampling with
// optional top-k and top-p cuts (/root/reference/src/main.cpp:40-83 does these
// on the host with a sort).  One workgroup per row of logits.
//
// Temperature sampling draws by inverse CDF over the index order from one
// uniform number per row, which the host derives from (seed, request, number of
// tokens generated), so a draw does not depend on what else is in the batch.
// The cuts are the k-th largest logit and the logit at which the descending
// cumulative mass reaches top_p, both found on the order-preserving integer
// image of the floats: by radix with many workgroups a row where there is a
// top-k cut, else by 32 steps of bisection each in one workgroup.  Every sum is
// reduced in a fixed order, so the result is reproducible.
#include <algorithm>
#include <mutex>

#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define SNT 1024

__device__ __forceinline__ uint32_t order_key(float f) {
  uint32_t u = __float_as_uint(f);
  if (u == 0x80000000u) u = 0u;                  // -0 and +0 are equal logits
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
// One workgroup walks the whole row some seventy times: the way for the rows that the four short
// kernels below do not serve, and for a caller without their workspace.
__device__ void sample_row_by_bisection(const float* __restrict__ logits, const float* __restrict__ temp,
                                        const int* __restrict__ top_k, const float* __restrict__ top_p,
                                        const float* __restrict__ uni, int* __restrict__ out, int V, int r) {
  __shared__ float s_val[SNT / TI_WAVE];
  __shared__ int s_idx[SNT / TI_WAVE];
  __shared__ float s_chunk[SNT];
  __shared__ int s_pick;
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

__global__ void __launch_bounds__(SNT)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temp, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ uni, int* __restrict__ out, int V) {
  sample_row_by_bisection(logits, temp, top_k, top_p, uni, out, V, blockIdx.x);
}

// ------------------------------------------------------------ the same draw in four short kernels
// A row of 151,936 logits cut to its 512 largest: the kernel above takes 0.9 ms (1.8 with a top-p
// cut), as long as a whole decode step, because one workgroup reads the row once per bit of the
// answer.  Here the k-th largest key is found by radix and many workgroups share a row:
//   pass 0  counts the keys of a row by their upper 11 bits (counts in LDS first, then added to the
//           row's histogram in memory: sums of integers, the same in any order);
//   pass 1  finds the bin that holds the k-th largest and counts its keys by their next 11 bits;
//   pass 2  collects the keys at or above the 22-bit prefix that holds the k-th largest: the k - 1
//           above it and those that share its prefix (few: for logits between 16 and 32 a prefix
//           is 0.002 wide), as (key, index) pairs;
//   finish  one workgroup per row sorts the collected pairs by (logit down, index up), cuts at the
//           k-th key (equals stay), sums the weights in that order for the top-p cut, sorts what
//           is left by index and draws by inverse CDF.  Sums are scans of a fixed shape.
// It draws what the kernel above draws, up to the rounding of sums that are taken in another order.
// Rows that it does not serve (no top-k cut, a cut beyond S_MAX_K, more than S_CAND keys collected:
// thousands of equal logits at the cut) are left to that kernel's walk, inside the last kernel.
// The row's words of the workspace start at zero and are left at zero.
#define S_BINS 2048
#define S_CAND 4096                              // pairs a row may collect (and the finish sorts in LDS)
#define S_MAX_K 3584                             // the largest cut served: room for equals and prefix-mates
#define S_LOADS 8                                // loads of a thread that are under way at a time
#define S_STAGE 512                              // pairs a workgroup gathers in LDS before it asks for room
#define S_HEAD_WORDS (2 * S_BINS + 64)           // two histograms, the count of pairs, pass 1's bin (and padding)
#define S_ROW_WORDS (S_HEAD_WORDS + 2 * S_CAND)

__device__ __forceinline__ float key_value(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}
// the cut that the radix kernels find for row r: a greedy row is a cut to the largest key; 0: not served
__device__ __forceinline__ int served_cut(const float* temp, const int* top_k, int r, int V) {
  const int k = temp[r] > 0.f ? top_k[r] : 1;
  return (k > 0 && k < V && k <= S_MAX_K) ? k : 0;
}

// Which of the S_BINS bins holds the k-th largest key, and how many keys lie in the bins above it.  Every
// thread of the workgroup calls it (256 or more: thread t < 256 owns bins 8 t .. 8 t + 7) and gets both.
// k beyond the number of keys: the lowest bin that holds a key.  No keys: bin -1.
__device__ void bin_of_kth(const int* __restrict__ hist, int k, int* s_sum, int* s_above, int* s_res, int& bin, int& above) {
  const int t = threadIdx.x;
  const bool own = t < 256;
  int c[8], mine = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    c[j] = own ? hist[8 * t + j] : 0;
    mine += c[j];
  }
  if (own) s_sum[t] = mine;
  if (t == 0) s_res[0] = -1, s_res[1] = 0;
  __syncthreads();
  if (t < TI_WAVE) {
    int q[4], s4 = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      q[j] = s_sum[4 * t + j];
      s4 += q[j];
    }
    int suf = s4;                                  // keys of the owners that lanes >= t stand for
#pragma unroll
    for (int o = 1; o < TI_WAVE; o <<= 1) {
      const int v = __shfl_down(suf, o, TI_WAVE);
      if (t + o < TI_WAVE) suf += v;
    }
    int run = suf - s4;
#pragma unroll
    for (int j = 3; j >= 0; --j) {
      s_above[4 * t + j] = run;                    // keys in the bins of owners beyond 4 t + j
      run += q[j];
    }
    if (t == 0) s_above[256] = run;                // all keys
  }
  __syncthreads();
  const int total = s_above[256];
  const int kk = k < total ? k : total;
  if (own && kk >= 1) {
    int run = s_above[t];
#pragma unroll
    for (int j = 7; j >= 0; --j) {
      if (run < kk && run + c[j] >= kk) s_res[0] = 8 * t + j, s_res[1] = run;
      run += c[j];
    }
  }
  __syncthreads();
  bin = s_res[0];
  above = s_res[1];
  __syncthreads();
}

template <int PASS>
__global__ void __launch_bounds__(256)
sample_pass_kernel(const float* __restrict__ logits, const float* __restrict__ temp, const int* __restrict__ top_k,
                   int* __restrict__ scratch, int V) {
  __shared__ int s_hist[PASS == 2 ? 1 : S_BINS];
  __shared__ unsigned long long s_stage[PASS == 2 ? S_STAGE : 1];
  __shared__ int s_sum[256], s_above[257], s_res[2], s_count, s_base;
  const int r = blockIdx.y;
  const int k = served_cut(temp, top_k, r, V);
  if (k == 0) return;                              // the whole workgroup
  const float* row = logits + (size_t)r * V;
  int* hist1 = scratch + (size_t)r * S_ROW_WORDS;
  int* hist2 = hist1 + S_BINS;
  int* n_cand = hist2 + S_BINS;
  unsigned long long* cand = reinterpret_cast<unsigned long long*>(hist1 + S_HEAD_WORDS);
  int b1 = 0, above1 = 0, b2 = 0, above2 = 0;
  if (PASS == 1) {
    bin_of_kth(hist1, k, s_sum, s_above, s_res, b1, above1);
    if (blockIdx.x == 0 && threadIdx.x == 0) n_cand[1] = b1, n_cand[2] = above1;   // pass 2 need not look again
    if (b1 < 0) return;                            // a row of NaN
  }
  if (PASS == 2) {
    b1 = n_cand[1];
    above1 = n_cand[2];
    if (b1 < 0) return;
    bin_of_kth(hist2, k - above1, s_sum, s_above, s_res, b2, above2);
    if (b2 < 0) return;
    if (threadIdx.x == 0) s_count = 0;
    __syncthreads();
  } else {
    for (int i = threadIdx.x; i < S_BINS; i += 256) s_hist[i] = 0;
    __syncthreads();
  }
  const uint32_t prefix = ((uint32_t)b1 << 11) | (uint32_t)b2;
  // S_LOADS loads are under way at a time: one load a turn leaves a wavefront waiting for memory 37 times over
  for (int base = blockIdx.x * (256 * S_LOADS) + threadIdx.x; base < V; base += gridDim.x * (256 * S_LOADS)) {
    float v[S_LOADS];
#pragma unroll
    for (int u = 0; u < S_LOADS; ++u) v[u] = base + 256 * u < V ? row[base + 256 * u] : __uint_as_float(0x7fc00000u);
#pragma unroll
    for (int u = 0; u < S_LOADS; ++u) {
      if (!(v[u] == v[u])) continue;               // NaN is never drawn
      const int i = base + 256 * u;
      const uint32_t key = order_key(v[u]);
      if (PASS == 0) {
        atomicAdd(&s_hist[key >> 21], 1);
      } else if (PASS == 1) {
        if ((key >> 21) == (uint32_t)b1) atomicAdd(&s_hist[(key >> 10) & (S_BINS - 1)], 1);
      } else if ((key >> 10) >= prefix) {
        const unsigned long long pair = ((unsigned long long)key << 32) | (uint32_t)~i;
        const int at = atomicAdd(&s_count, 1);
        if (at < S_STAGE) {
          s_stage[at] = pair;
        } else {                                   // more than the stage holds: one by one
          const int g = atomicAdd(n_cand, 1);
          if (g < S_CAND) cand[g] = pair;
        }
      }
    }
  }
  __syncthreads();
  if (PASS == 2) {
    const int mine = min(s_count, S_STAGE);
    if (threadIdx.x == 0 && mine > 0) s_base = atomicAdd(n_cand, mine);
    __syncthreads();
    for (int i = threadIdx.x; i < mine; i += 256)
      if (s_base + i < S_CAND) cand[s_base + i] = s_stage[i];
  } else {
    int* hist = PASS == 0 ? hist1 : hist2;
    for (int i = threadIdx.x; i < S_BINS; i += 256)
      if (s_hist[i]) atomicAdd(&hist[i], s_hist[i]);
  }
}

// sorts a[0..n) of LDS downwards by the entries' upper words, n <= S_CAND; every thread of the workgroup
// calls it.  Up to S_BY_RANK entries each thread counts the entries above its own and puts it there (n reads
// that the whole wavefront shares, a compare and an add each, no barrier between them); entries with equal
// upper words take neighbouring places in the order in which they come.  More entries are sorted by a
// bitonic network on the whole entries, a barrier a stage.  tmp: room for S_BY_RANK entries and as many counters.
#define S_BY_RANK 1024
__device__ void sort_down(unsigned long long* a, int n, unsigned long long* tmp) {
  if (n <= S_BY_RANK) {
    int* taken = reinterpret_cast<int*>(tmp + S_BY_RANK);
    const int i = threadIdx.x;
    if (i < n) taken[i] = 0;
    __syncthreads();
    if (i < n) {
      const unsigned long long x = a[i];
      const uint32_t mine = (uint32_t)(x >> 32);
      int above = 0;
      for (int j = 0; j < n; ++j) above += (uint32_t)(a[j] >> 32) > mine ? 1 : 0;
      tmp[above + atomicAdd(&taken[above], 1)] = x;
    }
    __syncthreads();
    if (i < n) a[i] = tmp[i];
    __syncthreads();
    return;
  }
  int p2 = 1;
  while (p2 < n) p2 <<= 1;
  for (int i = n + threadIdx.x; i < p2; i += SNT) a[i] = 0ull;     // below every pair
  __syncthreads();
  for (int size = 2; size <= p2; size <<= 1)
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = threadIdx.x; t < p2 / 2; t += SNT) {
        const int lo = ((t & ~(stride - 1)) << 1) | (t & (stride - 1)), hi = lo + stride;
        const bool down = (lo & size) == 0;
        const unsigned long long x = a[lo], y = a[hi];
        if ((x < y) == down) {
          a[lo] = y;
          a[hi] = x;
        }
      }
      __syncthreads();
    }
}

// running sums of w[0..n), n <= 4 SNT, in place (each entry's sum includes it); returns the sum of all.
// Thread t owns entries 4 t .. 4 t + 3; a wavefront scans its threads' sums with shuffles, the wavefronts'
// totals are added in order.
__device__ float scan_in_place(float* w, int n, float* s_wave) {
  const int t = threadIdx.x, lane = t & (TI_WAVE - 1), wave = t / TI_WAVE;
  float e[4], local = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    e[j] = 4 * t + j < n ? w[4 * t + j] : 0.f;
    local += e[j];
  }
  float run = local;
#pragma unroll
  for (int o = 1; o < TI_WAVE; o <<= 1) {
    const float v = __shfl_up(run, o, TI_WAVE);
    if (lane >= o) run += v;
  }
  const float upto = __shfl_up(run, 1, TI_WAVE);
  __syncthreads();
  if (lane == TI_WAVE - 1) s_wave[wave] = run;
  __syncthreads();
  float acc = 0.f, total = 0.f;
  for (int i = 0; i < SNT / TI_WAVE; ++i) {
    if (i == wave) acc = total;
    total += s_wave[i];
  }
  if (lane > 0) acc += upto;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    acc += e[j];
    if (4 * t + j < n) w[4 * t + j] = acc;
  }
  __syncthreads();
  return total;
}

// how many of the pairs a[0..n), sorted downwards by key, have a key of at least `key` (a[0] has)
__device__ int pairs_at_least(const unsigned long long* a, int n, uint32_t key, int* s_n) {
  for (int i = threadIdx.x; i < n; i += SNT)
    if ((uint32_t)(a[i] >> 32) >= key && (i + 1 == n || (uint32_t)(a[i + 1] >> 32) < key)) *s_n = i + 1;
  __syncthreads();
  const int m = *s_n;
  __syncthreads();
  return m;
}

__global__ void __launch_bounds__(SNT)
sample_finish_kernel(const float* __restrict__ logits, const float* __restrict__ temp, const int* __restrict__ top_k,
                     const float* __restrict__ top_p, const float* __restrict__ uni, int* __restrict__ out,
                     int* __restrict__ scratch, int V) {
  __shared__ unsigned long long s_pair[S_CAND];
  __shared__ float s_w[S_CAND];
  __shared__ float s_wave[SNT / TI_WAVE];
  __shared__ int s_n, s_at;
  const int r = blockIdx.x;
  const int k = served_cut(temp, top_k, r, V);
  if (k == 0) {
    sample_row_by_bisection(logits, temp, top_k, top_p, uni, out, V, r);
    return;
  }
  const float T = temp[r], p_keep = top_p[r], u = uni[r];
  int* head = scratch + (size_t)r * S_ROW_WORDS;
  const unsigned long long* cand = reinterpret_cast<const unsigned long long*>(head + S_HEAD_WORDS);
  const int n = head[2 * S_BINS];
  if (threadIdx.x == 0) s_at = 0x7fffffff;
  __syncthreads();                                 // every thread has the count: now the row's words go back to zero
  for (int i = threadIdx.x; i < S_HEAD_WORDS; i += SNT) head[i] = 0;
  if (n > S_CAND) {
    sample_row_by_bisection(logits, temp, top_k, top_p, uni, out, V, r);
    return;
  }
  if (n == 0) {                                    // a row of NaN
    if (threadIdx.x == 0) out[r] = 0;
    return;
  }
  for (int i = threadIdx.x; i < n; i += SNT) s_pair[i] = cand[i];
  __syncthreads();
  sort_down(s_pair, n, reinterpret_cast<unsigned long long*>(s_w));                            // by key
  if (!(T > 0.f)) {                                // of equal logits the lowest index
    const uint32_t top = (uint32_t)(s_pair[0] >> 32);
    for (int i = threadIdx.x; i < n; i += SNT)
      if ((uint32_t)(s_pair[i] >> 32) == top) atomicMin(&s_at, (int)~(uint32_t)s_pair[i]);
    __syncthreads();
    if (threadIdx.x == 0) out[r] = s_at;
    return;
  }
  int m = pairs_at_least(s_pair, n, (uint32_t)(s_pair[min(k, n) - 1] >> 32), &s_n);
  const float mx = key_value((uint32_t)(s_pair[0] >> 32));
  const float inv_t = 1.0f / T;
  if (p_keep < 1.0f) {
    for (int i = threadIdx.x; i < m; i += SNT) s_w[i] = expf((key_value((uint32_t)(s_pair[i] >> 32)) - mx) * inv_t);
    __syncthreads();
    const float need = p_keep * scan_in_place(s_w, m, s_wave);
    for (int i = threadIdx.x; i < m; i += SNT)
      if (s_w[i] >= need) atomicMin(&s_at, i);
    __syncthreads();
    const int j = s_at;                            // the first pair at which the mass from the top reaches need
    __syncthreads();
    if (threadIdx.x == 0) s_at = 0x7fffffff;
    if (j < m) m = pairs_at_least(s_pair, m, (uint32_t)(s_pair[j] >> 32), &s_n);   // its equals stay
    else __syncthreads();
  }
  // what is left, in the order of the indices
  for (int i = threadIdx.x; i < m; i += SNT) {
    const unsigned long long pr = s_pair[i];
    s_pair[i] = (pr << 32) | (pr >> 32);           // (~index, key)
  }
  __syncthreads();
  sort_down(s_pair, m, reinterpret_cast<unsigned long long*>(s_w));
  for (int i = threadIdx.x; i < m; i += SNT) s_w[i] = expf((key_value((uint32_t)s_pair[i]) - mx) * inv_t);
  __syncthreads();
  const float target = u * scan_in_place(s_w, m, s_wave);
  for (int i = threadIdx.x; i < m; i += SNT)
    if (target < s_w[i]) atomicMin(&s_at, i);
  __syncthreads();
  if (threadIdx.x == 0) {
    const int at = s_at < m ? s_at : m - 1;        // rounding pushed the target past the end: the last one kept
    out[r] = (int)~(uint32_t)(s_pair[at] >> 32);
  }
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

extern "C" long ti_sample_scratch_bytes(int n_rows) { return (long)n_rows * S_ROW_WORDS * 4; }

// scratch: ti_sample_scratch_bytes(n_rows) bytes that were zero before the first call and that only calls of
// this function (one at a time) have touched since, or nullptr (then one workgroup walks a whole row)
extern "C" int ti_sample(const float* logits, const float* temp, const int* top_k, const float* top_p,
                         const float* uni, int* out, void* scratch, int n_rows, int V, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && V > 0, "sample: bad sizes rows=%d V=%d", n_rows, V);
  if (n_rows == 0) return 0;
  if (!scratch) {
    sample_kernel<<<n_rows, SNT, 0, stream>>>(logits, temp, top_k, top_p, uni, out, V);
  } else {
    const int most = n_rows <= 8 ? 80 : (n_rows <= 32 ? 32 : 16), span = 256 * S_LOADS;
    const dim3 grid(std::min(most, (V + span - 1) / span), n_rows);
    sample_pass_kernel<0><<<grid, 256, 0, stream>>>(logits, temp, top_k, (int*)scratch, V);
    sample_pass_kernel<1><<<grid, 256, 0, stream>>>(logits, temp, top_k, (int*)scratch, V);
    sample_pass_kernel<2><<<grid, 256, 0, stream>>>(logits, temp, top_k, (int*)scratch, V);
    sample_finish_kernel<<<n_rows, SNT, 0, stream>>>(logits, temp, top_k, top_p, uni, out, (int*)scratch, V);
  }
  TI_LAUNCH_CHECK();
  return 0;
}
