// bfloat16 matrix products C = A W^T on the matrix cores of gfx950, 32-bit
// accumulation.  A is [M, K] (row stride lda), W is [N, K], both bfloat16 with K
// contiguous, which is the natural operand layout of MFMA for both sides.
//
// Two kernels:
//  * skinny (M <= 64, decode and small portions): every weight element is read
//    from memory exactly once per call.  A workgroup of four wavefronts owns 16
//    weight rows; the wavefronts split K between them in interleaved 128-byte
//    pieces and reduce through LDS in a fixed order.  The weights are the "A"
//    operand of v_mfma_f32_16x16x32_bf16, the tokens are the 16 columns.
//  * tiled (M > 64, prefill): 128 x 128 x 32 tiles through double-buffered LDS,
//    four wavefronts in 2 x 2, each 64 x 64 out of v_mfma_f32_32x32x16_bf16.
//
// Epilogues: store float, add into a float residual, store bfloat16, or SwiGLU
// over a stacked [gate; up] weight.  The reduction order of an output element
// never depends on M within one kernel.  (The reference's two products are
// /root/reference/src/cuda/gemm.cu:37-85 and 152-261; it reads the weights once
// per row of A for M <= 32.)
#include <algorithm>
#include <string>
#include "common.h"
#include "tinyinfer_kernels.h"
#include "tinyinfer_kernels_tuning.h"
#include "qk_prep.h"

TI_ERROR_API

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

typedef unsigned v4u __attribute__((ext_vector_type(4)));

union Frag {
  uint4 u;
  bf16x8 v;
};

__device__ __forceinline__ uint4 ld16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + __expf(-g)) * u; }

// ============================================================== skinny kernel
// grid.x = ceil(N / 16) (SwiGLU: ceil(F / 8): 8 gate rows and their 8 up rows).
// NW wavefronts split K between them.
// UN: 64-element chunks of K a wavefront has in flight at a time.  All loads of a pass are
// issued before the first product: out-of-range pieces read a valid address (piece 0 of the
// row) and get a zeroed weight instead of a branch, so that nothing waits in between.
template <int MT, int EPI, int NW = 4, int UN = 4>
__global__ void __launch_bounds__(NW * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ out_,
                   int M, int N, int K, long lda) {
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  __shared__ float red[NW][MT][16][17];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, j = lane >> 4;   // MFMA row / column, and k group
  // the weight row this lane feeds
  int wrow;
  if (SW) {
    const int n = blockIdx.x * 8 + (r & 7);
    wrow = (r < 8 ? 0 : N) + (n < N ? n : N - 1);
  } else {
    const int n = blockIdx.x * 16 + r;
    wrow = n < N ? n : N - 1;
  }
  const bf16_t* wp = W + (size_t)wrow * K;
  const bf16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    ap[t] = A + (size_t)(m < M ? m : 0) * lda;   // columns beyond M are computed from row 0 and never stored
  }
  // the residual this thread will add to, asked for before the product
  const int tok = threadIdx.x >> 4, row = threadIdx.x & 15;
  float prev[MT];
  if (EPI == TI_EPI_ADD_F32) {   // threads without an output element read a valid one: no branch
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + (tok & 15), n = blockIdx.x * 16 + row;
      prev[t] = ((const float*)out_)[(size_t)(m < M ? m : 0) * N + (n < N ? n : N - 1)];
    }
  }
  floatx4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const uint4 zero = make_uint4(0, 0, 0, 0);
  // chunk c covers k in [64 c, 64 c + 64); lane group j takes [64 c + 16 j, +16)
  const int chunks = (K + 63) / 64;
  for (int c0 = wave; c0 < chunks; c0 += NW * UN) {
    Frag w0[UN], w1[UN], a0[UN][MT], a1[UN][MT];
    bool ok0[UN], ok1[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = (c0 + NW * u) * 64 + j * 16;
      ok0[u] = k + 8 <= K;    // false too for chunks beyond the last
      ok1[u] = k + 16 <= K;
      w0[u].u = ld16(wp + (ok0[u] ? k : 0));
      w1[u].u = ld16(wp + (ok1[u] ? k + 8 : 0));
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = (c0 + NW * u) * 64 + j * 16;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        a0[u][t].u = ld16(ap[t] + (ok0[u] ? k : 0));
        a1[u][t].u = ld16(ap[t] + (ok1[u] ? k + 8 : 0));
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // every load above is issued before the first product waits
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (!ok0[u]) w0[u].u = zero;
      if (!ok1[u]) w1[u].u = zero;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u].v, a0[u][t].v, acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u].v, a1[u][t].v, acc[t], 0, 0, 0);
      }
    }
  }
  // acc[t][i]: weight row 4 j + i, token 16 t + r
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t][r][4 * j + i] = acc[t][i];
  __syncthreads();
  // thread -> (token = tid / 16, row = tid % 16): consecutive threads, consecutive columns
  if (NW > 4 && threadIdx.x >= 256) return;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + tok;
    if (m >= M) continue;
    if (SW) {
      if (row >= 8) continue;
      const int n = blockIdx.x * 8 + row;
      if (n >= N) continue;
      float g = 0.f, u = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        g += red[w][t][tok][row];
        u += red[w][t][tok][row + 8];
      }
      ((bf16_t*)out_)[(size_t)m * N + n] = f2bf(silu_mul(g, u));
    } else {
      const int n = blockIdx.x * 16 + row;
      if (n >= N) continue;
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) s += red[w][t][tok][row];
      const size_t o = (size_t)m * N + n;
      if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = s;
      if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] = prev[t] + s;
      if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(s);
    }
  }
}

// ================================== skinny kernel whose token rows are made in the kernel
// out = rows W^T for M <= 16 tokens, where the rows do not exist in memory yet: a producer
// makes them, as bfloat16 in LDS, in every workgroup for itself.  The rows are few and what
// they are made from lies in the cache; the first weight loads are already under way while
// the producer runs; and it costs no launch of its own.  The rounding to bfloat16 is the
// one every product operand gets, so the result equals that of the producer's own kernel
// followed by the plain product.
//
// A producer has `template <int NW> __device__ void fill(bf16_t* sA, int lda, int M, int K)`,
// called by all NW * 64 threads, writing sA[m * lda + k]; the kernel synchronizes after it.

// RMSNorm of float rows X [M, K] with weight Gw [K].  KC: float4 pieces of a row each lane
// holds (K <= 256 KC).  Wavefront w takes rows w, w + NW, ...; two rows' loads are issued
// together where the registers allow; a lane's pieces beyond K read piece 0 and are left
// out of the sum and the store.
template <int KC>
struct NormProducer {
  const float* X;
  const float* Gw;
  float eps;
  template <int NW, class IssueWeights>
  __device__ __forceinline__ void fill(bf16_t* sA, int lda, int M, int K, IssueWeights issue_weights) const {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int RB = KC <= 8 ? 2 : 1;
    float4 g[KC], v[RB][KC];
    auto load_rows = [&](int r0) {
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        const int m = r0 + NW * b < M ? r0 + NW * b : (r0 < M ? r0 : 0);
        const float* xr = X + (size_t)m * K;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
          const int k = lane * 4 + 256 * c;
          v[b][c] = *reinterpret_cast<const float4*>(xr + (k < K ? k : 0));
        }
      }
    };
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int k = lane * 4 + 256 * c;
      g[c] = *reinterpret_cast<const float4*>(Gw + (k < K ? k : 0));
    }
    load_rows(wave);
    // loads come back in the order they were issued: the rows (from the cache) before the
    // weights (from memory), so the norm does not wait for the weights
    __builtin_amdgcn_sched_barrier(0);
    issue_weights();
    __builtin_amdgcn_sched_barrier(0);
    for (int r0 = wave; r0 < M; r0 += NW * RB) {
      if (r0 != wave) load_rows(r0);
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        const int m = r0 + NW * b;
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < KC; ++c)
          if (lane * 4 + 256 * c < K) ss = rms_accumulate(ss, v[b][c]);
        const float scale = rms_scale(ss, K, eps);
        if (m < M) {
#pragma unroll
          for (int c = 0; c < KC; ++c) {
            const int k = lane * 4 + 256 * c;
            if (k < K) {
              const uint2 hb = make_uint2(pack_bf16x2(v[b][c].x * scale * g[c].x, v[b][c].y * scale * g[c].y),
                                          pack_bf16x2(v[b][c].z * scale * g[c].z, v[b][c].w * scale * g[c].w));
              *reinterpret_cast<uint2*>(sA + (size_t)m * lda + k) = hb;
            }
          }
        }
      }
    }
  }
};

// Rows that do exist in memory (bfloat16 [M, K], row stride lda): copied into LDS once per
// workgroup, 16 bytes per thread and load, instead of every wavefront fetching its token
// fragments from memory with one load instruction per fragment (for one token fifteen of
// sixteen lanes of such a load repeat a row): a compute unit takes a load instruction of 64
// lanes every 16 cycles or so, and the kernel for few tokens is bound by that.
struct CopyProducer {
  const bf16_t* A;
  long lda;
  template <int NW, class IssueWeights>
  __device__ __forceinline__ void fill(bf16_t* sA, int lds_stride, int M, int K, IssueWeights issue_weights) const {
    constexpr int NT = NW * 64, PB = 8;
    const int kp = K >> 3, pieces = M * kp;
    bool first = true;
    for (int p0 = threadIdx.x; first || p0 < pieces; p0 += NT * PB) {
      uint4 v[PB];
      int dst[PB];
      bool ok[PB];
#pragma unroll
      for (int b = 0; b < PB; ++b) {
        const int p = p0 + NT * b;
        ok[b] = p < pieces;
        const int pc = ok[b] ? p : 0;
        const int m = pc / kp, k8 = pc - m * kp;
        v[b] = ld16(A + (size_t)m * lda + k8 * 8);
        dst[b] = m * lds_stride + k8 * 8;
      }
      if (first) {
        __builtin_amdgcn_sched_barrier(0);
        issue_weights();
        __builtin_amdgcn_sched_barrier(0);
        first = false;
      }
#pragma unroll
      for (int b = 0; b < PB; ++b)
        if (ok[b]) *reinterpret_cast<uint4*>(sA + dst[b]) = v[b];
    }
  }
};

template <class Producer, int EPI, int NW, int UN = 4>
__global__ void __launch_bounds__(NW * 64)
gemm_skinny_staged_kernel(Producer producer, const bf16_t* __restrict__ W, void* __restrict__ out_, int M, int N,
                          int K) {
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_smem[];
  bf16_t* sA = reinterpret_cast<bf16_t*>(dyn_smem);          // [M][K + 8]
  __shared__ float red[NW][16][17];
  const int lda = K + 8;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, j = lane >> 4;
  int wrow;
  if (SW) {
    const int n = blockIdx.x * 8 + (r & 7);
    wrow = (r < 8 ? 0 : N) + (n < N ? n : N - 1);
  } else {
    const int n = blockIdx.x * 16 + r;
    wrow = n < N ? n : N - 1;
  }
  const bf16_t* wp = W + (size_t)wrow * K + j * 16;
  const uint4 zero = make_uint4(0, 0, 0, 0);
  const int chunks = K / 64;

  // the residual this thread will add to
  const int tok = threadIdx.x >> 4, row = threadIdx.x & 15;   // tok >= 16 for the wavefronts beyond four
  float prev = 0.f;
  if (EPI == TI_EPI_ADD_F32) {   // threads without an output element read a valid one: no branch
    const int n = blockIdx.x * 16 + row;
    prev = ((const float*)out_)[(size_t)(tok < M ? tok : 0) * N + (n < N ? n : N - 1)];
  }

  // the first weights of this wavefront: the producer asks for them right after its own first
  // loads, so that they are on their way while the rows are made.  A chunk beyond the last
  // reads chunk 0 and is zeroed afterwards: no branch between the loads.
  Frag w0[UN], w1[UN];
  auto issue_weights = [&]() {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int c = wave + NW * u < chunks ? wave + NW * u : 0;
      w0[u].u = ld16(wp + (size_t)c * 64);
      w1[u].u = ld16(wp + (size_t)c * 64 + 8);
    }
  };
  producer.template fill<NW>(sA, lda, M, K, issue_weights);
  __syncthreads();

  // ---- the product, as in the plain skinny kernel with the token fragments from LDS
  const bf16_t* ap = sA + (size_t)(r < M ? r : 0) * lda + j * 16;
  floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int c0 = wave; c0 < chunks; c0 += NW * UN) {
    if (c0 != wave) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int c = c0 + NW * u < chunks ? c0 + NW * u : 0;
        w0[u].u = ld16(wp + (size_t)c * 64);
        w1[u].u = ld16(wp + (size_t)c * 64 + 8);
      }
    }
    Frag a0[UN], a1[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int c = c0 + NW * u < chunks ? c0 + NW * u : 0;
      a0[u].u = ld16(ap + (size_t)c * 64);
      a1[u].u = ld16(ap + (size_t)c * 64 + 8);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (c0 + NW * u >= chunks) w0[u].u = w1[u].u = zero;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u].v, a0[u].v, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u].v, a1[u].v, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][r][4 * j + i] = acc[i];
  __syncthreads();
  if (tok >= M) return;
  if (SW) {
    if (row >= 8) return;
    const int n = blockIdx.x * 8 + row;
    if (n >= N) return;
    float gt = 0.f, up = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      gt += red[w][tok][row];
      up += red[w][tok][row + 8];
    }
    ((bf16_t*)out_)[(size_t)tok * N + n] = f2bf(silu_mul(gt, up));
  } else {
    const int n = blockIdx.x * 16 + row;
    if (n >= N) return;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += red[w][tok][row];
    const size_t o = (size_t)tok * N + n;
    if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = sum;
    if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] = prev + sum;
    if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(sum);
  }
}

// ================================== few tokens, any K: the token rows in pieces, loads never at rest
// out (op)= A W^T for M <= 16, K a multiple of 64.  As in the kernels above a workgroup of four
// wavefronts owns 16 weight rows, wavefront w takes the 64-wide chunks w, w + 4, ... of K, and the
// four sums meet in LDS in the order 0..3: with one workgroup per 16 rows the bits are those of
// the kernels above.  Two things differ.
//  * The token rows go through LDS in pieces of SP_PIECE columns, two buffers in turn: any K fits,
//    and any M <= 16 leaves room for two workgroups or more on a compute unit.
//  * While a piece is multiplied, the weights and the token rows of the next one are already on
//    their way: a wavefront always has 8 to 16 KB of weights in flight, where the kernels above
//    ask for a batch, wait for all of it, multiply, and only then ask again.  On weights of tens
//    to hundreds of megabytes that is the difference between ~3.5 and ~5.5 TB/s.
// grid (ceil(N / 16), KS) (SwiGLU: ceil(F / 8)).  KS > 1 (adding epilogue only): workgroup
// (., s) takes the pieces s, s + KS, ... and leaves its sums in partial [KS][M][N]; they are
// added to the residual in the order 0..KS-1 by whoever reads it next.
#define SP_PIECE 1024              // 16 chunks: four per wavefront, one batch of loads
#define SP_LD (SP_PIECE + 8)       // LDS row stride in bfloat16
// AV: 16-byte pieces of the token rows per thread and piece (M <= 2 AV)
template <int EPI, int AV, bool SPLIT>
__global__ void __launch_bounds__(256)
gemm_skinny_pieces_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, void* __restrict__ out_,
                          float* __restrict__ partial, int M, int N, int K) {
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_smem[];
  bf16_t* sA = reinterpret_cast<bf16_t*>(dyn_smem);          // [2][M][SP_LD]
  __shared__ float red[4][16][17];
  constexpr int NT = 256;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, j = lane >> 4;
  const int tile = blockIdx.x;               // 16 rows (SwiGLU: 8 gate and 8 up rows)
  int wrow;
  if (SW) {
    const int n = tile * 8 + (r & 7);
    wrow = (r < 8 ? 0 : N) + (n < N ? n : N - 1);
  } else {
    const int n = tile * 16 + r;
    wrow = n < N ? n : N - 1;
  }
  const bf16_t* wp = W + (size_t)wrow * K + j * 16;
  const int chunks = K / 64;
  const int n_pieces = (K + SP_PIECE - 1) / SP_PIECE;
  const int KS = SPLIT ? gridDim.y : 1, split = SPLIT ? blockIdx.y : 0;

  const int tok = threadIdx.x >> 4, row = threadIdx.x & 15;
  float prev = 0.f;
  if (EPI == TI_EPI_ADD_F32 && !SPLIT) {   // threads without an output element read a valid one: no branch
    const int n = tile * 16 + row;
    prev = ((const float*)out_)[(size_t)(tok < M ? tok : 0) * N + (n < N ? n : N - 1)];
  }

  // piece p: thread t copies the 16-byte pieces t, t + NT, ... of [M][SP_PIECE / 8]
  uint4 av[AV];
  auto ask_rows = [&](int p) {
#pragma unroll
    for (int b = 0; b < AV; ++b) {
      const int v = threadIdx.x + NT * b;
      const int m = v / (SP_PIECE / 8), k = p * SP_PIECE + (v % (SP_PIECE / 8)) * 8;
      const bool ok = m < M && k < K;
      av[b] = ld16(A + (ok ? (size_t)m * lda + k : 0));
    }
  };
  auto keep_rows = [&](int buf) {
#pragma unroll
    for (int b = 0; b < AV; ++b) {
      const int v = threadIdx.x + NT * b;
      const int m = v / (SP_PIECE / 8);
      if (m < M) *reinterpret_cast<uint4*>(sA + ((size_t)buf * M + m) * SP_LD + (v % (SP_PIECE / 8)) * 8) = av[b];
    }
  };
  // a chunk beyond the last reads chunk 0 and counts for nothing: no branch between the loads
  auto ask_weights = [&](int p, Frag (&w0)[4], Frag (&w1)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = p * (SP_PIECE / 64) + wave + 4 * u;
      const size_t at = (size_t)(c < chunks ? c : 0) * 64;
      w0[u].u = ld16(wp + at);
      w1[u].u = ld16(wp + at + 8);
    }
  };
  floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  auto multiply = [&](int p, int buf, Frag (&w0)[4], Frag (&w1)[4]) {
    const bf16_t* ap = sA + ((size_t)buf * M + (r < M ? r : 0)) * SP_LD + j * 16;
    Frag a0[4], a1[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      a0[u].u = *reinterpret_cast<const uint4*>(ap + (wave + 4 * u) * 64);
      a1[u].u = *reinterpret_cast<const uint4*>(ap + (wave + 4 * u) * 64 + 8);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (p * (SP_PIECE / 64) + wave + 4 * u >= chunks) w0[u].u = w1[u].u = zero;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u].v, a0[u].v, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u].v, a1[u].v, acc, 0, 0, 0);
    }
  };
  // one turn: piece p is multiplied out of `buf` and (w0, w1) while piece p + KS arrives in the
  // other buffer and (n0, n1).  Loads return in the order they were asked for: the rows of the
  // next piece are asked for before its weights, so that keeping them waits for nothing else.
  auto turn = [&](int p, int buf, Frag (&w0)[4], Frag (&w1)[4], Frag (&n0)[4], Frag (&n1)[4]) {
    const bool more = p + KS < n_pieces;
    if (more) {
      ask_rows(p + KS);
      __builtin_amdgcn_sched_barrier(0);
      ask_weights(p + KS, n0, n1);
      __builtin_amdgcn_sched_barrier(0);
    }
    multiply(p, buf, w0, w1);
    if (more) keep_rows(buf ^ 1);
    __syncthreads();
  };
  Frag wa0[4], wa1[4], wb0[4], wb1[4];
  int p = split;
  if (p < n_pieces) {
    ask_rows(p);
    __builtin_amdgcn_sched_barrier(0);
    ask_weights(p, wa0, wa1);
    __builtin_amdgcn_sched_barrier(0);
    keep_rows(0);
  }
  __syncthreads();
  while (p < n_pieces) {
    turn(p, 0, wa0, wa1, wb0, wb1);
    p += KS;
    if (p >= n_pieces) break;
    turn(p, 1, wb0, wb1, wa0, wa1);
    p += KS;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][r][4 * j + i] = acc[i];
  __syncthreads();
  if (tok >= M) return;
  if (SW) {
    if (row >= 8) return;
    const int n = tile * 8 + row;
    if (n >= N) return;
    float gt = 0.f, up = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      gt += red[w][tok][row];
      up += red[w][tok][row + 8];
    }
    ((bf16_t*)out_)[(size_t)tok * N + n] = f2bf(silu_mul(gt, up));
  } else {
    const int n = tile * 16 + row;
    if (n >= N) return;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) sum += red[w][tok][row];
    const size_t o = (size_t)tok * N + n;
    if (SPLIT) partial[(size_t)split * M * N + o] = sum;
    else if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = sum;
    else if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] = prev + sum;
    else if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(sum);
  }
}

// ================================== few tokens, a weight of few rows: a row per wavefront
// out (op)= A W^T for M <= MMAX tokens and a weight with so few rows that the kernels above,
// whose workgroups own 16 rows each, would leave most compute units idle (N = 1024: 64
// workgroups), while each busy unit would have hundreds of load instructions to get through
// (a unit takes one 64-lane load every ~25 cycles: measured 2.7 us to issue 256 of them).
// Here a wavefront owns one weight row: lane l holds the 8-element pieces l, l + 64, ... of
// it (every load instruction fetches 1 KiB that nobody else fetches), the token rows are
// copied into LDS once per workgroup, the products are v_dot2c_f32_bf16 (two multiply-adds
// on packed bfloat16, accumulated in 32-bit), and the lanes' partial sums meet in a
// butterfly.  N / 4 workgroups of four wavefronts.  A row's bits do not depend on the rows
// beside it.  K a multiple of 8, up to 512 NL (NL: pieces of the weight row per lane); MMAX: the
// most tokens.  Both are template parameters so that every load is unconditional and counted.
#define GR_LOADS 8
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(unsigned a, unsigned b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}

template <int EPI, int MMAX, int NL>
__global__ void __launch_bounds__(256)
gemv_rows_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ out_, int M, int N,
                 int K, long lda) {
  static_assert(EPI != TI_EPI_SWIGLU, "no SwiGLU here");
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_smem[];
  bf16_t* sA = reinterpret_cast<bf16_t*>(dyn_smem);          // [M][K]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + wave;
  const bf16_t* wp = W + (size_t)(n < N ? n : N - 1) * K;
  const uint4 zero = make_uint4(0, 0, 0, 0);

  // the residual lane m will add to (row m of the tokens): asked for first
  float prev = 0.f;
  if (EPI == TI_EPI_ADD_F32) prev = ((const float*)out_)[(size_t)(lane < M ? lane : 0) * N + (n < N ? n : N - 1)];
  // the token rows (from the cache), 16 bytes per thread and load, all in flight at once; then
  // this wavefront's weight row (from memory).  Loads come back in the order they were issued.
  constexpr int PB = (MMAX * NL + 3) / 4;                     // pieces per thread: all of [MMAX][512 NL]
  const int kp = K >> 3, pieces = M * kp;
  uint4 av[PB];
#pragma unroll
  for (int b = 0; b < PB; ++b) {
    const int p = threadIdx.x + 256 * b;
    const int pc = p < pieces ? p : 0;
    const int m = pc / kp, k8 = pc - m * kp;
    av[b] = ld16(A + (size_t)m * lda + k8 * 8);
  }
  __builtin_amdgcn_sched_barrier(0);
  uint4 wv[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int kk = (i * 64 + lane) * 8;
    wv[i] = ld16(wp + (kk < K ? kk : 0));
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int b = 0; b < PB; ++b) {
    const int p = threadIdx.x + 256 * b;
    if (p < pieces) {
      const int m = p / kp, k8 = p - m * kp;
      *reinterpret_cast<uint4*>(sA + (size_t)m * K + k8 * 8) = av[b];
    }
  }
  __syncthreads();

  // rows beyond M repeat row 0 and are dropped: all LDS reads of a piece go out together
  float acc[MMAX];
#pragma unroll
  for (int m = 0; m < MMAX; ++m) acc[m] = 0.f;
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int kk = (i * 64 + lane) * 8;
    const bool ok = kk < K;
    const uint4 w = ok ? wv[i] : zero;
    const bf16_t* ap = sA + (ok ? kk : 0);
    uint4 a[MMAX];
#pragma unroll
    for (int m = 0; m < MMAX; ++m) a[m] = *reinterpret_cast<const uint4*>(ap + (size_t)(m < M ? m : 0) * K);
#pragma unroll
    for (int m = 0; m < MMAX; ++m) {
      acc[m] = dot2_bf16(w.x, a[m].x, acc[m]);
      acc[m] = dot2_bf16(w.y, a[m].y, acc[m]);
      acc[m] = dot2_bf16(w.z, a[m].z, acc[m]);
      acc[m] = dot2_bf16(w.w, a[m].w, acc[m]);
    }
  }
  float mine = 0.f;
#pragma unroll
  for (int m = 0; m < MMAX; ++m) {
    const float t = group_sum<TI_WAVE>(acc[m]);
    if (lane == m) mine = t;
  }
  if (lane < M && n < N) {
    const size_t o = (size_t)lane * N + n;
    if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = mine;
    if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] = prev + mine;
    if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(mine);
  }
}

// The same product with the token rows straight from memory into registers: lane l fetches, for every
// token, the pieces of the row that go with its pieces of the weight row (all workgroups read the same few
// KB: they come from the caches), after its weights have been asked for.  Nothing goes through LDS, so
// nothing is written, waited for at a barrier and read back between the arrival of the weights and the
// products (8 tokens, a 1,024 x 2,048 weight, in a chain of dependent launches: 5.3 -> 4.75 us; 1,024 x
// 3,072: 6.3 -> 5.7 us).  The same order of sums, the same bits.  MMAX * NL * 4 registers hold the token
// rows: up to NL = 6 (K <= 3,072) at 8 tokens.
template <int EPI, int MMAX, int NL>
__global__ void __launch_bounds__(256)
gemv_rows_direct_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ out_, int M,
                        int N, int K, long lda) {
  static_assert(EPI != TI_EPI_SWIGLU, "no SwiGLU here");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + wave;
  const bf16_t* wp = W + (size_t)(n < N ? n : N - 1) * K;
  const uint4 zero = make_uint4(0, 0, 0, 0);
  float prev = 0.f;
  if (EPI == TI_EPI_ADD_F32) prev = ((const float*)out_)[(size_t)(lane < M ? lane : 0) * N + (n < N ? n : N - 1)];
  uint4 wv[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int kk = (i * 64 + lane) * 8;
    wv[i] = ld16(wp + (kk < K ? kk : 0));
  }
  __builtin_amdgcn_sched_barrier(0);
  uint4 a[NL][MMAX];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int kk = (i * 64 + lane) * 8;
#pragma unroll
    for (int m = 0; m < MMAX; ++m) a[i][m] = ld16(A + (size_t)(m < M ? m : 0) * lda + (kk < K ? kk : 0));
  }
  __builtin_amdgcn_sched_barrier(0);
  float acc[MMAX];
#pragma unroll
  for (int m = 0; m < MMAX; ++m) acc[m] = 0.f;
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int kk = (i * 64 + lane) * 8;
    const uint4 w = kk < K ? wv[i] : zero;
#pragma unroll
    for (int m = 0; m < MMAX; ++m) {
      acc[m] = dot2_bf16(w.x, a[i][m].x, acc[m]);
      acc[m] = dot2_bf16(w.y, a[i][m].y, acc[m]);
      acc[m] = dot2_bf16(w.z, a[i][m].z, acc[m]);
      acc[m] = dot2_bf16(w.w, a[i][m].w, acc[m]);
    }
  }
  float mine = 0.f;
#pragma unroll
  for (int m = 0; m < MMAX; ++m) {
    const float t = group_sum<TI_WAVE>(acc[m]);
    if (lane == m) mine = t;
  }
  if (lane < M && n < N) {
    const size_t o = (size_t)lane * N + n;
    if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = mine;
    if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] = prev + mine;
    if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(mine);
  }
}

// =============================================================== tiled kernel
#define TBM 128
#define TBN 128
#define TBK 32
#define TLD (TBK + 8)   // LDS row stride in bfloat16: 80 bytes, keeps 16-byte reads off the same banks
#define TPIECES (TBM * TBK / 8 / 256)   // 16-byte pieces per thread and operand tile
#define TKP (TBK / 8)                   // pieces per row

// SwiGLU: the workgroup covers 64 output columns; LDS row b of the weight tile is
// global row (b & 32 ? F : 0) + n0 + (b >> 6) * 32 + (b & 31), so that in every
// wavefront MFMA tile 0 holds gate columns and tile 1 the matching up columns.
template <int EPI>
__global__ void __launch_bounds__(256)
gemm_tiled_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ out_,
                  int M, int N, int K, long lda) {
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  __shared__ __attribute__((aligned(16))) bf16_t sA[2][TBM * TLD];
  __shared__ __attribute__((aligned(16))) bf16_t sB[2][TBN * TLD];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * TBM;
  const int n0 = blockIdx.x * (SW ? TBN / 2 : TBN);
  const int w_rows = SW ? 2 * N : N;

  // global -> LDS in pieces of 16 bytes, TPIECES per thread and operand tile
  constexpr int RSTEP = 256 / TKP;   // rows covered by one round of the workgroup
  const int lrow = tid / TKP, lkc = (tid % TKP) * 8;
  const bf16_t* gA[TPIECES];
  const bf16_t* gB[TPIECES];
  bool okA[TPIECES], okB[TPIECES];
#pragma unroll
  for (int i = 0; i < TPIECES; ++i) {
    const int row = lrow + RSTEP * i;
    const int am = m0 + row;
    okA[i] = am < M;
    gA[i] = A + (size_t)(okA[i] ? am : 0) * lda + lkc;
    int wr;
    if (SW) {
      const int n = n0 + (row >> 6) * 32 + (row & 31);
      okB[i] = n < N;
      wr = ((row & 32) ? N : 0) + (okB[i] ? n : 0);
    } else {
      wr = n0 + row;
      okB[i] = wr < N;
      if (!okB[i]) wr = 0;
    }
    (void)w_rows;
    gB[i] = W + (size_t)wr * K + lkc;
  }
  const uint4 zero = make_uint4(0, 0, 0, 0);
  uint4 ra[TPIECES], rb[TPIECES];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < TPIECES; ++i) {
      const bool kin = k0 + lkc + 8 <= K;
      ra[i] = (okA[i] && kin) ? ld16(gA[i] + k0) : zero;
      rb[i] = (okB[i] && kin) ? ld16(gB[i] + k0) : zero;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TPIECES; ++i) {
      *reinterpret_cast<uint4*>(&sA[buf][(lrow + RSTEP * i) * TLD + lkc]) = ra[i];
      *reinterpret_cast<uint4*>(&sB[buf][(lrow + RSTEP * i) * TLD + lkc]) = rb[i];
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  const int fr = lane & 31, fk = (lane >> 5) * 8;
  const int n_k = (K + TBK - 1) / TBK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int kt = 0; kt < n_k; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < n_k) fetch((kt + 1) * TBK);
#pragma unroll
    for (int ks = 0; ks < TBK; ks += 16) {
      Frag fa[2], fb[2];
#pragma unroll
      for (int a = 0; a < 2; ++a)
        fa[a].u = *reinterpret_cast<const uint4*>(&sA[buf][(wm * 64 + a * 32 + fr) * TLD + ks + fk]);
#pragma unroll
      for (int b = 0; b < 2; ++b)
        fb[b].u = *reinterpret_cast<const uint4*>(&sB[buf][(wn * 64 + b * 32 + fr) * TLD + ks + fk]);
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[a].v, fb[b].v, acc[a][b], 0, 0, 0);
    }
    if (kt + 1 < n_k) stash(buf ^ 1);
    __syncthreads();
  }

  // acc[a][b][i]: row wm*64 + a*32 + 8*(i/4) + 4*(lane/32) + i%4, column wn*64 + b*32 + lane%32
  const int ccol = lane & 31, crow = (lane >> 5) * 4;
#pragma unroll
  for (int a = 0; a < 2; ++a) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = m0 + wm * 64 + a * 32 + (i >> 2) * 8 + crow + (i & 3);
      if (m >= M) continue;
      if (SW) {
        const int n = n0 + wn * 32 + ccol;
        if (n < N) ((bf16_t*)out_)[(size_t)m * N + n] = f2bf(silu_mul(acc[a][0][i], acc[a][1][i]));
      } else {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int n = n0 + wn * 64 + b * 32 + ccol;
          if (n >= N) continue;
          const size_t o = (size_t)m * N + n;
          const float s = acc[a][b][i];
          if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = s;
          if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] += s;
          if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(s);
        }
      }
    }
  }
}

// ====================================================== tiled kernel, pipelined
// The same product with the tiles brought in by direct global-to-LDS loads
// (global_load_lds_dwordx4: each lane fetches 16 bytes, the wavefront's 64 pieces
// land in 1 KiB of LDS in lane order) three stages deep, so that two k-tiles are in
// flight while one is multiplied (K must be a multiple of 64; other K take the plain
// tiled kernel).  BK = 64: a tile row is 128 bytes = 8 pieces.  Rows
// are stored unpadded, and piece c of row r sits in slot c ^ ((r >> 1) & 7): the 16
// rows that one phase of a 16-byte LDS read touches then fall on all 64 banks once.
// The lane that fills slot (r, c) simply fetches piece c ^ ((r >> 1) & 7) of row r.
//
// WG tile BM x BN, four wavefronts as WAVES_M x WAVES_N, each (BM / WAVES_M) x
// (BN / WAVES_N) out of 32 x 32 x 16 MFMAs.  SwiGLU needs two 32-column tiles per
// wavefront: tile 0 holds gate columns, tile 1 the matching up columns.
#define PBK 64
#define PSTAGES 3

__device__ __forceinline__ void wait_vmcnt(int n) {
  // s_waitcnt with only vmcnt set (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
#define TI_W(N) case N: __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14)); break;
    TI_W(1) TI_W(2) TI_W(3) TI_W(4) TI_W(5) TI_W(6) TI_W(7) TI_W(8) TI_W(9) TI_W(10) TI_W(11) TI_W(12)
    TI_W(13) TI_W(14) TI_W(15) TI_W(16) TI_W(20) TI_W(24)
#undef TI_W
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
}

// What the epilogue TI_EPI_QKV_PREP needs: the product is the fused q/k/v projection of a step's
// rows, and instead of storing it the kernel finishes each head of each row: per-head norm and
// rotation for q heads (to q_out, T [M, n_head hd]) and k heads (into the cache page of the row's
// position), v heads copied into the cache transposed.  A workgroup's BN columns are whole heads.
struct QKVEpilogue {
  const float* q_w;          // per-head norm weights or nullptr
  const float* k_w;
  float eps;
  const float* inv_freq;     // nullptr: no rotation
  const float2* rope_table;  // (cos, sin) [table_len][hd / 2] or nullptr
  int table_len;
  const int* pos;            // position of each row
  const int* slot;           // block-table row of each row
  const int* table;
  int table_stride;
  bf16_t* pool;              // [pages][2][n_kv][P * hd]
  bf16_t* q_out;
  int n_head, n_kv, hd, P;
};

// A q or k head (unit u of the fused projection, head hh of the tile) of all BM rows of a tile that
// lies in LDS in 32-bit (row stride FS): eight lanes a row, 8 NWV rows a pass.  The angles of the
// next pass are asked for before a pass is finished; a lane reads its HD / 16 pairs from LDS as runs of
// 16 bytes and writes its finished elements to memory as two runs of HD / 8 bytes, the eight lanes
// together the row's 2 HD consecutive bytes.
template <int HD, int BM, int NWV, int FS, bool NORMED, bool ROTATE>
__device__ __forceinline__ void qkv_rows_by_lanes(const QKVEpilogue& ep, float* ft, const int* s_pos,
                                                  const int* s_page, const int* s_prow, const int* s_live, int hh,
                                                  int u, int m0) {
  constexpr int NP = HD / 16, PASSES = BM / (NWV * 8);
  const int tid = threadIdx.x;
  const bool is_q = u < ep.n_head;
  float wlo[NP], whi[NP];
  qk_lanes_weights<HD>(wlo, whi, NORMED ? (is_q ? ep.q_w : ep.k_w) : nullptr);
  float2 cs[NP], next[NP];
#pragma unroll 1
  for (int ps = -1; ps < PASSES; ++ps) {
    if (ROTATE && ps + 1 < PASSES)
      qk_lanes_angles<HD>(next, s_pos[(ps + 1) * NWV * 8 + tid / 8], ep.inv_freq, ep.rope_table, ep.table_len);
    if (ps >= 0) {
      const int r = ps * NWV * 8 + tid / 8;
      unsigned lo[NP / 2], hi[NP / 2];
      qk_head_lanes<HD, NORMED, ROTATE>(ft + r * FS + hh * HD, wlo, whi, ep.eps, cs, lo, hi);
      bf16_t* dst = nullptr;
      if (is_q) {
        if (s_live[r] >= 0) dst = ep.q_out + ((size_t)(m0 + r) * ep.n_head + u) * HD;
      } else if (s_page[r] >= 0) {
        dst = kv_page_slot<bf16_t>(ep.pool, s_page[r], 0, u - ep.n_head, s_prow[r], ep.n_kv, ep.P, HD);
      }
      if (dst) {
        bf16_t* mine = dst + NP * (tid & 7);
        if constexpr (NP == 8) {
          *reinterpret_cast<uint4*>(mine) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
          *reinterpret_cast<uint4*>(mine + HD / 2) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        } else {
          *reinterpret_cast<uint2*>(mine) = make_uint2(lo[0], lo[1]);
          *reinterpret_cast<uint2*>(mine + HD / 2) = make_uint2(hi[0], hi[1]);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < NP; ++k) cs[k] = next[k];
  }
}

template <int HD, int BM, int NWV, int FS>
__device__ __forceinline__ void qkv_rows_by_lanes(const QKVEpilogue& ep, float* ft, const int* s_pos,
                                                  const int* s_page, const int* s_prow, const int* s_live, int hh,
                                                  int u, int m0) {
  const bool normed = (u < ep.n_head ? ep.q_w : ep.k_w) != nullptr, rotate = ep.inv_freq != nullptr;
  if (normed && rotate)
    qkv_rows_by_lanes<HD, BM, NWV, FS, true, true>(ep, ft, s_pos, s_page, s_prow, s_live, hh, u, m0);
  else if (normed)
    qkv_rows_by_lanes<HD, BM, NWV, FS, true, false>(ep, ft, s_pos, s_page, s_prow, s_live, hh, u, m0);
  else if (rotate)
    qkv_rows_by_lanes<HD, BM, NWV, FS, false, true>(ep, ft, s_pos, s_page, s_prow, s_live, hh, u, m0);
  else
    qkv_rows_by_lanes<HD, BM, NWV, FS, false, false>(ep, ft, s_pos, s_page, s_prow, s_live, hh, u, m0);
}

// k-steps whose fragments are on their way from LDS while one is multiplied (two: a prompt of 2,048 tokens at
// Qwen3-0.6B's sizes 0.7 % faster, at Qwen3-8B's 3.7 % slower)
#define FRAG_AHEAD 1
template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, int STAGES = PSTAGES, int KT = PBK>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_pipelined_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ out_arg,
                      int M, int N, int K, long lda, int n_first, int xcd_rows, QKVEpilogue ep = QKVEpilogue{}) {
  // n_first: the output column the grid's first workgroup starts at (a launch may cover a range of columns)
  // xcd_rows > 0 (the grid's width is a multiple of 8 then): which tile a workgroup takes follows the eight
  // dies.  Workgroups go to the dies in turn, so die c has numbers c, c + 8, ...; it takes an eighth of the
  // column tiles, in blocks of xcd_rows row tiles, down the rows of a column first: the workgroups of a die
  // that run at the same time then share a few column tiles of the weight and xcd_rows row tiles of the
  // tokens in the die's own L2.
  int bx = blockIdx.x, by = blockIdx.y;
  if (xcd_rows > 0) {
    const int nx = gridDim.x, ny = gridDim.y, cx = nx >> 3;
    const int id = bx + nx * by, die = id & 7, local = id >> 3;
    const int full = ny / xcd_rows, per = xcd_rows * cx;
    int rb = local / per, rem = local - rb * per, rows = xcd_rows;
    if (rb >= full) {
      rb = full;
      rem = local - full * per;
      rows = ny - full * xcd_rows;
    }
    by = rb * xcd_rows + rem % rows;
    bx = die * cx + rem / rows;
  }
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
  constexpr int NWV = WAVES_M * WAVES_N;                     // wavefronts: 4 or 8
  static_assert(NWV == 4 || NWV == 8, "four or eight wavefronts");
  static_assert(!SW || TN % 2 == 0, "SwiGLU pairs the column tiles of a wavefront: the first half gate, the second half up");
  static_assert(STAGES >= 2 && STAGES <= 4, "two to four stages");
  // KT: the depth of a k-tile, 64 or 32.  A row of a stage is KT bfloat16 (CPR pieces of 16 bytes); a wavefront's
  // load of 1 KiB covers RPL rows; piece c of row r lies in slot c ^ swz(r), so that the sixteen lanes of a
  // fragment read (sixteen rows, one piece) touch sixteen different 16-byte columns of the banks
  static_assert(KT == 64 || KT == 32, "k-tiles of 64 or 32");
  constexpr int CPR = KT / 8, RPL = 64 / CPR, ROWB = KT * 2;
  auto swz = [](int r) { return KT == 64 ? (r >> 1) & 7 : (r >> 2) & 3; };

  constexpr int STAGE_BYTES = (BM + BN) * ROWB;
  constexpr int GROUPS_A = BM / RPL, GROUPS_B = BN / RPL;    // RPL rows = 1 KiB = one wavefront load
  static_assert((GROUPS_A + GROUPS_B) % NWV == 0, "every wavefront issues the same number of loads");
  constexpr int LOADS = (GROUPS_A + GROUPS_B) / NWV;         // per wavefront and k-tile
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  // gridDim.z > 1 (storing epilogue only): K is split; workgroup z takes its share of the k-tiles and
  // stores its sums into the z-th [M, N] of out
  const int kt0 = (int)((long)(K / KT) * blockIdx.z / gridDim.z);
  const int n_k = (int)((long)(K / KT) * (blockIdx.z + 1) / gridDim.z) - kt0;
  void* __restrict__ out_ = (EPI == TI_EPI_STORE_F32) ? (void*)((float*)out_arg + (size_t)blockIdx.z * M * N) : out_arg;
  // the wavefront's number in a scalar register: where its loads go in LDS is scalar arithmetic then
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int m0 = by * BM;
  const int n0 = n_first + bx * (SW ? BN / 2 : BN);
  const int lr = lane / CPR, lc = lane % CPR;                // row within a load's group of rows, slot within the row
  const bool spread = K >= 4096;

  // the global row each of this lane's loads reads (clamped into the matrix: rows
  // beyond it are computed and thrown away), as a pointer to its first element
  const bf16_t* gsrc[LOADS];
  int gpiece[LOADS];                                         // which 8-element piece of the row this lane fetches
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int g = wave + NWV * i;                            // groups 0..GROUPS_A-1: A, then B
    if (g < GROUPS_A) {
      const int row = g * RPL + lr;
      const int gm = min(m0 + row, M - 1);
      gsrc[i] = A + (size_t)gm * lda;
      gpiece[i] = lc ^ swz(row);
    } else {
      const int row = (g - GROUPS_A) * RPL + lr;
      int wr;
      if (SW) {
        constexpr int span = BN / WAVES_N, half = span / 2;  // LDS rows of one wavefront's columns: gate rows, then up rows
        const int n = n0 + (row / span) * half + (row % half);
        wr = ((row % span) >= half ? N : 0) + min(n, N - 1);
      } else {
        wr = min(n0 + row, N - 1);
      }
      gsrc[i] = W + (size_t)wr * K;
      gpiece[i] = lc ^ swz(row);
    }
  }

  // load i of this wavefront's LOADS loads of k-tile kt
  auto issue_one = [&](int kt, int i) {
    unsigned char* stage = smem + (kt % STAGES) * STAGE_BYTES;
    const int k0 = (kt0 + kt) * KT;
    const int g = wave + NWV * i;
    unsigned char* dst = stage + g * 1024;                   // the same in every lane
    // K is a multiple of 64 here (the dispatcher sees to it): no piece lies past the end
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void*)(gsrc[i] + k0 + gpiece[i] * 8),
        (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
  };
  auto issue = [&](int kt) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) issue_one(kt, i);
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  // The multiply loop is scheduled by hand.  The compiler does not know which LDS
  // bytes a direct load will write, so before any LDS read it can see, and at every
  // fence, it waits for all of them, the two k-tiles in flight included; that would
  // undo the pipeline.  So LDS is read with ds_read_b128 in inline assembly, the
  // barrier is the bare instruction, and the waits are written out: vmcnt before the
  // barrier (the tile about to be multiplied has landed), lgkmcnt before each group of
  // MFMAs (its fragments have arrived; those of the next k-step are still in flight).
  const int fr = lane & 31, fh = lane >> 5;                  // fragment row, and which half of a 16-wide k-step
  const unsigned lds0 = (unsigned)(size_t)smem;              // LDS byte address of the first stage
  const unsigned rowA = lds0 + (wm * (BM / WAVES_M) + fr) * ROWB;
  const unsigned rowB = lds0 + BM * ROWB + (wn * (BN / WAVES_N) + fr) * ROWB;
  unsigned xo[KT / 16];                                      // swizzled byte offset of this lane's piece, per k-step
#pragma unroll
  for (int ks = 0; ks < KT / 16; ++ks) xo[ks] = ((ks * 2 + fh) ^ swz(fr)) << 4;

  // the residual an adding epilogue adds to: asked for while the last k-tile is multiplied
  // (elements outside the matrix read a valid one and are not stored)
  // (a tile of many accumulators has no registers for it and reads the residual in the epilogue)
  constexpr bool PREV = EPI == TI_EPI_ADD_F32 && (NWV == 4 || TM * TN <= 4);
  float prev[PREV ? TM : 1][PREV ? TN : 1][16];
#pragma unroll
  for (int st = 0; st < STAGES - 1; ++st)
    if (st < n_k) issue(st);
  for (int kt = 0; kt < n_k; ++kt) {
    // tile kt has landed (its loads are older than those of the tiles after it), in every wavefront,
    // and every wavefront has finished with the stage that tile kt + STAGES - 1 goes into
    wait_vmcnt(min(STAGES - 2, n_k - 1 - kt) * LOADS);
    __builtin_amdgcn_s_barrier();
    // Tile kt + 2 goes into the stage that everyone has left.  Its loads go out between the k-steps
    // below, each behind a k-step's matrix instructions: the unit that takes the addresses handles 64
    // bytes a cycle for the whole compute unit, and eight wavefronts that ask for a whole tile at once
    // queue there with nothing on the matrix cores meanwhile.
    // (a prompt of 2,048 tokens 2.5 % faster at Qwen3-0.6B's sizes, 2.1 % at Qwen3-8B's; a k-tile of a 256 x 128
    // tile from 2,480 to 2,200 cycles)
    // (spread evenly between the matrix instructions where K is long, k-step by k-step where it is short: see below)
    const bool more = kt + STAGES - 1 < n_k, more_spread = more && spread, more_steps = more && !spread;
    if constexpr (PREV) {
      if (kt == n_k - 1) {
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
          for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int m = m0 + wm * (BM / WAVES_M) + a * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
              const int n = n0 + wn * (BN / WAVES_N) + b * 32 + (lane & 31);
              prev[a][b][i] = ((const float*)out_)[(size_t)min(m, M - 1) * N + min(n, N - 1)];
            }
      }
    }
    const unsigned st = (kt % STAGES) * STAGE_BYTES;
    // the fragments of FRAG_AHEAD k-steps are on their way from LDS while one is multiplied
    constexpr int SETS = FRAG_AHEAD + 1, KSTEPS = KT / 16;
    v4u fa[SETS][TM], fb[SETS][TN];
    auto read_step = [&](int ks, int set) {
      const unsigned pa = rowA + st + xo[ks], pb = rowB + st + xo[ks];
#pragma unroll
      for (int a = 0; a < TM; ++a)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa[set][a]) : "v"(pa), "n"(a * 32 * ROWB));
#pragma unroll
      for (int b = 0; b < TN; ++b)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb[set][b]) : "v"(pb), "n"(b * 32 * ROWB));
    };
#pragma unroll
    for (int ks = 0; ks < FRAG_AHEAD; ++ks) read_step(ks, ks);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int set = ks % SETS;
      if (ks + FRAG_AHEAD < KSTEPS) read_step(ks + FRAG_AHEAD, (ks + FRAG_AHEAD) % SETS);
      // this k-step's fragments are there when only the reads issued after them are outstanding:
      // those of the k-steps up to FRAG_AHEAD further on
      constexpr int PER = TM + TN;
      const int later = (KSTEPS - 1 - ks < FRAG_AHEAD ? KSTEPS - 1 - ks : FRAG_AHEAD) * PER;
      static_assert(FRAG_AHEAD * PER <= 15, "lgkmcnt counts to 15");
      switch (later) {
#define TI_LGKM(N) case N: asm volatile("s_waitcnt lgkmcnt(" #N ")" ::: "memory"); break;
        TI_LGKM(0) TI_LGKM(2) TI_LGKM(3) TI_LGKM(4) TI_LGKM(6) TI_LGKM(7) TI_LGKM(8) TI_LGKM(12) TI_LGKM(14)
#undef TI_LGKM
        default: asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); break;
      }
      // tie the fragments to the wait, so that no MFMA is moved above it
#pragma unroll
      for (int a = 0; a < TM; ++a) asm volatile("" : "+v"(fa[set][a]));
#pragma unroll
      for (int b = 0; b < TN; ++b) asm volatile("" : "+v"(fb[set][b]));
#pragma unroll
      for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b) {
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[set][a]),
                                                              __builtin_bit_cast(bf16x8, fb[set][b]), acc[a][b],
                                                              0, 0, 0);
          // load i goes out behind matrix instruction (2 i + 1) NM / (2 LOADS) of the k-tile's NM: spread evenly,
          // no two wavefronts' loads queue at the unit that takes the addresses (a prompt of 2,048 tokens at
          // Qwen3-8B's sizes 2.2 % faster, at Qwen3-32B's 3.1 %; at Qwen3-0.6B's, K = 1,024 to 3,072, 0.6 % slower
          // than with the loads behind each k-step's matrix instructions, which stays for K below 4,096)
          constexpr int NM = KSTEPS * TM * TN;
          const int g = (ks * TM + a) * TN + b;
          if (more_spread) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i)
              if ((2 * i + 1) * NM / (2 * LOADS) == g) issue_one(kt + STAGES - 1, i);
          }
        }
      if (more_steps) {
#pragma unroll
        for (int i = ks; i < LOADS; i += KT / 16) issue_one(kt + STAGES - 1, i);
      }
    }
  }

  // acc[a][b][i]: row wm*(BM/WAVES_M) + a*32 + 8*(i/4) + 4*(lane/32) + i%4, column wn*(BN/WAVES_N) + b*32 + lane%32
  const int ccol = lane & 31, crow = (lane >> 5) * 4;
  if constexpr (EPI == TI_EPI_QKV_PREP) {
    // The tile goes to LDS in 32-bit (the stages are free now); then, head by head of the tile, eight
    // lanes finish a row of a q or k head (the arithmetic of the kernel that prepares whole steps; a
    // row's eight lanes read its angles and write its result as runs of consecutive bytes), and a
    // thread a dim of a v head.
    static_assert((BM == 256 || BM == 128) && NWV == 8, "the first wavefronts look up a row each; 64 rows per pass of all eight");
    constexpr int FS = BN + 8;                              // row stride: the eight rows x eight lanes of a wavefront
                                                            // read 64 different banks
    static_assert(BM * FS * 4 + 4 * BM * 4 <= STAGES * STAGE_BYTES, "the 32-bit tile fits into the stages");
    float* ft = reinterpret_cast<float*>(smem);
    __syncthreads();
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int b = 0; b < TN; ++b)
          ft[(wm * (BM / WAVES_M) + a * 32 + (i >> 2) * 8 + crow + (i & 3)) * FS + wn * (BN / WAVES_N) + b * 32 + ccol] =
              acc[a][b][i];
    // each row's position, and where its key and value go
    int* s_page = reinterpret_cast<int*>(ft + BM * FS);     // [BM] page of the row's position, -1: none
    int* s_prow = s_page + BM;                              // [BM] row of the position in that page
    int* s_live = s_prow + BM;                              // [BM] block-table row (request) of the row, -1: none
    int* s_pos = s_live + BM;                               // [BM] position of the row
    const int hd = ep.hd, units = ep.n_head + 2 * ep.n_kv;
    if (tid < BM) {
      const int m = m0 + tid;
      const bool live = m < M;
      const int p = live ? ep.pos[m] : 0;
      // the host reserves pages first; a row without one (-1) writes nothing
      s_page[tid] = (live && ep.n_kv > 0) ? ep.table[(size_t)ep.slot[m] * ep.table_stride + p / ep.P] : -1;
      s_prow[tid] = p % ep.P;
      s_live[tid] = live ? ep.slot[m] : -1;
      s_pos[tid] = p;
    }
    __syncthreads();
    for (int hh = 0; hh < BN / hd; ++hh) {
      const int u = n0 / hd + hh;                            // the same in every thread
      if (u >= units) break;
      const bool is_q = u < ep.n_head, is_v = u >= ep.n_head + ep.n_kv;
      if (is_v) {
        // values go in transposed, [dim][row of the page]: thread -> one dim, for runs of 16 rows of
        // the tile; a run that is 16 consecutive rows of one page leaves as 32 contiguous bytes
        const int kvh = u - ep.n_head - ep.n_kv;
        const int d = tid % hd;
        for (int r0 = (tid / hd) * 16; r0 < BM; r0 += (NWV * 64 / hd) * 16) {
          const int pg = s_page[r0], pr = s_prow[r0];
          // rows of a run are consecutive positions of one request: its first and last row tell
          bool run = (pg >= 0) & (pr % 16 == 0) & (s_page[r0 + 15] == pg) & (s_prow[r0 + 15] == pr + 15) &
                     (s_live[r0] == s_live[r0 + 15]);
          const float* col = ft + r0 * FS + hh * hd + d;
          if (run) {
            float v[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) v[j] = col[j * FS];
            bf16_t* dst = kv_page_slot<bf16_t>(ep.pool, pg, 1, kvh, pr, ep.n_kv, ep.P, hd) + (size_t)d * ep.P;
            *reinterpret_cast<uint4*>(dst) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                                                        pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
            *reinterpret_cast<uint4*>(dst + 8) = make_uint4(pack_bf16x2(v[8], v[9]), pack_bf16x2(v[10], v[11]),
                                                            pack_bf16x2(v[12], v[13]), pack_bf16x2(v[14], v[15]));
          } else {
            for (int j = 0; j < 16; ++j) {
              const int pj = s_page[r0 + j];
              if (pj >= 0)
                kv_page_slot<bf16_t>(ep.pool, pj, 1, kvh, s_prow[r0 + j], ep.n_kv, ep.P, hd)[(size_t)d * ep.P] =
                    f2bf(col[j * FS]);
            }
          }
        }
        continue;
      }
      if (hd == 128)
        qkv_rows_by_lanes<128, BM, NWV, FS>(ep, ft, s_pos, s_page, s_prow, s_live, hh, u, m0);
      else
        qkv_rows_by_lanes<64, BM, NWV, FS>(ep, ft, s_pos, s_page, s_prow, s_live, hh, u, m0);
    }
    return;
  }
#pragma unroll
  for (int a = 0; a < TM; ++a) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = m0 + wm * (BM / WAVES_M) + a * 32 + (i >> 2) * 8 + crow + (i & 3);
      if (m >= M) continue;
      if (SW) {
#pragma unroll
        for (int b = 0; b < TN / 2; ++b) {
          const int n = n0 + wn * (BN / WAVES_N / 2) + b * 32 + ccol;
          if (n < N) ((bf16_t*)out_)[(size_t)m * N + n] = f2bf(silu_mul(acc[a][b][i], acc[a][b + TN / 2][i]));
        }
      } else {
#pragma unroll
        for (int b = 0; b < TN; ++b) {
          const int n = n0 + wn * (BN / WAVES_N) + b * 32 + ccol;
          if (n >= N) continue;
          const size_t o = (size_t)m * N + n;
          const float v = acc[a][b][i];
          if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = v;
          if constexpr (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] = (PREV ? prev[a][b][i] : ((const float*)out_)[o]) + v;
          if (EPI == TI_EPI_STORE_ACT) ((bf16_t*)out_)[o] = f2bf(v);
        }
      }
    }
  }
}

// Row tiles per block of the order in which a die takes its tiles (see the kernel), 0: tiles in the grid's
// order.  The dies' order pays where the weight is larger than the cache in front of the memory holds (256 MB):
// in the grid's order every row tile pulls the whole weight from memory again (Qwen3-32B's gate/up and down
// over 2,048 rows, 524 and 262 MB: a prompt of 2,048 tokens 9.6 % faster); a weight that cache holds is served
// from it either way (Qwen3-8B's, 201 MB: no change; Qwen3-0.6B's: 0.7 % slower).
static int g_xcd_rows = 0;       // a hook for measurements: > 0 forces the block's rows, -1 the grid's order
static int xcd_rows_for(const dim3& grid, int N, int K) {
  if (grid.x % 8 != 0 || g_xcd_rows < 0) return 0;
  if (g_xcd_rows > 0) return g_xcd_rows;
  return (long)N * K * 2 >= (192L << 20) ? 8 : 0;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, int STAGES = PSTAGES, int KT = PBK>
static int launch_pipelined(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda,
                            hipStream_t s, int ksplit = 1, int n_first = 0, int n_end = -1) {
  constexpr int bytes = STAGES * (BM + BN) * KT * 2;
  auto kernel = gemm_pipelined_kernel<BM, BN, WAVES_M, WAVES_N, EPI, STAGES, KT>;
  static bool ready = false;          // per instantiation: allow more than 64 KiB of dynamic LDS
  if (!ready) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
      ti_set_error("gemm_bf16: cannot reserve %d bytes of LDS", bytes);
      return 2;
    }
    ready = true;
  }
  const int bn = (EPI == TI_EPI_SWIGLU) ? BN / 2 : BN;
  // columns [n_first, n_end) of the output (all of them by default); n_end short of N is a multiple of the tile
  if (n_end < 0) n_end = N;
  dim3 grid((n_end - n_first + bn - 1) / bn, (M + BM - 1) / BM, (EPI == TI_EPI_STORE_F32) ? ksplit : 1);
  kernel<<<grid, WAVES_M * WAVES_N * 64, bytes, s>>>(A, W, out, M, N, K, lda, n_first,
                                                     xcd_rows_for(grid, (EPI == TI_EPI_SWIGLU ? 2 : 1) * N, K), QKVEpilogue{});
  return 0;
}

static int g_tiles_160 = 1;      // a hook for measurements: 0 = no tiles of 160 columns
static int g_tiles_256 = 1;      // a hook for measurements: 0 = no tiles of 256 x 256
static int g_two_ranges = 1;     // a hook for measurements: 0 = never split the columns between two tile shapes
static int g_qkv_rows = 0;       // hooks for measurements: 128 or 256 forces the tile's rows;
static int g_qkv_min_rows = 17;  // the fewest rows served (fewer take the kernels with the norm in front)

static int compute_units() {
  static int n = 0;
  if (!n) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) n = prop.multiProcessorCount;
    if (n <= 0) n = 256;
  }
  return n;
}

template <int BM, int WAVES_M, int WAVES_N>
static int launch_qkv_prep(const void* A, const void* W, int M, int N, int K, long lda, const QKVEpilogue& ep,
                           hipStream_t stream, int n_first = 0, int n_end = -1) {
  constexpr int BN = 128;
  constexpr int bytes = PSTAGES * (BM + BN) * PBK * 2;
  auto kernel = gemm_pipelined_kernel<BM, BN, WAVES_M, WAVES_N, TI_EPI_QKV_PREP>;
  static bool ready = false;
  if (!ready) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
      ti_set_error("gemm_bf16_qkv_prep: cannot reserve %d bytes of LDS", bytes);
      return 2;
    }
    ready = true;
  }
  if (n_end < 0) n_end = N;               // columns [n_first, n_end): whole heads
  dim3 grid((n_end - n_first + BN - 1) / BN, (M + BM - 1) / BM);
  kernel<<<grid, 512, bytes, stream>>>((const bf16_t*)A, (const bf16_t*)W, nullptr, M, N, K, lda, n_first,
                                       xcd_rows_for(grid, N, K), ep);
  return 0;
}

// The fused q/k/v projection of a step's rows with the per-head work in its epilogue (see
// QKVEpilogue): A [M, K] bf16, W [(n_head + 2 n_kv) hd, K] bf16 (n_kv = 0: q heads only, nothing is
// written to the cache).  Returns 3 for what it does not serve: M <= 16, K not a multiple of 64,
// head sizes other than 64 and 128.
extern "C" int ti_gemm_bf16_qkv_prep(const void* A, const void* W, int M, int K, long lda, const float* q_w,
                                     const float* k_w, float eps, const float* inv_freq, const float* rope_table,
                                     int table_len, const int* pos, const int* slot, const int* table,
                                     int table_stride, void* pool, void* q_out, int n_head, int n_kv, int hd,
                                     int page_size, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && K > 0 && lda >= K && n_head > 0 && n_kv >= 0 && hd > 0 && page_size > 0 && table_stride > 0,
             "gemm_bf16_qkv_prep: bad sizes");
  if (M < g_qkv_min_rows || K % 64 != 0 || lda % 8 != 0 || !(hd == 64 || hd == 128) || ((uintptr_t)A & 15) ||
      ((uintptr_t)W & 15) || ((uintptr_t)q_out & 15) || ((uintptr_t)pool & 15) || ((uintptr_t)rope_table & 15)) {
    ti_set_error("gemm_bf16_qkv_prep: M=%d K=%d head_dim=%d is not served (M > 16, K %% 64 == 0, head_dim 64 or 128)",
                 M, K, hd);
    return 3;
  }
  TI_REQUIRE(pos && slot && q_out && (n_kv == 0 || (table && pool)), "gemm_bf16_qkv_prep: a buffer is missing");
  TI_REQUIRE(inv_freq || !rope_table, "gemm_bf16_qkv_prep: a sin/cos table without inv_freq");
  QKVEpilogue ep{q_w, k_w, eps, inv_freq, (const float2*)rope_table, table_len, pos, slot, table, table_stride,
                 (bf16_t*)pool, (bf16_t*)q_out, n_head, n_kv, hd, page_size};
  const int N = (n_head + 2 * n_kv) * hd;
  // 128-row tiles while they make no more workgroups than there are compute units (1,024 rows of
  // the 32 column tiles of Qwen3-0.6B), else 256-row tiles, which load less per flop
  const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  // Few tiles (a short portion beside decoded tokens): a launch of tiles whose columns are whole heads
  // leaves most compute units idle, and each workgroup that does run finishes 128 rows of heads by
  // itself; the product in 64 x 64 tiles followed by the kernel that prepares whole steps is faster
  // then (8 decoded tokens beside 128 of a prompt, Qwen3-0.6B's sizes: 2.47 -> 2.29 ms a step; from
  // 512 rows on this kernel wins).  Not when a test asks for a tile.
  if (!g_qkv_rows && tiles128 * 2 < compute_units()) {
    ti_set_error("gemm_bf16_qkv_prep: %ld tiles of 128 x 128 are left to the product and the preparation kernel", tiles128);
    return 3;
  }
  const bool rows128 = g_qkv_rows ? g_qkv_rows == 128 : tiles128 <= compute_units();
  // 256-row tiles that leave a round short of three quarters (Qwen3-8B's 48 heads over 2,048 rows: 8 x 48
  // tiles on 256 units): the heads that make whole rounds take them, the other heads 128-row tiles in a
  // launch of their own, as in the plain product
  const int units = compute_units(), row_tiles = (M + 255) / 256;
  const long big = (long)row_tiles * ((N + 127) / 128);
  int rc_;
  if (!rows128 && !g_qkv_rows && g_two_ranges && big >= units && big < 4L * units && big % units != 0 &&
      big % units < units * 3 / 4 && (int)(big / units * units / row_tiles) >= 1) {
    const int n_big = (int)(big / units * units / row_tiles) * 128;
    rc_ = launch_qkv_prep<256, 4, 2>(A, W, M, N, K, lda, ep, stream, 0, n_big);
    if (!rc_) rc_ = launch_qkv_prep<128, 2, 4>(A, W, M, N, K, lda, ep, stream, n_big, N);
  } else {
    rc_ = rows128 ? launch_qkv_prep<128, 2, 4>(A, W, M, N, K, lda, ep, stream)
                  : launch_qkv_prep<256, 4, 2>(A, W, M, N, K, lda, ep, stream);
  }
  if (rc_) return rc_;
  TI_LAUNCH_CHECK();
  return 0;
}

// for measurements: 0 = choose the tile by the shape, 1 = 256 x 128, 3 = 128 x 64, 5 = 64 x 128 (SwiGLU only), 6 = 64 x 64,
// 8 = 128 x 160, 9 = 256 x 160 (neither for SwiGLU), 10 = 256 x 256
static int g_force_tile = 0;

// Three tiles.  256 x 128 with eight wavefronts does the most per byte it loads, one workgroup
// to a compute unit: it is taken when its workgroups come in (nearly) whole rounds of the 256
// units or in many rounds.  Otherwise 128 x 64 with four wavefronts, two workgroups to a unit;
// and where even those are fewer than two to a unit, 64 x 64 (three to a unit).
template <int EPI>
static int launch_tiled_best(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda,
                             hipStream_t s) {
  const int cols = (EPI == TI_EPI_SWIGLU) ? 2 : 1;   // a SwiGLU workgroup covers BN / 2 output columns
  constexpr bool SW = EPI == TI_EPI_SWIGLU;
  const long big = (long)((M + 255) / 256) * ((N * cols + 127) / 128);
  const long mid = (long)((M + 127) / 128) * ((N * cols + 63) / 64);
  const int units = compute_units();
  const bool whole_rounds = big >= units && (big % units == 0 || big % units >= units * 3 / 4);
  int tile = (big >= 4 * units || whole_rounds) ? 1 : (mid >= 2 * units ? 3 : 6);
  if (M <= 64 && tile == 1) tile = 6;                // few rows times a wide weight: no 256-row tile
  // Up to 64 rows times a stacked [gate; up] weight: such a product waits for the weight from memory, and
  // a 128 x 64 tile, half of whose rows are empty then, has 8 of its 24 KB a stage in weights.  A 64 x 128
  // tile has 16 of 24, two workgroups to a unit as well: twice the weight under way (Qwen3-32B's gate/up
  // at 64 rows 141 -> 115 us, 8B's 52 -> 45); a weight that gives it fewer workgroups than half the
  // units stays with the narrower tile (0.6B's: 10.0 against 10.6 us).
  if (SW && M <= 64 && (long)(N * cols + 127) / 128 * 2 >= compute_units()) tile = 5;
  // 65 to 520 rows (a portion of a prompt beside decoded tokens) times a large weight wait for the weight,
  // and every tile of rows pulls all of it in again.  129 to 256 rows under a stacked [gate; up] weight take
  // one 256-row tile, not two of 128 (Qwen3-8B's at 136 rows 89 -> 65 us, 32B's 185 -> 163, 4B's 48 -> 40);
  // from 385 rows on 128 x 64 tiles, not 64 x 64 (8B's q/k/v, o and down at 520 rows 63, 42 and 132 ->
  // 47, 39 and 104 us).  Small weights are not what such a step waits for: they stay as they were.
  const bool large = (long)N * cols * K >= (8L << 20);
  if (SW && large && M > 128 && M <= 256 && tile == 3) tile = 1;
  if (!SW && large && M > 384 && tile == 6) tile = 3;
  // Widths that 160 columns divide (2,560 and 5,120 among Qwen3's): where tiles of 256 x 160 or 128 x 160,
  // four wavefronts of 64 x 160 or 32 x 160, make whole rounds of the units, they are taken: a workgroup
  // to a unit, fewer LDS reads and bytes from memory per matrix instruction than 256 x 128 (Qwen3-32B's o
  // and down over 2,048 rows, 8 x 32 tiles: 212 and 604 us -> 180 and 554; Qwen3-4B's, 16 x 16 tiles of
  // 128 x 160: 88 and 170 -> 75 and 141).
  if constexpr (!SW) {
    if (!g_force_tile && g_tiles_160 && M > 64 && N % 160 == 0) {
      const long cols160 = N / 160;
      const long wg256 = (long)((M + 255) / 256) * cols160, wg128 = (long)((M + 127) / 128) * cols160;
      auto whole = [&](long wg) { return wg >= units && (wg % units == 0 || wg % units >= units * 7 / 8); };
      if (whole(wg256)) tile = 9;
      else if (whole(wg128) && wg128 <= 2L * units) tile = 8;
    }
  }
  // A stacked [gate; up] weight over many rows, K long: 256 x 256 tiles (eight wavefronts of 64 x 128, two
  // stages of 64 KB) load two thirds of what 256 x 128 tiles load per flop.  Taken where they come in whole
  // rounds of the units (Qwen3-8B's gate/up over 2,048 rows, 8 x 96 tiles: 382 -> 343 us); where rounds are
  // left over, the columns of the whole rounds take them and the rest 256 x 128 tiles in a launch of its own
  // (Qwen3-32B's, 8 x 200 tiles).  With the other epilogues they gain nothing or lose (o over 8,192 rows: 285 ->
  // 314 us).
  if constexpr (SW) {
    const long huge = (long)((M + 255) / 256) * ((N * cols + 255) / 256);
    if (!g_force_tile && g_tiles_256 && M > 256 && K >= 4096 && huge >= units) {
      const int row_tiles = (M + 255) / 256;
      if (huge % units == 0 || huge % units >= units * 7 / 8) return launch_pipelined<256, 256, 4, 2, EPI, 4, 32>(A, W, out, M, N, K, lda, s);
      const int col_tiles = (int)(huge / units * units / row_tiles);
      const int n_big = col_tiles * 128;                // output columns of the first range
      if (huge >= 2L * units && col_tiles >= 1 && n_big < N) {
        if (int rc = launch_pipelined<256, 256, 4, 2, EPI, 4, 32>(A, W, out, M, N, K, lda, s, 1, 0, n_big)) return rc;
        return launch_pipelined<256, 128, 4, 2, EPI>(A, W, out, M, N, K, lda, s, 1, n_big, N);
      }
    }
  }
  // 256 x 128 tiles that fill the units once or more and leave a round short of three quarters (Qwen3-32B's
  // o and down projections over 2,048 rows: 8 x 40 tiles on 256 units): the columns that make whole rounds
  // take those tiles, the rest 128 x 64 tiles in a launch of their own behind them, rather than everything
  // the smaller tile, which needs a third more time per flop (those projections 548 -> 420 us on average;
  // Qwen3-0.6B's gate/up, 8 x 48 tiles, likewise).
  if (tile == 3 && big >= units && !g_force_tile && g_two_ranges) {   // (not where a 160-column tile was chosen)
    const int row_tiles = (M + 255) / 256;
    const int col_tiles = (int)(big / units * units / row_tiles);
    const int n_big = col_tiles * (128 / cols);         // output columns of the first range
    if (col_tiles >= 1 && n_big < N) {
      if (int rc = launch_pipelined<256, 128, 4, 2, EPI>(A, W, out, M, N, K, lda, s, 1, 0, n_big)) return rc;
      return launch_pipelined<128, 64, 4, 1, EPI>(A, W, out, M, N, K, lda, s, 1, n_big, N);
    }
  }
  if (g_force_tile) tile = g_force_tile;
  if constexpr (!SW) {
    if (tile == 8) return launch_pipelined<128, 160, 4, 1, EPI>(A, W, out, M, N, K, lda, s);
    if (tile == 9) return launch_pipelined<256, 160, 4, 1, EPI>(A, W, out, M, N, K, lda, s);
  }
  if (tile == 1) return launch_pipelined<256, 128, 4, 2, EPI>(A, W, out, M, N, K, lda, s);
  if (tile == 10) return launch_pipelined<256, 256, 4, 2, EPI, 4, 32>(A, W, out, M, N, K, lda, s);
  if constexpr (EPI == TI_EPI_SWIGLU)
    if (tile == 5) return launch_pipelined<64, 128, 2, 2, EPI>(A, W, out, M, N, K, lda, s);
  if constexpr (EPI != TI_EPI_SWIGLU)                // a SwiGLU wavefront needs two column tiles
    if (tile == 6) return launch_pipelined<64, 64, 2, 2, EPI>(A, W, out, M, N, K, lda, s);
  return launch_pipelined<128, 64, 4, 1, EPI>(A, W, out, M, N, K, lda, s);
}

// ------------------------------------------------------------------- dispatch
// Wavefronts per workgroup of the skinny kernel (4 or 8).  A product with few output columns
// has few workgroups (one per 16 columns); more wavefronts in each, splitting K further, keep
// more loads in flight.  0 = choose by the shape.
static int g_skinny_waves = 0;
// 1 (default): eight chunks of K in flight per wavefront where its share of K is more than four
static int g_skinny_deep = 1;

template <int EPI>
static void launch_skinny(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda,
                          hipStream_t s) {
  const int grid = (EPI == TI_EPI_SWIGLU) ? (N + 7) / 8 : (N + 15) / 16;
  const int mt = (M + 15) / 16;
  int waves = g_skinny_waves;
  // by the weight's shape only, so that a row's bits do not depend on the rows beside it
  if (waves == 0) waves = (grid <= 128 && K >= 1024) ? 8 : 4;
#define TI_SKINNY(MTV)                                                               \
  if (mt == MTV) {                                                                   \
    if (waves == 8)                                                                  \
      gemm_skinny_kernel<MTV, EPI, 8><<<grid, 512, 0, s>>>(A, W, out, M, N, K, lda); \
    else                                                                             \
      gemm_skinny_kernel<MTV, EPI, 4><<<grid, 256, 0, s>>>(A, W, out, M, N, K, lda); \
  }
  // up to 16 tokens: a wavefront whose share of K is more than four chunks takes eight at a
  // time, so that one round trip to memory serves K up to 512 per wavefront
  if (mt == 1 && (K + 63) / 64 > 4 * waves && g_skinny_deep) {
    if (waves == 8)
      gemm_skinny_kernel<1, EPI, 8, 8><<<grid, 512, 0, s>>>(A, W, out, M, N, K, lda);
    else
      gemm_skinny_kernel<1, EPI, 4, 8><<<grid, 256, 0, s>>>(A, W, out, M, N, K, lda);
    return;
  }
  TI_SKINNY(1)
  TI_SKINNY(2)
  TI_SKINNY(3)
  TI_SKINNY(4)
#undef TI_SKINNY
}

template <int EPI>
static void launch_tiled(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda,
                         hipStream_t s) {
  const int bn = (EPI == TI_EPI_SWIGLU) ? TBN / 2 : TBN;
  dim3 grid((N + bn - 1) / bn, (M + TBM - 1) / TBM);
  gemm_tiled_kernel<EPI><<<grid, 256, 0, s>>>(A, W, out, M, N, K, lda);
}

// 1: the pipelined tiled kernel for M > 64 (default); 0: the plain tiled kernel (for comparison)
static int g_use_pipelined = 1;

// 17..64 rows: the kernels whose workgroups own 16 weight rows pull all token rows in once per 16
// rows, (1 + M / 16) times the weight's bytes through the caches.  Under a small weight that hides
// behind the launch; under a large one it is what the product waits for (Qwen3-8B's gate/up at 64
// rows: 110 us, 1.8 TB/s of weights), and the tiled kernels, which read the token rows once per
// 64 rows of the weight and take about the same time for 17 rows as for 64, are faster although
// their tile is partly empty (50 us).  Measured at the widths of Qwen3-0.6B to 8B: the tiled
// kernels win from about rows x weight elements = 280 Mi on.  13..16 rows: the 16-row kernels
// multiply without the matrix cores and under a large weight that is what they wait for (8B's
// gate/up at 16 rows: 72 us with the norm inside, 62 us as norm + tiled product; Qwen3-4B's: 50
// against 37 us); from rows x weight elements = 600 Mi on these take the tiled kernels too, and
// the norm a kernel of its own.  (At 9 to 12 rows that was measured as well, and loses.)
static long g_tiled_from = 280L << 20;           // 17..64 rows x weight elements from which steps take the tiled kernels
static long g_tiled_from_16 = 600L << 20;        // the same for 13..16 rows
static void set_tiled_from(long rows_times_elems) {
  g_tiled_from = rows_times_elems;
  g_tiled_from_16 = rows_times_elems >= (280L << 20) && rows_times_elems < (1L << 59) ? rows_times_elems / 280 * 600
                                                                                     : rows_times_elems;
}
static bool large_weight(int M, int N, int K, int epi) {
  const long rows = (epi == TI_EPI_SWIGLU) ? 2L * N : (long)N;
  if (M <= 12 || M > 64 || K % PBK != 0) return false;
  return rows * K * M >= (M <= 16 ? g_tiled_from_16 : g_tiled_from);
}

// 1 (default): up to GR_MMAX tokens and a weight of fewer than GR_ROWS_BELOW rows take the kernel
// with a weight row per wavefront; 0: they take the kernels whose workgroups own 16 rows
#define GR_MMAX 8
#define GR_ROWS_BELOW 4096
static int g_row_per_wave = 1;
// Every workgroup (four weight rows) copies all M token rows into LDS: M / 4 times the bytes of its
// weight rows.  Up to four tokens that is no more than the weight itself; beyond, the kernel is taken
// only while its workgroups are no more than the compute units (Qwen3-0.6B's o and down, 1,024 rows: 4.7
// against 7.5 us at 8 tokens), not for more rows (Qwen3-4B's o, 2,560 x 4,096: 10.8 us here, 6.1 in
// workgroups of 16 rows; 1.7B's, 2,048 x 2,048: 3.9 against 3.0).
static bool row_per_wave_serves(int M, int N, int K, int epi) {
  return g_row_per_wave && M <= GR_MMAX && N < GR_ROWS_BELOW && (M <= 4 || N <= 4 * compute_units()) && K % 8 == 0 &&
         K <= 64 * 8 * GR_LOADS && (epi == TI_EPI_STORE_F32 || epi == TI_EPI_ADD_F32);
}

static int g_rows_direct = 1;     // a hook for measurements: 0: the token rows go through LDS for every K
template <int EPI, int MMAX, int NL>
static int launch_rows_mk(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda, hipStream_t s) {
  if constexpr (MMAX * NL <= 48) {
    if (g_rows_direct) {
      gemv_rows_direct_kernel<EPI, MMAX, NL><<<(N + 3) / 4, 256, 0, s>>>(A, W, out, M, N, K, lda);
      return 0;
    }
  }
  const size_t lds = (size_t)M * K * 2;
  auto kern = gemv_rows_kernel<EPI, MMAX, NL>;
  static size_t allowed = 48 * 1024;
  if (lds > allowed) {
    TI_REQUIRE(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) ==
                   hipSuccess, "gemm_bf16: LDS size refused");
    allowed = lds;
  }
  kern<<<(N + 3) / 4, 256, lds, s>>>(A, W, out, M, N, K, lda);
  return 0;
}
template <int EPI, int MMAX>
static int launch_rows_m(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda, hipStream_t s) {
  if (K <= 1024) return launch_rows_mk<EPI, MMAX, 2>(A, W, out, M, N, K, lda, s);
  if (K <= 2048) return launch_rows_mk<EPI, MMAX, 4>(A, W, out, M, N, K, lda, s);
  if (K <= 3072) return launch_rows_mk<EPI, MMAX, 6>(A, W, out, M, N, K, lda, s);
  return launch_rows_mk<EPI, MMAX, GR_LOADS>(A, W, out, M, N, K, lda, s);
}
// the kernel is compiled for 1, 2, 4 and GR_MMAX tokens and four lengths of K; a row's bits are
// the same in all of them
template <int EPI>
static int launch_rows(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda, hipStream_t s) {
  if (M <= 1) return launch_rows_m<EPI, 1>(A, W, out, M, N, K, lda, s);
  if (M <= 2) return launch_rows_m<EPI, 2>(A, W, out, M, N, K, lda, s);
  if (M <= 4) return launch_rows_m<EPI, 4>(A, W, out, M, N, K, lda, s);
  return launch_rows_m<EPI, GR_MMAX>(A, W, out, M, N, K, lda, s);
}

template <class Producer, int EPI, int NW, int UN = 4>
static int launch_staged(const char* what, Producer producer, const bf16_t* w, void* out, int M, int N, int K,
                         int grid, hipStream_t stream) {
  const size_t lds = (size_t)M * (K + 8) * 2;
  auto kern = gemm_skinny_staged_kernel<Producer, EPI, NW, UN>;
  static size_t allowed = 48 * 1024;   // per instantiation: the largest size asked for so far
  if (lds > allowed) {
    TI_REQUIRE(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) ==
                   hipSuccess, "%s: LDS size refused", what);
    allowed = lds;
  }
  kern<<<grid, NW * 64, lds, stream>>>(producer, w, out, M, N, K);
  TI_LAUNCH_CHECK();
  return 0;
}

// The number of wavefronts the plain skinny kernel takes for this weight: the kernels that
// make their rows themselves take the same, so that they give the same bits.
// (not under a weight of 8 Mi elements or more: there the kernel that takes the token rows in pieces, four
// wavefronts, is faster: Qwen3-1.7B's down projection, 2,048 x 6,144, at 8 tokens 12.2 -> 9.2 us)
static int skinny_waves_for(int grid, int K) {
  return g_skinny_waves ? g_skinny_waves : ((grid <= 128 && K >= 1024 && (long)grid * K < (512L << 10)) ? 8 : 4);
}

static bool pieces_serves(int M, int N, int K, int epi);
#define NORMED_WEIGHT_BELOW (40L << 20)   // weight elements from which the norm stays a kernel of its own
static long g_normed_weight_below = NORMED_WEIGHT_BELOW;
// out = rmsnorm(x; nw, eps) W^T for M <= 16 (see gemm_skinny_staged_kernel).  Returns 3 for
// sizes it does not serve (M > 16, K not a multiple of 64 or above 4096).
extern "C" int ti_gemm_bf16_normed(const float* x, const float* nw, float eps, const void* W, void* out,
                                   int M, int N, int K, int epi, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16_normed: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M > 16 || K % 64 != 0 || K > 4096 || ((uintptr_t)W & 15) || ((uintptr_t)x & 15) || ((uintptr_t)nw & 15)) {
    ti_set_error("gemm_bf16_normed: M=%d K=%d is not served (M <= 16, K %% 64 == 0, K <= 4096)", M, K);
    return 3;
  }
  if (row_per_wave_serves(M, N, K, epi)) {
    // the plain product of these sizes takes another kernel, with another order of summation: the
    // caller norms first and takes that one too, so that the norm in front changes no bit
    ti_set_error("gemm_bf16_normed: M=%d N=%d is left to the kernel with a weight row per wavefront", M, N);
    return 3;
  }
  if (large_weight(M, N, K, epi) && g_use_pipelined) {
    ti_set_error("gemm_bf16_normed: M=%d times a weight of %d x %d is left to the tiled kernels", M, N, K);
    return 3;
  }
  // Every workgroup here norms all M rows for itself, which pulls as many bytes through the caches as
  // its share of the weight has.  Under a large weight the kernel that keeps loads in flight gains more
  // than the norm's own launch costs (Qwen3-8B's gate/up, 100 M elements, at 8 rows: 46 us here, 38 + 5 us
  // there; Qwen3-4B's, 50 M: 29 against 21 + 2.5; Qwen3-1.7B's, 25 M, and 8B's q/k/v are faster here).
  if ((long)(epi == TI_EPI_SWIGLU ? 2 : 1) * N * K >= g_normed_weight_below && pieces_serves(M, N, K, epi)) {
    ti_set_error("gemm_bf16_normed: a weight of %d x %d is left to the norm's kernel and the product's", N, K);
    return 3;
  }
  if (M == 0) return 0;
  const bf16_t* w = (const bf16_t*)W;
  const int grid = (epi == TI_EPI_SWIGLU) ? (N + 7) / 8 : (N + 15) / 16;
  const int kc = (K + 255) / 256;
  const int waves = skinny_waves_for(grid, K);
#define TI_GNK(E, KCV)                                                                                          \
  return waves == 8                                                                                             \
             ? launch_staged<NormProducer<KCV>, E, 8>("gemm_bf16_normed", NormProducer<KCV>{x, nw, eps}, w, out, \
                                                      M, N, K, grid, stream)                                    \
             : launch_staged<NormProducer<KCV>, E, 4>("gemm_bf16_normed", NormProducer<KCV>{x, nw, eps}, w, out, \
                                                      M, N, K, grid, stream);
#define TI_GN(E)                        \
  case E:                               \
    if (kc <= 4) TI_GNK(E, 4)           \
    else if (kc <= 8) TI_GNK(E, 8)      \
    else TI_GNK(E, 16)
  switch (epi) {
    TI_GN(TI_EPI_STORE_F32)
    TI_GN(TI_EPI_ADD_F32)
    TI_GN(TI_EPI_STORE_ACT)
    TI_GN(TI_EPI_SWIGLU)
    default:
      TI_REQUIRE(false, "gemm_bf16_normed: unknown epilogue %d", epi);
  }
#undef TI_GN
#undef TI_GNK
  return 0;
}

// 1 (default): up to 16 tokens with K a multiple of 64 up to 4096, the token rows are copied into
// LDS once per workgroup (see CopyProducer); 0: every wavefront fetches its fragments from memory
static int g_skinny_copy = 1;

template <int EPI>
static int launch_skinny_copied(const bf16_t* A, const bf16_t* W, void* out, int M, int N, int K, long lda,
                                hipStream_t s) {
  const int grid = (EPI == TI_EPI_SWIGLU) ? (N + 7) / 8 : (N + 15) / 16;
  int waves = g_skinny_waves;
  if (waves == 0) waves = (grid <= 128 && K >= 1024) ? 8 : 4;         // as the plain kernel: same bits
  const bool deep = K / 64 > 4 * waves && g_skinny_deep;
  CopyProducer pr{A, lda};
  if (waves == 8)
    return deep ? launch_staged<CopyProducer, EPI, 8, 8>("gemm_bf16", pr, W, out, M, N, K, grid, s)
                : launch_staged<CopyProducer, EPI, 8, 4>("gemm_bf16", pr, W, out, M, N, K, grid, s);
  return deep ? launch_staged<CopyProducer, EPI, 4, 8>("gemm_bf16", pr, W, out, M, N, K, grid, s)
              : launch_staged<CopyProducer, EPI, 4, 4>("gemm_bf16", pr, W, out, M, N, K, grid, s);
}

// ---------------------------------------------------------------------------------------------
// 17 to 64 rows: 16x16x32 MFMAs fed straight from memory.  A workgroup takes 16 rows of W (16
// output columns; SwiGLU: 8 gate and 8 up rows) and a range of K; its four wavefronts take the
// 64-wide k-blocks of that range in turn, each block as MB + 1 pairs of 16-byte loads per lane
// (lane -> row lane % 16, 8 k at 8 (lane / 16), first and second half of the block) and 2 MB
// MFMAs over all 16 MB rows of A.  The four wavefronts' sums meet in LDS, in the order 0..3.
// With a weight of few rows the launch would fill a fraction of the compute units and every
// workgroup would pull in all of A: then K is split over KS workgroups, which leave their sums
// in `partial` [KS][M][N], and gemm_partials_add_kernel adds them to the residual in the order
// 0..KS-1.  A row's bits do not depend on the other rows.
#define MBK_STRIDE 20   // floats per row of the LDS tile: the 4 x 16 lanes of a store hit 64 banks

template <int MB, int EPI>
__global__ void __launch_bounds__(256)
gemm_mblocks_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ out_,
                    float* __restrict__ partial, int M, int N, int K, long lda) {
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  constexpr int TILE = SW ? 8 : 16;                          // output columns of a workgroup
  __shared__ __attribute__((aligned(16))) float red[4][MB * 16][MBK_STRIDE];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * TILE;
  const int KS = gridDim.y, split = blockIdx.y;
  const int nb = K / 64;
  const int kb0 = (int)((long)nb * split / KS), kb1 = (int)((long)nb * (split + 1) / KS);

  // rows outside the matrices read a valid row; what they give is not stored
  const bf16_t* arow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) arow[mb] = A + (size_t)min(mb * 16 + r, M - 1) * lda + g * 8;
  int wr;
  if (SW) wr = (r < 8) ? min(n0 + r, N - 1) : N + min(n0 + r - 8, N - 1);
  else wr = min(n0 + r, N - 1);
  const bf16_t* wrow = W + (size_t)wr * K + g * 8;

  struct Block { uint4 a[MB][2]; uint4 b[2]; };
  auto load = [&](Block& f, int kb) {
    const int k = kb * 64;
    f.b[0] = *reinterpret_cast<const uint4*>(wrow + k);
    f.b[1] = *reinterpret_cast<const uint4*>(wrow + k + 32);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      f.a[mb][0] = *reinterpret_cast<const uint4*>(arow[mb] + k);
      f.a[mb][1] = *reinterpret_cast<const uint4*>(arow[mb] + k + 32);
    }
  };
  floatx4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
  int kb = kb0 + wave;
  if (kb < kb1) {
    Block cur;
    load(cur, kb);
    while (kb < kb1) {
      // the next block is asked for before this one is multiplied (after the last one, the last again)
      Block next;
      load(next, min(kb + 4, kb1 - 1));
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, cur.a[mb][h]),
                                                            __builtin_bit_cast(bf16x8, cur.b[h]), acc[mb], 0, 0, 0);
      cur = next;
      kb += 4;
    }
  }
  // acc[mb][q]: row 16 mb + 4 g + q, column r
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int q = 0; q < 4; ++q) red[wave][mb * 16 + 4 * g + q][r] = acc[mb][q];
  __syncthreads();
  if (SW) {
    // thread -> a row and 4 of the 8 columns: gate in columns 0..7 of the tile, up in 8..15
    const int row = tid >> 1, c = (tid & 1) * 4;
    if (row >= MB * 16 || row >= M) return;
    float gt[4] = {0.f, 0.f, 0.f, 0.f}, up[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        gt[i] += red[w][row][c + i];
        up[i] += red[w][row][8 + c + i];
      }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n0 + c + i < N) ((bf16_t*)out_)[(size_t)row * N + n0 + c + i] = f2bf(silu_mul(gt[i], up[i]));
    return;
  }
  const int row = tid >> 2, c = (tid & 3) * 4;
  if (row >= MB * 16 || row >= M) return;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < 4; ++w)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += red[w][row][c + i];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = n0 + c + i;
    if (n >= N) continue;
    const size_t o = (size_t)row * N + n;
    if (EPI == TI_EPI_ADD_F32 && KS > 1) partial[(size_t)split * M * N + o] = v[i];
    else if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] += v[i];
    else if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = v[i];
    else ((bf16_t*)out_)[o] = f2bf(v[i]);
  }
}

// out[i] += partial[0][i] + ... + partial[KS - 1][i], in that order
__global__ void __launch_bounds__(256)
gemm_partials_add_kernel(float* __restrict__ out, const float* __restrict__ partial, int KS, size_t count) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = out[i];
  for (int s = 0; s < KS; ++s) v += partial[(size_t)s * count + i];
  out[i] = v;
}

// 17 to 64 rows times a weight of very many rows (the head: 151,936): the same MFMAs, but a
// workgroup keeps its share of A in registers (wavefront w of NW the k-blocks w, w + NW, ..., at
// most four) and walks over tiles of 16 weight rows, blockIdx.x, blockIdx.x + gridDim.x, ...: the
// weight streams through once, and A is read once per workgroup instead of once per tile (with a
// workgroup per tile the 9,496 tiles of the head pulled 1.2 GB of A through the caches: 170 us at
// 64 rows, against ~60 us for the weight alone).  The next tile's weight fragments are asked for
// before this tile is multiplied.  Stores 32-bit results; a row's bits do not depend on the others.
template <int MB, int NW>
__global__ void __launch_bounds__(64 * NW)
gemm_wide_rows_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, float* __restrict__ out, int M,
                      int N, int K, long lda) {
  constexpr int BPW = 4;                                     // k-blocks of 64 per wavefront at most
  __shared__ __attribute__((aligned(16))) float red[2][NW][MB * 16][MBK_STRIDE];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int nb = K / 64, tiles = (N + 15) / 16;
  // this wavefront's k-blocks: block j is k-block wave + NW j (one past the end repeats the last
  // and is not multiplied)
  int kof[BPW];
  bool live[BPW];
#pragma unroll
  for (int j = 0; j < BPW; ++j) {
    live[j] = wave + NW * j < nb;
    kof[j] = min(wave + NW * j, nb - 1) * 64 + g * 8;
  }
  uint4 a[BPW][MB][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const bf16_t* arow = A + (size_t)min(mb * 16 + r, M - 1) * lda;
#pragma unroll
    for (int j = 0; j < BPW; ++j) {
      a[j][mb][0] = *reinterpret_cast<const uint4*>(arow + kof[j]);
      a[j][mb][1] = *reinterpret_cast<const uint4*>(arow + kof[j] + 32);
    }
  }
  auto load_w = [&](uint4 (&b)[BPW][2], int tile) {
    const bf16_t* wrow = W + (size_t)min(tile * 16 + r, N - 1) * K;
#pragma unroll
    for (int j = 0; j < BPW; ++j) {
      b[j][0] = *reinterpret_cast<const uint4*>(wrow + kof[j]);
      b[j][1] = *reinterpret_cast<const uint4*>(wrow + kof[j] + 32);
    }
  };
  int tile = blockIdx.x;
  if (tile >= tiles) return;
  uint4 cur[BPW][2];
  load_w(cur, tile);
  for (int it = 0; tile < tiles; ++it, tile += gridDim.x) {
    uint4 next[BPW][2];
    load_w(next, min(tile + (int)gridDim.x, tiles - 1));
    floatx4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < BPW; ++j)
      if (live[j]) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[j][mb][h]),
                                                              __builtin_bit_cast(bf16x8, cur[j][h]), acc[mb], 0, 0, 0);
      }
    // the wavefronts' sums meet in LDS, in the order 0..NW-1; two buffers take turns, so that one
    // barrier a tile is enough (a wavefront two tiles ahead would have to pass the barrier between)
    float (*rd)[MB * 16][MBK_STRIDE] = red[it & 1];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int q = 0; q < 4; ++q) rd[wave][mb * 16 + 4 * g + q][r] = acc[mb][q];
    __syncthreads();
    for (int e = tid; e < MB * 16 * 4; e += 64 * NW) {
      const int row = e >> 2, c = (e & 3) * 4;
      if (row >= M) continue;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += rd[w][row][c + i];
      const int n = tile * 16 + c;
      float* dst = out + (size_t)row * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) dst[i] = v[i];
      }
    }
#pragma unroll
    for (int j = 0; j < BPW; ++j) {
      cur[j][0] = next[j][0];
      cur[j][1] = next[j][1];
    }
  }
}

static int g_wide_rows = 1;      // a hook for measurements: 0: the kernel above serves nothing
#define WIDE_ROWS_MIN_N 16384

// whether gemm_wide_rows_kernel takes the product (storing 32-bit results)
static int g_wide_rows_min_n = WIDE_ROWS_MIN_N, g_wide_rows_grid = 0;     // hooks for measurements
static bool wide_rows_serves(int M, int N, int K, int epi) {
  return g_wide_rows && epi == TI_EPI_STORE_F32 && M > 16 && M <= 64 && N >= g_wide_rows_min_n && K % 64 == 0 &&
         K / 64 <= 4 * 8;
}

static void launch_wide_rows(const bf16_t* a, const bf16_t* w, float* out, int M, int N, int K, long lda,
                             hipStream_t s) {
  const int mb = (M + 15) / 16, tiles = (N + 15) / 16;
  const bool eight = K / 64 > 4 * 4;                         // more than 16 k-blocks: eight wavefronts
  int dev = 0, units = 256;
  hipDeviceProp_t prop;
  static int cached_units = 0;
  if (!cached_units) {
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) units = prop.multiProcessorCount;
    cached_units = units > 0 ? units : 256;
  }
  const int grid = g_wide_rows_grid > 0 ? min(tiles, g_wide_rows_grid) : min(tiles, cached_units);
#define TI_GO(MBV)                                                                                   \
  if (eight) gemm_wide_rows_kernel<MBV, 8><<<grid, 512, 0, s>>>(a, w, out, M, N, K, lda);            \
  else gemm_wide_rows_kernel<MBV, 4><<<grid, 256, 0, s>>>(a, w, out, M, N, K, lda)
  if (mb == 2) { TI_GO(2); }
  else if (mb == 3) { TI_GO(3); }
  else { TI_GO(4); }
#undef TI_GO
}

template <int EPI, int AV, bool SPLIT>
static int launch_pieces_av(const bf16_t* a, long lda, const bf16_t* w, void* out, float* partial, int M, int N, int K,
                            int KS, hipStream_t s) {
  const size_t lds = (size_t)2 * M * SP_LD * 2;
  auto kern = gemm_skinny_pieces_kernel<EPI, AV, SPLIT>;
  static size_t allowed = 48 * 1024;
  if (lds > allowed) {
    TI_REQUIRE(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,
               "gemm_bf16: LDS size refused");
    allowed = lds;
  }
  const int tile = (EPI == TI_EPI_SWIGLU) ? 8 : 16;
  kern<<<dim3((N + tile - 1) / tile, KS), 256, lds, s>>>(a, lda, w, out, partial, M, N, K);
  return 0;
}
template <int EPI, bool SPLIT>
static int launch_pieces(const bf16_t* a, long lda, const bf16_t* w, void* out, float* partial, int M, int N, int K, int KS,
                         hipStream_t s) {
  if (M <= 2) return launch_pieces_av<EPI, 1, SPLIT>(a, lda, w, out, partial, M, N, K, KS, s);
  if (M <= 4) return launch_pieces_av<EPI, 2, SPLIT>(a, lda, w, out, partial, M, N, K, KS, s);
  if (M <= 8) return launch_pieces_av<EPI, 4, SPLIT>(a, lda, w, out, partial, M, N, K, KS, s);
  return launch_pieces_av<EPI, 8, SPLIT>(a, lda, w, out, partial, M, N, K, KS, s);
}

// 1 (default): up to 16 rows times a weight whose K is a multiple of 64 and at least two pieces long
// take the kernel with the token rows in pieces; 0: the kernels above it (for comparison)
static int g_pieces = 1;
static bool pieces_serves(int M, int N, int K, int epi) {
  if (!g_pieces || M > 16 || K % 64 != 0 || K < 2 * SP_PIECE) return false;
  if (epi < TI_EPI_STORE_F32 || epi > TI_EPI_SWIGLU) return false;
  // few tokens times a weight of few rows: a row per wavefront wins (and fills the compute units)
  if (row_per_wave_serves(M, N, K, epi)) return false;
  // where the kernels with the norm in front take eight wavefronts, this one would give other bits
  const int grid = (epi == TI_EPI_SWIGLU) ? (N + 7) / 8 : (N + 15) / 16;
  return skinny_waves_for(grid, K) == 4;
}
// Into how many workgroups the pieces of K go when the product adds into the residual: a long K under
// few rows of weight leaves a launch of few workgroups that each walk a long way (Qwen3-32B's down
// projection: 320 workgroups, 25 pieces each, 3.1 TB/s; split four ways 4.8 TB/s).  By the weight's
// shape alone, so that a row's bits do not depend on the rows beside it.
static int pieces_splits(int N, int K, long partial_bytes) {
  const int n_pieces = (K + SP_PIECE - 1) / SP_PIECE;
  if (n_pieces < 16) return 1;      // (from 8 pieces on: Qwen3-4B's and 8B's down projections lose 1-3 % of the step)
  const int grid = (N + 15) / 16;
  int ks = std::min(n_pieces / 4, (4 * compute_units() + grid - 1) / grid);
  while (ks > 1 && (long)ks * 16 * N * 4 > partial_bytes) --ks;
  return ks < 1 ? 1 : ks;
}

static int g_add_split = 1;        // a hook for measurements: 0: ti_gemm_bf16_add_split serves nothing

template <int EPI>
static void launch_mblocks(const bf16_t* a, const bf16_t* w, void* out, float* partial, int M, int N, int K,
                           long lda, int KS, hipStream_t s) {
  const int tile = (EPI == TI_EPI_SWIGLU) ? 8 : 16;
  dim3 grid((N + tile - 1) / tile, KS);
  const int mb = (M + 15) / 16;
  if (mb == 1) gemm_mblocks_kernel<1, EPI><<<grid, 256, 0, s>>>(a, w, out, partial, M, N, K, lda);
  else if (mb == 2) gemm_mblocks_kernel<2, EPI><<<grid, 256, 0, s>>>(a, w, out, partial, M, N, K, lda);
  else if (mb == 3) gemm_mblocks_kernel<3, EPI><<<grid, 256, 0, s>>>(a, w, out, partial, M, N, K, lda);
  else gemm_mblocks_kernel<4, EPI><<<grid, 256, 0, s>>>(a, w, out, partial, M, N, K, lda);
}

// out[i] += partial[0][i] + ... + partial[KS - 1][i] for count elements: what a product with a split
// K leaves to do (see ti_gemm_bf16_add_split)
extern "C" int ti_gemm_bf16_partials_add(float* out, const float* partial, int KS, long count, hipStream_t stream) {
  TI_REQUIRE(KS >= 1 && count >= 0, "gemm_bf16_partials_add: bad sizes KS=%d count=%ld", KS, count);
  if (count == 0) return 0;
  gemm_partials_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(out, partial, KS, (size_t)count);
  TI_LAUNCH_CHECK();
  return 0;
}

// The product that adds into the 32-bit residual, for steps of more than 16 rows whose launch would
// leave most compute units idle (few rows times a weight of few rows): K is split over workgroups,
// which leave their sums in `partial` [KS][M][N] (workspace of partial_bytes).  17..64 rows:
// gemm_mblocks_kernel (measured against the kernels without MFMA at 64 rows: 1024 x 3072 19.7 ->
// 9.7 us with the addition of the partial sums as a kernel of its own, ~6 us without).  More rows:
// the pipelined kernel with 64 x 64 tiles, storing (136 rows: 18.5 -> ~8 us).
// Up to 16 rows: the kernel with the token rows in pieces, where pieces_splits says so.
// defer = 0: the partial sums are added to `out` here, and only what gains even so is served.
// defer = 1: they are left in `partial`, *splits gets their number, and the caller sees to the
// addition (ti_gemm_bf16_partials_add, or a kernel that reads the residual next and adds them on
// the way).  defer = 2: what defer = 1 serves, added here (the same bits).  Returns 3 for what
// it does not serve.
extern "C" int ti_gemm_bf16_add_split(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                                    void* partial, long partial_bytes, int defer, int* splits, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K, "gemm_bf16_add_split: bad sizes M=%d N=%d K=%d lda=%ld", M, N, K, lda);
  TI_REQUIRE(splits != nullptr, "gemm_bf16_add_split: splits must point to an int");
  *splits = 0;
  if (M <= 16 && M > 0 && g_add_split && epi == TI_EPI_ADD_F32 && partial && lda % 8 == 0 && !((uintptr_t)A & 15) &&
      !((uintptr_t)W & 15) && !((uintptr_t)partial & 15) && pieces_serves(M, N, K, epi)) {
    const int ks = pieces_splits(N, K, partial_bytes);
    if (ks > 1) {
      int rc_ = launch_pieces<TI_EPI_ADD_F32, true>((const bf16_t*)A, lda, (const bf16_t*)W, out, (float*)partial, M, N, K, ks,
                                                    stream);
      if (rc_) return rc_;
      if (defer == 1) {
        *splits = ks;
      } else {
        const size_t count = (size_t)M * N;
        gemm_partials_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((float*)out, (const float*)partial,
                                                                                    ks, count);
      }
      TI_LAUNCH_CHECK();
      return 0;
    }
  }
  int KS = 1;
  const bool small = M <= 64 && !(large_weight(M, N, K, epi) && g_use_pipelined);
  if (g_add_split && epi == TI_EPI_ADD_F32 && partial && M > 16 && K % 64 == 0 && lda % 8 == 0 &&
      !((uintptr_t)A & 15) && !((uintptr_t)W & 15) && !((uintptr_t)partial & 15) && (small || g_use_pipelined)) {
    // split K until the launch has about a workgroup per compute unit
    const long tiles = small ? (N + 15) / 16 : (long)((M + 63) / 64) * ((N + 63) / 64);
    const int nb = K / 64;
    // (a large weight is waited for from memory: then about four workgroups per unit, so that enough
    // of it is on its way at any time)
    // as long as the partial sums stay a small part of what the weight has in bytes
    const bool streamed = !small && (long)N * K >= (8L << 20);
    while (KS < 8 && tiles * KS * 2 <= compute_units() && nb / (KS * 2) >= 4) KS *= 2;
    if (streamed)
      while (KS < 8 && tiles * KS * 2 <= 4L * compute_units() && nb / (KS * 2) >= 4 && (long)KS * 2 * M * 16 <= K) KS *= 2;
    while (KS > 1 && (long)KS * M * N * 4 > partial_bytes) KS /= 2;
    // with the addition as a kernel of its own, only large products gain
    if (!defer && small && !((long)M * K >= 128 * 1024 || (K >= 3072 && (long)M * K >= 96 * 1024))) KS = 1;
    if (!defer && !small && KS < 4) KS = 1;
  }
  // Many rows times a weight of few rows (o and down of a whole prompt): 64 x 64 tiles are what fills
  // the chip, and they pull four bytes into a compute unit where a 128 x 128 tile pulls two.  When the
  // 128 x 128 tiles are at most half as many as the units, K is split between two to four workgroups
  // per tile instead: the same bytes as one round of 128 x 128 tiles, on all units.
  // (not under a weight of 64 Mi elements or more: Qwen3-32B's down projection at 264 rows 164 -> 199 us)
  if (KS == 1 && !small && g_add_split && g_use_pipelined && defer && epi == TI_EPI_ADD_F32 && partial && M >= 256 &&
      (long)N * K < (64L << 20) && K % 64 == 0 && lda % 8 == 0 && !((uintptr_t)A & 15) && !((uintptr_t)W & 15) && !((uintptr_t)partial & 15)) {
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    int ks = (int)std::min<long>(4, compute_units() / std::max<long>(1, tiles128));
    while (ks > 1 && ((K / 64) / ks < 8 || (long)ks * M * N * 4 > partial_bytes)) --ks;
    if (ks >= 2) {
      int rc_ = launch_pipelined<128, 128, 2, 4, TI_EPI_STORE_F32>((const bf16_t*)A, (const bf16_t*)W, partial, M, N, K, lda,
                                                                   stream, ks);
      if (rc_) return rc_;
      if (defer == 1) {
        *splits = ks;
      } else {
        const size_t count = (size_t)M * N;
        gemm_partials_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((float*)out, (const float*)partial,
                                                                                    ks, count);
      }
      TI_LAUNCH_CHECK();
      return 0;
    }
  }
  if (KS == 1) {
    ti_set_error("gemm_bf16_add_split: serves more than 16 rows added into a product of few tiles, K a multiple of 64");
    return 3;
  }
  if (small) {
    launch_mblocks<TI_EPI_ADD_F32>((const bf16_t*)A, (const bf16_t*)W, out, (float*)partial, M, N, K, lda, KS, stream);
  } else {
    int rc_ = launch_pipelined<64, 64, 2, 2, TI_EPI_STORE_F32>((const bf16_t*)A, (const bf16_t*)W, partial, M, N, K, lda,
                                                               stream, KS);
    if (rc_) return rc_;
  }
  if (defer == 1) {
    *splits = KS;
  } else {
    const size_t count = (size_t)M * N;
    gemm_partials_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((float*)out, (const float*)partial,
                                                                                KS, count);
  }
  TI_LAUNCH_CHECK();
  return 0;
}

// the kernel with the token rows in pieces alone, for tests and measurements: any epilogue, 1..16
// rows, K a multiple of 64 split ks ways (1: not split; partial sums are added here)
extern "C" int ti_gemm_bf16_pieces_any(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                                       void* partial, int ks, hipStream_t stream) {
  TI_REQUIRE(M > 0 && M <= 16 && N > 0 && K > 0 && K % 64 == 0 && lda >= K && lda % 8 == 0 && ks >= 1 &&
                 ks <= (K + SP_PIECE - 1) / SP_PIECE,
             "gemm_bf16_pieces_any: bad sizes M=%d N=%d K=%d lda=%ld ks=%d", M, N, K, lda, ks);
  TI_REQUIRE(ks == 1 || (epi == TI_EPI_ADD_F32 && partial), "gemm_bf16_pieces_any: a split K needs the adding epilogue");
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  int rc = 0;
  switch (epi) {
    case TI_EPI_STORE_F32: rc = launch_pieces<TI_EPI_STORE_F32, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
    case TI_EPI_STORE_ACT: rc = launch_pieces<TI_EPI_STORE_ACT, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
    case TI_EPI_SWIGLU: rc = launch_pieces<TI_EPI_SWIGLU, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
    case TI_EPI_ADD_F32:
      if (ks == 1) {
        rc = launch_pieces<TI_EPI_ADD_F32, false>(a, lda, w, out, nullptr, M, N, K, 1, stream);
      } else {
        rc = launch_pieces<TI_EPI_ADD_F32, true>(a, lda, w, out, (float*)partial, M, N, K, ks, stream);
        const size_t count = (size_t)M * N;
        gemm_partials_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((float*)out, (const float*)partial,
                                                                                    ks, count);
      }
      break;
    default:
      TI_REQUIRE(false, "gemm_bf16_pieces_any: unknown epilogue %d", epi);
  }
  if (rc) return rc;
  TI_LAUNCH_CHECK();
  return 0;
}

// out[i] = partial[0][i] + ... + partial[KS - 1][i], in that order
__global__ void __launch_bounds__(256)
gemm_partials_sum_kernel(float* __restrict__ out, const float* __restrict__ partial, int KS, size_t count) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = partial[i];
  for (int s = 1; s < KS; ++s) v += partial[(size_t)s * count + i];
  out[i] = v;
}

// The product that stores 32-bit results, for 17 to 64 rows times a large weight whose 64 x 64 tiles
// are few (the q/k/v projection of a decode step of many requests with a large model: 96 to 160
// workgroups that wait for the weight from memory with too little of it under way).  K is split over
// four or eight workgroups a tile, which store their sums into `partial` [KS][M][N]; a kernel of its
// own adds them up into `out` (Qwen3-8B's q/k/v at 64 rows: 27 -> 17 us).  The number of shares
// depends on the weight's shape alone.  Returns 3 for what it does not serve.
extern "C" int ti_gemm_bf16_store_split(const void* A, const void* W, void* out, int M, int N, int K, long lda,
                                        void* partial, long partial_bytes, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K, "gemm_bf16_store_split: bad sizes M=%d N=%d K=%d lda=%ld", M, N, K, lda);
  int KS = 1;
  if (g_add_split && g_use_pipelined && partial && M > 16 && M <= 64 && K % 64 == 0 && lda % 8 == 0 &&
      !((uintptr_t)A & 15) && !((uintptr_t)W & 15) && !((uintptr_t)partial & 15) &&
      large_weight(M, N, K, TI_EPI_STORE_F32) && !wide_rows_serves(M, N, K, TI_EPI_STORE_F32)) {
    const long tiles = (N + 63) / 64;
    const int nb = K / 64;
    while (KS < 8 && tiles * KS * 2 <= 4L * compute_units() && nb / (KS * 2) >= 4 && (long)KS * 2 * 64 * 16 <= K) KS *= 2;
    while (KS > 1 && (long)KS * M * N * 4 > partial_bytes) KS /= 2;
  }
  if (KS < 4) {
    ti_set_error("gemm_bf16_store_split: serves 17 to 64 rows times a large weight of few tiles, K a multiple of 64");
    return 3;
  }
  int rc_ = launch_pipelined<64, 64, 2, 2, TI_EPI_STORE_F32>((const bf16_t*)A, (const bf16_t*)W, partial, M, N, K, lda, stream,
                                                             KS);
  if (rc_) return rc_;
  const size_t count = (size_t)M * N;
  gemm_partials_sum_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((float*)out, (const float*)partial, KS, count);
  TI_LAUNCH_CHECK();
  return 0;
}

// hooks for tests of the kernel alone: any epilogue, K split `ks` ways (1: not split; partial sums
// are added here)
extern "C" int ti_gemm_bf16_mblocks_any(const void* A, const void* W, void* out, int M, int N, int K, long lda,
                                        int epi, void* partial, int ks, hipStream_t stream) {
  TI_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0 && K % 64 == 0 && lda >= K && lda % 8 == 0 && ks >= 1 && ks <= K / 64,
             "gemm_bf16_mblocks_any: bad sizes M=%d N=%d K=%d lda=%ld ks=%d", M, N, K, lda, ks);
  TI_REQUIRE(ks == 1 || (epi == TI_EPI_ADD_F32 && partial), "gemm_bf16_mblocks_any: a split K needs the adding epilogue");
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  switch (epi) {
    case TI_EPI_STORE_F32: launch_mblocks<TI_EPI_STORE_F32>(a, w, out, nullptr, M, N, K, lda, 1, stream); break;
    case TI_EPI_STORE_ACT: launch_mblocks<TI_EPI_STORE_ACT>(a, w, out, nullptr, M, N, K, lda, 1, stream); break;
    case TI_EPI_SWIGLU: launch_mblocks<TI_EPI_SWIGLU>(a, w, out, nullptr, M, N, K, lda, 1, stream); break;
    case TI_EPI_ADD_F32:
      launch_mblocks<TI_EPI_ADD_F32>(a, w, out, (float*)partial, M, N, K, lda, ks, stream);
      if (ks > 1) {
        const size_t count = (size_t)M * N;
        gemm_partials_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>((float*)out, (const float*)partial,
                                                                                    ks, count);
      }
      break;
    default:
      TI_REQUIRE(false, "gemm_bf16_mblocks_any: unknown epilogue %d", epi);
  }
  TI_LAUNCH_CHECK();
  return 0;
}


// N: output columns (SwiGLU: F, with W holding 2F rows).  Returns 3 for a shape
// these kernels do not serve (the caller takes the generic kernel then).
extern "C" int ti_gemm_bf16(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                            hipStream_t stream) {
  TI_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K, "gemm_bf16: bad sizes M=%d N=%d K=%d lda=%ld", M, N, K, lda);
  if (K % 8 != 0 || lda % 8 != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) {
    ti_set_error("gemm_bf16: K=%d / lda=%ld not multiples of 8 or operands not 16-byte aligned", K, lda);
    return 3;
  }
  if ((M + TBM - 1) / TBM > 65535) {
    ti_set_error("gemm_bf16: M=%d too large for one launch", M);
    return 3;
  }
  if (M == 0) return 0;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  const bool skinny = M <= 64 && !(large_weight(M, N, K, epi) && g_use_pipelined);
  const bool copied = g_skinny_copy && M <= 16 && K % 64 == 0 && K <= 4096 && skinny;
  if (pieces_serves(M, N, K, epi)) {
    int rc_ = 0;
    switch (epi) {
      case TI_EPI_STORE_F32: rc_ = launch_pieces<TI_EPI_STORE_F32, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
      case TI_EPI_ADD_F32: rc_ = launch_pieces<TI_EPI_ADD_F32, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
      case TI_EPI_STORE_ACT: rc_ = launch_pieces<TI_EPI_STORE_ACT, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
      default: rc_ = launch_pieces<TI_EPI_SWIGLU, false>(a, lda, w, out, nullptr, M, N, K, 1, stream); break;
    }
    if (rc_) return rc_;
    TI_LAUNCH_CHECK();
    return 0;
  }
  if (wide_rows_serves(M, N, K, epi)) {
    launch_wide_rows(a, w, (float*)out, M, N, K, lda, stream);
    TI_LAUNCH_CHECK();
    return 0;
  }
  if (row_per_wave_serves(M, N, K, epi)) {
    int rc_ = 0;
    if (epi == TI_EPI_STORE_F32) rc_ = launch_rows<TI_EPI_STORE_F32>(a, w, out, M, N, K, lda, stream);
    else rc_ = launch_rows<TI_EPI_ADD_F32>(a, w, out, M, N, K, lda, stream);
    if (rc_) return rc_;
    TI_LAUNCH_CHECK();
    return 0;
  }
#define TI_GO(E)                                                  \
  case E:                                                         \
    if (copied) {                                                 \
      int rc_ = launch_skinny_copied<E>(a, w, out, M, N, K, lda, stream); \
      if (rc_) return rc_;                                        \
    } else if (skinny)                                            \
      launch_skinny<E>(a, w, out, M, N, K, lda, stream);          \
    else if (g_use_pipelined && K % PBK == 0) {                   \
      int rc_ = launch_tiled_best<E>(a, w, out, M, N, K, lda, stream); \
      if (rc_) return rc_;                                        \
    } else                                                        \
      launch_tiled<E>(a, w, out, M, N, K, lda, stream);           \
    break;
  switch (epi) {
    TI_GO(TI_EPI_STORE_F32)
    TI_GO(TI_EPI_ADD_F32)
    TI_GO(TI_EPI_STORE_ACT)
    TI_GO(TI_EPI_SWIGLU)
    default:
      TI_REQUIRE(false, "gemm_bf16: unknown epilogue %d", epi);
  }
#undef TI_GO
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------- tests and measurements
// One entry for every shape rule above that a test or a measurement may want to force: `name` as in
// tinyinfer_kernels_tuning.h, value 0 (or what the table says) restores the rule's own choice.
// The rules are the library's, process-wide; the host library's Ops applies an object's own
// overrides around its calls and resets them afterwards.  Returns 0, or 1 for an unknown name.
extern "C" void ti_tuning_reset() {
  g_xcd_rows = 0; g_tiles_160 = 1; g_tiles_256 = 1; g_two_ranges = 1; g_qkv_rows = 0; g_qkv_min_rows = 17; g_force_tile = 0; g_skinny_waves = 0;
  g_skinny_deep = 1; g_use_pipelined = 1; set_tiled_from(280L << 20); g_row_per_wave = 1;
  g_normed_weight_below = NORMED_WEIGHT_BELOW; g_skinny_copy = 1; g_wide_rows = 1; g_pieces = 1; g_add_split = 1;
  g_rows_direct = 1;
  g_wide_rows_min_n = WIDE_ROWS_MIN_N;
  g_wide_rows_grid = 0;
}
extern "C" int ti_tuning_set(const char* name, long value) {
  const std::string n = name ? name : "";
  if (n == "force_tile") g_force_tile = (int)value;
  else if (n == "normed_weight_below") g_normed_weight_below = value > 0 ? value : NORMED_WEIGHT_BELOW;
  else if (n == "tiles_160") g_tiles_160 = (int)value;
  else if (n == "tiles_256") g_tiles_256 = (int)value;
  else if (n == "two_ranges") g_two_ranges = (int)value;
  else if (n == "xcd_rows") g_xcd_rows = (int)value;
  else if (n == "skinny_waves") g_skinny_waves = (int)value;
  else if (n == "qkv_prep_min_rows") g_qkv_min_rows = (int)value;
  else if (n == "qkv_prep_rows") g_qkv_rows = (int)value;
  else if (n == "wide_rows") g_wide_rows = (int)value;
  else if (n == "tiled_from") set_tiled_from(value);
  else if (n == "add_split") g_add_split = (int)value;
  else if (n == "use_pipelined") g_use_pipelined = (int)value;
  else if (n == "row_per_wave") g_row_per_wave = (int)value;
  else if (n == "skinny_copy") g_skinny_copy = (int)value;
  else if (n == "pieces") g_pieces = (int)value;
  else if (n == "skinny_deep") g_skinny_deep = (int)value;
  else if (n == "rows_direct") g_rows_direct = (int)value;
  else if (n == "wide_rows_min_n") g_wide_rows_min_n = value > 0 ? (int)value : WIDE_ROWS_MIN_N;
  else if (n == "wide_rows_grid") g_wide_rows_grid = (int)value;
  else return 1;
  return 0;
}
