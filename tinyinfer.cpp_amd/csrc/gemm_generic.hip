// C = A W^T for any M, N, K, in true 32-bit arithmetic (FMA, no matrix-core
// mode): the matrix product of the float32 path, and the fallback of the
// bfloat16 path for shapes its fast kernels refuse (operands are widened to
// float, exactly).  A is [M, K], W is [N, K], both row-major in T.
//
// Every output element sums its K products in ascending k, whatever M is, so a
// token's result does not depend on what else is in the batch.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define GT 64   // tile of C: GT x GT
#define GK 16   // depth of one LDS stage

template <typename T, int EPI>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const T* __restrict__ A, const T* __restrict__ W, void* __restrict__ out_,
                    int M, int N, int K, long lda) {
  constexpr bool SW = (EPI == TI_EPI_SWIGLU);
  __shared__ float As[GK][GT + 4];
  __shared__ float Ws[GK][GT + 4];
  __shared__ float Us[SW ? GK : 1][GT + 4];   // the up rows, for SwiGLU
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  const int tid = threadIdx.x;
  const int ty = tid / 16, tx = tid % 16;
  const int lrow = tid / 4, lk = (tid % 4) * 4;
  float acc[4][4] = {};
  float accu[SW ? 4 : 1][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + j][lrow] = (am < M && k < K) ? ld<T>(A + (size_t)am * lda + k) : 0.f;
      Ws[lk + j][lrow] = (wn < N && k < K) ? ld<T>(W + (size_t)wn * K + k) : 0.f;
      if (SW) Us[lk + j][lrow] = (wn < N && k < K) ? ld<T>(W + (size_t)(wn + N) * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
      if (SW) {
        float u[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] = Us[kk][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) accu[i][j] = fmaf(a[i], u[j], accu[i][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      const size_t o = (size_t)m * N + n;
      if (EPI == TI_EPI_STORE_F32) ((float*)out_)[o] = acc[i][j];
      if (EPI == TI_EPI_ADD_F32) ((float*)out_)[o] += acc[i][j];
      if (EPI == TI_EPI_STORE_ACT) st<T>((T*)out_ + o, acc[i][j]);
      if (EPI == TI_EPI_SWIGLU) {
        const float g = acc[i][j];
        st<T>((T*)out_ + o, g / (1.0f + expf(-g)) * accu[SW ? i : 0][j]);
      }
    }
  }
}

template <typename T>
static int launch(const void* A, const void* W, void* out, int M, int N, int K, long lda, int epi,
                  hipStream_t stream) {
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
  switch (epi) {
    case TI_EPI_STORE_F32:
      gemm_generic_kernel<T, TI_EPI_STORE_F32><<<grid, 256, 0, stream>>>((const T*)A, (const T*)W, out, M, N, K, lda);
      break;
    case TI_EPI_ADD_F32:
      gemm_generic_kernel<T, TI_EPI_ADD_F32><<<grid, 256, 0, stream>>>((const T*)A, (const T*)W, out, M, N, K, lda);
      break;
    case TI_EPI_STORE_ACT:
      gemm_generic_kernel<T, TI_EPI_STORE_ACT><<<grid, 256, 0, stream>>>((const T*)A, (const T*)W, out, M, N, K, lda);
      break;
    case TI_EPI_SWIGLU:
      gemm_generic_kernel<T, TI_EPI_SWIGLU><<<grid, 256, 0, stream>>>((const T*)A, (const T*)W, out, M, N, K, lda);
      break;
    default:
      ti_set_error("gemm_generic: unknown epilogue %d", epi);
      return 1;
  }
  return 0;
}

// N is the number of output columns (for SwiGLU: F, with W holding 2F rows).
extern "C" int ti_gemm_generic(int dtype, const void* A, const void* W, void* out, int M, int N, int K,
                               long lda, int epi, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K, "gemm_generic: bad sizes M=%d N=%d K=%d lda=%ld", M, N, K, lda);
  TI_REQUIRE((M + GT - 1) / GT <= 65535, "gemm_generic: M=%d too large for one launch", M);
  if (M == 0) return 0;
  int rc;
  if (dtype == TI_F32)
    rc = launch<float>(A, W, out, M, N, K, lda, epi, stream);
  else if (dtype == TI_BF16)
    rc = launch<bf16_t>(A, W, out, M, N, K, lda, epi, stream);
  else {
    ti_set_error("gemm_generic: unknown dtype %d", dtype);
    return 1;
  }
  if (rc) return rc;
  TI_LAUNCH_CHECK();
  return 0;
}
