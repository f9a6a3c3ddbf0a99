// A kernel library that is no part of the framework: built by tests/test_plugin_gpu.py, registered by the
// plugin beside it under the name "toy_relu", and called through tinyinfer::kernel_symbol.
//   y[i] = T(alpha * max(u[i], 0))      u float32, y float32 (bf16 = 0) or bfloat16 (bf16 = 1)
#include <hip/hip_runtime.h>
#include <stdint.h>

__global__ void toy_relu_scale_kernel(const float* __restrict__ u, void* __restrict__ y, long n, float alpha, int bf16) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = alpha * fmaxf(u[i], 0.0f);
    if (bf16) {
      const uint32_t bits = __float_as_uint(v);
      ((uint16_t*)y)[i] = (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);      // to nearest, ties to even
    } else {
      ((float*)y)[i] = v;
    }
  }
}

extern "C" int toy_relu_scale(const float* u, void* y, long n, float alpha, int bf16, hipStream_t stream) {
  if (n <= 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024);
  toy_relu_scale_kernel<<<blocks, 256, 0, stream>>>(u, y, n, alpha, bf16);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}
