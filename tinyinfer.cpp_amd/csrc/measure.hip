// What this GPU delivers, measured: the bandwidth of a kernel that only reads memory, and the rate of
// matrix-core instructions whose operands never leave the registers.  bench.py reports its figures
// as fractions of these beside the fractions of the published peaks.  The reference times its own
// GEMV against the clock in the same spirit (/root/reference/src/selftest.cpp:392-428).
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

// every thread reads 16-byte pieces with a grid stride and adds them up; one word per workgroup is
// written so that the loads cannot be dropped
__global__ void __launch_bounds__(256) read_kernel(const uint4* __restrict__ p, long n16, unsigned* __restrict__ sink) {
  unsigned acc = 0;
  const long stride = (long)gridDim.x * blockDim.x;
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = p[i], b = p[i + stride], c = p[i + 2 * stride], d = p[i + 3 * stride];
    acc += a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n16; i += stride) {
    const uint4 a = p[i];
    acc += a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) sink[blockIdx.x] = acc;      // all but never true
}

// reads `bytes` bytes (a multiple of 16) once with `blocks` workgroups; sink: at least `blocks` words
extern "C" int ti_measure_read(const void* p, long bytes, void* sink, int blocks, hipStream_t stream) {
  TI_REQUIRE(bytes > 0 && bytes % 16 == 0 && blocks > 0, "measure_read: bad sizes bytes=%ld blocks=%d", bytes, blocks);
  read_kernel<<<blocks, 256, 0, stream>>>((const uint4*)p, bytes / 16, (unsigned*)sink);
  TI_LAUNCH_CHECK();
  return 0;
}

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// every wavefront runs `iters` rounds of four independent 32x32x16 bfloat16 MFMAs on registers.  The
// operands are scattered values (what the chip draws, and with it its clock, depends on the bits that
// toggle: all-zero operands run a fifth faster than a model's), different in every lane and round.
__global__ void __launch_bounds__(256) mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8_t a[4], b[4];
  unsigned h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 8; ++i) {
      h = h * 1664525u + 1013904223u;
      a[j][i] = (__bf16)(((int)(h >> 16) % 2001 - 1000) * 1e-3f);
      h = h * 1664525u + 1013904223u;
      b[j][i] = (__bf16)(((int)(h >> 16) % 2001 - 1000) * 2e-5f);
    }
  float16_t c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  for (int it = 0; it < iters; it += 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], b[j], c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 1) & 3], b[j], c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 2) & 3], b[j], c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 3) & 3], b[j], c3, 0, 0, 0);
    }
  }
  float s = 0.f;
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 12345.678f) sink[blockIdx.x] = s;
}

// `blocks` workgroups of four wavefronts; flops = blocks * 4 * iters * 4 * (2 * 32 * 32 * 16)
extern "C" int ti_measure_mfma(int blocks, int iters, void* sink, hipStream_t stream) {
  TI_REQUIRE(blocks > 0 && iters > 0, "measure_mfma: bad sizes blocks=%d iters=%d", blocks, iters);
  mfma_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  TI_LAUNCH_CHECK();
  return 0;
}

// every workgroup reads one word every `stride` bytes of [p, p + bytes): address translations and nothing else
__global__ void __launch_bounds__(64) touch_kernel(const char* __restrict__ p, long bytes, long stride, unsigned* __restrict__ sink) {
  unsigned acc = 0;
  for (long off = (long)threadIdx.x * stride; off < bytes; off += 64 * stride) acc += *(const unsigned*)(p + off);
  if (acc == 0x9e3779b9u) sink[blockIdx.x] = acc;
}

extern "C" int ti_measure_touch(const void* p, long bytes, long stride, void* sink, int blocks, hipStream_t stream) {
  TI_REQUIRE(bytes > 0 && stride >= 4 && stride % 4 == 0 && blocks > 0, "measure_touch: bad sizes");
  touch_kernel<<<blocks, 64, 0, stream>>>((const char*)p, bytes, stride, (unsigned*)sink);
  TI_LAUNCH_CHECK();
  return 0;
}
