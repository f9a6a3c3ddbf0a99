// Sampling parameters, the counter-based random stream, and the device sampler.
//
// The reference samples on the host: greedy argmax when the temperature is 0, else the K largest
// logits (K = --top-k, or 512 when that is 0), weights exp(l/T - max), an optional top-p cut, and
// one draw from a process-wide mt19937 shared by all sequences in turn
// (/root/reference/src/main.cpp:23-84).  Here the same options run on the device
// (csrc/sampling.hip), and the random stream is keyed by (seed, request number, index of the
// generated token): what a request draws does not depend on which other requests share its
// steps, nor on being preempted.
#include <hip/hip_runtime_api.h>

#include "../include/inference.h"

namespace tinyinfer {

static inline uint64_t mix(uint64_t z) {      // splitmix64's output function
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// A number in [0, 1) with 24 random bits (exact in float32), a pure function of its three keys.
float uniform(uint64_t seed, uint64_t request, uint64_t n_generated) {
  uint64_t z = mix(seed);
  z = mix(z ^ request);
  z = mix(z ^ n_generated);
  return (float)(z >> 40) / 16777216.0f;
}

struct Sampler::Buffers {
  int cap = 0;
  float* f_host = nullptr;     // temperature | top_p | uniform
  int* i_host = nullptr;       // top_k | ids read back
  DeviceBuffer f_dev, i_dev, out_dev;
  ~Buffers() {
    if (f_host) (void)hipHostFree(f_host);
    if (i_host) (void)hipHostFree(i_host);
  }
};

Sampler::Sampler(Ops& ops) : ops_(ops), b_(new Buffers()) {}
Sampler::~Sampler() {}

static void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw KernelError(std::string(what) + ": " + hipGetErrorString(e));
}

std::vector<int> Sampler::sample(const Tensor& logits, const std::vector<SamplingParams>& params,
                                 const std::vector<int64_t>& requests, const std::vector<int64_t>& counters) {
  const int n = (int)logits.shape[0];
  if ((int)params.size() != n || (int)requests.size() != n || (int)counters.size() != n)
    throw KernelError("sample: one set of parameters, one request number and one counter per row of logits");
  hipStream_t stream = (hipStream_t)ops_.stream();
  Buffers& b = *b_;
  if (n > b.cap) {
    hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    const int cap = std::max(64, 2 * n);
    if (b.f_host) (void)hipHostFree(b.f_host);
    if (b.i_host) (void)hipHostFree(b.i_host);
    hip_check(hipHostMalloc((void**)&b.f_host, (size_t)3 * cap * 4, hipHostMallocDefault), "hipHostMalloc");
    hip_check(hipHostMalloc((void**)&b.i_host, (size_t)2 * cap * 4, hipHostMallocDefault), "hipHostMalloc");
    b.f_dev = DeviceBuffer((size_t)3 * cap * 4);
    b.i_dev = DeviceBuffer((size_t)cap * 4);
    b.out_dev = DeviceBuffer((size_t)cap * 4);
    b.cap = cap;
  }
  bool greedy = true;
  for (const auto& p : params) greedy = greedy && p.temperature <= 0.f;
  int* out = (int*)b.out_dev.data();
  if (greedy) {
    ops_.argmax(logits, out);
  } else {
    const int cap = b.cap;
    for (int i = 0; i < n; ++i) {
      b.f_host[i] = params[i].temperature;
      b.f_host[cap + i] = params[i].top_p;
      b.f_host[2 * cap + i] = uniform(params[i].seed, (uint64_t)requests[i], (uint64_t)counters[i]);
      b.i_host[i] = params[i].effective_top_k();
    }
    // the previous call ended with a read-back of its result, so the earlier copies out of the
    // pinned buffers have finished
    ops_.flush();
    hip_check(hipMemcpyAsync(b.f_dev.data(), b.f_host, (size_t)3 * cap * 4, hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
    hip_check(hipMemcpyAsync(b.i_dev.data(), b.i_host, (size_t)cap * 4, hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
    const float* fd = (const float*)b.f_dev.data();
    ops_.sample(logits, fd, (const int*)b.i_dev.data(), fd + cap, fd + 2 * cap, out);
  }
  int* back = b.i_host + b.cap;
  hip_check(hipMemcpyAsync(back, out, (size_t)n * 4, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
  hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
  return std::vector<int>(back, back + n);
}

}  // namespace tinyinfer
