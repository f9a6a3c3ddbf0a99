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

// Two sets of pinned host buffers take turns, so that a call can be prepared while the call before
// it is still under way on the device.
struct Sampler::Buffers {
  struct Turn {
    float* f_host = nullptr;     // temperature | top_p | uniform | top_k (as integers): one copy takes them to the device
    int* i_host = nullptr;       // ids read back
    hipEvent_t read_back = nullptr;
    int n = 0;
    uint64_t ticket = 0;         // the call whose ids lie here (0: none)
    bool collected = true;
  };
  int cap = 0;
  Turn turns[2];
  uint64_t issued = 0;
  DeviceBuffer f_dev, out_dev;
  void free_host() {
    for (Turn& t : turns) {
      if (t.f_host) (void)hipHostFree(t.f_host);
      if (t.i_host) (void)hipHostFree(t.i_host);
      t.f_host = nullptr;
      t.i_host = nullptr;
    }
  }
  ~Buffers() {
    free_host();
    for (Turn& t : turns)
      if (t.read_back) (void)hipEventDestroy(t.read_back);
  }
};

Sampler::Sampler(Ops& ops) : ops_(ops), b_(new Buffers()) {}
Sampler::~Sampler() {}

static void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw KernelError(std::string(what) + ": " + hipGetErrorString(e));
}

uint64_t Sampler::sample_async(const Tensor& logits, const std::vector<SamplingParams>& params,
                               const std::vector<int64_t>& requests, const std::vector<int64_t>& counters, int* device_out) {
  const int n = (int)logits.shape[0];
  if ((int)params.size() != n || (int)requests.size() != n || (int)counters.size() != n)
    throw KernelError("sample: one set of parameters, one request number and one counter per row of logits");
  hipStream_t stream = (hipStream_t)ops_.stream();
  Buffers& b = *b_;
  Buffers::Turn& t = b.turns[b.issued & 1];
  if (!t.collected)
    throw KernelError("sample: two calls are under way whose ids have not been collected (Sampler::collect)");
  if (n > b.cap) {
    for (const Buffers::Turn& other : b.turns)
      if (!other.collected) throw KernelError("sample: more rows than before while a call is under way: collect it first");
    hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    const int cap = std::max(64, 2 * n);
    b.free_host();
    for (Buffers::Turn& u : b.turns) {
      hip_check(hipHostMalloc((void**)&u.f_host, (size_t)4 * cap * 4, hipHostMallocDefault), "hipHostMalloc");
      hip_check(hipHostMalloc((void**)&u.i_host, (size_t)cap * 4, hipHostMallocDefault), "hipHostMalloc");
      if (!u.read_back) hip_check(hipEventCreateWithFlags(&u.read_back, hipEventDisableTiming), "hipEventCreate");
    }
    b.f_dev = DeviceBuffer((size_t)4 * cap * 4);
    b.out_dev = DeviceBuffer((size_t)cap * 4);
    b.cap = cap;
  }
  bool greedy = true;
  for (const auto& p : params) greedy = greedy && p.temperature <= 0.f;
  int* out = device_out ? device_out : (int*)b.out_dev.data();
  if (greedy) {
    ops_.argmax(logits, out);
  } else {
    const int cap = b.cap;
    for (int i = 0; i < n; ++i) {
      t.f_host[i] = params[i].temperature;
      t.f_host[cap + i] = params[i].top_p;
      t.f_host[2 * cap + i] = uniform(params[i].seed, (uint64_t)requests[i], (uint64_t)counters[i]);
      reinterpret_cast<int*>(t.f_host)[3 * cap + i] = params[i].effective_top_k();
    }
    // this turn's earlier call has been collected: its copies out of these pinned buffers have
    // finished.  The device copies are shared: the stream puts this call's behind the last call's kernel.
    ops_.flush();
    hip_check(hipMemcpyAsync(b.f_dev.data(), t.f_host, (size_t)4 * cap * 4, hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
    const float* fd = (const float*)b.f_dev.data();
    ops_.sample(logits, fd, reinterpret_cast<const int*>(fd + 3 * cap), fd + cap, fd + 2 * cap, out);
  }
  hip_check(hipMemcpyAsync(t.i_host, out, (size_t)n * 4, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
  hip_check(hipEventRecord(t.read_back, stream), "hipEventRecord");
  t.n = n;
  t.collected = false;
  t.ticket = ++b.issued;
  return t.ticket;
}

std::vector<int> Sampler::collect(uint64_t ticket) {
  Buffers& b = *b_;
  for (Buffers::Turn& t : b.turns) {
    if (t.ticket != ticket || t.collected) continue;
    hip_check(hipEventSynchronize(t.read_back), "hipEventSynchronize");
    t.collected = true;
    const int* back = t.i_host;
    return std::vector<int>(back, back + t.n);
  }
  throw KernelError("sample: no call with ticket " + std::to_string(ticket) + " is waiting to be collected");
}

void Sampler::drop(uint64_t ticket) {
  for (Buffers::Turn& t : b_->turns)
    if (t.ticket == ticket && !t.collected) {
      (void)hipEventSynchronize(t.read_back);
      t.collected = true;
    }
}

std::vector<int> Sampler::sample(const Tensor& logits, const std::vector<SamplingParams>& params,
                                 const std::vector<int64_t>& requests, const std::vector<int64_t>& counters) {
  return collect(sample_async(logits, params, requests, counters, nullptr));
}

}  // namespace tinyinfer
