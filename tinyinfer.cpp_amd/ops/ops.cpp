// Tensors, device memory, the table of kernel libraries, and `Ops`: the kernels as calls on
// tensors.  Each call checks shapes and dtypes on the host, then launches the hand-written HIP
// kernel through the C interface of the kernel libraries (tinyinfer_kernels.h).  Nothing here
// computes, and nothing falls back to the CPU or to a library: a kernel library that is not
// built is an error.
//
// How a step's rows reach the bfloat16 matrix-core attention kernels: rows of single-token
// entries go to the flash-decoding kernel (split over the context so that the launch fills the
// chip), rows of longer entries to the tiled prefill kernels.  Head or page sizes those do not
// serve are left to the generic kernel.  The reference runs one kernel for both
// (/root/reference/src/cuda/attention.cu:89-214).
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>

#include "../include/inference.h"
#include "../csrc/tinyinfer_kernels.h"

namespace tinyinfer {

// ------------------------------------------------------------------------------------ tensors
size_t dtype_size(DType dt) {
  switch (dt) {
    case DType::F32: case DType::I32: return 4;
    case DType::BF16: case DType::F16: return 2;
    case DType::F64: case DType::I64: return 8;
  }
  return 0;
}
const char* dtype_name(DType dt) {
  switch (dt) {
    case DType::F32: return "float32";
    case DType::BF16: return "bfloat16";
    case DType::I32: return "int32";
    case DType::F16: return "float16";
    case DType::F64: return "float64";
    case DType::I64: return "int64";
  }
  return "?";
}
DType dtype_from_name(const std::string& n) {
  if (n == "float32") return DType::F32;
  if (n == "bfloat16") return DType::BF16;
  throw EngineError("dtype must be one of ['bfloat16', 'float32'], got '" + n + "'");
}

Tensor::Tensor(void* p, DType dt, std::initializer_list<int64_t> dims) : Tensor(p, dt, std::vector<int64_t>(dims)) {}
Tensor::Tensor(void* p, DType dt, const std::vector<int64_t>& dims) : data(p), dtype(dt), ndim((int)dims.size()) {
  if (ndim > 4) throw KernelError("a tensor has at most 4 dimensions");
  int64_t s = 1;
  for (int i = ndim - 1; i >= 0; --i) {
    shape[i] = dims[i];
    stride[i] = s;
    s *= dims[i];
  }
}
int64_t Tensor::numel() const {
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) n *= shape[i];
  return n;
}
bool Tensor::contiguous() const {
  int64_t s = 1;
  for (int i = ndim - 1; i >= 0; --i) {
    if (shape[i] != 1 && stride[i] != s) return false;
    s *= shape[i];
  }
  return true;
}
Tensor Tensor::rows(int64_t first, int64_t count) const {
  Tensor t = *this;
  t.data = (char*)data + first * stride[0] * (int64_t)dtype_size(dtype);
  t.shape[0] = count;
  return t;
}
Tensor Tensor::cols(int64_t first, int64_t count) const {
  Tensor t = *this;
  t.data = (char*)data + first * stride[ndim - 1] * (int64_t)dtype_size(dtype);
  t.shape[ndim - 1] = count;
  return t;
}
std::string Tensor::describe() const {
  std::string s = std::string(dtype_name(dtype)) + "[";
  for (int i = 0; i < ndim; ++i) s += (i ? ", " : "") + std::to_string(shape[i]);
  return s + "]";
}

// ------------------------------------------------------------------------------ device memory
namespace {
void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw KernelError(std::string(what) + ": " + hipGetErrorString(e));
}
void* default_alloc(void*, size_t bytes) {
  void* p = nullptr;
  hip_check(hipMalloc(&p, bytes ? bytes : 4), "hipMalloc");
  return p;
}
void default_release(void*, void* p) { (void)hipFree(p); }
Allocator g_allocator = {default_alloc, default_release, nullptr};
}  // namespace

static void no_release(void*, void*) {}
void detach_allocator() { g_allocator.release = no_release; }

void set_allocator(const Allocator& a) {
  if (a.alloc && a.release) g_allocator = a;
  else g_allocator = {default_alloc, default_release, nullptr};
}

static thread_local bool g_host_memory = false;
HostMemoryScope::HostMemoryScope() : before(g_host_memory) { g_host_memory = true; }
HostMemoryScope::~HostMemoryScope() { g_host_memory = before; }

static void give_back(void* p, bool host) {
  if (!p) return;
  if (host) free(p);
  else g_allocator.release(g_allocator.user, p);
}
DeviceBuffer::DeviceBuffer(size_t bytes) : n_(bytes), host_(g_host_memory) {
  p_ = host_ ? calloc(1, bytes ? bytes : 4) : g_allocator.alloc(g_allocator.user, bytes ? bytes : 4);
  if (!p_) throw KernelError(std::string("out of ") + (host_ ? "host" : "device") + " memory: " + std::to_string(bytes) + " bytes");
}
DeviceBuffer::~DeviceBuffer() { give_back(p_, host_); }
DeviceBuffer::DeviceBuffer(DeviceBuffer&& o) noexcept : p_(o.p_), n_(o.n_), host_(o.host_) { o.p_ = nullptr; o.n_ = 0; }
DeviceBuffer& DeviceBuffer::operator=(DeviceBuffer&& o) noexcept {
  if (this != &o) {
    give_back(p_, host_);
    p_ = o.p_;
    n_ = o.n_;
    host_ = o.host_;
    o.p_ = nullptr;
    o.n_ = 0;
  }
  return *this;
}

void* Workspace::get(const std::string& name, size_t bytes) {
  auto it = bufs_.find(name);
  if (it != bufs_.end() && it->second.bytes() >= bytes) return it->second.data();
  if (frozen)
    throw EngineError("workspace buffer '" + name + "' would have to grow while a captured graph reads its address");
  size_t cap = bytes ? bytes : 4;
  if (it != bufs_.end()) cap = std::max(cap, it->second.bytes() + it->second.bytes() / 2);
  cap = (cap + 255) & ~(size_t)255;
  bufs_[name] = DeviceBuffer(cap);
  return bufs_[name].data();
}
Tensor Workspace::tensor(const std::string& name, DType dt, std::initializer_list<int64_t> dims) {
  Tensor t(nullptr, dt, dims);
  t.data = get(name + (dt == DType::F32 ? ":f" : dt == DType::BF16 ? ":b" : ":i"), t.bytes());
  return t;
}
size_t Workspace::total_bytes() const {
  size_t n = 0;
  for (const auto& kv : bufs_) n += kv.second.bytes();
  return n;
}

// ---------------------------------------------------------------------------- kernel libraries
namespace {
std::mutex g_lib_mutex;
std::map<std::string, std::string>& lib_paths() {
  static std::map<std::string, std::string> m;
  return m;
}
std::map<std::string, void*>& lib_handles() {
  static std::map<std::string, void*> m;
  return m;
}

std::string own_directory() {
  Dl_info info;
  if (dladdr((void*)&own_directory, &info) && info.dli_fname) {
    std::string p = info.dli_fname;
    const size_t k = p.rfind('/');
    return k == std::string::npos ? "." : p.substr(0, k);
  }
  return ".";
}

// kernels.manifest: one "name path" a line, written by the build
void read_manifest(const std::string& dir) {
  std::ifstream f(dir + "/kernels.manifest");
  std::string name, path;
  while (f >> name >> path) {
    if (path.size() && path[0] != '/') path = dir + "/" + path;
    if (!lib_paths().count(name)) lib_paths()[name] = path;
  }
}

void* library(const std::string& name) {
  std::lock_guard<std::mutex> lock(g_lib_mutex);
  auto h = lib_handles().find(name);
  if (h != lib_handles().end()) return h->second;
  if (!lib_paths().count(name)) {
    if (const char* env = getenv("TINYINFER_KERNEL_DIR")) read_manifest(env);
    read_manifest(own_directory());
  }
  auto p = lib_paths().find(name);
  if (p == lib_paths().end())
    throw KernelError("the kernel library '" + name + "' is not built (no path registered and none in kernels.manifest): "
                      "build the kernels first; there is no fallback");
  void* handle = dlopen(p->second.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!handle) throw KernelError("cannot load the kernel library '" + name + "' from " + p->second + ": " + dlerror());
  lib_handles()[name] = handle;
  return handle;
}

template <class Fn> Fn symbol(const char* lib, const char* name) {
  void* s = dlsym(library(lib), name);
  if (!s) throw KernelError(std::string("kernel library '") + lib + "' does not export " + name);
  return (Fn)s;
}

// a function of a kernel library, resolved at its first call
#define KERNEL(lib, fn) ([]() { static auto f = symbol<decltype(&::fn)>(lib, #fn); return f; }())

std::string last_error(const char* lib) {
  using Fn = const char* (*)();
  static std::map<std::string, Fn> cache;
  Fn f;
  {
    auto it = cache.find(lib);
    if (it == cache.end()) it = cache.emplace(lib, symbol<Fn>(lib, "ti_last_error")).first;
    f = it->second;
  }
  return f();
}
void check(const char* lib, int rc, const char* what) {
  if (rc != 0) throw KernelError(std::string(what) + ": " + last_error(lib));
}
int code(DType dt, const char* what) {
  if (dt == DType::F32) return 0;
  if (dt == DType::BF16) return 1;
  throw KernelError(std::string(what) + ": dtype " + dtype_name(dt) + " is not served by the kernels (float32, bfloat16)");
}
void require(bool ok, const std::string& message) {
  if (!ok) throw KernelError(message);
}
}  // namespace

void register_kernel_library(const std::string& name, const std::string& path) {
  std::lock_guard<std::mutex> lock(g_lib_mutex);
  auto it = lib_paths().find(name);
  if (it != lib_paths().end() && it->second != path && lib_handles().count(name))
    throw KernelError("kernel library '" + name + "' is already loaded from " + it->second);
  lib_paths()[name] = path;
}

void* kernel_symbol(const std::string& lib, const std::string& name) {
  void* s = dlsym(library(lib), name.c_str());
  if (!s) throw KernelError("kernel library '" + lib + "' does not export " + name);
  return s;
}

void load_plugin(const std::string& path) {
  void* handle = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
  if (!handle) throw FileError("cannot load the plugin " + path + ": " + dlerror());
  if (void* init = dlsym(handle, "tinyinfer_plugin_init")) ((void (*)())init)();
}

bool kernel_library_available(const std::string& name) {
  try {
    library(name);
    return true;
  } catch (const KernelError&) {
    return false;
  }
}

// ---------------------------------------------------------------------------------------- Ops
// An object's overrides of a kernel library's shape rules, in force for the calls of one scope.
static std::mutex g_tuning_mutex;
struct TunedScope {
  const char* lib = nullptr;
  TunedScope(Ops& ops, const char* library) {
    if (ops.tuning_.empty()) return;
    auto it = ops.tuning_.find(library);
    if (it == ops.tuning_.end() || it->second.empty()) return;
    lib = library;
    g_tuning_mutex.lock();
    auto set = symbol<int (*)(const char*, long)>(library, "ti_tuning_set");
    for (const auto& kv : it->second)
      if (set(kv.first.c_str(), kv.second) != 0) {
        symbol<void (*)()>(library, "ti_tuning_reset")();
        g_tuning_mutex.unlock();
        lib = nullptr;
        throw KernelError(std::string("kernel library '") + library + "' has no shape rule '" + kv.first + "'");
      }
  }
  ~TunedScope() {
    if (!lib) return;
    symbol<void (*)()>(lib, "ti_tuning_reset")();
    g_tuning_mutex.unlock();
  }
};
void Ops::tune(const std::string& library, const std::string& name, long value) { tuning_[library][name] = value; }
void Ops::untune() { tuning_.clear(); }

static const int64_t PARTIALS_BYTES = 32 << 20;
static const int NORMED_MAX_ROWS = 16;

struct Ops::Timing {
  struct Rec { std::string name; hipEvent_t a, b; };
  std::vector<Rec> recs;
  int depth = 0;
  bool names_only = false;      // calls are listed, not timed: nothing is recorded on the stream, nothing is flushed
  std::string tag;              // what the call under way says about the kernel it took
};
Ops::Ops(void* stream) : stream_(stream) {}
Ops::~Ops() {
  if (timing_)
    for (auto& r : timing_->recs)
      if (r.a) {
        (void)hipEventDestroy(r.a);
        (void)hipEventDestroy(r.b);
      }
}

void Ops::timing(bool on) {
  flush();
  if (on && !timing_) timing_.reset(new Timing());
  if (!on && timing_) {
    timing_report();
    timing_.reset();
  }
}

void Ops::count_calls(bool on) {
  if (timing_ && !timing_->names_only) timing(false);
  if (on && !timing_) {
    timing_.reset(new Timing());
    timing_->names_only = true;
  }
  if (!on) timing_.reset();
}

void Ops::took(const char* what) {
  if (timing_ && timing_->depth == 1) timing_->tag = what;
}

std::vector<Ops::Timed> Ops::timing_report() {
  std::vector<Timed> out;
  if (!timing_) return out;
  if (!timing_->names_only) hip_check(hipStreamSynchronize((hipStream_t)stream_), "hipStreamSynchronize");
  std::map<std::string, size_t> index;
  for (auto& r : timing_->recs) {
    float ms = 0.f;
    if (r.a) (void)hipEventElapsedTime(&ms, r.a, r.b);
    auto it = index.find(r.name);
    if (it == index.end()) {
      it = index.emplace(r.name, out.size()).first;
      out.push_back({r.name, 0, 0.0});
    }
    out[it->second].calls += 1;
    out[it->second].us += ms * 1e3;
    if (r.a) {
      (void)hipEventDestroy(r.a);
      (void)hipEventDestroy(r.b);
    }
  }
  timing_->recs.clear();
  return out;
}

// Events around what one call launches, when timing is on (the outermost call only).
struct TimedScope {
  Ops& ops;
  bool active = false;
  size_t index = 0;
  template <class F> TimedScope(Ops& o, F&& name) : ops(o) {
    if (!ops.timing_) return;
    if (ops.timing_->depth++ > 0) return;
    Ops::Timing::Rec r;
    r.name = name();
    r.a = r.b = nullptr;
    ops.timing_->tag.clear();
    if (!ops.timing_->names_only) {
      if (ops.pending_.out) ops.flush();          // the sums of the call before are not this call's time
      if (hipEventCreate(&r.a) != hipSuccess || hipEventCreate(&r.b) != hipSuccess) return;
      (void)hipEventRecord(r.a, (hipStream_t)ops.stream_);
    }
    index = ops.timing_->recs.size();
    ops.timing_->recs.push_back(r);
    active = true;
  }
  ~TimedScope() {
    if (!ops.timing_) return;
    --ops.timing_->depth;
    if (!active) return;
    Ops::Timing::Rec& r = ops.timing_->recs[index];
    if (!ops.timing_->tag.empty()) r.name += " " + ops.timing_->tag;
    if (r.b) (void)hipEventRecord(r.b, (hipStream_t)ops.stream_);
  }
};
static std::string dims(const Tensor& t) {
  std::string s;
  for (int i = 0; i < t.ndim; ++i) s += (i ? "x" : "") + std::to_string(t.shape[i]);
  return s;
}
#define TIMED(expr) TimedScope timed_scope_(*this, [&]() -> std::string { return expr; })

int Ops::compute_units() {
  if (!units_) {
    int dev = 0, n = 0;
    hip_check(hipGetDevice(&dev), "hipGetDevice");
    hip_check(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev), "hipDeviceGetAttribute");
    units_ = n > 0 ? n : 256;
  }
  return units_;
}

void* Ops::launch_stream() {
  if (pending_.out) flush();
  return stream_;
}

void Ops::flush() {
  if (!pending_.out) return;
  auto p = pending_;
  pending_ = {};
  int rc = KERNEL("gemm_bf16", ti_gemm_bf16_partials_add)((float*)p.out, (const float*)partials_.data(), p.splits,
                                                          (long)p.count, (hipStream_t)stream_);
  check("gemm_bf16", rc, "linear(bf16): adding the partial sums");
}

const Tensor& Rows::materialize(Ops& ops) const {
  if (lazy) {
    ops.rmsnorm(x, weight, eps, t);
    const_cast<Rows*>(this)->lazy = false;
  }
  return t;
}

void Ops::embed(const Tensor& table, const int* tokens, int64_t M, const Tensor& x, const int* fed, int n_fed) {
  TIMED("embed " + dims(x));
  require(table.ndim == 2 && x.ndim == 2, "embed: table and x must be matrices");
  const int64_t V = table.shape[0], H = table.shape[1];
  require(x.shape[0] == M && x.shape[1] == H && x.dtype == DType::F32,
          "embed: x " + x.describe() + " does not fit [" + std::to_string(M) + "," + std::to_string(H) + "] float32");
  require(table.contiguous() && x.contiguous(), "embed: table and x must be contiguous");
  int rc = KERNEL("core", ti_embed_fed)(code(table.dtype, "embed"), table.data, tokens, fed, fed ? n_fed : 0, (float*)x.data,
                                        (int)M, (int)H, (int)V, (hipStream_t)launch_stream());
  check("core", rc, "embed");
}

void Ops::rmsnorm(const Tensor& x, const Tensor& w, float eps, const Tensor& out, const int* rows, int64_t n_rows) {
  TIMED(std::string(pending_.out ? "rmsnorm+partials " : "rmsnorm ") + std::to_string(rows ? n_rows : x.shape[0]) + "x" + std::to_string(x.shape[1]));
  require(x.ndim == 2, "rmsnorm: x must be a matrix");
  const int64_t H = x.shape[1];
  const int64_t n = rows ? n_rows : x.shape[0];
  require(x.dtype == DType::F32 && w.dtype == DType::F32 && w.numel() == H,
          "rmsnorm: x " + x.describe() + " / weight " + w.describe() + " do not fit width " + std::to_string(H));
  require(out.ndim == 2 && out.shape[0] == n && out.shape[1] == H && out.contiguous() && x.contiguous(),
          "rmsnorm: out " + out.describe() + " does not fit [" + std::to_string(n) + "," + std::to_string(H) +
              "] or is not contiguous");
  const int oc = code(out.dtype, "rmsnorm");
  if (pending_.out && !rows && pending_.out == x.data && pending_.count == x.numel()) {
    // the product before left its partial sums: this norm adds them on its way
    int rc = KERNEL("core", ti_rmsnorm_add_partials)(oc, (float*)x.data, (const float*)partials_.data(), pending_.splits,
                                                     (const float*)w.data, out.data, (int)n, (int)H, eps,
                                                     (hipStream_t)stream_);
    if (rc == 0) {
      pending_ = {};
      return;
    }
    if (rc != 3) check("core", rc, "rmsnorm");
  }
  int rc = KERNEL("core", ti_rmsnorm)(oc, (const float*)x.data, (const float*)w.data, rows, out.data, (int)n, (int)H, eps,
                                      (hipStream_t)launch_stream());
  check("core", rc, "rmsnorm");
}

void Ops::rope_neox(const Tensor& x, const int* positions, const Tensor& inv_freq) {
  TIMED("rope_neox " + dims(x));
  require(x.ndim == 3 && x.dtype == DType::F32 && x.stride[2] == 1 && x.stride[1] == x.shape[2],
          "rope: x must be float32 [M, heads, hd] with contiguous heads");
  const int64_t M = x.shape[0], heads = x.shape[1], hd = x.shape[2];
  require(inv_freq.numel() == hd / 2 && inv_freq.dtype == DType::F32, "rope: inv_freq must be float32 [hd/2]");
  int rc = KERNEL("core", ti_rope_neox)((float*)x.data, positions, (const float*)inv_freq.data, (int)M, (int)heads, (int)hd,
                                        (long)x.stride[0], (hipStream_t)launch_stream());
  check("core", rc, "rope");
}

void Ops::rope_table(const Tensor& inv_freq, const Tensor& table) {
  require(table.ndim == 3 && table.shape[2] == 2 && table.shape[1] == inv_freq.numel() && table.dtype == DType::F32 &&
              table.contiguous(),
          "rope_table: the table must be float32 [positions, hd/2, 2]");
  int rc = KERNEL("core", ti_rope_table)((float*)table.data, (const float*)inv_freq.data, (int)inv_freq.numel(),
                                         (int)table.shape[0], (hipStream_t)launch_stream());
  check("core", rc, "rope_table");
}

static void check_pool(const char* what, const Tensor& pool, int kv_heads, int head_dim, DType dt) {
  // a pool of one cache layer is [pages][2 * kv_heads][P][hd]: the K|V dimension is folded into
  // the second one (a tensor here has at most four dimensions)
  require(pool.ndim == 4 && pool.shape[1] == 2 * (int64_t)kv_heads && pool.shape[3] == head_dim && pool.dtype == dt &&
              pool.contiguous(),
          std::string(what) + ": pool " + pool.describe() + " does not fit [pages, 2 x " + std::to_string(kv_heads) +
              ", P, " + std::to_string(head_dim) + "] of " + dtype_name(dt));
}

void Ops::qk_norm_rope_kv_write(const Tensor& qkv, const float* q_w, const float* k_w, float eps, const Rotation& rot,
                                const int* positions, const int* slots, const CacheView& view, const Tensor& pool,
                                const Tensor& q_out, int heads, int kv_heads, int head_dim) {
  TIMED("qk_norm_rope_kv_write " + dims(qkv));
  const int64_t M = qkv.shape[0];
  const int64_t width = (int64_t)(heads + 2 * kv_heads) * head_dim;
  require(qkv.ndim == 2 && qkv.shape[1] == width && qkv.dtype == DType::F32 && qkv.contiguous(),
          "qk_norm_rope_kv_write: qkv " + qkv.describe() + " does not fit [" + std::to_string(M) + "," +
              std::to_string(width) + "]");
  require(q_out.ndim == 2 && q_out.shape[0] == M && q_out.shape[1] == (int64_t)heads * head_dim && q_out.contiguous(),
          "qk_norm_rope_kv_write: q_out has the wrong shape");
  int page = view.page_size > 0 ? view.page_size : 16;
  if (kv_heads > 0) {
    check_pool("qk_norm_rope_kv_write", pool, kv_heads, head_dim, q_out.dtype);
    page = (int)pool.shape[2];
  }
  int rc = KERNEL("core", ti_qk_norm_rope_kv_write)(
      code(q_out.dtype, "qk_norm_rope_kv_write"), (const float*)qkv.data, q_w, k_w, rot.inv_freq, rot.table, rot.table_len,
      positions, slots, view.table, view.table_width, pool.data, q_out.data, (int)M, heads, kv_heads, head_dim, page, eps,
      (hipStream_t)launch_stream());
  check("core", rc, "qk_norm_rope_kv_write");
}

void Ops::qk_norm_inplace(const Tensor& qkv, const float* q_w, const float* k_w, float eps, int heads, int kv_heads,
                          int head_dim) {
  TIMED("qk_norm_inplace " + dims(qkv));
  require(qkv.ndim == 2 && qkv.dtype == DType::F32 && qkv.contiguous() &&
              qkv.shape[1] >= (int64_t)(heads + kv_heads) * head_dim,
          "qk_norm_inplace: qkv " + qkv.describe() + " does not hold " + std::to_string(heads) + " + " +
              std::to_string(kv_heads) + " heads of " + std::to_string(head_dim));
  int rc = KERNEL("core", ti_qk_norm_inplace)((float*)qkv.data, (int)qkv.shape[1], q_w, k_w, (int)qkv.shape[0], heads,
                                              kv_heads, head_dim, eps, (hipStream_t)launch_stream());
  check("core", rc, "qk_norm_inplace");
}

// ---------------------------------------------------------------------------- matrix products
bool Ops::can_fuse_norm(int64_t n_rows, DType dtype) const {
  return use.fused_norm && use.fast_gemm && dtype == DType::BF16 && n_rows > 0 && n_rows <= NORMED_MAX_ROWS &&
         kernel_library_available("gemm_bf16");
}

bool Ops::linear_with_norm(const Rows& a, const Tensor& w, const Tensor& out, Epilogue epi) {
  TunedScope tuned(*this, "gemm_bf16");
  static const char* EPI_NAMES[] = {"store", "add", "store_act", "swiglu"};
  TIMED(std::string("norm+linear.") + EPI_NAMES[epi] + " " + dims(a.t) + " * " + dims(w));
  const int64_t M = a.t.shape[0], K = a.t.shape[1];
  if (!can_fuse_norm(M, a.t.dtype) || w.dtype != DType::BF16) return false;
  // the rows wait for partial sums: the norm's own kernel adds them on its way
  if (pending_.out && pending_.out == a.x.data) return false;
  const int64_t rows = w.shape[0];
  const int64_t N = epi == SwiGLU ? rows / 2 : rows;
  require(w.ndim == 2 && w.shape[1] == K && w.contiguous() && !(epi == SwiGLU && rows % 2),
          "linear: normed rows " + a.t.describe() + " and w " + w.describe() + " do not fit");
  require(a.x.ndim == 2 && a.x.shape[0] == M && a.x.shape[1] == K && a.x.dtype == DType::F32 && a.x.contiguous() &&
              a.weight.numel() == K && a.weight.dtype == DType::F32,
          "linear: the rows to norm must be float32 [M, K] with a float32 weight [K]");
  const DType want = (epi == Store || epi == Add) ? DType::F32 : DType::BF16;
  require(out.ndim == 2 && out.shape[0] == M && out.shape[1] == N && out.dtype == want && out.contiguous(),
          "linear: out " + out.describe() + " does not fit the product");
  int rc = KERNEL("gemm_bf16", ti_gemm_bf16_normed)((const float*)a.x.data, (const float*)a.weight.data, a.eps, w.data,
                                                    out.data, (int)M, (int)N, (int)K, (int)epi,
                                                    (hipStream_t)launch_stream());
  if (rc == 3) return false;
  check("gemm_bf16", rc, "linear(normed)");
  took("[fused]");
  return true;
}

void Ops::linear(const Rows& a, const Tensor& w, const Tensor& out, Epilogue epi, bool may_defer) {
  if (a.lazy) {
    if (linear_with_norm(a, w, out, epi)) return;
    a.materialize(*this);
  }
  linear(a.t, w, out, epi, may_defer);
}

void Ops::linear(const Tensor& a, const Tensor& w, const Tensor& out, Epilogue epi, bool may_defer) {
  TunedScope tuned(*this, "gemm_bf16");
  static const char* EPI_NAMES[] = {"store", "add", "store_act", "swiglu"};
  TIMED(std::string("linear.") + EPI_NAMES[epi] + " " + dims(a) + " * " + dims(w));
  require(a.ndim == 2 && w.ndim == 2, "linear: a and w must be matrices");
  const int64_t M = a.shape[0], K = a.shape[1], rows = w.shape[0];
  const int64_t N = epi == SwiGLU ? rows / 2 : rows;
  require(w.shape[1] == K && a.dtype == w.dtype && a.stride[1] == 1 && w.contiguous(),
          "linear: a " + a.describe() + " and w " + w.describe() + " do not fit");
  require(!(epi == SwiGLU && rows % 2), "linear: a SwiGLU weight needs an even number of rows");
  const DType want = (epi == Store || epi == Add) ? DType::F32 : a.dtype;
  require(out.ndim == 2 && out.shape[0] == M && out.shape[1] == N && out.dtype == want && out.contiguous(),
          "linear: out " + out.describe() + " does not fit [" + std::to_string(M) + "," + std::to_string(N) + "] " +
              dtype_name(want));
  if (M == 0) return;
  const int dt = code(a.dtype, "linear");
  const long lda = (long)a.stride[0];
  if (a.dtype == DType::BF16 && use.fast_gemm && kernel_library_available("gemm_bf16") && K % 8 == 0 && lda % 8 == 0 &&
      ((uintptr_t)a.data % 16) == 0 && ((uintptr_t)w.data % 16) == 0) {
    if (epi == Add && use.split_k_add) {
      // a product of few tiles: K split over workgroups; their sums go through a workspace
      void* stream = launch_stream();
      if (!partials_.data()) partials_ = DeviceBuffer(PARTIALS_BYTES);
      // 1: the sums are left for the next norm; 2: the same product, added at once
      const int defer = !may_defer ? 0 : use.deferred_add ? 1 : 2;
      int splits = 0;
      int rc = KERNEL("gemm_bf16", ti_gemm_bf16_add_split)(a.data, w.data, out.data, (int)M, (int)N, (int)K, lda, (int)epi,
                                                           partials_.data(), (long)PARTIALS_BYTES, defer, &splits,
                                                           (hipStream_t)stream);
      if (rc == 0) {
        if (splits) {
          pending_.out = out.data;
          pending_.count = out.numel();
          pending_.splits = splits;
        }
        took(splits ? "[mfma, K split, sums left]" : "[mfma]");
        return;
      }
      if (rc != 3) check("gemm_bf16", rc, "linear(bf16, split K)");
    }
    if (epi == Store && M > 16 && M <= 64 && use.split_k_add) {
      void* stream = launch_stream();
      if (!partials_.data()) partials_ = DeviceBuffer(PARTIALS_BYTES);
      int rc = KERNEL("gemm_bf16", ti_gemm_bf16_store_split)(a.data, w.data, out.data, (int)M, (int)N, (int)K, lda,
                                                             partials_.data(), (long)PARTIALS_BYTES, (hipStream_t)stream);
      if (rc == 0) {
        took("[mfma, K split]");
        return;
      }
      if (rc != 3) check("gemm_bf16", rc, "linear(bf16, split K, stored)");
    }
    int rc = KERNEL("gemm_bf16", ti_gemm_bf16)(a.data, w.data, out.data, (int)M, (int)N, (int)K, lda, (int)epi,
                                               (hipStream_t)launch_stream());
    if (rc == 0) {
      took("[mfma]");
      return;
    }
    if (rc != 3) check("gemm_bf16", rc, "linear(bf16)");     // 3: shape not served, the generic kernel takes it
  }
  took("[generic]");
  int rc = KERNEL("gemm_generic", ti_gemm_generic)(dt, a.data, w.data, out.data, (int)M, (int)N, (int)K, lda, (int)epi,
                                                   (hipStream_t)launch_stream());
  check("gemm_generic", rc, "linear");
}

bool Ops::qkv_prepared(const Rows& a, const Tensor& w, const float* q_w, const float* k_w, float eps, const Rotation& rot,
                       const int* positions, const int* slots, const CacheView& view, const Tensor& pool,
                       const Tensor& q_out, int heads, int kv_heads, int head_dim) {
  TunedScope tuned(*this, "gemm_bf16");
  TIMED("qkv_prepared " + dims(a.t) + " * " + dims(w));
  if (!(use.fused_qkv_prefill && use.fast_gemm) || a.lazy) return false;
  if (a.t.dtype != DType::BF16 || w.dtype != DType::BF16 || q_out.dtype != DType::BF16) return false;
  if (!kernel_library_available("gemm_bf16")) return false;
  const int64_t M = a.t.shape[0], K = a.t.shape[1];
  const int64_t N = (int64_t)(heads + 2 * kv_heads) * head_dim;
  require(w.ndim == 2 && w.shape[0] == N && w.shape[1] == K && a.t.stride[1] == 1 && w.contiguous(),
          "qkv_prepared: a " + a.t.describe() + " and w " + w.describe() + " do not fit " + std::to_string(N) +
              " rows of heads");
  require(q_out.ndim == 2 && q_out.shape[0] == M && q_out.shape[1] == (int64_t)heads * head_dim && q_out.contiguous(),
          "qkv_prepared: q_out has the wrong shape");
  int page = view.page_size > 0 ? view.page_size : 16;
  if (kv_heads > 0) {
    check_pool("qkv_prepared", pool, kv_heads, head_dim, DType::BF16);
    page = (int)pool.shape[2];
  }
  int rc = KERNEL("gemm_bf16", ti_gemm_bf16_qkv_prep)(
      a.t.data, w.data, (int)M, (int)K, (long)a.t.stride[0], q_w, k_w, eps, rot.inv_freq, rot.table, rot.table_len,
      positions, slots, view.table, view.table_width, pool.data, q_out.data, heads, kv_heads, head_dim, page,
      (hipStream_t)launch_stream());
  if (rc == 3) return false;
  check("gemm_bf16", rc, "qkv_prepared");
  took("[fused]");
  return true;
}

// ---------------------------------------------------------------------------------- attention
void Ops::attention_rows(const Tensor& q, const Tensor& pool, const CacheView& view, const int* positions, const int* slots,
                         const Tensor& out, int heads, int kv_heads, int head_dim, float scale, int window) {
  TIMED("attention_rows " + dims(q));
  const int64_t M = q.shape[0];
  require(q.ndim == 2 && q.shape[1] == (int64_t)heads * head_dim && out.ndim == 2 && out.shape[0] == M &&
              out.shape[1] == q.shape[1] && q.dtype == pool.dtype && out.dtype == q.dtype,
          "attention: q/out/pool shapes or dtypes do not fit");
  check_pool("attention", pool, kv_heads, head_dim, q.dtype);
  require(q.contiguous() && out.contiguous(), "attention: arguments must be contiguous");
  int rc = KERNEL("attention_generic", ti_attention_rows)(
      code(q.dtype, "attention"), q.data, pool.data, view.table, view.table_width, positions, slots, out.data, (int)M, heads,
      kv_heads, head_dim, (int)pool.shape[2], scale, window, (hipStream_t)launch_stream());
  check("attention_generic", rc, "attention");
}

// What a launch of the decode kernel costs, as measured on an MI355X at a head size of 128 (a
// workgroup per row, kv head and split; a compute unit streams about as fast with one workgroup
// as with two, so workgroups beyond one per unit wait for a second round).
static const int MAX_SPLITS = 64;             // the merge kernel's limit
static const int MIN_BLOCKS_PER_SPLIT = 16;   // four 16-key blocks per wavefront at least
static const double SPLIT_PROLOGUE_US = 5.0;  // position, table row, query, page ids: before a workgroup's first key arrives
static const double SPLIT_TOKEN_US = 0.019;   // per token of context that one workgroup walks, at 512 bytes of key and value a token
static const double SPLIT_MERGE_US = 4.0;     // the merge kernel, which a launch without splits does without

// Into how many runs the decode kernel splits the context.  `context`: the longest context the
// launch is sized for (it bounds the number); `typical`: the context the choice is made for (a
// captured graph is sized for the longest sequence, but replayed mostly on shorter ones).  The
// number that makes rounds x (prologue + run) + merge the least, rounds being the workgroups over
// the compute units, rounded up.
int Ops::decode_splits(int n_rows, int kv_heads, int heads, int context, int typical, int units, int head_dim) {
  if (typical <= 0) typical = context;
  const int parts = (heads / kv_heads + 15) / 16;
  const long base = std::max(1L, (long)n_rows * kv_heads * parts);
  const int blocks = (std::max(1, context) + 15) / 16;
  const int limit = std::max(1, std::min(blocks / MIN_BLOCKS_PER_SPLIT, MAX_SPLITS));
  const double walk = SPLIT_TOKEN_US * std::max(1, typical) * (head_dim > 0 ? head_dim / 128.0 : 1.0);
  int best = 1;
  double best_cost = -1.0;
  for (int s = 1; s <= limit; ++s) {
    const long rounds = (base * s + units - 1) / units;
    const double cost = rounds * (SPLIT_PROLOGUE_US + walk / s) + (s > 1 ? SPLIT_MERGE_US : 0.0);
    if (best_cost < 0 || cost < best_cost - 1e-9) {
      best = s;
      best_cost = cost;
    }
  }
  return best;
}

static int typical_context(const AttentionWork& w) {
  return w.split_context > w.max_context ? std::max(w.max_context, w.split_context / 2) : w.max_context;
}

static const int PORTION_SPLIT_KEYS = 512;   // a portion's keys are cut into runs of at least this many ...
static const int PORTION_SPLIT_MAX = 8;      // ... at most this many runs
static const int PAIRED_BELOW = 1025;        // (tiles of 128 rows) x heads below which a launch takes the paired kernel

// A launch whose tiles all find a compute unit at once gives each tile a workgroup of its own (it
// lasts as long as its heaviest tile then); a larger one pairs the heaviest tile with the lightest.
// The keys are cut into runs when the launch would leave most units idle (a short portion) while
// every workgroup walks a long context.
int Ops::portion_launch(int n_tiles_small, int heads, int portion_context, int window, int units, bool* paired) {
  const int context = window == 0 ? portion_context : std::min(portion_context, window + 64);
  const bool pair = n_tiles_small * heads > units;
  if (paired) *paired = pair;
  const int workgroups = std::max(1, (pair ? (n_tiles_small + 1) / 2 : n_tiles_small) * heads);
  if (workgroups * 2 > units || context < 2 * PORTION_SPLIT_KEYS) return 1;
  return std::max(1, std::min({PORTION_SPLIT_MAX, units / workgroups, context / PORTION_SPLIT_KEYS}));
}

bool Ops::attention_from_projections(const AttentionWork& work, Workspace& ws, const CacheView& view, const Tensor& qkv,
                                     const float* q_w, const float* k_w, float eps, const Rotation& rot,
                                     const Tensor& pool, bool write_kv, const Tensor& out, int heads, int kv_heads,
                                     int head_dim, float scale, int window) {
  TunedScope tuned(*this, "attention_bf16");
  TIMED("attention.decode_prepared rows=" + std::to_string(work.M) + " context<=" + std::to_string(work.max_context));
  if (!(use.fused_qk_decode && use.fast_attention && work.decode_only && pool.dtype == DType::BF16)) return false;
  if (!kernel_library_available("attention_bf16")) return false;
  const int64_t M = qkv.shape[0];
  const int64_t width = (int64_t)(heads + (write_kv ? 2 * kv_heads : 0)) * head_dim;
  require(qkv.ndim == 2 && qkv.shape[1] >= width && qkv.dtype == DType::F32 && qkv.contiguous(),
          "attention_from_projections: qkv " + qkv.describe() + " does not fit [" + std::to_string(M) + ", >= " +
              std::to_string(width) + "] float32");
  require(out.ndim == 2 && out.shape[0] == M && out.shape[1] == (int64_t)heads * head_dim && out.dtype == DType::BF16 &&
              out.contiguous(),
          "attention_from_projections: out has the wrong shape or dtype");
  check_pool("attention_from_projections", pool, kv_heads, head_dim, DType::BF16);
  const int P = (int)pool.shape[2];
  if ((head_dim != 64 && head_dim != 128) || P % 16 != 0 || heads / kv_heads > 16) return false;
  const int n = (int)work.M;
  const int context = window == 0 ? work.split_context : std::min(work.split_context, window + 16);
  int S = decode_splits(n, kv_heads, heads, context, std::min(context, typical_context(work)), compute_units(), head_dim);
  if (use.force_decode_splits > 0) S = std::min(use.force_decode_splits, std::max(1, (context + 15) / 16));
  float *part_o = nullptr, *part_ml = nullptr;
  if (S > 1) {
    part_o = (float*)ws.get("attn.part_o", (size_t)n * heads * S * head_dim * 4);
    part_ml = (float*)ws.get("attn.part_ml", (size_t)n * heads * S * 2 * 4);
  }
  int rc = KERNEL("attention_bf16", ti_attention_decode_prepared_bf16)(
      (const float*)qkv.data, (int)qkv.shape[1], q_w, k_w, eps, rot.inv_freq, rot.table, rot.table_len, pool.data,
      write_kv ? 1 : 0, view.table, view.table_width, work.positions,
      (work.slots_are_rows && view.table_width <= 1024 && use.early_page_ids) ? nullptr : work.slots, out.data, part_o, part_ml, n,
      heads, kv_heads, head_dim, P, scale, window, S, (hipStream_t)launch_stream());
  if (rc == 3) return false;
  check("attention_bf16", rc, "attention(decode, prepared)");
  took(S > 1 ? "[fused, runs]" : "[fused]");
  return true;
}

void Ops::attention(const AttentionWork& work, Workspace& ws, const CacheView& view, const Tensor& q, const Tensor& pool,
                    const Tensor& out, int heads, int kv_heads, int head_dim, float scale, int window) {
  TunedScope tuned(*this, "attention_bf16");
  TIMED("attention rows=" + std::to_string(work.M) + (work.decode_only ? " decode" : " tiles=" + std::to_string(work.n_tiles) + " single=" + std::to_string(work.n_decode_rows)) + " context<=" + std::to_string(work.max_context));
  bool done = false;
  if (q.dtype == DType::BF16 && use.fast_attention && kernel_library_available("attention_bf16")) {
    check_pool("attention", pool, kv_heads, head_dim, DType::BF16);
    const int P = (int)pool.shape[2];
    const bool served = (head_dim == 32 || head_dim == 64 || head_dim == 128) && P % 16 == 0;
    if (served) {
      done = true;
      void* stream = launch_stream();
      const int units = compute_units();
      // the portions first: with their keys cut into runs, the merge writes every row of the step, and
      // the rows of single tokens get their own result afterwards
      if (work.n_tiles && (head_dim == 64 || head_dim == 128) && work.n_tiles * heads < PAIRED_BELOW && work.tiles_small &&
          use.paired_prefill) {
        // few tiles: under a causal mask they differ much in work, and a launch lasts as long as its
        // heaviest workgroup; the paired kernel gives every workgroup a heavy and a light tile
        bool paired = false;
        int S = portion_launch(work.n_tiles_small, heads, work.portion_context, window, units, &paired);
        if (!use.portion_splits) S = 1;
        if (use.force_paired_tiles >= 0) paired = use.force_paired_tiles != 0;
        float *part_o = nullptr, *part_ml = nullptr;
        if (S > 1) {
          part_o = (float*)ws.get("attn.portion_o", (size_t)work.M * heads * S * head_dim * 4);
          part_ml = (float*)ws.get("attn.portion_ml", (size_t)work.M * heads * S * 2 * 4);
        }
        int rc = KERNEL("attention_bf16", ti_attention_prefill_paired_bf16)(
            q.data, pool.data, view.table, view.table_width, work.tiles_small, work.entry_meta, out.data, work.n_tiles_small,
            heads, kv_heads, head_dim, P, scale, window, (int)work.M, part_o, part_ml, S, paired ? 1 : 0,
            (hipStream_t)stream);
        if (rc == 3) done = false;
        else check("attention_bf16", rc, "attention(prefill, paired)");
      } else if (work.n_tiles) {
        int rc = KERNEL("attention_bf16", ti_attention_prefill_bf16)(
            q.data, pool.data, view.table, view.table_width, work.tiles, work.entry_meta, out.data, work.n_tiles, heads,
            kv_heads, head_dim, P, scale, window, (hipStream_t)stream);
        if (rc == 3) done = false;
        else check("attention_bf16", rc, "attention(prefill)");
      }
      const int n_dec = work.decode_only ? (int)work.M : work.n_decode_rows;
      if (done && n_dec) {
        const int* rows = work.decode_only ? nullptr : work.decode_rows;
        const int context = window == 0 ? work.split_context : std::min(work.split_context, window + 16);
        const int S = decode_splits(n_dec, kv_heads, heads, context, std::min(context, typical_context(work)), units, head_dim);
        float *part_o = nullptr, *part_ml = nullptr;
        if (S > 1) {
          part_o = (float*)ws.get("attn.part_o", (size_t)n_dec * heads * S * head_dim * 4);
          part_ml = (float*)ws.get("attn.part_ml", (size_t)n_dec * heads * S * 2 * 4);
        }
        int rc = KERNEL("attention_bf16", ti_attention_decode_bf16)(
            q.data, pool.data, view.table, view.table_width, work.positions,
            (work.slots_are_rows && !rows && view.table_width <= 1024 && use.early_page_ids) ? nullptr : work.slots, rows, out.data,
            part_o, part_ml, n_dec, heads, kv_heads, head_dim, P, scale, window, S, (hipStream_t)stream);
        if (rc == 3) done = false;
        else check("attention_bf16", rc, "attention(decode)");
      }
    }
  }
  took(done ? "[mfma]" : "[generic]");
  if (!done)
    attention_rows(q, pool, view, work.positions, work.slots, out, heads, kv_heads, head_dim, scale, window);
}

// ----------------------------------------------------------------------------------- sampling
void Ops::argmax(const Tensor& logits, int* out) {
  TIMED("argmax " + dims(logits));
  require(logits.ndim == 2 && logits.dtype == DType::F32 && logits.contiguous(),
          "argmax: logits must be contiguous float32 [n, V]");
  const int64_t n = logits.shape[0];
  const size_t need = (size_t)2 * 64 * std::max<int64_t>(n, 64) * 4;
  if (argmax_scratch_.bytes() < need) {
    flush();
    argmax_scratch_ = DeviceBuffer(need);
  }
  int rc = KERNEL("sampling", ti_argmax)((const float*)logits.data, out, argmax_scratch_.data(), (int)n,
                                         (int)logits.shape[1], (hipStream_t)launch_stream());
  check("sampling", rc, "argmax");
}

void Ops::sample(const Tensor& logits, const float* temperature, const int* top_k, const float* top_p,
                 const float* uniform, int* out) {
  TIMED("sample " + dims(logits));
  require(logits.ndim == 2 && logits.dtype == DType::F32 && logits.contiguous(),
          "sample: logits must be contiguous float32 [n, V]");
  void* scratch = nullptr;
  if (use.radix_sample) {
    const int64_t rows = std::max<int64_t>(logits.shape[0], 8);
    const size_t need = (size_t)KERNEL("sampling", ti_sample_scratch_bytes)((int)rows);
    if (sample_scratch_.bytes() < need) {
      flush();
      sample_scratch_ = DeviceBuffer(need);
      fill_zero(sample_scratch_.data(), need);     // the kernels leave it at zero
    }
    scratch = sample_scratch_.data();
  }
  int rc = KERNEL("sampling", ti_sample)((const float*)logits.data, temperature, top_k, top_p, uniform, out, scratch,
                                         (int)logits.shape[0], (int)logits.shape[1], (hipStream_t)launch_stream());
  check("sampling", rc, "sample");
}

void Ops::fill_zero(void* p, size_t bytes) {
  int rc = KERNEL("core", ti_fill_zero)(p, (long)bytes, (hipStream_t)launch_stream());
  check("core", rc, "fill_zero");
}

void Ops::fill_random(const Tensor& t, const std::string& init, double a, double b, uint64_t seed) {
  require(t.contiguous(), "fill_random: the tensor must be contiguous");
  const int kind = init == "normal" ? 0 : init == "uniform" ? 1 : init == "constant" ? 2 : -1;
  require(kind >= 0, "fill_random: unknown init '" + init + "'");
  const int dt = t.dtype == DType::I32 ? 2 : code(t.dtype, "fill_random");
  int rc = KERNEL("core", ti_fill_random)(dt, t.data, (long)t.numel(), dt == 2 ? 1 : kind, (float)a, (float)b,
                                          (unsigned long)seed, (hipStream_t)launch_stream());
  check("core", rc, "fill_random");
}

}  // namespace tinyinfer
