// Weights: safetensors files read and written, and the three places a model's tensors come from
// while it loads (a model folder, tensors in memory, the random generator).
//
// safetensors: 8 bytes little-endian header length n, n bytes of JSON
// `{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`, then the tensor
// bytes; offsets count from the end of the header.  (The reference's GGUF loader once treated data
// offsets as file-absolute: /root/reference/docs/report.md:84-91.)  The file is mapped; nothing
// in it is executed.
//
// Every fault of a checkpoint is reported in one error: tensors the model asks for and the files
// lack, tensors the files hold and nothing asks for, tensors of the wrong shape (the full shape
// is compared; the reference compares element counts only, /root/reference/src/model.cpp:74-80,
// 104-109, so a transposed matrix would pass there) or of the wrong kind of dtype.
//
// Dtypes on the device, by the role a part gives the tensor: a matrix takes the engine's compute
// dtype (bfloat16 stays bfloat16; under float32 every matrix is widened exactly; a matrix stored
// in 32-bit is rounded to bfloat16 only for a bfloat16 engine, and a line on stderr says so), a
// vector float32, a table int32.  Tensors go from the mapping through two pinned staging buffers
// straight into the part's own (fused) buffers: a model's weights are in device memory once.
#include <dirent.h>
#include <fcntl.h>
#include <hip/hip_runtime_api.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <thread>

#include "../include/inference.h"
#include "weights.h"

namespace tinyinfer {

WeightsError::WeightsError(const std::string& where, std::vector<std::string> missing_, std::vector<std::string> unexpected_,
                           std::vector<std::string> wrong_shape_, std::vector<std::string> wrong_dtype_)
    : Error([&] {
        auto list = [](const std::vector<std::string>& v) {
          std::string s;
          for (size_t i = 0; i < v.size(); ++i) s += (i ? ", " : "") + v[i];
          return s;
        };
        std::string m = where + ": the weights do not fit the model";
        if (!missing_.empty()) m += "\n  missing (" + std::to_string(missing_.size()) + "): " + list(missing_);
        if (!unexpected_.empty()) m += "\n  unexpected (" + std::to_string(unexpected_.size()) + "): " + list(unexpected_);
        if (!wrong_shape_.empty()) m += "\n  wrong shape (" + std::to_string(wrong_shape_.size()) + "): " + list(wrong_shape_);
        if (!wrong_dtype_.empty()) m += "\n  wrong dtype (" + std::to_string(wrong_dtype_.size()) + "): " + list(wrong_dtype_);
        return m;
      }()),
      missing(std::move(missing_)), unexpected(std::move(unexpected_)), wrong_shape(std::move(wrong_shape_)),
      wrong_dtype(std::move(wrong_dtype_)) {}

// ------------------------------------------------------------------------------- safetensors
namespace {
struct StoredType { const char* name; DType dtype; };
const StoredType STORED[] = {{"F32", DType::F32}, {"BF16", DType::BF16}, {"F16", DType::F16},
                             {"F64", DType::F64}, {"I32", DType::I32},   {"I64", DType::I64}};
std::string shape_text(const std::vector<int64_t>& s) {
  std::string t = "[";
  for (size_t i = 0; i < s.size(); ++i) t += (i ? ", " : "") + std::to_string(s[i]);
  return t + "]";
}
const char* stored_name(DType dt) {
  for (const auto& s : STORED)
    if (s.dtype == dt) return s.name;
  return "?";
}
}  // namespace

SafetensorsFile::SafetensorsFile(const std::string& path_) : path(path_) {
  const int fd = open(path.c_str(), O_RDONLY);
  if (fd < 0) throw FileError(path + ": cannot be opened");
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 8) {
    close(fd);
    throw FileError(path + ": too short to be a safetensors file");
  }
  size_ = (size_t)st.st_size;
  void* m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (m == MAP_FAILED) throw FileError(path + ": cannot be mapped");
  map_ = (const uint8_t*)m;
  uint64_t n = 0;
  memcpy(&n, map_, 8);
  if (n == 0 || 8 + n > size_)
    throw FileError(path + ": header length " + std::to_string(n) + " does not fit the file (" + std::to_string(size_) + " bytes)");
  Json header;
  try {
    header = Json::parse(std::string((const char*)map_ + 8, (size_t)n));
  } catch (const Error& e) {
    throw FileError(path + ": header is not JSON (" + e.what() + ")");
  }
  base_ = map_ + 8 + n;
  const size_t data_bytes = size_ - 8 - (size_t)n;
  for (const auto& kv : header.members()) {
    if (kv.first == "__metadata__") continue;
    const Json& e = kv.second;
    Entry en;
    const std::string dt = e.at("dtype").as_string();
    bool known = false;
    for (const auto& s : STORED)
      if (dt == s.name) {
        en.dtype = s.dtype;
        known = true;
      }
    if (!known) throw FileError(path + ": tensor '" + kv.first + "' has dtype '" + dt + "', which is not served");
    int64_t numel = 1;
    for (const Json& s : e.at("shape").items()) {
      en.shape.push_back(s.as_int());
      numel *= s.as_int();
    }
    const Json& off = e.at("data_offsets");
    en.begin = (size_t)off[0].as_int();
    en.end = (size_t)off[1].as_int();
    const size_t need = (size_t)numel * dtype_size(en.dtype);
    if (en.end < en.begin || en.end - en.begin != need || en.end > data_bytes)
      throw FileError(path + ": tensor '" + kv.first + "' " + dt + shape_text(en.shape) + " needs " + std::to_string(need) +
                      " bytes but its offsets [" + std::to_string(en.begin) + ", " + std::to_string(en.end) + ") give " +
                      std::to_string(en.end - en.begin) + " (file holds " + std::to_string(data_bytes) + " data bytes)");
    index_[kv.first] = entries_.size();
    entries_.emplace_back(kv.first, std::move(en));
  }
}

SafetensorsFile::~SafetensorsFile() {
  if (map_) munmap((void*)map_, size_);
}

const SafetensorsFile::Entry* SafetensorsFile::find(const std::string& name) const {
  auto it = index_.find(name);
  return it == index_.end() ? nullptr : &entries_[it->second].second;
}

void write_safetensors(const std::string& path, const std::vector<HostTensor>& tensors,
                       const std::vector<std::pair<std::string, std::string>>& metadata) {
  Json header = Json::object();
  if (!metadata.empty()) {
    Json m = Json::object();
    for (const auto& kv : metadata) m.set(kv.first, kv.second);
    header.set("__metadata__", m);
  }
  size_t off = 0;
  for (const auto& t : tensors) {
    int64_t numel = 1;
    Json shape = Json::array();
    for (int64_t s : t.shape) {
      numel *= s;
      shape.push(s);
    }
    const size_t n = (size_t)numel * dtype_size(t.dtype);
    Json e = Json::object();
    e.set("dtype", stored_name(t.dtype));
    e.set("shape", shape);
    Json o = Json::array();
    o.push((int64_t)off);
    o.push((int64_t)(off + n));
    e.set("data_offsets", o);
    header.set(t.name, e);
    off += n;
  }
  std::string hj = header.dump();
  while (hj.size() % 8) hj += ' ';
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) throw FileError(path + ": cannot be written");
  const uint64_t n = hj.size();
  bool ok = fwrite(&n, 8, 1, f) == 1 && fwrite(hj.data(), 1, hj.size(), f) == hj.size();
  for (const auto& t : tensors) {
    int64_t numel = 1;
    for (int64_t s : t.shape) numel *= s;
    const size_t bytes = (size_t)numel * dtype_size(t.dtype);
    if (bytes) ok = ok && fwrite(t.data, 1, bytes, f) == bytes;
  }
  ok = (fclose(f) == 0) && ok;
  if (!ok) throw FileError(path + ": short write");
}

// -------------------------------------------------------------------------------- conversions
namespace {
inline float bf16_to_f32(uint16_t v) {
  uint32_t u = (uint32_t)v << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
inline uint16_t f32_to_bf16(float f) {      // round to nearest even; NaN stays NaN
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
inline float f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else {
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while (!(man & 0x400u));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp - 15 + 127) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

bool is_float(DType dt) { return dt == DType::F32 || dt == DType::BF16 || dt == DType::F16 || dt == DType::F64; }

// n elements from `src` (stored as `from`) to `dst` (as `to`), on the host
void convert(const void* src, DType from, void* dst, DType to, size_t n) {
  if (from == to) {
    memcpy(dst, src, n * dtype_size(to));
    return;
  }
  auto read = [&](size_t i) -> double {
    switch (from) {
      case DType::F32: return ((const float*)src)[i];
      case DType::BF16: return bf16_to_f32(((const uint16_t*)src)[i]);
      case DType::F16: return f16_to_f32(((const uint16_t*)src)[i]);
      case DType::F64: return ((const double*)src)[i];
      case DType::I32: return ((const int32_t*)src)[i];
      case DType::I64: return (double)((const int64_t*)src)[i];
    }
    return 0.0;
  };
  for (size_t i = 0; i < n; ++i) {
    const double v = read(i);
    switch (to) {
      case DType::F32: ((float*)dst)[i] = (float)v; break;
      case DType::BF16: ((uint16_t*)dst)[i] = f32_to_bf16((float)v); break;
      case DType::I32: ((int32_t*)dst)[i] = (int32_t)v; break;
      default: throw KernelError(std::string("weights: cannot convert to ") + dtype_name(to));
    }
  }
}

void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw KernelError(std::string(what) + ": " + hipGetErrorString(e));
}

// Two pinned buffers take turns: while one is on its way to the device the host converts into
// the other.
class Staging {
 public:
  static const size_t CHUNK = 32u << 20;
  Staging() {
    for (int i = 0; i < 2; ++i) {
      hip_check(hipHostMalloc(&buf_[i], CHUNK, hipHostMallocDefault), "hipHostMalloc");
      hip_check(hipEventCreateWithFlags(&done_[i], hipEventDisableTiming), "hipEventCreate");
    }
    hip_check(hipStreamCreate(&stream_), "hipStreamCreate");
  }
  ~Staging() {
    (void)hipStreamSynchronize(stream_);
    for (int i = 0; i < 2; ++i) {
      (void)hipHostFree(buf_[i]);
      (void)hipEventDestroy(done_[i]);
    }
    (void)hipStreamDestroy(stream_);
  }
  // n elements of `from` at src -> device dst as `to`
  void send(const void* src, DType from, void* dst, DType to, size_t n) {
    const size_t in = dtype_size(from), out = dtype_size(to);
    const size_t per = CHUNK / std::max(in, out);
    for (size_t i = 0; i < n; i += per) {
      const size_t k = std::min(per, n - i);
      if (used_[turn_]) hip_check(hipEventSynchronize(done_[turn_]), "hipEventSynchronize");
      convert((const char*)src + i * in, from, buf_[turn_], to, k);
      hip_check(hipMemcpyAsync((char*)dst + i * out, buf_[turn_], k * out, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
      hip_check(hipEventRecord(done_[turn_], stream_), "hipEventRecord");
      used_[turn_] = true;
      turn_ ^= 1;
    }
  }
  void finish() { hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }

 private:
  void* buf_[2] = {nullptr, nullptr};
  hipEvent_t done_[2];
  bool used_[2] = {false, false};
  hipStream_t stream_ = nullptr;
  int turn_ = 0;
};

DType role_dtype(TensorNeed::Role role, DType matrix) {
  return role == TensorNeed::Matrix ? matrix : role == TensorNeed::Vector ? DType::F32 : DType::I32;
}
}  // namespace

Tensor WeightSource::alloc(DType dt, const std::vector<int64_t>& shape) {
  Tensor t(nullptr, dt, shape);
  owner->emplace_back(t.bytes());
  t.data = owner->back().data();
  return t;
}

Tensor WeightSource::fetch(const std::string& name, const TensorNeed& need) {
  auto it = fetched_.find(name);
  if (it != fetched_.end()) return it->second;      // a tied head reads the embedding's copy
  Tensor t = alloc(role_dtype(need.role, matrix_dtype), need.shape);
  fill(name, t);
  fetched_[name] = t;
  return t;
}

// ------------------------------------------------------------------------------ the sources
namespace {
// A model folder: `model.safetensors`, or the shards an index file lists, or every *.safetensors.
class FolderSource final : public WeightSource {
 public:
  explicit FolderSource(const std::string& dir) {
    std::vector<std::string> files;
    struct stat st;
    const std::string single = dir + "/model.safetensors", index = dir + "/model.safetensors.index.json";
    if (stat(single.c_str(), &st) == 0) {
      files.push_back(single);
    } else if (stat(index.c_str(), &st) == 0) {
      std::ifstream f(index);
      std::stringstream ss;
      ss << f.rdbuf();
      const Json j = Json::parse(ss.str());
      for (const auto& kv : j.at("weight_map").members()) {
        const std::string p = dir + "/" + kv.second.as_string();
        if (std::find(files.begin(), files.end(), p) == files.end()) files.push_back(p);
      }
      std::sort(files.begin(), files.end());
    } else if (DIR* d = opendir(dir.c_str())) {
      while (dirent* e = readdir(d)) {
        const std::string n = e->d_name;
        if (n.size() > 12 && n.compare(n.size() - 12, 12, ".safetensors") == 0) files.push_back(dir + "/" + n);
      }
      closedir(d);
      std::sort(files.begin(), files.end());
    }
    if (files.empty()) throw FileError(dir + ": no model.safetensors (and no other *.safetensors) in the model folder");
    for (const auto& p : files) files_.emplace_back(new SafetensorsFile(p));
  }
  std::vector<std::pair<std::string, SourceInfo>> list() const override {
    std::vector<std::pair<std::string, SourceInfo>> out;
    for (const auto& f : files_)
      for (const auto& e : f->entries()) out.emplace_back(e.first, SourceInfo{e.second.dtype, e.second.shape});
    return out;
  }
  bool has(const std::string& name) const override {
    for (const auto& f : files_)
      if (f->find(name)) return true;
    return false;
  }
  void fill(const std::string& name, const Tensor& dst) override {
    for (const auto& f : files_)
      if (const auto* e = f->find(name)) {
        if (dst.dtype == DType::BF16 && (e->dtype == DType::F32 || e->dtype == DType::F64)) rounded.push_back(name);
        if (to_host) {
          convert(f->bytes(*e), e->dtype, dst.data, dst.dtype, (size_t)dst.numel());
          return;
        }
        if (!staging_) staging_.reset(new Staging());
        staging_->send(f->bytes(*e), e->dtype, dst.data, dst.dtype, (size_t)dst.numel());
        return;
      }
    throw Error("tensor '" + name + "' is not in the model folder");
  }
  void finish() override {
    if (staging_) staging_->finish();
    if (!rounded.empty())
      fprintf(stderr, "[tinyinfer] %zu matrices stored in 32-bit are rounded to bfloat16 for --dtype bfloat16 (first: %s)\n",
              rounded.size(), rounded[0].c_str());
  }
  std::vector<std::string> rounded;

 private:
  std::vector<std::unique_ptr<SafetensorsFile>> files_;
  std::unique_ptr<Staging> staging_;
};

// Tensors in memory (host or device).  Device tensors must already have the dtype their role asks for.
class TensorsSource final : public WeightSource {
 public:
  TensorsSource(const std::vector<HostTensor>& tensors, bool on_device) : tensors_(tensors), on_device_(on_device) {
    for (size_t i = 0; i < tensors_.size(); ++i) index_[tensors_[i].name] = i;
  }
  std::vector<std::pair<std::string, SourceInfo>> list() const override {
    std::vector<std::pair<std::string, SourceInfo>> out;
    for (const auto& t : tensors_) out.emplace_back(t.name, SourceInfo{t.dtype, t.shape});
    return out;
  }
  bool has(const std::string& name) const override { return index_.count(name) != 0; }
  void fill(const std::string& name, const Tensor& dst) override {
    const HostTensor& t = tensors_[index_.at(name)];
    if (to_host) {
      if (on_device_) throw KernelError("tensors on the device cannot be loaded into host memory");
      convert(t.data, t.dtype, dst.data, dst.dtype, (size_t)dst.numel());
    } else if (on_device_) {
      if (t.dtype != dst.dtype)
        throw KernelError("tensor '" + name + "' is " + dtype_name(t.dtype) + " on the device, the model holds it as " +
                          dtype_name(dst.dtype));
      hip_check(hipMemcpy(dst.data, t.data, dst.bytes(), hipMemcpyDeviceToDevice), "hipMemcpy");
    } else {
      if (!staging_) staging_.reset(new Staging());
      staging_->send(t.data, t.dtype, dst.data, dst.dtype, (size_t)dst.numel());
    }
  }
  void finish() override {
    if (staging_) staging_->finish();
  }

 private:
  const std::vector<HostTensor>& tensors_;
  bool on_device_;
  std::map<std::string, size_t> index_;
  std::unique_ptr<Staging> staging_;
};
}  // namespace

uint64_t tensor_seed(uint64_t seed, const std::string& name) {
  // FNV-1a of the name, mixed with the seed: a tensor's values depend on its name and the seed only
  uint64_t h = 0xcbf29ce484222325ull;
  for (unsigned char c : name) h = (h ^ c) * 0x100000001b3ull;
  return h ^ (seed * 0x9E3779B97F4A7C15ull + 0x632BE59BD9B4E019ull);
}

namespace {
// The random generator on the device: values drawn where they are needed, nothing on the host.
class RandomSource final : public WeightSource {
 public:
  RandomSource(const std::vector<std::pair<std::string, TensorNeed>>& needs, uint64_t seed, Ops& ops)
      : seed_(seed), ops_(ops) {
    for (const auto& kv : needs)
      if (!kv.second.optional) needs_[kv.first] = kv.second;
  }
  std::vector<std::pair<std::string, SourceInfo>> list() const override {
    std::vector<std::pair<std::string, SourceInfo>> out;
    for (const auto& kv : needs_)
      out.emplace_back(kv.first, SourceInfo{kv.second.role == TensorNeed::Table ? DType::I32 : DType::F32, kv.second.shape});
    return out;
  }
  bool has(const std::string& name) const override { return needs_.count(name) != 0; }
  void fill(const std::string& name, const Tensor& dst) override {
    const TensorNeed& n = needs_.at(name);
    // a part may fill a range of rows of a fused matrix: the values of a tensor do not depend on where it lands
    ops_.fill_random(dst, n.init, n.a, n.b, tensor_seed(seed_, name));
  }
  void finish() override { hip_check(hipStreamSynchronize((hipStream_t)ops_.stream()), "hipStreamSynchronize"); }

 private:
  std::map<std::string, TensorNeed> needs_;
  uint64_t seed_;
  Ops& ops_;
};
}  // namespace

std::unique_ptr<WeightSource> make_folder_source(const std::string& dir) { return std::unique_ptr<WeightSource>(new FolderSource(dir)); }
std::unique_ptr<WeightSource> make_tensors_source(const std::vector<HostTensor>& t, bool on_device) {
  return std::unique_ptr<WeightSource>(new TensorsSource(t, on_device));
}
std::unique_ptr<WeightSource> make_random_source(const std::vector<std::pair<std::string, TensorNeed>>& needs, uint64_t seed, Ops& ops) {
  return std::unique_ptr<WeightSource>(new RandomSource(needs, seed, ops));
}

// What the device's generator computes (csrc/core.hip, fill_random_kernel), on the host: the
// values of a model folder written here.  Element i is a pure function of (seed, i).
static inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
void host_random(const TensorNeed& need, uint64_t seed, DType dt, void* out) {
  int64_t n = 1;
  for (int64_t s : need.shape) n *= s;
  const uint64_t base = mix64(seed);
  const int kind = need.init == "normal" ? 0 : need.init == "uniform" ? 1 : need.init == "constant" ? 2 : -1;
  if (kind < 0) throw ConfigError("unknown init '" + need.init + "'");
  auto work = [&](int64_t lo, int64_t hi) {
    for (int64_t i = lo; i < hi; ++i) {
      const uint64_t z = mix64(base ^ (uint64_t)i);
      if (dt == DType::I32) {
        const int a = (int)need.a, b = (int)need.b;
        ((int32_t*)out)[i] = a + (int)((z >> 11) % (uint64_t)(b > a ? b - a : 1));
        continue;
      }
      // in double precision, rounded to 32-bit once at the end, with the parameters as the device gets them
      // (32-bit): the same bits as csrc/core.hip's fill_random_kernel draws
      const double u1 = ((double)((z >> 40) & 0xffffffu) + 1.0) * (1.0 / 16777216.0);
      const double u2 = (double)((z >> 16) & 0xffffffu) * (1.0 / 16777216.0);
      const double a = (double)(float)need.a, b = (double)(float)need.b;
      float v;
      if (kind == 0) v = (float)(a + b * (std::sqrt(-2.0 * std::log(u1)) * std::cos(6.28318530717958647692 * u2)));
      else if (kind == 1) v = (float)(a + (b - a) * u2);
      else v = (float)need.a;
      if (dt == DType::BF16) ((uint16_t*)out)[i] = f32_to_bf16(v);
      else ((float*)out)[i] = v;
    }
  };
  const int threads = n > (1 << 20) ? 8 : 1;
  if (threads == 1) {
    work(0, n);
  } else {
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t) pool.emplace_back(work, n * t / threads, n * (t + 1) / threads);
    for (auto& th : pool) th.join();
  }
}

// Check a source against what the model asks for; every fault in one error.
void check_source(const std::string& where, const std::vector<std::pair<std::string, TensorNeed>>& needs,
                  const WeightSource& src) {
  std::map<std::string, SourceInfo> have;
  std::vector<std::string> order;
  for (auto& kv : src.list()) {
    if (!have.count(kv.first)) order.push_back(kv.first);
    have[kv.first] = kv.second;
  }
  std::map<std::string, const TensorNeed*> wanted;
  for (const auto& kv : needs) wanted[kv.first] = &kv.second;
  std::vector<std::string> missing, unexpected, wrong_shape, wrong_dtype;
  for (const auto& kv : needs) {
    auto it = have.find(kv.first);
    if (it == have.end()) {
      if (!kv.second.optional) missing.push_back(kv.first);
      continue;
    }
    if (it->second.shape != kv.second.shape)
      wrong_shape.push_back(kv.first + " is " + shape_text(it->second.shape) + ", expected " + shape_text(kv.second.shape));
    const bool fl = is_float(it->second.dtype);
    if (kv.second.role == TensorNeed::Table && fl)
      wrong_dtype.push_back(kv.first + " is " + dtype_name(it->second.dtype) + ", expected an integer type");
    if (kv.second.role != TensorNeed::Table && !fl)
      wrong_dtype.push_back(kv.first + " is " + dtype_name(it->second.dtype) + ", expected a floating-point type");
  }
  for (const auto& n : order)
    if (!wanted.count(n)) unexpected.push_back(n);
  if (!missing.empty() || !unexpected.empty() || !wrong_shape.empty() || !wrong_dtype.empty())
    throw WeightsError(where, missing, unexpected, wrong_shape, wrong_dtype);
}

}  // namespace tinyinfer
