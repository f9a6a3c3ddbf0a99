// tinyinfer for AMD MI355X: the programming interface of the engine, in one header.
//
// The reference's counterpart is `class Inference` with `init / forward / reset_kv /
// set_use_cuda_graph` (/root/reference/src/inference.h:12-44) over `Qwen3Model::load`
// (/root/reference/src/model.h:39-53).  Here the same step-function shape (a flat batch of
// tokens with positions, logits at chosen rows) sits on a paged cache with a scheduler above
// it, and the model is put together from registered parts.
//
//   auto model  = tinyinfer::Model::from_folder("model_dir", "bfloat16");
//   tinyinfer::EngineOptions opt;  opt.max_seq = 2048;  opt.max_tokens = 16 * 2048;
//   tinyinfer::Engine engine(model, opt);
//   auto out = tinyinfer::generate(engine, {{1, 2, 3}}, 16, tinyinfer::SamplingParams{});
//
// Everything that touches a token's numbers is a HIP kernel of the libraries declared in
// tinyinfer_kernels.h; this library (libtinyinfer) is the host around them: configuration,
// weights, parts, cache manager, step function, scheduler, sampler.  The same objects serve
// the Python package through the C interface at the end of this file.
//
// Request ids are 64-bit integers chosen by the caller.  All device pointers belong to the
// current HIP device; an engine launches on the stream it was given (the null stream by
// default).  Errors are exceptions derived from tinyinfer::Error.
#pragma once
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace tinyinfer {

// ------------------------------------------------------------------------------------ errors
struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
  virtual const char* kind() const { return "Error"; }
};
#define TINYINFER_ERROR(Name, Base)                       \
  struct Name : Base {                                    \
    using Base::Base;                                     \
    const char* kind() const override { return #Name; }   \
  }
TINYINFER_ERROR(ConfigError, Error);      // a config.json that cannot be served; the text names the key
TINYINFER_ERROR(CacheError, Error);
TINYINFER_ERROR(OutOfPages, CacheError);  // a reservation the free pages cannot cover; nothing was taken
TINYINFER_ERROR(EngineError, Error);
TINYINFER_ERROR(SchedulerError, Error);
TINYINFER_ERROR(KernelError, Error);      // a kernel refused its arguments, is not built, or failed to launch
TINYINFER_ERROR(FileError, Error);
// the weights do not fit the model: every fault in one error
struct WeightsError : Error {
  std::vector<std::string> missing, unexpected, wrong_shape, wrong_dtype;
  WeightsError(const std::string& where, std::vector<std::string> missing, std::vector<std::string> unexpected,
               std::vector<std::string> wrong_shape, std::vector<std::string> wrong_dtype);
  const char* kind() const override { return "WeightsError"; }
};

// -------------------------------------------------------------------------------------- JSON
// A small JSON value: what config.json, a safetensors header and a part's parameters need.
// Integers and other numbers are kept apart (3 and 3.0 are integers, 3.5 is not).
class Json {
 public:
  enum Type { Null, Bool, Int, Float, String, Array, Object };
  Json() = default;
  Json(std::nullptr_t) {}
  Json(bool b) : type_(Bool), b_(b) {}
  Json(int v) : type_(Int), i_(v) {}
  Json(int64_t v) : type_(Int), i_(v) {}
  Json(double v) : type_(Float), d_(v) {}
  Json(const char* s) : type_(String), s_(s) {}
  Json(std::string s) : type_(String), s_(std::move(s)) {}
  static Json array() { Json j; j.type_ = Array; return j; }
  static Json object() { Json j; j.type_ = Object; return j; }
  static Json parse(const std::string& text);          // throws Error with the offset
  std::string dump() const;

  Type type() const { return type_; }
  bool is_null() const { return type_ == Null; }
  bool is_number() const { return type_ == Int || type_ == Float; }
  bool as_bool() const { return b_; }
  int64_t as_int() const { return type_ == Int ? i_ : (int64_t)d_; }
  double as_double() const { return type_ == Int ? (double)i_ : d_; }
  const std::string& as_string() const { return s_; }
  // arrays
  size_t size() const { return type_ == Object ? members_.size() : items_.size(); }
  const Json& operator[](size_t i) const { return items_[i]; }
  void push(Json v) { items_.push_back(std::move(v)); }
  const std::vector<Json>& items() const { return items_; }
  // objects (members keep their order)
  const Json* find(const std::string& key) const;
  bool has(const std::string& key) const { const Json* j = find(key); return j && !j->is_null(); }
  const Json& at(const std::string& key) const;          // throws Error if absent
  void set(const std::string& key, Json v);
  const std::vector<std::pair<std::string, Json>>& members() const { return members_; }

 private:
  Type type_ = Null;
  bool b_ = false;
  int64_t i_ = 0;
  double d_ = 0.0;
  std::string s_;
  std::vector<Json> items_;
  std::vector<std::pair<std::string, Json>> members_;
};

// ----------------------------------------------------------------------------- configuration
// The hyper-parameters of the Qwen3 dense decoder, read from the keys of its config.json
// (the reference reads nine of them from GGUF keys: /root/reference/src/model.h:11-21,
// src/model.cpp:32-47).  Options that would change the math and are not served
// (attention_bias, rope_scaling, another hidden_act) are refused by name.
struct Qwen3Config {
  int64_t vocab_size = 0, hidden_size = 0, intermediate_size = 0, num_hidden_layers = 0;
  int64_t num_attention_heads = 0, num_key_value_heads = 0, head_dim = 0;
  double rms_norm_eps = 1e-6, rope_theta = 1e6;
  int tie_word_embeddings = -1;                 // 1, 0, or -1: decided by whether the weights hold lm_head.weight
  std::vector<std::string> layer_types;         // "full_attention" | "sliding_attention", one per layer
  int64_t sliding_window = 0;                   // 0: no layer slides
  int64_t max_position_embeddings = 0;          // 0: absent
  std::vector<int64_t> eos_token_ids;
  std::string architecture = "Qwen3ForCausalLM";

  static Qwen3Config from_json(const Json& config);     // reads and validates
  void validate() const;
  Json to_json() const;                                 // the config.json that reads back as this
};
Json read_config_json(const std::string& model_dir);

// ------------------------------------------------------------------------------ model as data
struct PartSpec {
  std::string kind;      // the registered kind within the part's family
  Json params = Json::object();   // every size and constant the part needs; a nested part is {"kind", "params", "name"}
  std::string name;      // appended to the owner's tensor-name prefix ("self_attn", "mlp")
  Json to_json() const;
  static PartSpec from_json(const Json&);
};
struct LayerSpec {
  std::string prefix;
  PartSpec block;
  std::vector<std::pair<std::string, PartSpec>> parts;   // slot of the block arrangement -> part
  int cache_from = -1;   // index of another layer whose cache this layer's mixer reads (-1: its own)
};
struct ModelSpec {
  std::string architecture;
  int64_t vocab_size = 0, hidden_size = 0;
  PartSpec embedding, final_norm, lm_head;
  std::vector<LayerSpec> layers;
  std::vector<int> schedule;              // order in which layers run (empty: 0, 1, 2, ...); an index may come twice
  std::vector<int64_t> eos_token_ids;
  int64_t max_position_embeddings = 0;
  std::vector<int> run_order() const;
  Json to_json() const;
  static ModelSpec from_json(const Json&);
};

// An architecture: config.json -> ModelSpec.  The reference gates on one string
// (/root/reference/src/model.cpp:26-30); here that compare is a table.
using SpecBuilder = std::function<ModelSpec(const Json& config)>;
// The architecture's typed configuration: config.json read, validated and written back with its defaults
// filled in (what a model folder's config.json says after a round trip).  Optional.
using ConfigReader = std::function<Json(const Json& config)>;
void register_architecture(const std::vector<std::string>& names, SpecBuilder builder, ConfigReader typed = nullptr);
// {"architecture": the registered name that matched, "config": the typed configuration (the input itself if
// the architecture registered no reader)}; ConfigError as spec_from_config
Json typed_config(const Json& config);
std::vector<std::string> registered_architectures();
bool architecture_registered(const Json& config);
ModelSpec spec_from_config(const Json& config);   // by architectures[0], else model_type; ConfigError lists what is registered

// ------------------------------------------------------------------------------------ tensors
enum class DType : int { F32 = 0, BF16 = 1, I32 = 2, F16 = 3, F64 = 4, I64 = 5 };   // the kernels serve 0 and 1
size_t dtype_size(DType);
const char* dtype_name(DType);
DType dtype_from_name(const std::string&);     // "float32" | "bfloat16"

// A view of device (or host) memory: up to 4 dims, strides in elements.
struct Tensor {
  void* data = nullptr;
  DType dtype = DType::F32;
  int ndim = 0;
  int64_t shape[4] = {0, 0, 0, 0};
  int64_t stride[4] = {0, 0, 0, 0};
  Tensor() = default;
  Tensor(void* p, DType dt, std::initializer_list<int64_t> dims);      // contiguous
  Tensor(void* p, DType dt, const std::vector<int64_t>& dims);
  bool defined() const { return data != nullptr; }
  int64_t numel() const;
  size_t bytes() const { return (size_t)numel() * dtype_size(dtype); }
  bool contiguous() const;
  Tensor rows(int64_t first, int64_t count) const;   // a range of the first dimension
  Tensor cols(int64_t first, int64_t count) const;   // a range of the last dimension of a 2-D tensor
  template <class T> T* ptr() const { return (T*)data; }
  std::string describe() const;
};

// Where device memory comes from.  Default: hipMalloc / hipFree.  The Python package installs
// torch's allocator, so that every buffer here is also a torch tensor there.
struct Allocator {
  void* (*alloc)(void* user, size_t bytes) = nullptr;
  void (*release)(void* user, void* p) = nullptr;
  void* user = nullptr;
};
void set_allocator(const Allocator&);
void detach_allocator();      // from now on memory is no longer given back (the allocator's owner is going away)
class DeviceBuffer {        // owns one allocation
 public:
  DeviceBuffer() = default;
  explicit DeviceBuffer(size_t bytes);
  ~DeviceBuffer();
  DeviceBuffer(DeviceBuffer&&) noexcept;
  DeviceBuffer& operator=(DeviceBuffer&&) noexcept;
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  void* data() const { return p_; }
  size_t bytes() const { return n_; }
 private:
  void* p_ = nullptr;
  size_t n_ = 0;
  bool host_ = false;
};
// While one of these lives, the thread's DeviceBuffers are host memory (a model loaded without a
// GPU, to look at its weights).
struct HostMemoryScope {
  HostMemoryScope();
  ~HostMemoryScope();
  bool before;
};

// --------------------------------------------------------------------- what parts declare
struct TensorNeed {
  enum Role { Matrix, Vector, Table };   // held in the engine's compute dtype / float32 / int32
  std::vector<int64_t> shape;
  Role role = Matrix;
  std::string init = "normal";           // random-weights mode: "normal" (a = mean, b = std), "uniform" [a, b), "constant" a
  double a = 0.0, b = 0.02;
  bool optional = false;                 // absent from the checkpoint is allowed
};
struct CacheNeed {
  // PagedKV: keys and values per token, in the layout the attention kernels read.  PagedRows: whatever a
  // token keeps, `row_shape` elements per token and layer in pages of their own layout [page][row][...]
  // (a mixer with another kind of memory than keys and values).  State: a fixed size per request.
  enum Kind { PagedKV, State, PagedRows } kind = PagedKV;
  int kv_heads = 0, head_dim = 0, window = 0;    // PagedKV; window (PagedRows too) 0: every token is kept
  std::vector<int64_t> state_shape;              // State: float32 per request and layer, zeroed at admission
  std::vector<int64_t> row_shape;                // PagedRows: one or two dimensions, in the compute dtype ...
  bool rows_f32 = false;                         // ... or in float32
  bool paged() const { return kind != State; }
  bool operator==(const CacheNeed& o) const;
};

// ------------------------------------------------------------------------------------ kernels
// Where the kernel libraries are: name ("core", "gemm_bf16", ...) -> shared library.  Unregistered
// names are looked up in kernels.manifest beside this library or in $TINYINFER_KERNEL_DIR.
void register_kernel_library(const std::string& name, const std::string& path);
bool kernel_library_available(const std::string& name);
// A function of a kernel library by name; the library is opened at the first call.  A part that lives
// outside this library and brings kernels of its own registers their library and calls into it through
// this (KernelError if the library or the function is not there).
void* kernel_symbol(const std::string& library, const std::string& name);
// Opens a shared library whose static initialisers (or its `extern "C" void tinyinfer_plugin_init()`)
// register parts, architectures or kernel libraries: a model made of parts this library does not
// know then builds, loads and steps like any other.  The plugin links with this library.
void load_plugin(const std::string& path);

class Workspace;       // named scratch buffers of a step
struct Rows;           // activation rows, maybe a norm not computed yet
struct AttentionWork;  // the work lists the attention kernels read

// The kernels as calls on tensors: shapes and dtypes are checked on the host, then the kernel
// is launched on this object's stream.  No fallback to the CPU or to a library.  One object per
// engine: it holds the partial sums a split product left for the next norm (see `flush`).
class Ops {
 public:
  explicit Ops(void* stream = nullptr);
  ~Ops();
  void* stream() const { return stream_; }
  void set_stream(void* s) { flush(); stream_ = s; }
  int compute_units();

  // a token below zero stands for fed[-1 - token] (device memory, n_fed ids; may be null)
  void embed(const Tensor& table, const int* tokens, int64_t M, const Tensor& x, const int* fed = nullptr, int n_fed = 0);
  // out[r] = rmsnorm(x[rows ? rows[r] : r]) * w
  void rmsnorm(const Tensor& x, const Tensor& w, float eps, const Tensor& out, const int* rows = nullptr, int64_t n_rows = 0);
  void rope_neox(const Tensor& x, const int* positions, const Tensor& inv_freq);      // in place on f32 [M, heads, hd]
  void rope_table(const Tensor& inv_freq, const Tensor& table);                       // f32 [n_pos, hd/2, 2]
  struct Rotation { const float* inv_freq = nullptr; const float* table = nullptr; int table_len = 0; };
  struct CacheView { const int* table = nullptr; int table_width = 0; int page_size = 0; };
  void qk_norm_rope_kv_write(const Tensor& qkv, const float* q_w, const float* k_w, float eps, const Rotation& rot,
                             const int* positions, const int* slots, const CacheView& view, const Tensor& pool,
                             const Tensor& q_out, int heads, int kv_heads, int head_dim);
  void qk_norm_inplace(const Tensor& qkv, const float* q_w, const float* k_w, float eps, int heads, int kv_heads, int head_dim);
  // out (op)= a w^T.  epilogue: "store" f32 = ; "add" f32 += ; "store_act" T = ; "swiglu" w = [gate; up].
  // may_defer (with "add"): the caller promises that `out` is read next through this object.
  enum Epilogue { Store = 0, Add = 1, StoreAct = 2, SwiGLU = 3 };
  void linear(const Rows& a, const Tensor& w, const Tensor& out, Epilogue epi, bool may_defer = false);
  void linear(const Tensor& a, const Tensor& w, const Tensor& out, Epilogue epi, bool may_defer = false);
  bool can_fuse_norm(int64_t n_rows, DType dtype) const;
  // rmsnorm and product in one kernel; false if no kernel serves the shape (nothing was launched)
  bool linear_with_norm(const Rows& a, const Tensor& w, const Tensor& out, Epilogue epi);
  // product + per-head norm + rotation + cache write in one kernel (steps of many tokens, bfloat16)
  bool qkv_prepared(const Rows& a, const Tensor& w, const float* q_w, const float* k_w, float eps, const Rotation& rot,
                    const int* positions, const int* slots, const CacheView& view, const Tensor& pool,
                    const Tensor& q_out, int heads, int kv_heads, int head_dim);
  void attention_rows(const Tensor& q, const Tensor& pool, const CacheView& view, const int* positions, const int* slots,
                      const Tensor& out, int heads, int kv_heads, int head_dim, float scale, int window);
  void attention(const AttentionWork& work, Workspace& ws, const CacheView& view, const Tensor& q, const Tensor& pool,
                 const Tensor& out, int heads, int kv_heads, int head_dim, float scale, int window);
  bool attention_from_projections(const AttentionWork& work, Workspace& ws, const CacheView& view, const Tensor& qkv,
                                  const float* q_w, const float* k_w, float eps, const Rotation& rot, const Tensor& pool,
                                  bool write_kv, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                                  int window);
  void argmax(const Tensor& logits, int* out);
  void sample(const Tensor& logits, const float* temperature, const int* top_k, const float* top_p, const float* uniform,
              int* out);
  void fill_zero(void* p, size_t bytes);
  void fill_random(const Tensor& t, const std::string& init, double a, double b, uint64_t seed);
  // Partial sums that a product left in the workspace are added now (same order, same bits as
  // the norm that would have added them).  Every launch through this object does it first.
  void flush();
  int pending_splits() const { return pending_.out ? pending_.splits : 0; }   // 0: no sums are waiting
  // Per-call timing with events (the reference's selftest times its kernels the same way:
  // /root/reference/src/selftest.cpp:404-424): while on, every call records an event before and
  // after what it launches; the report waits for them and gives (name with sizes, calls, microseconds).
  void timing(bool on);
  // the same list of calls without the times: nothing is recorded on the stream and no sum is added early, so
  // the step runs exactly as it does unobserved; a name ends in what the call took ("[mfma]", "[generic]",
  // "[fused]", ...).  For tests that check which kernel served a shape.
  void count_calls(bool on);
  struct Timed { std::string name; int calls = 0; double us = 0; };
  std::vector<Timed> timing_report();

  // switches for tests and measurements: each leaves the results the same up to the order of sums
  struct Switches {
    bool fast_gemm = true, fast_attention = true, fused_norm = true, fused_qk_decode = true, fused_qkv_prefill = true;
    bool split_k_add = true, deferred_add = true, paired_prefill = true, portion_splits = true;
    bool early_page_ids = true;     // a step of single tokens: the decode attention fetches a row's page ids beside its position
    bool radix_sample = true;       // draws with a top-k cut: many workgroups share a row (else one walks it bit by bit)
    int force_paired_tiles = -1;    // 1 / 0: that kernel with / without pairs, whatever the launch
    int force_decode_splits = 0;    // > 0: the decode attention cuts every context into this many runs
  } use;
  // A shape rule of a kernel library forced for this object's calls (tests and measurements; the names are listed
  // in csrc/tinyinfer_kernels_tuning.h).  The rules are the libraries' own, process-wide: this object sets its
  // overrides before each of its calls into that library and resets them afterwards.
  void tune(const std::string& library, const std::string& name, long value);
  void untune();
  static int decode_splits(int n_rows, int kv_heads, int heads, int context, int typical, int units, int head_dim = 128);
  // runs of keys for the prefill kernel with 64-row tiles, and whether it pairs a heavy with a light tile
  static int portion_launch(int n_tiles_small, int heads, int portion_context, int window, int units, bool* paired);

 private:
  void* launch_stream();
  void took(const char* what);       // the call under way names the kernel it took (seen in the list of calls)
  void* stream_ = nullptr;
  int units_ = 0;
  DeviceBuffer partials_;
  DeviceBuffer argmax_scratch_;
  DeviceBuffer sample_scratch_;       // zero between calls
  struct { void* out = nullptr; int64_t count = 0; int splits = 0; } pending_;
  std::map<std::string, std::map<std::string, long>> tuning_;
  friend struct TunedScope;
  struct Timing;
  friend struct TimedScope;
  std::unique_ptr<Timing> timing_;
};

// Activation rows handed from a norm to its consumer: computed (`t`), or, when the consumer
// takes them into one product and nothing else, the norm itself not computed yet
// (`lazy`: t is the buffer they would go to).
struct Rows {
  Tensor t;
  bool lazy = false;
  Tensor x, weight;
  float eps = 0.f;
  const Tensor& materialize(Ops& ops) const;
};

class Workspace {
 public:
  // the same memory for the same name in every layer and step; grows when more is asked for
  void* get(const std::string& name, size_t bytes);
  Tensor tensor(const std::string& name, DType dt, std::initializer_list<int64_t> dims);
  size_t total_bytes() const;
  bool frozen = false;            // a captured graph reads these addresses: growing is an error
 private:
  std::map<std::string, DeviceBuffer> bufs_;
};

// The lists the attention kernels walk, in device memory (the step's metadata).
struct AttentionWork {
  int64_t M = 0;
  const int* positions = nullptr;    // [M]
  const int* slots = nullptr;        // [M] row of the block table
  const int* entry_meta = nullptr;   // [R][4] = (row0, n_tokens, start_pos, state slot)
  const int* tiles = nullptr;        // [n_tiles][2] = (entry, first row) of 128 query rows
  int n_tiles = 0;
  const int* tiles_small = nullptr;  // the same in tiles of 64 rows, from the most visible keys to the fewest
  int n_tiles_small = 0;
  const int* decode_rows = nullptr;  // rows of single-token entries (null when every entry is one)
  int n_decode_rows = 0;
  bool decode_only = false;
  bool slots_are_rows = false;       // slots[m] == m for every row (a step of single tokens, one entry a row)
  int max_context = 0;               // longest context any row reads
  int portion_context = 0;           // ... over rows of entries of several tokens
  int split_context = 0;             // the context the decode kernel's runs are sized for
};

// ---------------------------------------------------------------------------------- the step
// In place of a token id: the id that the sampler's last call wrote to row `row` of the engine's
// token feedback buffer (Engine::token_feedback).  The step then needs no id that the host has not
// read yet, so it can be launched before the step before it has finished.
inline int token_from_feedback(int row) { return -1 - row; }
struct StepEntry {
  int64_t request = 0;
  std::vector<int> tokens;     // the request's next tokens (ids, or token_from_feedback(row))
  std::vector<int> want;       // places among them (0-based) whose logits are wanted
  int start = -1;              // the position of the first token, if the caller knows it: checked against the cache
};
struct EntryRecord { int row0, n_tokens, start, state_slot; };

class Engine;
class Part;
// What a part may add to a step before its metadata goes to the device: integer lists of its
// own.  `ints(key, n)` returns host memory for n ints that will lie in the step's metadata;
// the same key asked for twice is the same list (the layers of a model share theirs).
class StepPlan {
 public:
  const std::vector<EntryRecord>& entries() const { return *entries_; }
  int64_t M() const { return M_; }
  bool decode_only() const { return decode_only_; }
  int max_seq() const { return max_seq_; }
  bool sized_for_longest() const { return sized_for_longest_; }   // a graph is being captured: size launches for max_seq
  bool has(const std::string& key) const { return lists_.count(key) != 0; }
  int* ints(const std::string& key, size_t n);
  void set_value(const std::string& key, int64_t v) { values_[key] = v; }
 private:
  friend class Engine;
  friend class StepContext;
  struct List { size_t offset = 0, n = 0; std::vector<int> host; };
  std::map<std::string, List> lists_;
  std::map<std::string, int64_t> values_;
  const std::vector<EntryRecord>* entries_ = nullptr;
  int64_t M_ = 0;
  bool decode_only_ = false, sized_for_longest_ = false;
  int max_seq_ = 0;
};

// Everything a part may touch during one step.
class StepContext {
 public:
  Ops& ops;
  Workspace& ws;
  DType act_dtype;                        // dtype of activations and cache: the engine's compute dtype
  int64_t M = 0;                          // tokens in the step
  const int* tokens = nullptr;            // device int32 [M]; an id below zero: fed_tokens[-1 - id] (token_from_feedback)
  const int* fed_tokens = nullptr;        // device int32 [n_fed_tokens]: ids the sampler left on the device, or null
  int n_fed_tokens = 0;
  const int* positions = nullptr;         // device int32 [M]
  const int* slots = nullptr;             // device int32 [M]: the token's entry = row of the block tables
  const int* out_rows = nullptr;          // device int32 [n_out]
  int64_t n_out = 0;
  const int* entry_meta = nullptr;        // device int32 [R][4]
  std::vector<EntryRecord> entries;       // the same on the host
  bool decode_only = false;               // every entry is a single token
  int max_context = 0;
  int run = 0;                            // index into the model's run order

  StepContext(Ops& ops, Workspace& ws, DType act_dtype) : ops(ops), ws(ws), act_dtype(act_dtype) {}
  Tensor buf(const std::string& name, DType dt, std::initializer_list<int64_t> dims) { return ws.tensor(name, dt, dims); }
  // the cache of the part that is running: (group, cache layer) as the model bound it for this run
  std::pair<int, int> binding(const Part* part) const;
  Tensor kv_pool(int group, int layer) const;                 // [pages][2 x kv heads][P][head_dim]; PagedRows: [pages][P][row...]
  Ops::CacheView cache_view(int group) const;                 // the block-table rows of the step's entries
  Tensor state(int group, int layer) const;                   // f32 [slots][...]
  // a list a part planned for this step (device memory), and values
  const int* planned(const std::string& key) const;
  size_t planned_size(const std::string& key) const;
  int64_t value(const std::string& key, int64_t fallback = 0) const;

  Engine* engine = nullptr;               // null for a part run on its own
  const StepPlan* plan = nullptr;
  const int* meta_dev = nullptr;
  std::vector<Ops::CacheView> views;      // per cache group
};

// -------------------------------------------------------------------------------------- parts
// A part holds sizes, constants and weights and computes through the kernels it finds in the
// step context.  It never looks at the model it sits in.  Families and their calls:
//   embedding  forward(ctx, x)                       fills x f32 [M, H] from ctx.tokens
//   norm       forward(ctx, x, rows, n_rows, lazy)   -> Rows in the compute dtype
//   pos        fused(rot) / apply(ctx, q, k)         rotation in the fused kernels, or in place on f32 views
//   mixer      forward(ctx, h, x)                    adds its output into x
//   ffn        forward(ctx, h, x)                    adds its output into x
//   block      forward(ctx, x)                       arranges its parts around x
//   head       forward(ctx, h) -> logits f32 [N, V]
class WeightSource;
class Part {
 public:
  explicit Part(std::string prefix) : prefix(std::move(prefix)) {}
  virtual ~Part() = default;
  virtual const char* family() const = 0;
  virtual const char* kind_name() const { return ""; }
  // checkpoint tensors of this part itself (children report their own), in a fixed order
  virtual std::vector<std::pair<std::string, TensorNeed>> tensors() const { return {}; }
  // take the tensors named in tensors() from the source (absent optional ones: src.has() is false)
  virtual void load(WeightSource& src) {}
  virtual std::vector<std::shared_ptr<Part>> children() const { return {}; }
  // the tensors the part holds after load(), by the name of the member (for looking at them)
  virtual std::vector<std::pair<std::string, Tensor>> held() const { return {}; }
  virtual bool has_cache() const { return false; }
  virtual CacheNeed cache_need() const { return {}; }
  virtual void prepare(Ops& ops, int max_seq) {}            // tables that depend on the longest sequence
  virtual void plan(StepPlan& plan) const {}                // lists of this part's own in the step's metadata
  // the part reads the residual stream only through ctx.ops (so a product before it may leave
  // partial sums for the next norm); parts that do not say so find the residual complete
  virtual bool reads_through_ops() const { return false; }
  // names of children(), in their order ("norm1", "mixer", ...; default "0", "1", ...)
  virtual std::vector<std::string> child_slots() const;
  void walk(const std::function<void(Part&)>& fn);
  std::string prefix;
  uint64_t foreign_id = 0;     // non-zero: the part is implemented outside this library (see ForeignCalls)
  std::string built_kind;      // what build_part made it from
  Json built_from;
};
class EmbeddingPart : public Part { public: using Part::Part; const char* family() const override { return "embedding"; }
  virtual void forward(StepContext& ctx, const Tensor& x) = 0; };
class NormPart : public Part { public: using Part::Part; const char* family() const override { return "norm"; }
  virtual Rows forward(StepContext& ctx, const Tensor& x, const int* rows = nullptr, int64_t n_rows = 0, bool lazy = false) = 0;
  virtual bool can_be_lazy() const { return false; } };
class PositionPart : public Part { public: using Part::Part; const char* family() const override { return "pos"; }
  virtual bool fused(Ops::Rotation& rot) const { return false; }    // arguments for the fused q/k kernels
  virtual void apply(StepContext& ctx, const Tensor& q, const Tensor& k) = 0; };   // f32 [M, heads, hd] views; k may be undefined
class MixerPart : public Part { public: using Part::Part; const char* family() const override { return "mixer"; }
  virtual void forward(StepContext& ctx, const Rows& h, const Tensor& x) = 0;
  virtual bool takes_lazy_norm() const { return false; } };        // h goes into exactly one Ops::linear
class FeedForwardPart : public Part { public: using Part::Part; const char* family() const override { return "ffn"; }
  virtual void forward(StepContext& ctx, const Rows& h, const Tensor& x) = 0;
  virtual bool takes_lazy_norm() const { return false; } };
class BlockPart : public Part { public: using Part::Part; const char* family() const override { return "block"; }
  virtual void forward(StepContext& ctx, const Tensor& x) = 0; };
class HeadPart : public Part { public: using Part::Part; const char* family() const override { return "head"; }
  virtual Tensor forward(StepContext& ctx, const Rows& h) = 0; };

// A factory gets the tensor-name prefix, the part's parameters and, for arrangements, its
// children by slot name.  `children` is also where an already built nested part arrives (the
// "pos" of an attention).
using PartChildren = std::vector<std::pair<std::string, std::shared_ptr<Part>>>;
using PartFactory = std::function<std::shared_ptr<Part>(const std::string& prefix, const Json& params, const PartChildren& children)>;
// slots: for a block arrangement, which family each named slot is built from
void register_part(const std::string& family, const std::string& kind, PartFactory factory,
                   std::vector<std::pair<std::string, std::string>> slots = {});
bool part_registered(const std::string& family, const std::string& kind);
std::vector<std::string> registered_parts(const std::string& family);
std::vector<std::pair<std::string, std::string>> block_slots(const std::string& kind);
std::shared_ptr<Part> build_part(const std::string& family, const PartSpec& spec, const std::string& prefix,
                                 const PartChildren& children = {});

// Parts implemented outside this library (the Python package's): one table of calls, the part
// named by its foreign_id.  Tensors cross as descriptors.  A call returns 0, or non-zero after
// leaving a message with set_foreign_error().
struct ForeignCalls {
  // op: "forward", "apply", "load", "prepare"; args/n_args by family (see parts.cpp)
  int (*call)(uint64_t id, const char* op, StepContext* ctx, const Tensor* args, int n_args, const char* names,
              Tensor* result) = nullptr;
};
void set_foreign_calls(const ForeignCalls&);
void set_foreign_error(const std::string& message);
std::string take_foreign_error();      // the message left last on this thread; it is cleared
// description: {"tensors": {name: {shape, role, init, a, b, optional}}, "cache_need": {...} | null, "fused": false}
std::shared_ptr<Part> make_foreign_part(const std::string& family, uint64_t id, const std::string& prefix,
                                        const Json& description, const PartChildren& children);

// ------------------------------------------------------------------------------------ weights
// Where a part's tensors come from while it loads: a model folder, tensors in memory, or the
// random generator.  `fill` writes the named tensor into `dst` (device memory the part owns, of
// the dtype its role asks for), converting from the stored dtype on the way.
struct SourceInfo { DType dtype; std::vector<int64_t> shape; };
class WeightSource {
 public:
  virtual ~WeightSource() = default;
  virtual std::vector<std::pair<std::string, SourceInfo>> list() const = 0;   // every tensor the source holds
  virtual bool has(const std::string& name) const = 0;
  virtual void fill(const std::string& name, const Tensor& dst) = 0;
  virtual void finish() {}                    // every copy has arrived
  DType matrix_dtype = DType::BF16;
  bool to_host = false;                       // the destinations are host memory
  // device memory that lives as long as the model
  Tensor alloc(DType dt, const std::vector<int64_t>& shape);
  // alloc by role + fill; the same name asked for twice is the same memory (a tied head)
  Tensor fetch(const std::string& name, const TensorNeed& need);
  std::vector<DeviceBuffer>* owner = nullptr;
 private:
  std::map<std::string, Tensor> fetched_;
};

class SafetensorsFile {     // one mapped file; nothing is executed from it
 public:
  struct Entry { DType dtype; std::vector<int64_t> shape; size_t begin, end; };
  explicit SafetensorsFile(const std::string& path);
  ~SafetensorsFile();
  const std::vector<std::pair<std::string, Entry>>& entries() const { return entries_; }
  const Entry* find(const std::string& name) const;
  const uint8_t* bytes(const Entry& e) const { return base_ + e.begin; }
  std::string path;
 private:
  std::vector<std::pair<std::string, Entry>> entries_;
  std::map<std::string, size_t> index_;
  const uint8_t* map_ = nullptr;
  const uint8_t* base_ = nullptr;
  size_t size_ = 0;
};
struct HostTensor { std::string name; DType dtype; std::vector<int64_t> shape; const void* data; };
void write_safetensors(const std::string& path, const std::vector<HostTensor>& tensors,
                       const std::vector<std::pair<std::string, std::string>>& metadata = {});

// -------------------------------------------------------------------------------------- model
class Model {
 public:
  // parts built through the registry from a spec
  explicit Model(const ModelSpec& spec);
  // parts built by the caller (the Python package builds them one by one)
  Model(const ModelSpec& meta, std::shared_ptr<Part> embedding, std::vector<std::shared_ptr<Part>> blocks,
        std::shared_ptr<Part> final_norm, std::shared_ptr<Part> head);
  // config.json -> registry -> parts -> weights from the folder's safetensors
  static std::shared_ptr<Model> from_folder(const std::string& dir, const std::string& dtype);
  // random weights drawn on the device (no folder is written)
  static std::shared_ptr<Model> from_config(const Json& config, uint64_t seed, const std::string& dtype);
  // config.json and model.safetensors with random weights drawn on the host
  static void write_folder(const std::string& dir, const Json& config, uint64_t seed, const std::string& store_dtype);
  void write_random_folder(const std::string& dir, const Json& config_out, uint64_t seed, const std::string& store_dtype);

  std::vector<std::pair<std::string, TensorNeed>> tensors() const;     // every tensor the model asks for, fixed order
  // to_host: the weights stay in host memory (no GPU is touched; such a model cannot run)
  void load_folder(const std::string& dir, const std::string& dtype, bool to_host = false);
  void load_tensors(const std::vector<HostTensor>& tensors, bool on_device, const std::string& dtype, const std::string& where,
                    bool to_host = false);
  void load_random(uint64_t seed, const std::string& dtype);
  void walk(const std::function<void(Part&)>& fn) const;

  ModelSpec spec;
  std::shared_ptr<EmbeddingPart> embedding;
  std::vector<std::shared_ptr<BlockPart>> blocks;
  std::shared_ptr<NormPart> final_norm;
  std::shared_ptr<HeadPart> head;
  std::vector<int> run_order;
  // groups of cache layers with the same need; bindings[run][part] = (group, cache layer)
  std::vector<std::pair<CacheNeed, int>> cache_groups;
  std::vector<std::map<const Part*, std::pair<int, int>>> bindings;
  std::string dtype;          // set by load_*: "bfloat16" | "float32"
  bool has_foreign_parts() const;
 private:
  void finish_construction();
  void group_cache();
  void load_from(WeightSource& src, const std::string& dtype, bool to_host);
  std::vector<DeviceBuffer> storage_;
};

// ------------------------------------------------------------------------------ cache manager
// Keys and values in pages with a block table per request, one pool per group of layers with the
// same need, slots for per-request state of fixed size.  Host bookkeeping only.  The reference
// keeps one slab for max_batch x max_seq tokens that is never given back per request
// (/root/reference/src/inference.cu:146-148,174-176).
class PagePool {
 public:
  PagePool(int num_pages, int scatter_window = 0);
  int num_pages() const { return num_pages_; }
  int num_free() const { return (int)free_.size(); }
  int take();
  void give_back(int page);
  int high_water = 0;
  int64_t taken_total = 0;
  const std::vector<int>& free_list() const { return free_; }
 private:
  int num_pages_;
  std::vector<int> free_;
  std::vector<char> held_;
};
class CacheManager {
 public:
  CacheManager(const std::vector<std::pair<CacheNeed, int>>& groups, int page_size, int num_pages, int max_requests,
               int max_seq, int scatter_window = 0);
  // queries
  bool has(int64_t req) const { return requests_.count(req) != 0; }
  std::vector<int64_t> live_requests() const;
  int length(int64_t req) const;
  int reserved(int64_t req) const;
  int slot(int64_t req) const;
  int num_free_slots() const { return (int)free_slots_.size(); }
  int num_free_pages() const;                         // of the tightest group
  int num_groups() const { return (int)groups_.size(); }
  bool group_is_paged(int g) const { return groups_[g].paged; }
  const CacheNeed& group_need(int g) const { return groups_[g].need; }
  int group_layers(int g) const { return groups_[g].n_layers; }
  const std::vector<int>& paged_groups() const { return paged_; }
  PagePool& pool(int g);
  const PagePool& pool(int g) const { return const_cast<CacheManager*>(this)->pool(g); }
  const std::vector<int>& table(int g, int64_t req) const;      // -1: given back behind the window
  const int* table_row(int g, int64_t req) const;               // the same, table_width ints, -1 padded
  int pages_to_cover(int g, int64_t req, bool admitted, int upto) const;
  int pages_needed(int64_t req, bool admitted, int n_tokens, int length = -1) const;
  bool can_reserve(int64_t req, int n_tokens) const;
  // actions
  int admit(int64_t req);                    // a slot (cleared before first use) and empty tables
  void reserve(int64_t req, int n_tokens);   // all groups or OutOfPages and nothing taken
  void commit(int64_t req, int n_tokens);    // gives back pages the window has passed
  std::vector<int> reserve_one_each(const std::vector<int64_t>& reqs);
  void commit_one_each(const std::vector<int64_t>& reqs);
  void rollback(int64_t req);                // forget a reservation that was not committed
  void release(int64_t req);
  void check() const;                        // throws CacheError naming the invariant that is broken

  const int page_size, max_requests, max_seq, table_width;
  std::vector<int> slots_to_clear;
 private:
  struct Req { int slot = 0, length = 0, reserved = 0; };
  struct Group {
    bool paged = false;
    CacheNeed need;
    int n_layers = 0;
    std::unique_ptr<PagePool> pool;
    std::map<int64_t, std::vector<int>> tables;
    std::map<int64_t, std::vector<int>> rows;
  };
  int first_needed_page(const Group& g, int next_pos) const;
  void give_back_page(Group& g, int64_t req, int index);
  std::vector<Group> groups_;
  std::vector<int> paged_;
  std::map<int64_t, Req> requests_;
  std::vector<int> free_slots_;
};

// ------------------------------------------------------------------------------------- engine
struct EngineOptions {
  std::string dtype = "";        // empty: the dtype the model was loaded in
  int page_size = 16;
  int64_t max_tokens = 0;        // the cache pool's size in tokens ...
  int64_t num_pages = 0;         // ... or in pages (one of the two)
  int max_requests = 64;
  int max_seq = 0;               // 0: the pool's size, bounded by max_position_embeddings
  void* stream = nullptr;
  int page_scatter_window = 512;
  int max_step_graphs = 32;      // graphs of steps that are not plain decode steps kept at a time (least recently used goes)
};

class Engine {
 public:
  Engine(std::shared_ptr<Model> model, const EngineOptions& options);
  ~Engine();
  // One batch: portions of prompts beside single tokens, cut anywhere.  Reserves pages (the whole
  // step or nothing), runs exactly the tokens given against the cache earlier steps left, and
  // returns device float32 logits [wanted, vocab] in the order of the entries and their `want`
  // (an undefined tensor if nothing is wanted).  The memory is the engine's: valid until the next step.
  Tensor step(const std::vector<StepEntry>& entries);
  // the same, replayed from a captured HIP graph where there is one (decode steps by batch size,
  // other steps by shape once a shape has come twice)
  Tensor step_graph(const std::vector<StepEntry>& entries);
  void release(int64_t request);
  // Device int32 [feedback_rows()]: where a sampler may leave the ids it draws, so that the next
  // step can name them with token_from_feedback(row).  Null for a model with parts from outside
  // the library (their embedding reads ids only).
  int* token_feedback();
  int feedback_rows() const;
  void logits_to_host(const Tensor& logits, float* out);    // synchronous copy
  void synchronize();

  std::shared_ptr<Model> model;
  std::unique_ptr<CacheManager> cache;
  Ops ops;
  const DType act_dtype;
  const std::string dtype;
  const int page_size, max_seq;
  int64_t num_pages;
  int64_t steps_run = 0;
  size_t num_graphs() const;
  std::vector<std::string> graph_keys() const;   // "d<batch>" for decode graphs, "s<tokens>:<want>,..;..." for shapes
  size_t cache_bytes() const;
  Tensor kv_pool(int group, int layer) const;
  Tensor state(int group, int layer) const;
  struct Impl;
 private:
  friend class StepContext;
  std::unique_ptr<Impl> impl_;
};

// ----------------------------------------------------------------------------------- sampling
// temperature <= 0: greedy (/root/reference/src/main.cpp:24,31-38); top_k 0 means the reference's
// 512 (src/main.cpp:47-48); seed 42 (src/main.cpp:27).  The n-th token of a request is drawn with
// uniform(seed, request number, n): neither batching nor preemption changes what is sampled.
struct SamplingParams {
  float temperature = 0.f;
  int top_k = 0;
  float top_p = 1.f;
  uint64_t seed = 42;
  int effective_top_k() const { return top_k > 0 ? top_k : 512; }
};
float uniform(uint64_t seed, uint64_t request, uint64_t n_generated);     // [0, 1), 24 random bits
class Sampler {
 public:
  explicit Sampler(Ops& ops);
  ~Sampler();
  // logits f32 [n, V] on the device; row i belongs to request number requests[i], which has
  // generated counters[i] tokens so far.  Reads the ids back (a full synchronisation).
  std::vector<int> sample(const Tensor& logits, const std::vector<SamplingParams>& params,
                          const std::vector<int64_t>& requests, const std::vector<int64_t>& counters);
  // The same without waiting: the ids are drawn and copied back behind whatever the stream holds,
  // and `collect(ticket)` waits for them.  `device_out` (device int32 [n], e.g. the engine's token
  // feedback) receives the ids too, for a step that is launched before they are read.  At most two
  // calls may be under way; `drop` gives up a call whose ids are not needed.
  uint64_t sample_async(const Tensor& logits, const std::vector<SamplingParams>& params, const std::vector<int64_t>& requests,
                        const std::vector<int64_t>& counters, int* device_out = nullptr);
  std::vector<int> collect(uint64_t ticket);
  void drop(uint64_t ticket);
 private:
  Ops& ops_;
  struct Buffers;
  std::unique_ptr<Buffers> b_;
};

// ---------------------------------------------------------------------------------- scheduler
// Which tokens of which requests the next step runs.  The reference has none: every prompt is
// prefilled whole in one batch, then every unfinished sequence decodes one token a step
// (/root/reference/src/main.cpp:210-297).
struct Request {
  int64_t number = 0;                  // order of submission; keys the random stream and the cache
  std::vector<int> prompt;
  int max_new_tokens = 0;
  SamplingParams params;
  std::vector<int> eos_token_ids;
  std::vector<int> tokens;             // prompt + generated so far
  int n_fed = 0;                       // tokens whose keys and values are in the cache
  std::vector<int> generated;
  std::string finish_reason;           // "", "length", "eos", "abort"
  int preemptions = 0;
  int64_t admitted_at = -1;
  int64_t key() const { return key_base + number; }
  int64_t key_base = 0;
  int pending() const { return (int)tokens.size() - n_fed; }
};
struct PlannedEntry { std::shared_ptr<Request> request; int start = 0, n_tokens = 0; bool sample = false; };
struct Plan { std::vector<PlannedEntry> entries; std::vector<std::shared_ptr<Request>> preempted; };
class Scheduler {
 public:
  Scheduler(CacheManager& cache, int max_batched_tokens = 2048, int chunk_size = 512, int max_running = 0);
  std::shared_ptr<Request> add(const std::vector<int>& prompt, int max_new_tokens, const SamplingParams& params = {},
                               const std::vector<int>& eos_token_ids = {});
  bool has_work() const { return !waiting.empty() || !running.empty(); }
  Plan plan();
  // the step after `last` (launched, not yet committed) if it does not depend on what `last`
  // samples: one more token of every running request; else an empty plan
  Plan plan_ahead(const Plan& last) const;
  // the step ran; sampled[request number] for every entry that asked.  Returns the requests that
  // finished: their pages and slots are the caller's to give back.
  std::vector<std::shared_ptr<Request>> commit(const Plan& plan, const std::map<int64_t, int>& sampled);
  void abort(const std::shared_ptr<Request>& req);       // gives its pages and slot back
  void abort_all();
  void set_next_number(int64_t n) { submitted_ = n; }   // the number the next request gets (it keys its random stream)
  CacheManager& cache;
  const int max_batched_tokens, chunk_size;
  int max_running;
  std::vector<std::shared_ptr<Request>> waiting, running, finished;   // waiting: front first
 private:
  int new_pages(const std::vector<std::pair<std::shared_ptr<Request>, int>>& batch) const;
  void preempt(const std::shared_ptr<Request>& req, Plan& plan);
  int64_t submitted_ = 0, admissions_ = 0;
  int64_t key_base_ = 0;
};

struct GenerationStats {
  double prefill_ms = 0, decode_ms = 0;
  int64_t prefill_tokens = 0, decode_tokens = 0, steps = 0, preemptions = 0;
  int64_t steps_ahead = 0;             // of `steps`: launched before the ids of the step before were read
};
// Run until the scheduler has no work: plan, step, sample, commit, release.  When anything
// throws, every request the scheduler still holds is given back to the cache first.
// `run_ahead`: while every running request decodes and nobody waits, the next step is launched
// before the ids of the last one are read (it takes them from the device), so the device does
// not wait for the host between steps; tokens are the same, `on_token` hears them one step later.
// `on_prompt_logits`: called with the 32-bit logits (host memory, `vocab` of them) behind the last token of a
// request's prompt, before its first token is drawn (what the reference's --verbose prints:
// /root/reference/src/main.cpp:233-249); it costs a copy and a wait per such step.
using PromptLogits = std::function<void(const Request&, const float* logits, int64_t vocab)>;
void run_requests(Engine& engine, Scheduler& scheduler, Sampler* sampler = nullptr, GenerationStats* stats = nullptr,
                  const std::function<void(const Request&, int token)>& on_token = nullptr, bool use_graph = false,
                  bool run_ahead = true, const PromptLogits& on_prompt_logits = nullptr);
struct GenerateOptions {
  int max_new_tokens = 128;
  SamplingParams sampling;
  std::vector<int> eos_token_ids;      // empty with use_model_eos: the model's own
  bool use_model_eos = true;
  int chunk_size = 512, max_batched_tokens = 2048;
  bool use_graph = false;
  bool run_ahead = true;
};
std::vector<std::vector<int>> generate(Engine& engine, const std::vector<std::vector<int>>& prompts,
                                       const GenerateOptions& options = {}, GenerationStats* stats = nullptr);

}  // namespace tinyinfer

// ============================================================================ the C interface
// What the Python package binds.  Every function returns 0, or non-zero after an error whose
// class name and text `ti_error_kind()` / `ti_error_message()` give (per thread).  Strings that
// come back (`char**`) are owned by the library until the same thread's next call that returns
// a string.  Structured values cross as JSON text.
extern "C" {
const char* ti_error_kind();
const char* ti_error_message();
typedef struct ti_tensor { void* data; int dtype; int ndim; int64_t shape[4]; int64_t stride[4]; } ti_tensor;

int ti_kernels_register(const char* name, const char* path);
int ti_load_plugin(const char* path);
int ti_set_allocator(void* (*alloc)(void*, size_t), void (*release)(void*, void*), void* user);
void ti_detach_allocator();
int ti_set_foreign_calls(int (*call)(uint64_t, const char*, void*, const ti_tensor*, int, const char*, ti_tensor*));
void ti_set_foreign_error(const char* message);

// configuration and registries
int ti_qwen3_config(const char* config_json, const char** out_json);       // the typed configuration, validated
int ti_typed_config(const char* config_json, const char** out_json);       // {"architecture", "config"} of whatever architecture config.json names
int ti_spec_from_config(const char* config_json, const char** out_spec_json);
int ti_architecture_registered(const char* config_json, int* out);
int ti_registered_architectures(const char** out_json);
int ti_registered_parts(const char* family, const char** out_json);
int ti_block_slots(const char* kind, const char** out_json);

// parts (handles are shared references: release each with ti_part_release)
int ti_part_create(const char* family, const char* kind, const char* prefix, const char* params_json, int n_children,
                   const char* const* child_slots, void* const* children, void** out);
int ti_part_create_foreign(const char* family, uint64_t id, const char* prefix, const char* description_json,
                           int n_children, const char* const* child_slots, void* const* children, void** out);
// kinds implemented outside this library: `make` builds one and returns a handle the caller owns (the library
// takes a reference of its own); `ti_register_foreign_kind` enters the kind into the table of parts, so that a
// spec that names it builds like any other (slots_json: for a block arrangement, {slot: family})
int ti_set_foreign_factory(int (*make)(const char* family, const char* kind, const char* prefix, const char* params_json,
                                       int n_children, const char* const* child_slots, void* const* children, void** out));
int ti_register_foreign_kind(const char* family, const char* kind, const char* slots_json);
void ti_part_release(void* part);
int ti_part_child(void* part, int index, void** out);                  // a new handle to the index-th of the part's children
int ti_part_tensors(void* part, const char** out_json);
int ti_part_cache_need(void* part, const char** out_json);
int ti_part_info(void* part, const char** out_json);
// load one part from tensors in device memory (names '\n'-joined)
int ti_part_load(void* part, int n, const char* names, const ti_tensor* tensors, const char* matrix_dtype, int on_host);
int ti_part_held(void* part, const char* member, ti_tensor* out);     // a tensor the part holds ("weight", "w_qkv", ...)
int ti_part_pointer(void* part, void** out);                           // the part's identity
// a context for running parts on their own
int ti_ctx_create(const char* dtype, void* stream, void** out);
void ti_ctx_release(void* ctx);
int ti_ctx_set_rows(void* ctx, int64_t M, const int* positions, const int* tokens);
int ti_part_call(void* part, const char* op, void* ctx, const ti_tensor* args, int n_args, int flags, ti_tensor* result);
// what a foreign part asks of the context it was called with
int ti_ctx_info(void* ctx, const char** out_json);         // M, decode_only, run, entries, dtype
int ti_ctx_pointers(void* ctx, const int** tokens, const int** positions, const int** slots);
int ti_ctx_binding(void* ctx, void* part, int* group, int* layer);
int ti_ctx_kv_pool(void* ctx, int group, int layer, ti_tensor* out);
int ti_ctx_state(void* ctx, int group, int layer, ti_tensor* out);
int ti_ctx_cache_view(void* ctx, int group, ti_tensor* out_table, int* page_size);
int ti_ctx_buf(void* ctx, const char* name, int dtype, int ndim, const int64_t* shape, ti_tensor* out);
int ti_ctx_ops(void* ctx, void** out_ops);

// model
int ti_model_from_spec(const char* spec_json, void** out);              // every part through the table of parts
// a new handle to a part of the model: which = "embedding" | "block" (index) | "final_norm" | "head"
int ti_model_part(void* model, const char* which, int index, void** out);
int ti_model_create(const char* meta_json, void* embedding, int n_blocks, void* const* blocks, void* final_norm,
                    void* head, void** out);
void ti_model_release(void* model);
int ti_model_tensors(void* model, const char** out_json);
int ti_model_cache_groups(void* model, const char** out_json);
int ti_model_bindings(void* model, const char** out_json);             // per run: [[part identity, group, cache layer], ...]
int ti_model_load_folder(void* model, const char* dir, const char* dtype, int to_host);
int ti_model_load_tensors(void* model, int n, const char* names, const ti_tensor* tensors, int on_device,
                          const char* dtype, const char* where, int to_host);
int ti_model_load_random(void* model, uint64_t seed, const char* dtype);
int ti_model_write_random_folder(void* model, const char* dir, const char* config_json, uint64_t seed, const char* store_dtype);
int ti_weights_error_lists(const char** out_json);          // of the last WeightsError of this thread

// cache manager (also on its own, without a GPU)
int ti_cache_create(const char* groups_json, int page_size, int num_pages, int max_requests, int max_seq,
                    int scatter_window, void** out);
void ti_cache_release(void* cache);
int ti_cache_call(void* cache, const char* op, int64_t req, int64_t a, int64_t b, int64_t* out);
int ti_cache_table(void* cache, int group, int64_t req, const char** out_json);
int ti_cache_many(void* cache, const char* op, int n, const int64_t* reqs, const char** out_json);
int ti_cache_dump(void* cache, const char** out_json);
int ti_pool_create(int num_pages, int scatter_window, void** out);
void ti_pool_release(void* pool);
int ti_pool_call(void* pool, const char* op, int64_t a, int64_t* out);
int ti_pool_free_list(void* pool, const char** out_json);

// engine
int ti_engine_create(void* model, const char* options_json, void** out);
void ti_engine_release(void* engine);
int ti_engine_info(void* engine, const char** out_json);
int ti_engine_cache(void* engine, void** out_cache);            // borrowed
int ti_engine_ops(void* engine, void** out_ops);                // borrowed
int ti_engine_step(void* engine, int use_graph, int n_entries, const int64_t* requests, const int* n_tokens,
                   const int* tokens, const int* n_want, const int* want, ti_tensor* out_logits);
int ti_engine_release_request(void* engine, int64_t request);
int ti_engine_kv_pool(void* engine, int group, int layer, ti_tensor* out);
int ti_engine_state(void* engine, int group, int layer, ti_tensor* out);
int ti_engine_synchronize(void* engine);

// sampling and scheduling
float ti_uniform(uint64_t seed, uint64_t request, uint64_t n_generated);
int ti_sampler_create(void* ops, void** out);
void ti_sampler_release(void* sampler);
int ti_sampler_sample(void* sampler, const ti_tensor* logits, int n, const float* temperature, const int* top_k,
                      const float* top_p, const uint64_t* seeds, const int64_t* requests, const int64_t* counters, int* out);
// without waiting: `ti_sampler_collect` waits for the ids.  `feed_engine` (or null): the ids also go to that engine's
// token feedback, where its next step finds them under the token ids -1 - row.
int ti_sampler_sample_async(void* sampler, const ti_tensor* logits, int n, const float* temperature, const int* top_k,
                            const float* top_p, const uint64_t* seeds, const int64_t* requests, const int64_t* counters,
                            void* feed_engine, uint64_t* out_ticket);
int ti_sampler_collect(void* sampler, uint64_t ticket, int n, int* out);
int ti_scheduler_create(void* cache, int max_batched_tokens, int chunk_size, int max_running, void** out);
void ti_scheduler_release(void* scheduler);
int ti_scheduler_add(void* scheduler, int n_prompt, const int* prompt, int max_new_tokens, float temperature, int top_k,
                     float top_p, uint64_t seed, int n_eos, const int* eos, int64_t* out_number);
int ti_scheduler_plan(void* scheduler, const char** out_json);
// the step behind the last plan, before that one is committed (Scheduler::plan_ahead); `ti_scheduler_commit` then
// commits the last plan first and what was planned ahead at its next call
int ti_scheduler_plan_ahead(void* scheduler, const char** out_json);
int ti_scheduler_commit(void* scheduler, int n, const int64_t* numbers, const int* tokens, const char** out_finished_json);
int ti_scheduler_abort(void* scheduler, int64_t number);
int ti_scheduler_set_next_number(void* scheduler, int64_t number);
int ti_scheduler_state(void* scheduler, const char** out_json);
int ti_scheduler_request(void* scheduler, int64_t number, const char** out_json);
// on_token returns 0; anything else stops the run (the requests still held are given back, and the call fails)
// on_logits (or null): the logits behind the last token of a request's prompt, as run_requests' on_prompt_logits
int ti_run_requests(void* engine, void* scheduler, void* sampler, int use_graph, int run_ahead,
                    int (*on_token)(int64_t number, int token), int (*on_logits)(int64_t number, const float* row, int64_t vocab),
                    const char** out_stats_json);

// the kernels through an Ops object (what the kernel tests and foreign parts call)
int ti_ops_create(void* stream, void** out);
void ti_ops_release(void* ops);
int ti_ops_switch(void* ops, const char* name, int value, int* old);
int ti_ops_call(void* ops, const char* op, const ti_tensor* t, int n_t, const double* scalars, int n_scalars,
                const char* text, ti_tensor* result);
int ti_ops_timing_report(void* ops, const char** out_json);     // [{"name", "calls", "us"}] since timing was switched on
int ti_decode_splits(int n_rows, int kv_heads, int heads, int context, int typical, int units, int head_dim);
int ti_portion_launch(int n_tiles_small, int heads, int portion_context, int window, int units, int* paired);
}
