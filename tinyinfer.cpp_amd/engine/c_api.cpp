// The C interface of the library: what the Python package binds (ctypes).  Handles are plain
// pointers to the C++ objects of inference.h; structured values cross as JSON text; an error
// becomes a non-zero return with its class name and text kept per thread.
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <mutex>
#include <sstream>

#include "../include/inference.h"

using namespace tinyinfer;

static_assert(sizeof(ti_tensor) == sizeof(Tensor), "ti_tensor and Tensor must have one layout");

namespace {
thread_local std::string g_kind, g_message, g_text, g_weights_lists = "{}";

int fail(const char* kind, const std::string& message) {
  g_kind = kind;
  g_message = message;
  return 1;
}
#define TI_BEGIN try {
#define TI_END                                                                  \
  return 0;                                                                     \
  }                                                                             \
  catch (const WeightsError& e) {                                               \
    Json j = Json::object();                                                    \
    auto put = [&](const char* k, const std::vector<std::string>& v) {          \
      Json a = Json::array();                                                   \
      for (const auto& s : v) a.push(s);                                        \
      j.set(k, a);                                                              \
    };                                                                          \
    put("missing", e.missing);                                                  \
    put("unexpected", e.unexpected);                                            \
    put("wrong_shape", e.wrong_shape);                                          \
    put("wrong_dtype", e.wrong_dtype);                                          \
    g_weights_lists = j.dump();                                                 \
    return fail(e.kind(), e.what());                                            \
  }                                                                             \
  catch (const Error& e) { return fail(e.kind(), e.what()); }                   \
  catch (const std::exception& e) { return fail("Error", e.what()); }

int give(const char** out, std::string text) {
  g_text = std::move(text);
  *out = g_text.c_str();
  return 0;
}

const Tensor& T(const ti_tensor* t, int i) { return reinterpret_cast<const Tensor*>(t)[i]; }
std::shared_ptr<Part>& P(void* h) { return *static_cast<std::shared_ptr<Part>*>(h); }
std::shared_ptr<Model>& M(void* h) { return *static_cast<std::shared_ptr<Model>*>(h); }

std::vector<std::string> split_lines(const char* s) {
  std::vector<std::string> out;
  if (!s || !*s) return out;
  std::stringstream ss(s);
  std::string line;
  while (std::getline(ss, line, '\n')) out.push_back(line);
  return out;
}

Json need_json(const TensorNeed& n) {
  Json j = Json::object();
  Json shape = Json::array();
  for (int64_t s : n.shape) shape.push(s);
  j.set("shape", shape);
  j.set("role", n.role == TensorNeed::Matrix ? "matrix" : n.role == TensorNeed::Vector ? "vector" : "table");
  j.set("init", n.init);
  j.set("a", n.a);
  j.set("b", n.b);
  j.set("optional", n.optional);
  return j;
}
Json needs_json(const std::vector<std::pair<std::string, TensorNeed>>& needs) {
  Json j = Json::object();
  for (const auto& kv : needs) j.set(kv.first, need_json(kv.second));
  return j;
}
Json cache_need_json(const CacheNeed& n) {
  Json j = Json::object();
  if (n.kind == CacheNeed::PagedKV) {
    j.set("kind", "paged_kv");
    j.set("kv_heads", n.kv_heads);
    j.set("head_dim", n.head_dim);
    j.set("window", n.window > 0 ? Json(n.window) : Json());
  } else if (n.kind == CacheNeed::PagedRows) {
    j.set("kind", "paged_rows");
    Json s = Json::array();
    for (int64_t v : n.row_shape) s.push(v);
    j.set("row_shape", s);
    j.set("float32", n.rows_f32);
    j.set("window", n.window > 0 ? Json(n.window) : Json());
  } else {
    j.set("kind", "state");
    Json s = Json::array();
    for (int64_t v : n.state_shape) s.push(v);
    j.set("shape", s);
  }
  return j;
}
CacheNeed cache_need_from(const Json& c) {
  CacheNeed n;
  if (c.at("kind").as_string() == "state") {
    n.kind = CacheNeed::State;
    for (const Json& s : c.at("shape").items()) n.state_shape.push_back(s.as_int());
  } else if (c.at("kind").as_string() == "paged_rows") {
    n.kind = CacheNeed::PagedRows;
    for (const Json& s : c.at("row_shape").items()) n.row_shape.push_back(s.as_int());
    n.rows_f32 = c.has("float32") && c.at("float32").as_bool();
    n.window = (c.has("window") && !c.at("window").is_null()) ? (int)c.at("window").as_int() : 0;
  } else {
    n.kind = CacheNeed::PagedKV;
    n.kv_heads = (int)c.at("kv_heads").as_int();
    n.head_dim = (int)c.at("head_dim").as_int();
    n.window = c.has("window") ? (int)c.at("window").as_int() : 0;
  }
  return n;
}
PartChildren children_of(int n, const char* const* slots, void* const* handles) {
  PartChildren c;
  for (int i = 0; i < n; ++i) c.emplace_back(slots[i], P(handles[i]));
  return c;
}

// contexts for running parts on their own
struct OwnContext {
  Ops ops;
  Workspace ws;
  StepContext ctx;
  OwnContext(DType dt, void* stream) : ops(stream), ctx(ops, ws, dt) {}
};
std::mutex g_ctx_mutex;
std::map<StepContext*, std::unique_ptr<OwnContext>> g_contexts;
std::map<Ops*, std::unique_ptr<Workspace>> g_ops_workspaces;
std::map<Ops*, std::unique_ptr<Ops>> g_own_ops;

Workspace& workspace_of(Ops* ops) {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  auto& w = g_ops_workspaces[ops];
  if (!w) w.reset(new Workspace());
  return *w;
}

struct SchedulerHandle {
  std::unique_ptr<Scheduler> s;
  Plan last, ahead;          // `ahead`: planned behind `last` before `last` was committed; it is next to be committed
  std::map<int64_t, std::shared_ptr<Request>> all;
};
Json request_json(const Request& r) {
  Json j = Json::object();
  auto ints = [](const std::vector<int>& v) {
    Json a = Json::array();
    for (int x : v) a.push(x);
    return a;
  };
  j.set("number", r.number);
  j.set("key", r.key());
  j.set("prompt", ints(r.prompt));
  j.set("max_new_tokens", r.max_new_tokens);
  j.set("tokens", ints(r.tokens));
  j.set("generated", ints(r.generated));
  j.set("n_fed", r.n_fed);
  j.set("finish_reason", r.finish_reason.empty() ? Json() : Json(r.finish_reason));
  j.set("preemptions", r.preemptions);
  j.set("admitted_at", r.admitted_at);
  j.set("eos_token_ids", ints(r.eos_token_ids));
  return j;
}
}  // namespace

extern "C" {

const char* ti_error_kind() { return g_kind.c_str(); }
const char* ti_error_message() { return g_message.c_str(); }

int ti_kernels_register(const char* name, const char* path) {
  TI_BEGIN
  register_kernel_library(name, path);
  TI_END
}
int ti_load_plugin(const char* path) {
  TI_BEGIN
  load_plugin(path);
  TI_END
}
int ti_set_allocator(void* (*alloc)(void*, size_t), void (*release)(void*, void*), void* user) {
  TI_BEGIN
  Allocator a;
  a.alloc = alloc;
  a.release = release;
  a.user = user;
  set_allocator(a);
  TI_END
}
int ti_set_foreign_calls(int (*call)(uint64_t, const char*, void*, const ti_tensor*, int, const char*, ti_tensor*)) {
  TI_BEGIN
  ForeignCalls f;
  f.call = reinterpret_cast<int (*)(uint64_t, const char*, StepContext*, const Tensor*, int, const char*, Tensor*)>(call);
  set_foreign_calls(f);
  TI_END
}
void ti_detach_allocator() { detach_allocator(); }
void ti_set_foreign_error(const char* message) { set_foreign_error(message ? message : ""); }

// ------------------------------------------------------------------------------ configuration
int ti_qwen3_config(const char* config_json, const char** out_json) {
  TI_BEGIN
  const Qwen3Config c = Qwen3Config::from_json(Json::parse(config_json));
  Json j = c.to_json();
  return give(out_json, j.dump());
  TI_END
}
int ti_typed_config(const char* config_json, const char** out) {
  TI_BEGIN
  return give(out, typed_config(Json::parse(config_json)).dump());
  TI_END
}
int ti_spec_from_config(const char* config_json, const char** out) {
  TI_BEGIN
  return give(out, spec_from_config(Json::parse(config_json)).to_json().dump());
  TI_END
}
int ti_architecture_registered(const char* config_json, int* out) {
  TI_BEGIN
  *out = architecture_registered(Json::parse(config_json)) ? 1 : 0;
  TI_END
}
int ti_registered_architectures(const char** out) {
  TI_BEGIN
  Json a = Json::array();
  for (const auto& n : registered_architectures()) a.push(n);
  return give(out, a.dump());
  TI_END
}
int ti_registered_parts(const char* family, const char** out) {
  TI_BEGIN
  Json a = Json::array();
  for (const auto& n : registered_parts(family)) a.push(n);
  return give(out, a.dump());
  TI_END
}
int ti_block_slots(const char* kind, const char** out) {
  TI_BEGIN
  Json j = Json::object();
  for (const auto& kv : block_slots(kind)) j.set(kv.first, kv.second);
  return give(out, j.dump());
  TI_END
}

// -------------------------------------------------------------------------------------- parts
int ti_part_create(const char* family, const char* kind, const char* prefix, const char* params_json, int n_children,
                   const char* const* child_slots, void* const* children, void** out) {
  TI_BEGIN
  PartSpec spec;
  spec.kind = kind;
  spec.params = Json::parse(params_json && *params_json ? params_json : "{}");
  *out = new std::shared_ptr<Part>(build_part(family, spec, prefix, children_of(n_children, child_slots, children)));
  TI_END
}
int ti_part_create_foreign(const char* family, uint64_t id, const char* prefix, const char* description_json, int n_children,
                           const char* const* child_slots, void* const* children, void** out) {
  TI_BEGIN
  *out = new std::shared_ptr<Part>(make_foreign_part(family, id, prefix, Json::parse(description_json),
                                                     children_of(n_children, child_slots, children)));
  TI_END
}
namespace {
int (*g_foreign_make)(const char*, const char*, const char*, const char*, int, const char* const*, void* const*, void**) = nullptr;
}
int ti_set_foreign_factory(int (*make)(const char*, const char*, const char*, const char*, int, const char* const*, void* const*,
                                       void**)) {
  TI_BEGIN
  g_foreign_make = make;
  TI_END
}
int ti_register_foreign_kind(const char* family_, const char* kind_, const char* slots_json) {
  TI_BEGIN
  const std::string family = family_, kind = kind_;
  std::vector<std::pair<std::string, std::string>> slots;
  if (slots_json && *slots_json) {
    const Json parsed = Json::parse(slots_json);
    for (const auto& kv : parsed.members()) slots.emplace_back(kv.first, kv.second.as_string());
  }
  register_part(family, kind, [family, kind](const std::string& prefix, const Json& params, const PartChildren& children) {
    if (!g_foreign_make) throw ConfigError("the " + family + " part '" + kind + "' is implemented outside the library, which is gone");
    // the children cross as handles that the other side owns from here on
    std::vector<const char*> names;
    std::vector<void*> handles;
    for (const auto& c : children) {
      names.push_back(c.first.c_str());
      handles.push_back(new std::shared_ptr<Part>(c.second));
    }
    void* made = nullptr;
    const std::string text = params.dump();
    const int rc = g_foreign_make(family.c_str(), kind.c_str(), prefix.c_str(), text.c_str(), (int)children.size(), names.data(),
                                  handles.data(), &made);
    // (the handles to the children are the maker's now: it releases each with ti_part_release)
    if (rc != 0 || !made) {
      const std::string why = take_foreign_error();
      throw ConfigError("building the " + family + " part '" + kind + "' outside the library failed" + (why.empty() ? "" : ": " + why));
    }
    return *static_cast<std::shared_ptr<Part>*>(made);       // a reference of our own; the handle stays the maker's
  }, slots);
  TI_END
}
void ti_part_release(void* part) { delete static_cast<std::shared_ptr<Part>*>(part); }
int ti_part_child(void* part, int index, void** out) {
  TI_BEGIN
  const auto kids = P(part)->children();
  if (index < 0 || index >= (int)kids.size()) throw Error("ti_part_child: the part has no child " + std::to_string(index));
  *out = new std::shared_ptr<Part>(kids[index]);
  TI_END
}
int ti_part_tensors(void* part, const char** out) {
  TI_BEGIN
  return give(out, needs_json(P(part)->tensors()).dump());
  TI_END
}
int ti_part_cache_need(void* part, const char** out) {
  TI_BEGIN
  return give(out, P(part)->has_cache() ? cache_need_json(P(part)->cache_need()).dump() : std::string("null"));
  TI_END
}
int ti_part_info(void* part, const char** out) {
  TI_BEGIN
  Part& p = *P(part);
  Json j = Json::object();
  j.set("family", p.family());
  j.set("kind", p.kind_name());
  j.set("prefix", p.prefix);
  j.set("reads_through_ops", p.reads_through_ops());
  bool lazy_in = false, lazy_out = false;
  if (auto* m = dynamic_cast<MixerPart*>(&p)) lazy_in = m->takes_lazy_norm();
  if (auto* f = dynamic_cast<FeedForwardPart*>(&p)) lazy_in = f->takes_lazy_norm();
  if (auto* n = dynamic_cast<NormPart*>(&p)) lazy_out = n->can_be_lazy();
  j.set("takes_lazy_norm", lazy_in);
  j.set("can_be_lazy", lazy_out);
  j.set("built_kind", p.built_kind);
  j.set("params", p.built_from.type() == Json::Object ? p.built_from : Json::object());
  j.set("foreign_id", (int64_t)p.foreign_id);
  Json slots = Json::array();
  for (const auto& n : p.child_slots()) slots.push(n);
  j.set("slots", slots);
  return give(out, j.dump());
  TI_END
}

namespace {
// one part's tensors from device memory the caller owns: copied into memory the part keeps
struct PartStorage {
  std::vector<DeviceBuffer> buffers;
};
std::mutex g_part_storage_mutex;
std::map<Part*, std::unique_ptr<PartStorage>> g_part_storage;
class GivenTensors final : public WeightSource {
 public:
  GivenTensors(const std::vector<std::string>& names, const ti_tensor* ts) {
    for (size_t i = 0; i < names.size(); ++i) given_[names[i]] = T(ts, (int)i);
  }
  std::vector<std::pair<std::string, SourceInfo>> list() const override { return {}; }
  bool has(const std::string& name) const override { return given_.count(name) != 0; }
  void fill(const std::string& name, const Tensor& dst) override {
    auto it = given_.find(name);
    if (it == given_.end()) throw WeightsError("weights", {name}, {}, {}, {});
    const Tensor& src = it->second;
    if (src.numel() != dst.numel()) throw WeightsError("weights", {}, {}, {name + " is " + src.describe() + ", expected " + dst.describe()}, {});
    if (src.dtype != dst.dtype)
      throw KernelError("tensor '" + name + "' is " + dtype_name(src.dtype) + ", the part holds it as " + dtype_name(dst.dtype));
    if (!src.contiguous()) throw KernelError("tensor '" + name + "' must be contiguous");
    if (to_host) memcpy(dst.data, src.data, dst.bytes());
    else if (hipMemcpy(dst.data, src.data, dst.bytes(), hipMemcpyDeviceToDevice) != hipSuccess)
      throw KernelError("copying tensor '" + name + "' failed");
  }
 private:
  std::map<std::string, Tensor> given_;
};
}  // namespace

int ti_part_held(void* part, const char* member, ti_tensor* out) {
  TI_BEGIN
  *reinterpret_cast<Tensor*>(out) = Tensor();
  for (const auto& kv : P(part)->held())
    if (kv.first == member) *reinterpret_cast<Tensor*>(out) = kv.second;
  TI_END
}
int ti_part_pointer(void* part, void** out) {
  TI_BEGIN
  *out = P(part).get();
  TI_END
}
int ti_part_load(void* part, int n, const char* names, const ti_tensor* tensors, const char* matrix_dtype, int on_host) {
  TI_BEGIN
  auto ns = split_lines(names);
  if ((int)ns.size() != n) throw Error("ti_part_load: names and tensors differ in number");
  GivenTensors src(ns, tensors);
  src.matrix_dtype = dtype_from_name(matrix_dtype);
  src.to_host = on_host != 0;
  std::unique_ptr<HostMemoryScope> scope;
  if (on_host) scope.reset(new HostMemoryScope());
  Part* p = P(part).get();
  std::unique_ptr<PartStorage> st(new PartStorage());
  st->buffers.reserve(64);
  src.owner = &st->buffers;
  p->load(src);
  std::lock_guard<std::mutex> lock(g_part_storage_mutex);
  g_part_storage[p] = std::move(st);
  TI_END
}

int ti_ctx_create(const char* dtype, void* stream, void** out) {
  TI_BEGIN
  std::unique_ptr<OwnContext> own(new OwnContext(dtype_from_name(dtype), stream));
  StepContext* ctx = &own->ctx;
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  g_contexts[ctx] = std::move(own);
  *out = ctx;
  TI_END
}
void ti_ctx_release(void* ctx) {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  g_contexts.erase(static_cast<StepContext*>(ctx));
}
int ti_ctx_set_rows(void* ctx, int64_t M_, const int* positions, const int* tokens) {
  TI_BEGIN
  StepContext& c = *static_cast<StepContext*>(ctx);
  c.M = M_;
  c.positions = positions;
  c.tokens = tokens;
  TI_END
}

int ti_part_call(void* part, const char* op_, void* ctx_, const ti_tensor* args, int n_args, int flags, ti_tensor* result) {
  TI_BEGIN
  Part& p = *P(part);
  const std::string op = op_;
  StepContext* ctx = static_cast<StepContext*>(ctx_);
  Tensor* res = reinterpret_cast<Tensor*>(result);
  auto arg = [&](int i) -> const Tensor& {
    if (i >= n_args) throw Error("ti_part_call: '" + op + "' needs more arguments");
    return T(args, i);
  };
  if (op == "prepare") {
    Ops local;
    p.prepare(ctx ? ctx->ops : local, flags);
    return 0;
  }
  if (!ctx) throw Error("ti_part_call: '" + op + "' needs a context");
  const std::string family = p.family();
  if (family == "embedding" && op == "forward") {
    static_cast<EmbeddingPart&>(p).forward(*ctx, arg(0));
  } else if (family == "norm" && op == "forward") {
    const Tensor rows = n_args > 1 ? arg(1) : Tensor();
    Rows r = static_cast<NormPart&>(p).forward(*ctx, arg(0), rows.defined() ? rows.ptr<int>() : nullptr,
                                               rows.defined() ? rows.numel() : 0, false);
    *res = r.materialize(ctx->ops);
  } else if (family == "pos" && op == "apply") {
    static_cast<PositionPart&>(p).apply(*ctx, arg(0), n_args > 1 ? arg(1) : Tensor());
  } else if (family == "pos" && op == "fused") {
    Ops::Rotation rot;
    const bool ok = static_cast<PositionPart&>(p).fused(rot);
    res[0] = Tensor();
    res[1] = Tensor();
    if (ok) {
      // result[0] = inv_freq [hd/2], result[1] = table [len, hd/2, 2] (flags = head_dim)
      res[0] = Tensor((void*)rot.inv_freq, DType::F32, {(int64_t)flags / 2});
      if (rot.table) res[1] = Tensor((void*)rot.table, DType::F32, {(int64_t)rot.table_len, (int64_t)flags / 2, 2});
    }
  } else if (family == "mixer" && op == "forward") {
    Rows h;
    h.t = arg(0);
    static_cast<MixerPart&>(p).forward(*ctx, h, arg(1));
  } else if (family == "ffn" && op == "forward") {
    Rows h;
    h.t = arg(0);
    static_cast<FeedForwardPart&>(p).forward(*ctx, h, arg(1));
  } else if (family == "block" && op == "forward") {
    static_cast<BlockPart&>(p).forward(*ctx, arg(0));
  } else if (family == "head" && op == "forward") {
    Rows h;
    h.t = arg(0);
    *res = static_cast<HeadPart&>(p).forward(*ctx, h);
  } else {
    throw Error("ti_part_call: a " + family + " part has no call '" + op + "'");
  }
  ctx->ops.flush();          // whoever reads the results next need not know about deferred sums
  TI_END
}

int ti_ctx_info(void* ctx_, const char** out) {
  TI_BEGIN
  StepContext& c = *static_cast<StepContext*>(ctx_);
  Json j = Json::object();
  j.set("M", c.M);
  j.set("decode_only", c.decode_only);
  j.set("max_context", c.max_context);
  j.set("run", c.run);
  j.set("dtype", dtype_name(c.act_dtype));
  j.set("n_out", c.n_out);
  Json es = Json::array();
  for (const auto& e : c.entries) {
    Json r = Json::array();
    r.push(e.row0);
    r.push(e.n_tokens);
    r.push(e.start);
    r.push(e.state_slot);
    es.push(r);
  }
  j.set("entries", es);
  return give(out, j.dump());
  TI_END
}
int ti_ctx_pointers(void* ctx_, const int** tokens, const int** positions, const int** slots) {
  TI_BEGIN
  StepContext& c = *static_cast<StepContext*>(ctx_);
  *tokens = c.tokens;
  *positions = c.positions;
  *slots = c.slots;
  TI_END
}
int ti_ctx_binding(void* ctx_, void* part, int* group, int* layer) {
  TI_BEGIN
  const auto b = static_cast<StepContext*>(ctx_)->binding(P(part).get());
  *group = b.first;
  *layer = b.second;
  TI_END
}
int ti_ctx_kv_pool(void* ctx_, int group, int layer, ti_tensor* out) {
  TI_BEGIN
  *reinterpret_cast<Tensor*>(out) = static_cast<StepContext*>(ctx_)->kv_pool(group, layer);
  TI_END
}
int ti_ctx_state(void* ctx_, int group, int layer, ti_tensor* out) {
  TI_BEGIN
  *reinterpret_cast<Tensor*>(out) = static_cast<StepContext*>(ctx_)->state(group, layer);
  TI_END
}
int ti_ctx_cache_view(void* ctx_, int group, ti_tensor* out_table, int* page_size) {
  TI_BEGIN
  StepContext& c = *static_cast<StepContext*>(ctx_);
  const Ops::CacheView v = c.cache_view(group);
  *reinterpret_cast<Tensor*>(out_table) = Tensor((void*)v.table, DType::I32, {(int64_t)c.entries.size(), (int64_t)v.table_width});
  *page_size = v.page_size;
  TI_END
}
int ti_ctx_buf(void* ctx_, const char* name, int dtype, int ndim, const int64_t* shape, ti_tensor* out) {
  TI_BEGIN
  StepContext& c = *static_cast<StepContext*>(ctx_);
  Tensor t(nullptr, (DType)dtype, std::vector<int64_t>(shape, shape + ndim));
  t.data = c.ws.get(std::string("py.") + name + ":" + std::to_string(dtype), t.bytes());
  *reinterpret_cast<Tensor*>(out) = t;
  TI_END
}
int ti_ctx_ops(void* ctx_, void** out) {
  TI_BEGIN
  *out = &static_cast<StepContext*>(ctx_)->ops;
  TI_END
}

// -------------------------------------------------------------------------------------- model
int ti_model_from_spec(const char* spec_json, void** out) {
  TI_BEGIN
  *out = new std::shared_ptr<Model>(new Model(ModelSpec::from_json(Json::parse(spec_json))));
  TI_END
}
int ti_model_part(void* model, const char* which_, int index, void** out) {
  TI_BEGIN
  Model& m = *M(model);
  const std::string which = which_;
  std::shared_ptr<Part> p;
  if (which == "embedding") p = m.embedding;
  else if (which == "final_norm") p = m.final_norm;
  else if (which == "head") p = m.head;
  else if (which == "block") {
    if (index < 0 || index >= (int)m.blocks.size()) throw Error("ti_model_part: the model has no layer " + std::to_string(index));
    p = m.blocks[index];
  } else {
    throw Error("ti_model_part: unknown part '" + which + "'");
  }
  *out = new std::shared_ptr<Part>(p);
  TI_END
}
int ti_model_create(const char* meta_json, void* embedding, int n_blocks, void* const* blocks, void* final_norm, void* head,
                    void** out) {
  TI_BEGIN
  const Json meta = Json::parse(meta_json);
  ModelSpec spec;
  spec.architecture = meta.at("architecture").as_string();
  spec.vocab_size = meta.at("vocab_size").as_int();
  spec.hidden_size = meta.at("hidden_size").as_int();
  if (meta.has("schedule"))
    for (const Json& v : meta.at("schedule").items()) spec.schedule.push_back((int)v.as_int());
  if (meta.has("eos_token_ids"))
    for (const Json& v : meta.at("eos_token_ids").items()) spec.eos_token_ids.push_back(v.as_int());
  if (meta.has("max_position_embeddings")) spec.max_position_embeddings = meta.at("max_position_embeddings").as_int();
  spec.layers.resize(n_blocks);
  if (meta.has("cache_from")) {
    const Json& cf = meta.at("cache_from");
    for (size_t i = 0; i < cf.size() && i < (size_t)n_blocks; ++i)
      if (!cf[i].is_null()) spec.layers[i].cache_from = (int)cf[i].as_int();
  }
  std::vector<std::shared_ptr<Part>> bs;
  for (int i = 0; i < n_blocks; ++i) bs.push_back(P(blocks[i]));
  *out = new std::shared_ptr<Model>(new Model(spec, P(embedding), bs, P(final_norm), P(head)));
  TI_END
}
void ti_model_release(void* model) { delete static_cast<std::shared_ptr<Model>*>(model); }
int ti_model_tensors(void* model, const char** out) {
  TI_BEGIN
  return give(out, needs_json(M(model)->tensors()).dump());
  TI_END
}
int ti_model_cache_groups(void* model, const char** out) {
  TI_BEGIN
  Json a = Json::array();
  for (const auto& g : M(model)->cache_groups) {
    Json j = Json::object();
    j.set("need", cache_need_json(g.first));
    j.set("layers", g.second);
    a.push(j);
  }
  return give(out, a.dump());
  TI_END
}
int ti_model_bindings(void* model, const char** out) {
  TI_BEGIN
  Json runs = Json::array();
  for (const auto& run : M(model)->bindings) {
    Json r = Json::array();
    for (const auto& kv : run) {
      Json b = Json::array();
      b.push((int64_t)(uintptr_t)kv.first);
      b.push(kv.second.first);
      b.push(kv.second.second);
      r.push(b);
    }
    runs.push(r);
  }
  return give(out, runs.dump());
  TI_END
}
int ti_model_load_folder(void* model, const char* dir, const char* dtype, int to_host) {
  TI_BEGIN
  M(model)->load_folder(dir, dtype, to_host != 0);
  TI_END
}
int ti_model_load_tensors(void* model, int n, const char* names, const ti_tensor* tensors, int on_device, const char* dtype,
                          const char* where, int to_host) {
  TI_BEGIN
  auto ns = split_lines(names);
  if ((int)ns.size() != n) throw Error("ti_model_load_tensors: names and tensors differ in number");
  std::vector<HostTensor> ts;
  for (int i = 0; i < n; ++i) {
    const Tensor& t = T(tensors, i);
    if (!t.contiguous()) throw KernelError("tensor '" + ns[i] + "' must be contiguous");
    ts.push_back(HostTensor{ns[i], t.dtype, std::vector<int64_t>(t.shape, t.shape + t.ndim), t.data});
  }
  M(model)->load_tensors(ts, on_device != 0, dtype, where ? where : "weights", to_host != 0);
  TI_END
}
int ti_model_load_random(void* model, uint64_t seed, const char* dtype) {
  TI_BEGIN
  M(model)->load_random(seed, dtype);
  TI_END
}
int ti_model_write_random_folder(void* model, const char* dir, const char* config_json, uint64_t seed, const char* store_dtype) {
  TI_BEGIN
  M(model)->write_random_folder(dir, Json::parse(config_json), seed, store_dtype);
  TI_END
}
int ti_weights_error_lists(const char** out) { return give(out, g_weights_lists); }

// ------------------------------------------------------------------------------ cache manager
int ti_cache_create(const char* groups_json, int page_size, int num_pages, int max_requests, int max_seq, int scatter_window,
                    void** out) {
  TI_BEGIN
  std::vector<std::pair<CacheNeed, int>> groups;
  const Json parsed = Json::parse(groups_json);
  for (const Json& g : parsed.items()) groups.emplace_back(cache_need_from(g.at("need")), (int)g.at("layers").as_int());
  *out = new CacheManager(groups, page_size, num_pages, max_requests, max_seq, scatter_window);
  TI_END
}
void ti_cache_release(void* cache) { delete static_cast<CacheManager*>(cache); }
int ti_cache_call(void* cache, const char* op_, int64_t req, int64_t a, int64_t b, int64_t* out) {
  TI_BEGIN
  CacheManager& c = *static_cast<CacheManager*>(cache);
  const std::string op = op_;
  int64_t r = 0;
  if (op == "has") r = c.has(req);
  else if (op == "length") r = c.length(req);
  else if (op == "reserved") r = c.reserved(req);
  else if (op == "slot") r = c.slot(req);
  else if (op == "num_free_slots") r = c.num_free_slots();
  else if (op == "num_free_pages") r = c.num_free_pages();
  else if (op == "pages_needed") r = c.pages_needed(req, a != 0, (int)b);
  else if (op == "can_reserve") r = c.can_reserve(req, (int)a);
  else if (op == "admit") r = c.admit(req);
  else if (op == "reserve") c.reserve(req, (int)a);
  else if (op == "commit") c.commit(req, (int)a);
  else if (op == "rollback") c.rollback(req);
  else if (op == "release") c.release(req);
  else if (op == "check") c.check();
  else if (op == "pool_num_free") r = c.pool((int)a).num_free();
  else if (op == "pool_num_pages") r = c.pool((int)a).num_pages();
  else if (op == "pool_high_water") r = c.pool((int)a).high_water;
  else if (op == "pool_taken_total") r = c.pool((int)a).taken_total;
  else if (op == "pool_give_back") c.pool((int)a).give_back((int)b);
  else if (op == "pool_take") r = c.pool((int)a).take();
  else if (op == "clear_slots_list") c.slots_to_clear.clear();
  else throw Error("ti_cache_call: unknown call '" + op + "'");
  if (out) *out = r;
  TI_END
}
int ti_cache_table(void* cache, int group, int64_t req, const char** out) {
  TI_BEGIN
  Json a = Json::array();
  for (int p : static_cast<CacheManager*>(cache)->table(group, req)) a.push(p);
  return give(out, a.dump());
  TI_END
}
int ti_cache_many(void* cache, const char* op_, int n, const int64_t* reqs, const char** out) {
  TI_BEGIN
  CacheManager& c = *static_cast<CacheManager*>(cache);
  const std::string op = op_;
  std::vector<int64_t> rs(reqs, reqs + n);
  Json a = Json::array();
  if (op == "reserve_one_each") {
    for (int s : c.reserve_one_each(rs)) a.push(s);
  } else if (op == "commit_one_each") {
    c.commit_one_each(rs);
  } else {
    throw Error("ti_cache_many: unknown call '" + op + "'");
  }
  return give(out, a.dump());
  TI_END
}
int ti_cache_dump(void* cache, const char** out) {
  TI_BEGIN
  CacheManager& c = *static_cast<CacheManager*>(cache);
  Json j = Json::object();
  j.set("page_size", c.page_size);
  j.set("max_requests", c.max_requests);
  j.set("max_seq", c.max_seq);
  j.set("table_width", c.table_width);
  Json live = Json::array();
  for (int64_t r : c.live_requests()) live.push(r);
  j.set("live", live);
  Json clear = Json::array();
  for (int s : c.slots_to_clear) clear.push(s);
  j.set("slots_to_clear", clear);
  Json groups = Json::array();
  for (int g = 0; g < c.num_groups(); ++g) {
    Json gj = Json::object();
    gj.set("need", cache_need_json(c.group_need(g)));
    gj.set("layers", c.group_layers(g));
    gj.set("paged", c.group_is_paged(g));
    if (c.group_is_paged(g)) {
      gj.set("num_free", c.pool(g).num_free());
      gj.set("num_pages", c.pool(g).num_pages());
    }
    groups.push(gj);
  }
  j.set("groups", groups);
  return give(out, j.dump());
  TI_END
}
int ti_pool_create(int num_pages, int scatter_window, void** out) {
  TI_BEGIN
  *out = new PagePool(num_pages, scatter_window);
  TI_END
}
void ti_pool_release(void* pool) { delete static_cast<PagePool*>(pool); }
int ti_pool_call(void* pool, const char* op_, int64_t a, int64_t* out) {
  TI_BEGIN
  PagePool& p = *static_cast<PagePool*>(pool);
  const std::string op = op_;
  int64_t r = 0;
  if (op == "take") r = p.take();
  else if (op == "give_back") p.give_back((int)a);
  else if (op == "num_free") r = p.num_free();
  else if (op == "num_pages") r = p.num_pages();
  else throw Error("ti_pool_call: unknown call '" + op + "'");
  if (out) *out = r;
  TI_END
}
int ti_pool_free_list(void* pool, const char** out) {
  TI_BEGIN
  Json a = Json::array();
  for (int p : static_cast<PagePool*>(pool)->free_list()) a.push(p);
  return give(out, a.dump());
  TI_END
}

// ------------------------------------------------------------------------------------- engine
int ti_engine_create(void* model, const char* options_json, void** out) {
  TI_BEGIN
  const Json o = Json::parse(options_json);
  EngineOptions opt;
  if (o.has("dtype")) opt.dtype = o.at("dtype").as_string();
  if (o.has("page_size")) opt.page_size = (int)o.at("page_size").as_int();
  if (o.has("max_tokens")) opt.max_tokens = o.at("max_tokens").as_int();
  if (o.has("num_pages")) opt.num_pages = o.at("num_pages").as_int();
  if (o.has("max_requests")) opt.max_requests = (int)o.at("max_requests").as_int();
  if (o.has("max_seq")) opt.max_seq = (int)o.at("max_seq").as_int();
  if (o.has("stream")) opt.stream = (void*)(uintptr_t)o.at("stream").as_int();
  if (o.has("page_scatter_window")) opt.page_scatter_window = (int)o.at("page_scatter_window").as_int();
  if (o.has("max_step_graphs")) opt.max_step_graphs = (int)o.at("max_step_graphs").as_int();
  *out = new Engine(M(model), opt);
  TI_END
}
void ti_engine_release(void* engine) { delete static_cast<Engine*>(engine); }
int ti_engine_info(void* engine, const char** out) {
  TI_BEGIN
  Engine& e = *static_cast<Engine*>(engine);
  Json j = Json::object();
  j.set("dtype", e.dtype);
  j.set("page_size", e.page_size);
  j.set("max_seq", e.max_seq);
  j.set("num_pages", e.num_pages);
  j.set("steps_run", e.steps_run);
  j.set("num_graphs", (int64_t)e.num_graphs());
  j.set("cache_bytes", (int64_t)e.cache_bytes());
  j.set("table_width", e.cache->table_width);
  j.set("feedback_rows", e.feedback_rows());
  Json keys = Json::array();
  for (const auto& k : e.graph_keys()) keys.push(k);
  j.set("graphs", keys);
  return give(out, j.dump());
  TI_END
}
int ti_engine_cache(void* engine, void** out) {
  TI_BEGIN
  *out = static_cast<Engine*>(engine)->cache.get();
  TI_END
}
int ti_engine_ops(void* engine, void** out) {
  TI_BEGIN
  *out = &static_cast<Engine*>(engine)->ops;
  TI_END
}
int ti_engine_step(void* engine, int use_graph, int n_entries, const int64_t* requests, const int* n_tokens, const int* tokens,
                   const int* n_want, const int* want, ti_tensor* out_logits) {
  TI_BEGIN
  std::vector<StepEntry> entries(n_entries);
  size_t t = 0, w = 0;
  for (int i = 0; i < n_entries; ++i) {
    entries[i].request = requests[i];
    entries[i].tokens.assign(tokens + t, tokens + t + n_tokens[i]);
    entries[i].want.assign(want + w, want + w + n_want[i]);
    t += n_tokens[i];
    w += n_want[i];
  }
  Engine& e = *static_cast<Engine*>(engine);
  *reinterpret_cast<Tensor*>(out_logits) = use_graph ? e.step_graph(entries) : e.step(entries);
  TI_END
}
int ti_engine_release_request(void* engine, int64_t request) {
  TI_BEGIN
  static_cast<Engine*>(engine)->release(request);
  TI_END
}
int ti_engine_kv_pool(void* engine, int group, int layer, ti_tensor* out) {
  TI_BEGIN
  *reinterpret_cast<Tensor*>(out) = static_cast<Engine*>(engine)->kv_pool(group, layer);
  TI_END
}
int ti_engine_state(void* engine, int group, int layer, ti_tensor* out) {
  TI_BEGIN
  *reinterpret_cast<Tensor*>(out) = static_cast<Engine*>(engine)->state(group, layer);
  TI_END
}
int ti_engine_synchronize(void* engine) {
  TI_BEGIN
  static_cast<Engine*>(engine)->synchronize();
  TI_END
}

// -------------------------------------------------------------------- sampling and scheduling
float ti_uniform(uint64_t seed, uint64_t request, uint64_t n_generated) { return uniform(seed, request, n_generated); }
int ti_sampler_create(void* ops, void** out) {
  TI_BEGIN
  *out = new Sampler(*static_cast<Ops*>(ops));
  TI_END
}
void ti_sampler_release(void* sampler) { delete static_cast<Sampler*>(sampler); }
static std::vector<SamplingParams> sampling_params(int n, const float* temperature, const int* top_k, const float* top_p,
                                                   const uint64_t* seeds) {
  std::vector<SamplingParams> params(n);
  for (int i = 0; i < n; ++i) {
    params[i].temperature = temperature[i];
    params[i].top_k = top_k[i];
    params[i].top_p = top_p[i];
    params[i].seed = seeds[i];
  }
  return params;
}
int ti_sampler_sample(void* sampler, const ti_tensor* logits, int n, const float* temperature, const int* top_k,
                      const float* top_p, const uint64_t* seeds, const int64_t* requests, const int64_t* counters, int* out) {
  TI_BEGIN
  const std::vector<int> ids = static_cast<Sampler*>(sampler)->sample(T(logits, 0), sampling_params(n, temperature, top_k, top_p, seeds),
                                                                      std::vector<int64_t>(requests, requests + n),
                                                                      std::vector<int64_t>(counters, counters + n));
  memcpy(out, ids.data(), (size_t)n * 4);
  TI_END
}
int ti_sampler_sample_async(void* sampler, const ti_tensor* logits, int n, const float* temperature, const int* top_k,
                            const float* top_p, const uint64_t* seeds, const int64_t* requests, const int64_t* counters,
                            void* feed_engine, uint64_t* out_ticket) {
  TI_BEGIN
  int* feed = nullptr;
  if (feed_engine) {
    Engine& e = *static_cast<Engine*>(feed_engine);
    if (!e.token_feedback()) throw EngineError("this engine has no token feedback (its model has parts from outside the library)");
    if (n > e.feedback_rows())
      throw EngineError(std::to_string(n) + " rows of logits but the token feedback holds " + std::to_string(e.feedback_rows()));
    feed = e.token_feedback();
  }
  *out_ticket = static_cast<Sampler*>(sampler)->sample_async(T(logits, 0), sampling_params(n, temperature, top_k, top_p, seeds),
                                                             std::vector<int64_t>(requests, requests + n),
                                                             std::vector<int64_t>(counters, counters + n), feed);
  TI_END
}
int ti_sampler_collect(void* sampler, uint64_t ticket, int n, int* out) {
  TI_BEGIN
  const std::vector<int> ids = static_cast<Sampler*>(sampler)->collect(ticket);
  if ((int)ids.size() != n) throw KernelError("sample: the call drew " + std::to_string(ids.size()) + " ids, not " + std::to_string(n));
  memcpy(out, ids.data(), (size_t)n * 4);
  TI_END
}

int ti_scheduler_create(void* cache, int max_batched_tokens, int chunk_size, int max_running, void** out) {
  TI_BEGIN
  std::unique_ptr<SchedulerHandle> h(new SchedulerHandle());
  h->s.reset(new Scheduler(*static_cast<CacheManager*>(cache), max_batched_tokens, chunk_size, max_running));
  *out = h.release();
  TI_END
}
void ti_scheduler_release(void* scheduler) { delete static_cast<SchedulerHandle*>(scheduler); }
int ti_scheduler_add(void* scheduler, int n_prompt, const int* prompt, int max_new_tokens, float temperature, int top_k,
                     float top_p, uint64_t seed, int n_eos, const int* eos, int64_t* out_number) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  SamplingParams sp;
  sp.temperature = temperature;
  sp.top_k = top_k;
  sp.top_p = top_p;
  sp.seed = seed;
  auto r = h.s->add(std::vector<int>(prompt, prompt + n_prompt), max_new_tokens, sp, std::vector<int>(eos, eos + n_eos));
  h.all[r->number] = r;
  *out_number = r->number;
  TI_END
}
static Json plan_json(const Plan& plan) {
  Json j = Json::object();
  Json es = Json::array();
  for (const auto& e : plan.entries) {
    Json r = Json::object();
    r.set("number", e.request->number);
    r.set("start", e.start);
    r.set("n_tokens", e.n_tokens);
    r.set("sample", e.sample);
    es.push(r);
  }
  j.set("entries", es);
  Json pre = Json::array();
  for (const auto& r : plan.preempted) pre.push(r->number);
  j.set("preempted", pre);
  return j;
}
int ti_scheduler_plan(void* scheduler, const char** out) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  if (!h.ahead.entries.empty()) throw SchedulerError("a step planned ahead waits to be committed");
  h.last = h.s->plan();
  return give(out, plan_json(h.last).dump());
  TI_END
}
int ti_scheduler_plan_ahead(void* scheduler, const char** out) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  if (!h.ahead.entries.empty()) throw SchedulerError("a step planned ahead waits to be committed");
  h.ahead = h.s->plan_ahead(h.last);
  return give(out, plan_json(h.ahead).dump());
  TI_END
}
int ti_scheduler_commit(void* scheduler, int n, const int64_t* numbers, const int* tokens, const char** out) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  std::map<int64_t, int> sampled;
  for (int i = 0; i < n; ++i) sampled[numbers[i]] = tokens[i];
  Json done = Json::array();
  for (const auto& r : h.s->commit(h.last, sampled)) done.push(r->number);
  // what was planned ahead is the next to be committed, without the requests that have just ended
  h.last = Plan();
  for (const auto& e : h.ahead.entries)
    if (e.request->finish_reason.empty()) h.last.entries.push_back(e);
  h.ahead = Plan();
  return give(out, done.dump());
  TI_END
}
int ti_scheduler_abort(void* scheduler, int64_t number) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  auto it = h.all.find(number);
  if (it == h.all.end()) throw SchedulerError("no request " + std::to_string(number));
  h.s->abort(it->second);
  TI_END
}
int ti_scheduler_set_next_number(void* scheduler, int64_t number) {
  TI_BEGIN
  static_cast<SchedulerHandle*>(scheduler)->s->set_next_number(number);
  TI_END
}
int ti_scheduler_state(void* scheduler, const char** out) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  Json j = Json::object();
  auto list = [](const std::vector<std::shared_ptr<Request>>& v) {
    Json a = Json::array();
    for (const auto& r : v) a.push(r->number);
    return a;
  };
  j.set("waiting", list(h.s->waiting));
  j.set("running", list(h.s->running));
  j.set("finished", list(h.s->finished));
  j.set("max_batched_tokens", h.s->max_batched_tokens);
  j.set("chunk_size", h.s->chunk_size);
  j.set("max_running", h.s->max_running);
  return give(out, j.dump());
  TI_END
}
int ti_scheduler_request(void* scheduler, int64_t number, const char** out) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  auto it = h.all.find(number);
  if (it == h.all.end()) throw SchedulerError("no request " + std::to_string(number));
  return give(out, request_json(*it->second).dump());
  TI_END
}
int ti_run_requests(void* engine, void* scheduler, void* sampler, int use_graph, int run_ahead, int (*on_token)(int64_t, int),
                    int (*on_logits)(int64_t, const float*, int64_t), const char** out_stats) {
  TI_BEGIN
  SchedulerHandle& h = *static_cast<SchedulerHandle*>(scheduler);
  GenerationStats st;
  std::function<void(const Request&, int)> cb;
  if (on_token)
    cb = [on_token](const Request& r, int tok) {
      if (on_token(r.number, tok) != 0) throw EngineError("the token callback stopped the run");
    };
  PromptLogits lcb;
  if (on_logits)
    lcb = [on_logits](const Request& r, const float* row, int64_t vocab) {
      if (on_logits(r.number, row, vocab) != 0) throw EngineError("the logits callback stopped the run");
    };
  run_requests(*static_cast<Engine*>(engine), *h.s, static_cast<Sampler*>(sampler), &st, cb, use_graph != 0, run_ahead != 0, lcb);
  Json j = Json::object();
  j.set("prefill_ms", st.prefill_ms);
  j.set("prefill_tokens", st.prefill_tokens);
  j.set("decode_ms", st.decode_ms);
  j.set("decode_tokens", st.decode_tokens);
  j.set("steps", st.steps);
  j.set("preemptions", st.preemptions);
  j.set("steps_ahead", st.steps_ahead);
  return give(out_stats, j.dump());
  TI_END
}

// ---------------------------------------------------------------------------------------- ops
int ti_ops_create(void* stream, void** out) {
  TI_BEGIN
  std::unique_ptr<Ops> o(new Ops(stream));
  Ops* p = o.get();
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  g_own_ops[p] = std::move(o);
  *out = p;
  TI_END
}
void ti_ops_release(void* ops) {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  g_ops_workspaces.erase(static_cast<Ops*>(ops));
  g_own_ops.erase(static_cast<Ops*>(ops));
}
int ti_ops_switch(void* ops_, const char* name_, int value, int* old) {
  TI_BEGIN
  Ops& ops = *static_cast<Ops*>(ops_);
  const std::string name = name_;
  auto flag = [&](bool& f) {
    if (old) *old = f;
    if (value >= 0) f = value != 0;
  };
  if (name == "fast_gemm") flag(ops.use.fast_gemm);
  else if (name == "fast_attention") flag(ops.use.fast_attention);
  else if (name == "fused_norm") flag(ops.use.fused_norm);
  else if (name == "fused_qk_decode") flag(ops.use.fused_qk_decode);
  else if (name == "fused_qkv_prefill") flag(ops.use.fused_qkv_prefill);
  else if (name == "split_k_add") flag(ops.use.split_k_add);
  else if (name == "early_page_ids") flag(ops.use.early_page_ids);
  else if (name == "radix_sample") flag(ops.use.radix_sample);
  else if (name == "deferred_add") flag(ops.use.deferred_add);
  else if (name == "paired_prefill") flag(ops.use.paired_prefill);
  else if (name == "portion_splits") flag(ops.use.portion_splits);
  else if (name == "force_decode_splits") {
    if (old) *old = ops.use.force_decode_splits;
    if (value >= 0) ops.use.force_decode_splits = value;
  } else if (name == "force_paired_tiles") {
    if (old) *old = ops.use.force_paired_tiles;
    if (value >= -1) ops.use.force_paired_tiles = value;
  } else {
    throw Error("ti_ops_switch: unknown switch '" + name + "'");
  }
  TI_END
}

int ti_ops_call(void* ops_, const char* op_, const ti_tensor* t, int n_t, const double* s, int n_s, const char* text,
                ti_tensor* result) {
  TI_BEGIN
  Ops& ops = *static_cast<Ops*>(ops_);
  const std::string op = op_;
  auto arg = [&](int i) -> const Tensor& {
    if (i >= n_t) throw Error("ti_ops_call: '" + op + "' needs more tensors");
    return T(t, i);
  };
  auto num = [&](int i) -> double {
    if (i >= n_s) throw Error("ti_ops_call: '" + op + "' needs more numbers");
    return s[i];
  };
  auto fptr = [&](int i) -> const float* { return arg(i).defined() ? arg(i).ptr<float>() : nullptr; };
  auto iptr = [&](int i) -> const int* { return arg(i).defined() ? arg(i).ptr<int>() : nullptr; };
  auto rotation = [&](int inv, int table) {
    Ops::Rotation r;
    r.inv_freq = fptr(inv);
    r.table = fptr(table);
    r.table_len = arg(table).defined() ? (int)arg(table).shape[0] : 0;
    return r;
  };
  auto view_of = [&](int table, const Tensor& pool) {
    Ops::CacheView v;
    v.table = iptr(table);
    v.table_width = arg(table).defined() ? (int)arg(table).shape[arg(table).ndim - 1] : 0;
    v.page_size = pool.defined() ? (int)pool.shape[2] : 0;
    return v;
  };
  Tensor* res = reinterpret_cast<Tensor*>(result);
  auto answer = [&](int64_t v) {
    if (res) {
      *res = Tensor();
      res->shape[0] = v;
    }
  };
  if (op == "embed") {
    ops.embed(arg(0), iptr(1), arg(1).numel(), arg(2));
  } else if (op == "rmsnorm") {
    const bool rows = n_t > 3 && arg(3).defined();
    ops.rmsnorm(arg(0), arg(1), (float)num(0), arg(2), rows ? iptr(3) : nullptr, rows ? arg(3).numel() : 0);
  } else if (op == "rope_neox") {
    ops.rope_neox(arg(0), iptr(1), arg(2));
  } else if (op == "rope_table") {
    ops.rope_table(arg(0), arg(1));
  } else if (op == "qk_norm_rope_kv_write") {
    // qkv, q_w, k_w, inv_freq, rope_table, positions, slots, table, pool, q_out; eps, heads, kv_heads, head_dim
    ops.qk_norm_rope_kv_write(arg(0), fptr(1), fptr(2), (float)num(0), rotation(3, 4), iptr(5), iptr(6), view_of(7, arg(8)), arg(8),
                              arg(9), (int)num(1), (int)num(2), (int)num(3));
  } else if (op == "qk_norm_inplace") {
    ops.qk_norm_inplace(arg(0), fptr(1), fptr(2), (float)num(0), (int)num(1), (int)num(2), (int)num(3));
  } else if (op == "linear") {
    ops.linear(arg(0), arg(1), arg(2), (Ops::Epilogue)(int)num(0), num(1) != 0);
  } else if (op == "linear_normed") {
    // x, norm weight, the buffer the normed rows would go to, w, out; eps, epilogue, may_defer
    Rows r;
    r.lazy = true;
    r.x = arg(0);
    r.weight = arg(1);
    r.t = arg(2);
    r.eps = (float)num(0);
    ops.linear(r, arg(3), arg(4), (Ops::Epilogue)(int)num(1), num(2) != 0);
  } else if (op == "linear_normed_only") {
    Rows r;
    r.lazy = true;
    r.x = arg(0);
    r.weight = arg(1);
    r.t = arg(2);
    r.eps = (float)num(0);
    answer(ops.linear_with_norm(r, arg(3), arg(4), (Ops::Epilogue)(int)num(1)));
  } else if (op == "qkv_prepared") {
    // a, w, q_w, k_w, inv_freq, rope_table, positions, slots, table, pool, q_out; eps, heads, kv_heads, head_dim
    Rows r;
    r.t = arg(0);
    answer(ops.qkv_prepared(r, arg(1), fptr(2), fptr(3), (float)num(0), rotation(4, 5), iptr(6), iptr(7), view_of(8, arg(9)), arg(9),
                            arg(10), (int)num(1), (int)num(2), (int)num(3)));
  } else if (op == "attention_rows") {
    // q, pool, table, positions, slots, out; heads, kv_heads, head_dim, scale, window
    ops.attention_rows(arg(0), arg(1), view_of(2, arg(1)), iptr(3), iptr(4), arg(5), (int)num(0), (int)num(1), (int)num(2),
                       (float)num(3), (int)num(4));
  } else if (op == "attention" || op == "attention_from_projections") {
    // q | qkv, pool, table, out, positions, slots, entry_meta, tiles, tiles_small, decode_rows, [q_w, k_w, inv_freq, rope_table];
    // heads, kv_heads, head_dim, scale, window, M, n_tiles, n_tiles_small, n_decode_rows, decode_only, max_context,
    // portion_context, split_context, [eps, write_kv]
    AttentionWork w;
    w.M = (int64_t)num(5);
    w.positions = iptr(4);
    w.slots = iptr(5);
    w.entry_meta = iptr(6);
    w.tiles = iptr(7);
    w.n_tiles = (int)num(6);
    w.tiles_small = iptr(8);
    w.n_tiles_small = (int)num(7);
    w.decode_rows = iptr(9);
    w.n_decode_rows = (int)num(8);
    w.decode_only = num(9) != 0;
    w.max_context = (int)num(10);
    w.portion_context = (int)num(11);
    w.split_context = (int)num(12);
    w.slots_are_rows = n_s > 15 && s[15] != 0;
    Workspace& ws = workspace_of(&ops);
    if (op == "attention") {
      ops.attention(w, ws, view_of(2, arg(1)), arg(0), arg(1), arg(3), (int)num(0), (int)num(1), (int)num(2), (float)num(3), (int)num(4));
    } else {
      answer(ops.attention_from_projections(w, ws, view_of(2, arg(1)), arg(0), fptr(10), fptr(11), (float)num(13), rotation(12, 13),
                                            arg(1), num(14) != 0, arg(3), (int)num(0), (int)num(1), (int)num(2), (float)num(3),
                                            (int)num(4)));
    }
  } else if (op == "argmax") {
    ops.argmax(arg(0), arg(1).ptr<int>());
  } else if (op == "sample") {
    ops.sample(arg(0), fptr(1), iptr(2), fptr(3), fptr(4), arg(5).ptr<int>());
  } else if (op == "flush") {
    ops.flush();
  } else if (op == "timing") {
    ops.timing(num(0) != 0);
  } else if (op == "pending") {
    answer(ops.pending_splits());
  } else if (op == "can_fuse_norm") {
    answer(ops.can_fuse_norm((int64_t)num(0), (DType)(int)num(1)));
  } else if (op == "compute_units") {
    answer(ops.compute_units());
  } else if (op == "fill_random") {
    ops.fill_random(arg(0), text ? text : "normal", num(0), num(1), (uint64_t)num(2));
  } else if (op == "tune") {
    // text = "library name"; no text: every override of this object goes
    if (!text || !*text) {
      ops.untune();
    } else {
      const std::string t = text;
      const size_t sp = t.find(' ');
      if (sp == std::string::npos) throw Error("ti_ops_call: 'tune' takes \"library name\"");
      ops.tune(t.substr(0, sp), t.substr(sp + 1), (long)num(0));
    }
  } else if (op == "count_calls") {
    ops.count_calls(num(0) != 0);
  } else if (op == "fill_zero") {
    ops.fill_zero(arg(0).data, arg(0).bytes());
  } else {
    throw Error("ti_ops_call: unknown call '" + op + "'");
  }
  TI_END
}

int ti_portion_launch(int n_tiles_small, int heads, int portion_context, int window, int units, int* paired) {
  bool p = false;
  const int s = Ops::portion_launch(n_tiles_small, heads, portion_context, window, units, &p);
  if (paired) *paired = p ? 1 : 0;
  return s;
}
int ti_ops_timing_report(void* ops_, const char** out) {
  TI_BEGIN
  Json a = Json::array();
  for (const auto& t : static_cast<Ops*>(ops_)->timing_report()) {
    Json j = Json::object();
    j.set("name", t.name);
    j.set("calls", t.calls);
    j.set("us", t.us);
    a.push(j);
  }
  return give(out, a.dump());
  TI_END
}
int ti_decode_splits(int n_rows, int kv_heads, int heads, int context, int typical, int units, int head_dim) {
  return Ops::decode_splits(n_rows, kv_heads, heads, context, typical, units, head_dim);
}

}  // extern "C"
