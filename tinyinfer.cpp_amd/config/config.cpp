// Typed configuration of the Qwen3 dense decoder, the model as data (specs), and the registry
// from an architecture's name to its model.
//
// The reference fills `Qwen3Config` from GGUF keys and refuses a model whose required sizes are
// zero (/root/reference/src/model.h:11-21, src/model.cpp:32-47); its architecture gate is one
// string compare (src/model.cpp:26-30).  Layer order and formulas: src/inference.cu:28-72; tensor
// names follow the checkpoint convention (`model.layers.{i}.…`), onto which the reference's GGUF
// names (`blk.{i}.attn_q.weight`, src/model.cpp:120-150) map one to one.
#include <cmath>
#include <fstream>
#include <mutex>
#include <sstream>

#include "../include/inference.h"

namespace tinyinfer {

namespace {
const char* FULL = "full_attention";
const char* SLIDING = "sliding_attention";

bool present(const Json& d, const char* key) { return d.has(key); }

std::string show(const Json& v) { return v.dump(); }

int64_t take_int(const Json& d, const char* key, const int64_t* fallback = nullptr) {
  if (!present(d, key)) {
    if (!fallback) throw ConfigError(std::string("config.json: required key '") + key + "' is missing");
    return *fallback;
  }
  const Json& v = d.at(key);
  if (v.type() == Json::Int) return v.as_int();
  if (v.type() == Json::Float && v.as_double() == std::floor(v.as_double())) return (int64_t)v.as_double();
  throw ConfigError(std::string("config.json: '") + key + "' must be an integer, got " + show(v));
}
double take_float(const Json& d, const char* key, double fallback) {
  if (!present(d, key)) return fallback;
  const Json& v = d.at(key);
  if (!v.is_number()) throw ConfigError(std::string("config.json: '") + key + "' must be a number, got " + show(v));
  return v.as_double();
}
bool take_bool(const Json& d, const char* key, bool fallback) {
  if (!present(d, key)) return fallback;
  const Json& v = d.at(key);
  if (v.type() != Json::Bool)
    throw ConfigError(std::string("config.json: '") + key + "' must be true or false, got " + show(v));
  return v.as_bool();
}
std::string take_string(const Json& d, const char* key, const std::string& fallback) {
  if (!present(d, key)) return fallback;
  const Json& v = d.at(key);
  if (v.type() != Json::String)
    throw ConfigError(std::string("config.json: '") + key + "' must be a string, got " + show(v));
  return v.as_string();
}
}  // namespace

Qwen3Config Qwen3Config::from_json(const Json& d) {
  if (d.type() != Json::Object) throw ConfigError("config.json: top level must be a JSON object");
  Qwen3Config c;
  c.num_hidden_layers = take_int(d, "num_hidden_layers");
  c.hidden_size = take_int(d, "hidden_size");
  c.num_attention_heads = take_int(d, "num_attention_heads");
  c.num_key_value_heads = take_int(d, "num_key_value_heads", &c.num_attention_heads);
  if (c.num_attention_heads <= 0) throw ConfigError("config.json: 'num_attention_heads' must be positive");
  if (present(d, "head_dim")) {
    c.head_dim = take_int(d, "head_dim");
  } else {
    if (c.hidden_size % c.num_attention_heads)
      throw ConfigError("config.json: 'head_dim' is absent and 'hidden_size' (" + std::to_string(c.hidden_size) +
                        ") is not a multiple of 'num_attention_heads' (" + std::to_string(c.num_attention_heads) + ")");
    c.head_dim = c.hidden_size / c.num_attention_heads;
  }
  const std::string act = take_string(d, "hidden_act", "silu");
  if (act != "silu") throw ConfigError("config.json: 'hidden_act' = '" + act + "' is not served (only 'silu')");
  if (take_bool(d, "attention_bias", false))
    throw ConfigError("config.json: 'attention_bias' = true is not served (the projections carry no bias)");
  if (present(d, "rope_scaling")) {
    const Json& sc = d.at("rope_scaling");
    std::string kind;
    if (sc.type() == Json::Object) {
      const Json* k = sc.find("rope_type");
      if (!k) k = sc.find("type");
      if (k && k->type() == Json::String) kind = k->as_string();
    } else if (sc.type() == Json::String) {
      kind = sc.as_string();
    }
    if (kind != "default") throw ConfigError("config.json: 'rope_scaling' = " + show(sc) + " is not served");
  }

  const int64_t zero = 0;
  int64_t window = take_int(d, "sliding_window", &zero);
  const bool has_window = present(d, "sliding_window");
  const bool use_window = take_bool(d, "use_sliding_window", false);
  const int64_t L = c.num_hidden_layers;
  if (present(d, "layer_types")) {
    const Json& types = d.at("layer_types");
    if (types.type() != Json::Array || (int64_t)types.size() != L)
      throw ConfigError("config.json: 'layer_types' must list one entry per layer (" + std::to_string(L) + "), got " +
                        show(types));
    for (const Json& t : types.items()) {
      if (t.type() != Json::String || (t.as_string() != FULL && t.as_string() != SLIDING))
        throw ConfigError("config.json: 'layer_types' entry " + show(t) + " is not served");
      c.layer_types.push_back(t.as_string());
    }
  } else if (use_window && has_window) {
    const int64_t first = take_int(d, "max_window_layers", &L);
    for (int64_t i = 0; i < L; ++i) c.layer_types.push_back(i >= first ? SLIDING : FULL);
  } else {
    for (int64_t i = 0; i < L; ++i) c.layer_types.push_back(FULL);
  }
  bool slides = false;
  for (const auto& t : c.layer_types) slides = slides || t == SLIDING;
  if (slides) {
    if (!has_window) throw ConfigError("config.json: a layer slides but 'sliding_window' is absent");
    if (window <= 0) throw ConfigError("config.json: 'sliding_window' must be positive");
  } else {
    window = 0;
  }
  c.sliding_window = window;

  if (present(d, "eos_token_id")) {
    const Json& eos = d.at("eos_token_id");
    if (eos.type() == Json::Array) {
      for (const Json& e : eos.items()) c.eos_token_ids.push_back(e.as_int());
    } else {
      c.eos_token_ids.push_back(take_int(d, "eos_token_id"));
    }
  }
  if (const Json* archs = d.find("architectures"))
    if (archs->type() == Json::Array && archs->size() && (*archs)[0].type() == Json::String)
      c.architecture = (*archs)[0].as_string();
  if (const Json* tie = d.find("tie_word_embeddings")) {
    if (!tie->is_null()) {
      if (tie->type() != Json::Bool)
        throw ConfigError("config.json: 'tie_word_embeddings' must be true or false, got " + show(*tie));
      c.tie_word_embeddings = tie->as_bool() ? 1 : 0;
    }
  }
  c.vocab_size = take_int(d, "vocab_size");
  c.intermediate_size = take_int(d, "intermediate_size");
  // defaults of the reference's loader: src/model.cpp:39-40
  c.rms_norm_eps = take_float(d, "rms_norm_eps", 1e-6);
  c.rope_theta = take_float(d, "rope_theta", 1000000.0);
  c.max_position_embeddings = take_int(d, "max_position_embeddings", &zero);
  c.validate();
  return c;
}

void Qwen3Config::validate() const {
  const std::pair<const char*, int64_t> sizes[] = {
      {"vocab_size", vocab_size}, {"hidden_size", hidden_size}, {"intermediate_size", intermediate_size},
      {"num_hidden_layers", num_hidden_layers}, {"num_attention_heads", num_attention_heads},
      {"num_key_value_heads", num_key_value_heads}, {"head_dim", head_dim}};
  for (const auto& kv : sizes)
    if (kv.second <= 0)
      throw ConfigError(std::string("config.json: '") + kv.first + "' must be positive, got " + std::to_string(kv.second));
  if (num_attention_heads % num_key_value_heads)
    throw ConfigError("config.json: 'num_attention_heads' (" + std::to_string(num_attention_heads) +
                      ") must be a multiple of 'num_key_value_heads' (" + std::to_string(num_key_value_heads) + ")");
  if (head_dim % 2)
    throw ConfigError("config.json: 'head_dim' (" + std::to_string(head_dim) +
                      ") must be even (rotation pairs k with k + head_dim/2)");
  // what the attention kernels take (the reference refuses a head size at the launch:
  // /root/reference/src/cuda/attention.cu:321-324); said here, before any weight is read
  if (head_dim % 16 || head_dim > 256)
    throw ConfigError("config.json: 'head_dim' = " + std::to_string(head_dim) +
                      " is not served: the attention kernels take head sizes in steps of 16 up to 256");
  if (!(rms_norm_eps > 0.0)) throw ConfigError("config.json: 'rms_norm_eps' must be positive");
  if (!(rope_theta > 0.0)) throw ConfigError("config.json: 'rope_theta' must be positive");
  if (sliding_window < 0) throw ConfigError("config.json: 'sliding_window' must be positive");
  if ((int64_t)layer_types.size() != num_hidden_layers)
    throw ConfigError("config.json: 'layer_types' must list one entry per layer");
}

Json Qwen3Config::to_json() const {
  Json d = Json::object();
  Json archs = Json::array();
  archs.push(architecture);
  d.set("architectures", archs);
  d.set("model_type", "qwen3");
  d.set("vocab_size", vocab_size);
  d.set("hidden_size", hidden_size);
  d.set("intermediate_size", intermediate_size);
  d.set("num_hidden_layers", num_hidden_layers);
  d.set("num_attention_heads", num_attention_heads);
  d.set("num_key_value_heads", num_key_value_heads);
  d.set("head_dim", head_dim);
  d.set("hidden_act", "silu");
  d.set("rms_norm_eps", rms_norm_eps);
  d.set("rope_theta", rope_theta);
  d.set("rope_scaling", Json());
  d.set("attention_bias", false);
  d.set("tie_word_embeddings", tie_word_embeddings < 0 ? Json() : Json(tie_word_embeddings == 1));
  Json types = Json::array();
  bool slides = false;
  for (const auto& t : layer_types) {
    types.push(t);
    slides = slides || t == SLIDING;
  }
  d.set("layer_types", types);
  d.set("sliding_window", sliding_window > 0 ? Json(sliding_window) : Json());
  d.set("use_sliding_window", slides);
  if (max_position_embeddings > 0) d.set("max_position_embeddings", max_position_embeddings);
  if (eos_token_ids.size() == 1) {
    d.set("eos_token_id", eos_token_ids[0]);
  } else if (!eos_token_ids.empty()) {
    Json e = Json::array();
    for (int64_t v : eos_token_ids) e.push(v);
    d.set("eos_token_id", e);
  }
  return d;
}

Json read_config_json(const std::string& model_dir) {
  const std::string path = model_dir + "/config.json";
  std::ifstream f(path, std::ios::binary);
  if (!f) throw ConfigError(path + ": no config.json in the model folder");
  std::stringstream ss;
  ss << f.rdbuf();
  Json d;
  try {
    d = Json::parse(ss.str());
  } catch (const Error& e) {
    throw ConfigError(path + ": not valid JSON (" + e.what() + ")");
  }
  if (d.type() != Json::Object) throw ConfigError(path + ": top level must be a JSON object");
  return d;
}

// ------------------------------------------------------------------------------------- specs
Json PartSpec::to_json() const {
  Json j = Json::object();
  j.set("kind", kind);
  j.set("params", params);
  j.set("name", name);
  return j;
}
PartSpec PartSpec::from_json(const Json& j) {
  PartSpec p;
  p.kind = j.at("kind").as_string();
  if (const Json* q = j.find("params")) p.params = q->is_null() ? Json::object() : *q;
  if (const Json* n = j.find("name")) p.name = n->is_null() ? "" : n->as_string();
  return p;
}

std::vector<int> ModelSpec::run_order() const {
  if (!schedule.empty()) return schedule;
  std::vector<int> r(layers.size());
  for (size_t i = 0; i < r.size(); ++i) r[i] = (int)i;
  return r;
}

Json ModelSpec::to_json() const {
  Json j = Json::object();
  j.set("architecture", architecture);
  j.set("vocab_size", vocab_size);
  j.set("hidden_size", hidden_size);
  j.set("embedding", embedding.to_json());
  Json ls = Json::array();
  for (const auto& l : layers) {
    Json lj = Json::object();
    lj.set("prefix", l.prefix);
    lj.set("block", l.block.to_json());
    Json parts = Json::object();
    for (const auto& kv : l.parts) parts.set(kv.first, kv.second.to_json());
    lj.set("parts", parts);
    lj.set("cache_from", l.cache_from < 0 ? Json() : Json(l.cache_from));
    ls.push(lj);
  }
  j.set("layers", ls);
  j.set("final_norm", final_norm.to_json());
  j.set("lm_head", lm_head.to_json());
  if (schedule.empty()) {
    j.set("schedule", Json());
  } else {
    Json s = Json::array();
    for (int v : schedule) s.push(v);
    j.set("schedule", s);
  }
  Json eos = Json::array();
  for (int64_t v : eos_token_ids) eos.push(v);
  j.set("eos_token_ids", eos);
  j.set("max_position_embeddings", max_position_embeddings > 0 ? Json(max_position_embeddings) : Json());
  return j;
}

ModelSpec ModelSpec::from_json(const Json& j) {
  ModelSpec s;
  s.architecture = j.at("architecture").as_string();
  s.vocab_size = j.at("vocab_size").as_int();
  s.hidden_size = j.at("hidden_size").as_int();
  if (j.has("embedding")) s.embedding = PartSpec::from_json(j.at("embedding"));
  if (j.has("final_norm")) s.final_norm = PartSpec::from_json(j.at("final_norm"));
  if (j.has("lm_head")) s.lm_head = PartSpec::from_json(j.at("lm_head"));
  if (j.has("layers"))
    for (const Json& lj : j.at("layers").items()) {
      LayerSpec l;
      l.prefix = lj.at("prefix").as_string();
      if (lj.has("block")) l.block = PartSpec::from_json(lj.at("block"));
      if (lj.has("parts"))
        for (const auto& kv : lj.at("parts").members()) l.parts.emplace_back(kv.first, PartSpec::from_json(kv.second));
      if (lj.has("cache_from")) l.cache_from = (int)lj.at("cache_from").as_int();
      s.layers.push_back(std::move(l));
    }
  if (j.has("schedule"))
    for (const Json& v : j.at("schedule").items()) s.schedule.push_back((int)v.as_int());
  if (j.has("eos_token_ids"))
    for (const Json& v : j.at("eos_token_ids").items()) s.eos_token_ids.push_back(v.as_int());
  if (j.has("max_position_embeddings")) s.max_position_embeddings = j.at("max_position_embeddings").as_int();
  return s;
}

// ---------------------------------------------------------------------------------- registry
namespace {
std::mutex g_arch_mutex;
struct Architecture {
  std::string name;
  SpecBuilder builder;
  ConfigReader typed;
};
std::vector<Architecture>& architectures() {
  static std::vector<Architecture> table;
  return table;
}

ModelSpec build_qwen3_spec(const Json& config) {
  const Qwen3Config cfg = Qwen3Config::from_json(config);
  const int64_t H = cfg.hidden_size;
  ModelSpec spec;
  spec.architecture = cfg.architecture;
  spec.vocab_size = cfg.vocab_size;
  spec.hidden_size = H;
  auto norm = [&](const char* name) {
    PartSpec p;
    p.kind = "rmsnorm";
    p.params.set("dim", H);
    p.params.set("eps", cfg.rms_norm_eps);
    p.name = name;
    return p;
  };
  for (int64_t i = 0; i < cfg.num_hidden_layers; ++i) {
    LayerSpec l;
    l.prefix = "model.layers." + std::to_string(i);
    l.block.kind = "pre_norm";
    PartSpec attn;
    attn.kind = "attention";
    attn.name = "self_attn";
    attn.params.set("hidden", H);
    attn.params.set("heads", cfg.num_attention_heads);
    attn.params.set("kv_heads", cfg.num_key_value_heads);
    attn.params.set("head_dim", cfg.head_dim);
    attn.params.set("qk_norm", true);
    attn.params.set("eps", cfg.rms_norm_eps);
    attn.params.set("window", cfg.layer_types[i] == SLIDING ? Json(cfg.sliding_window) : Json());
    PartSpec pos;
    pos.kind = "rope_neox";
    pos.params.set("head_dim", cfg.head_dim);
    pos.params.set("theta", cfg.rope_theta);
    attn.params.set("pos", pos.to_json());
    PartSpec ffn;
    ffn.kind = "swiglu";
    ffn.name = "mlp";
    ffn.params.set("hidden", H);
    ffn.params.set("intermediate", cfg.intermediate_size);
    l.parts.emplace_back("norm1", norm("input_layernorm"));
    l.parts.emplace_back("mixer", attn);
    l.parts.emplace_back("norm2", norm("post_attention_layernorm"));
    l.parts.emplace_back("ffn", ffn);
    spec.layers.push_back(std::move(l));
  }
  spec.embedding.kind = "table";
  spec.embedding.name = "model.embed_tokens";
  spec.embedding.params.set("vocab", cfg.vocab_size);
  spec.embedding.params.set("dim", H);
  spec.final_norm = norm("model.norm");
  spec.lm_head.kind = "linear";
  spec.lm_head.name = "lm_head";
  spec.lm_head.params.set("vocab", cfg.vocab_size);
  spec.lm_head.params.set("dim", H);
  spec.lm_head.params.set("tied", cfg.tie_word_embeddings < 0 ? Json() : Json(cfg.tie_word_embeddings == 1));
  spec.lm_head.params.set("tied_to", "model.embed_tokens.weight");
  spec.eos_token_ids = cfg.eos_token_ids;
  spec.max_position_embeddings = cfg.max_position_embeddings;
  return spec;
}

void ensure_builtin_architectures() {
  static std::once_flag once;
  std::call_once(once, [] {
    std::lock_guard<std::mutex> lock(g_arch_mutex);
    const ConfigReader typed = [](const Json& config) { return Qwen3Config::from_json(config).to_json(); };
    architectures().push_back({"Qwen3ForCausalLM", build_qwen3_spec, typed});
    architectures().push_back({"qwen3", build_qwen3_spec, typed});
  });
}

std::vector<std::string> candidates(const Json& config) {
  std::vector<std::string> c;
  if (const Json* a = config.find("architectures"))
    if (a->type() == Json::Array)
      for (const Json& v : a->items())
        if (v.type() == Json::String) c.push_back(v.as_string());
  if (const Json* m = config.find("model_type"))
    if (m->type() == Json::String) c.push_back(m->as_string());
  return c;
}

std::string list_of(const std::vector<std::string>& v) {
  std::string s = "[";
  for (size_t i = 0; i < v.size(); ++i) s += (i ? ", '" : "'") + v[i] + "'";
  return s + "]";
}
}  // namespace

void register_architecture(const std::vector<std::string>& names, SpecBuilder builder, ConfigReader typed) {
  ensure_builtin_architectures();
  std::lock_guard<std::mutex> lock(g_arch_mutex);
  for (const auto& n : names) {
    bool found = false;
    for (auto& a : architectures())
      if (a.name == n) {
        a.builder = builder;
        a.typed = typed;
        found = true;
      }
    if (!found) architectures().push_back({n, builder, typed});
  }
}

std::vector<std::string> registered_architectures() {
  ensure_builtin_architectures();
  std::lock_guard<std::mutex> lock(g_arch_mutex);
  std::vector<std::string> names;
  for (const auto& a : architectures()) names.push_back(a.name);
  std::sort(names.begin(), names.end());
  return names;
}

bool architecture_registered(const Json& config) {
  ensure_builtin_architectures();
  std::lock_guard<std::mutex> lock(g_arch_mutex);
  for (const auto& c : candidates(config))
    for (const auto& a : architectures())
      if (a.name == c) return true;
  return false;
}

namespace {
Architecture architecture_of(const Json& config) {
  ensure_builtin_architectures();
  const auto cand = candidates(config);
  if (cand.empty())
    throw ConfigError("config.json: neither 'architectures' nor 'model_type' names the model; registered: " +
                      list_of(registered_architectures()));
  {
    std::lock_guard<std::mutex> lock(g_arch_mutex);
    for (const auto& c : cand)
      for (const auto& a : architectures())
        if (a.name == c) return a;
  }
  throw ConfigError("config.json: architecture " + list_of(cand) + " is not registered; registered: " +
                    list_of(registered_architectures()));
}
}  // namespace

ModelSpec spec_from_config(const Json& config) { return architecture_of(config).builder(config); }

Json typed_config(const Json& config) {
  const Architecture a = architecture_of(config);
  Json j = Json::object();
  j.set("architecture", a.name);
  j.set("config", a.typed ? a.typed(config) : config);
  return j;
}

}  // namespace tinyinfer
