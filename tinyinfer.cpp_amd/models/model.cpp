// A model put together from a `ModelSpec`: parts built through the part registry, cache needs
// gathered into groups, the run order kept as a list, and the three ways its weights arrive.
#include <sys/stat.h>

#include <algorithm>
#include <cstdio>
#include <fstream>

#include "../include/inference.h"
#include "../weights/weights.h"

namespace tinyinfer {

static std::string join(const std::string& prefix, const std::string& name) {
  if (prefix.empty()) return name;
  if (name.empty()) return prefix;
  return prefix + "." + name;
}

Model::Model(const ModelSpec& s) : spec(s) {
  embedding = std::dynamic_pointer_cast<EmbeddingPart>(build_part("embedding", spec.embedding, spec.embedding.name));
  for (const auto& ls : spec.layers) {
    PartChildren built;
    for (const auto& slot : block_slots(ls.block.kind)) {
      const PartSpec* ps = nullptr;
      for (const auto& kv : ls.parts)
        if (kv.first == slot.first) ps = &kv.second;
      if (!ps) throw ConfigError("layer '" + ls.prefix + "': block '" + ls.block.kind + "' needs a '" + slot.first + "' part");
      built.emplace_back(slot.first, build_part(slot.second, *ps, join(ls.prefix, ps->name)));
    }
    blocks.push_back(std::dynamic_pointer_cast<BlockPart>(build_part("block", ls.block, ls.prefix, built)));
  }
  final_norm = std::dynamic_pointer_cast<NormPart>(build_part("norm", spec.final_norm, spec.final_norm.name));
  head = std::dynamic_pointer_cast<HeadPart>(build_part("head", spec.lm_head, spec.lm_head.name));
  finish_construction();
}

Model::Model(const ModelSpec& meta, std::shared_ptr<Part> emb, std::vector<std::shared_ptr<Part>> blks,
             std::shared_ptr<Part> norm, std::shared_ptr<Part> hd)
    : spec(meta) {
  embedding = std::dynamic_pointer_cast<EmbeddingPart>(emb);
  for (auto& b : blks) {
    auto bp = std::dynamic_pointer_cast<BlockPart>(b);
    if (!bp) throw ConfigError("a layer's part is not a block arrangement");
    blocks.push_back(bp);
  }
  final_norm = std::dynamic_pointer_cast<NormPart>(norm);
  head = std::dynamic_pointer_cast<HeadPart>(hd);
  finish_construction();
}

void Model::finish_construction() {
  if (!embedding || !final_norm || !head) throw ConfigError("a model needs an embedding, a final norm and a head");
  run_order = spec.run_order();
  if (spec.layers.size() != blocks.size()) {
    // built from parts: the spec carries one (empty) layer record per block for cache_from
    if (spec.layers.empty()) spec.layers.resize(blocks.size());
    else throw ConfigError("the spec lists " + std::to_string(spec.layers.size()) + " layers, " + std::to_string(blocks.size()) + " were built");
    run_order = spec.run_order();
  }
  for (int i : run_order)
    if (i < 0 || i >= (int)blocks.size())
      throw ConfigError("schedule names layer " + std::to_string(i) + ", but there are " + std::to_string(blocks.size()));
  group_cache();
}

void Model::walk(const std::function<void(Part&)>& fn) const {
  embedding->walk(fn);
  for (const auto& b : blocks) b->walk(fn);
  final_norm->walk(fn);
  head->walk(fn);
}

bool Model::has_foreign_parts() const {
  bool any = false;
  walk([&](Part& p) { any = any || p.foreign_id != 0; });
  return any;
}

// Every checkpoint tensor the model asks for, in a fixed order.  A name asked for twice (a tied
// head) must be asked for with one shape; it is optional only if every asker says so.
std::vector<std::pair<std::string, TensorNeed>> Model::tensors() const {
  std::vector<std::pair<std::string, TensorNeed>> out;
  std::map<std::string, size_t> index;
  walk([&](Part& p) {
    for (auto& kv : p.tensors()) {
      auto it = index.find(kv.first);
      if (it == index.end()) {
        index[kv.first] = out.size();
        out.push_back(kv);
        continue;
      }
      TensorNeed& old = out[it->second].second;
      if (old.shape != kv.second.shape || old.role != kv.second.role)
        throw ConfigError("tensor '" + kv.first + "' is asked for with two shapes or roles");
      if (old.optional && !kv.second.optional) old = kv.second;
    }
  });
  return out;
}

// Give every run of a layer that keeps a cache a cache layer of its own, and gather cache layers
// with the same need into groups (one page id addresses a token's slot in every cache layer of
// its group).  A layer named twice in the run order computes different keys and values each time,
// so each run has its own cache layer.  A layer with `cache_from = j` keeps none: it reads what
// the latest earlier run of layer j wrote (the first run of j if none came earlier).
void Model::group_cache() {
  std::vector<CacheNeed> needs;
  std::vector<int> counts;
  bindings.assign(run_order.size(), {});
  std::map<int, std::vector<int>> runs_of;
  auto cached_parts = [](BlockPart& b) {
    std::vector<Part*> v;
    b.walk([&](Part& p) {
      if (p.has_cache()) v.push_back(&p);
    });
    return v;
  };
  for (size_t r = 0; r < run_order.size(); ++r) {
    const int i = run_order[r];
    runs_of[i].push_back((int)r);
    if (spec.layers[i].cache_from >= 0) continue;
    for (Part* p : cached_parts(*blocks[i])) {
      const CacheNeed need = p->cache_need();
      int g = -1;
      for (size_t k = 0; k < needs.size(); ++k)
        if (needs[k] == need) g = (int)k;
      if (g < 0) {
        g = (int)needs.size();
        needs.push_back(need);
        counts.push_back(0);
      }
      bindings[r][p] = {g, counts[g]++};
    }
  }
  for (size_t r = 0; r < run_order.size(); ++r) {
    const int i = run_order[r];
    const int j = spec.layers[i].cache_from;
    if (j < 0) continue;
    if (!runs_of.count(j) || spec.layers[j].cache_from >= 0)
      throw ConfigError("layer " + std::to_string(i) + " reads the cache of layer " + std::to_string(j) + ", which keeps none");
    int src = runs_of[j][0];
    for (int q : runs_of[j])
      if (q < (int)r) src = q;
    const auto theirs_parts = cached_parts(*blocks[j]);
    const auto mine = cached_parts(*blocks[i]);
    if (theirs_parts.size() != mine.size())
      throw ConfigError("layer " + std::to_string(i) + " cannot read the cache of layer " + std::to_string(j) +
                        ": they keep different numbers of caches");
    for (size_t k = 0; k < mine.size(); ++k) bindings[r][mine[k]] = bindings[src].at(theirs_parts[k]);
  }
  cache_groups.clear();
  for (size_t k = 0; k < needs.size(); ++k) cache_groups.emplace_back(needs[k], counts[k]);
}

// ------------------------------------------------------------------------------------ loading
void Model::load_from(WeightSource& src, const std::string& dt, bool to_host) {
  const DType matrix = dtype_from_name(dt);
  src.matrix_dtype = matrix;
  src.to_host = to_host;
  std::unique_ptr<HostMemoryScope> scope;
  if (to_host) scope.reset(new HostMemoryScope());
  storage_.clear();
  size_t n_parts = 0;
  walk([&](Part&) { ++n_parts; });
  storage_.reserve(8 * n_parts + 64);        // the tensors handed out point into these; they must not move
  src.owner = &storage_;
  walk([&](Part& p) { p.load(src); });
  src.finish();
  dtype = to_host ? "" : dt;
}

void Model::load_folder(const std::string& dir, const std::string& dt, bool to_host) {
  dtype_from_name(dt);
  auto src = make_folder_source(dir);
  check_source(dir, tensors(), *src);
  load_from(*src, dt, to_host);
}

void Model::load_tensors(const std::vector<HostTensor>& ts, bool on_device, const std::string& dt, const std::string& where,
                         bool to_host) {
  dtype_from_name(dt);
  auto src = make_tensors_source(ts, on_device);
  check_source(where, tensors(), *src);
  load_from(*src, dt, to_host);
}

void Model::load_random(uint64_t seed, const std::string& dt) {
  dtype_from_name(dt);
  Ops ops;
  auto src = make_random_source(tensors(), seed, ops);
  load_from(*src, dt, false);
}

std::shared_ptr<Model> Model::from_folder(const std::string& dir, const std::string& dtype) {
  auto model = std::make_shared<Model>(spec_from_config(read_config_json(dir)));
  model->load_folder(dir, dtype);
  return model;
}

std::shared_ptr<Model> Model::from_config(const Json& config, uint64_t seed, const std::string& dtype) {
  auto model = std::make_shared<Model>(spec_from_config(config));
  model->load_random(seed, dtype);
  return model;
}

// config.json and model.safetensors with random weights drawn on the host: matrices and the
// embedding ~ N(0, 0.02); every RMSNorm weight = 1 + N(0, 0.1), so that a norm weight that is
// forgotten or put in the wrong place changes the logits.  The distribution of each tensor is the
// one its part declares.  Matrices are stored as `store_dtype`, vectors in float32; optional
// tensors (the duplicate of a tied head) are not written.
void Model::write_random_folder(const std::string& dir, const Json& config_out, uint64_t seed, const std::string& store_dtype) {
  const DType matrix = dtype_from_name(store_dtype);
  mkdir(dir.c_str(), 0777);
  std::vector<std::vector<uint8_t>> blobs;
  std::vector<HostTensor> out;
  for (const auto& kv : tensors()) {
    if (kv.second.optional) continue;
    const DType dt = kv.second.role == TensorNeed::Matrix ? matrix : kv.second.role == TensorNeed::Vector ? DType::F32 : DType::I32;
    int64_t n = 1;
    for (int64_t s : kv.second.shape) n *= s;
    blobs.emplace_back((size_t)n * dtype_size(dt));
    host_random(kv.second, tensor_seed(seed, kv.first), dt, blobs.back().data());
    out.push_back(HostTensor{kv.first, dt, kv.second.shape, blobs.back().data()});
  }
  Json cfg = config_out;
  cfg.set("torch_dtype", store_dtype);
  {
    std::ofstream f(dir + "/config.json");
    if (!f) throw FileError(dir + "/config.json: cannot be written");
    f << cfg.dump() << "\n";
  }
  write_safetensors(dir + "/model.safetensors", out, {{"format", "pt"}, {"seed", std::to_string(seed)}});
}

void Model::write_folder(const std::string& dir, const Json& config, uint64_t seed, const std::string& store_dtype) {
  Model model(spec_from_config(config));
  // a typed configuration writes itself back with its defaults filled in
  const Json out = typed_config(config).at("config");
  model.write_random_folder(dir, out, seed, store_dtype);
}

}  // namespace tinyinfer
