// The step function.
//
// `Engine::step(entries)` takes a batch of (request, its next tokens, the places whose logits are
// wanted): portions of prompts beside single decoded tokens, cut anywhere.  It reserves pages,
// runs exactly the tokens it is given as one flat batch against the cache that earlier steps
// left, and returns the logits at the wanted places.  The reference's `Inference::forward` has
// the same shape (flat tokens with a position and a sequence id each, logits for chosen rows:
// /root/reference/src/inference.h:26-42, src/inference.cu:178-265) over a non-paged cache; its
// kernel sequence is src/inference.cu:28-72, its graphs src/inference.cu:267-295.
//
// Per-step metadata (tokens, positions, block-table rows, output rows, the parts' own lists) is
// packed into one pinned host buffer and reaches the device in one copy.  What a part needs beyond
// the common lists it plans itself (`Part::plan`): the engine knows no kernel's tiling.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstring>
#include <list>
#include <set>

#include "../include/inference.h"

namespace tinyinfer {

namespace {
void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw EngineError(std::string(what) + ": " + hipGetErrorString(e));
}
const int STEP_GRAPH_AFTER = 2;    // a step's shape is captured when it comes for this many times ...
                                   // ... and EngineOptions::max_step_graphs such graphs are kept
}  // namespace

int* StepPlan::ints(const std::string& key, size_t n) {
  List& l = lists_[key];
  l.n = n;
  l.host.assign(n, 0);
  return l.host.data();
}

struct Engine::Impl {
  struct Graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    DeviceBuffer meta;
    Workspace ws;
    Tensor logits;
    ~Graph() {
      if (exec) (void)hipGraphExecDestroy(exec);
      if (graph) (void)hipGraphDestroy(graph);
    }
  };
  // one step, between prepare and finish
  struct Prepared {
    std::unique_ptr<StepContext> ctx;
    StepPlan plan;
    std::vector<int64_t> requests;
    std::vector<int> n_tokens;
    std::vector<int64_t> admitted_here;
    bool decode_fast = false;
  };

  Engine& e;
  std::vector<Part*> parts;                 // every part, once
  // storage behind the cache manager: per group, [cache layer][page][K|V][kv head][row][hd] of the
  // compute dtype, or [cache layer][slot][...] float32
  std::vector<DeviceBuffer> storage;
  std::vector<size_t> layer_bytes;
  Workspace ws;
  // metadata: two pinned host buffers take turns, one device buffer
  int* meta_host[2] = {nullptr, nullptr};
  hipEvent_t meta_event[2] = {nullptr, nullptr};
  bool meta_used[2] = {false, false};
  size_t meta_cap = 0;
  DeviceBuffer meta_dev;
  int turn = 0;
  hipStream_t stream = nullptr;
  hipStream_t capture_stream = nullptr;
  std::map<std::string, std::unique_ptr<Graph>> graphs;
  std::list<std::string> shape_order;       // shape keys, least recently used first
  std::map<std::string, int> shapes_seen;
  bool foreign = false;
  size_t max_step_graphs = 32;
  DeviceBuffer feedback;                    // int32 [max_requests]: ids a sampler left for the next step
  int feedback_rows = 0;

  // a token is an id of the vocabulary, or names a row of the feedback buffer
  bool token_ok(int t, int64_t V) const { return t >= 0 ? t < V : -1 - t < feedback_rows; }

  explicit Impl(Engine& e) : e(e) {}
  ~Impl() {
    (void)hipStreamSynchronize(stream);
    graphs.clear();
    for (int i = 0; i < 2; ++i) {
      if (meta_host[i]) (void)hipHostFree(meta_host[i]);
      if (meta_event[i]) (void)hipEventDestroy(meta_event[i]);
    }
    if (capture_stream) (void)hipStreamDestroy(capture_stream);
  }

  void meta_buffers(size_t n_ints) {
    if (meta_cap >= n_ints) return;
    hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    const size_t cap = std::max<size_t>(4096, n_ints + n_ints / 2);
    for (int i = 0; i < 2; ++i) {
      if (meta_host[i]) (void)hipHostFree(meta_host[i]);
      hip_check(hipHostMalloc((void**)&meta_host[i], cap * 4, hipHostMallocDefault), "hipHostMalloc");
      if (!meta_event[i]) hip_check(hipEventCreateWithFlags(&meta_event[i], hipEventDisableTiming), "hipEventCreate");
      meta_used[i] = false;
    }
    meta_dev = DeviceBuffer(cap * 4);
    meta_cap = cap;
  }

  void clear_slots() {
    CacheManager& c = *e.cache;
    if (c.slots_to_clear.empty()) return;
    for (int g = 0; g < c.num_groups(); ++g) {
      if (c.group_is_paged(g)) continue;
      const size_t slot_bytes = layer_bytes[g] / c.max_requests;
      for (int l = 0; l < c.group_layers(g); ++l)
        for (int s : c.slots_to_clear)
          e.ops.fill_zero((char*)storage[g].data() + (size_t)l * layer_bytes[g] + (size_t)s * slot_bytes, slot_bytes);
    }
    c.slots_to_clear.clear();
  }

  // The common step, checked and reserved in one pass: every entry is one token of a request that
  // is admitted already.  False for any other step (nothing has been done then).
  bool reserve_decode_step(const std::vector<StepEntry>& entries, std::vector<int>& starts) {
    CacheManager& c = *e.cache;
    const int64_t V = e.model->spec.vocab_size;
    std::vector<int64_t> reqs;
    reqs.reserve(entries.size());
    for (const auto& en : entries) {
      if (en.tokens.size() != 1 || !c.has(en.request) || c.reserved(en.request) != c.length(en.request)) return false;
      if (!token_ok(en.tokens[0], V)) return false;                      // the general path names the token
      for (int w : en.want)
        if (w != 0) return false;
      if (en.start >= 0 && en.start != c.length(en.request)) return false;
      reqs.push_back(en.request);
    }
    std::set<int64_t> distinct(reqs.begin(), reqs.end());
    if (distinct.size() != reqs.size()) return false;                    // the general path names the request
    try {
      starts = c.reserve_one_each(reqs);
    } catch (const OutOfPages&) {
      throw;
    } catch (const CacheError& err) {
      throw EngineError(err.what());
    }
    return true;
  }

  std::unique_ptr<Prepared> prepare(const std::vector<StepEntry>& entries, Graph* graph, bool capturing) {
    if (entries.empty()) throw EngineError("a step needs at least one entry");
    CacheManager& c = *e.cache;
    const int64_t V = e.model->spec.vocab_size;
    auto p = std::unique_ptr<Prepared>(new Prepared());
    std::vector<int> starts;
    p->decode_fast = reserve_decode_step(entries, starts);
    int64_t M = 0, n_want = 0;
    const size_t R = entries.size();
    if (!p->decode_fast) {
      std::set<int64_t> seen;
      for (const auto& en : entries) {
        const std::string name = std::to_string(en.request);
        if (!seen.insert(en.request).second) throw EngineError("request " + name + " appears twice in one step");
        if (en.tokens.empty()) throw EngineError("request " + name + ": an entry needs at least one token");
        for (int t : en.tokens)
          if (!token_ok(t, V))
            throw EngineError("request " + name + ": token id " + std::to_string(t) + " is outside the vocabulary [0, " +
                              std::to_string(V) + ")" +
                              (t < 0 && feedback_rows ? " and names no row of the token feedback (" + std::to_string(feedback_rows) + " rows)" : ""));
        for (int w : en.want)
          if (w < 0 || w >= (int)en.tokens.size())
            throw EngineError("request " + name + ": wanted place " + std::to_string(w) + " is outside its " +
                              std::to_string(en.tokens.size()) + " tokens");
        if (en.start >= 0 && en.start != (c.has(en.request) ? c.length(en.request) : 0))
          throw EngineError("request " + name + ": the entry starts at position " + std::to_string(en.start) + " but the cache holds " +
                            std::to_string(c.has(en.request) ? c.length(en.request) : 0) + " tokens of it");
      }
      // all or nothing: see that every group can cover every entry before taking a page
      int n_new = 0;
      for (const auto& en : entries) n_new += c.has(en.request) ? 0 : 1;
      if (n_new > c.num_free_slots())
        throw EngineError(std::to_string(n_new) + " new requests but only " + std::to_string(c.num_free_slots()) + " free request slots");
      for (int g : c.paged_groups()) {
        int need = 0;
        for (const auto& en : entries) {
          const bool known = c.has(en.request);
          const int upto = (known ? c.reserved(en.request) : 0) + (int)en.tokens.size();
          if (upto > c.max_seq)
            throw EngineError("request " + std::to_string(en.request) + ": " + std::to_string(upto) + " tokens exceed max_seq = " +
                              std::to_string(c.max_seq));
          need += c.pages_to_cover(g, en.request, known, upto);
        }
        if (need > c.pool(g).num_free())
          throw OutOfPages("the step needs " + std::to_string(need) + " new pages in cache group " + std::to_string(g) + ", " +
                           std::to_string(c.pool(g).num_free()) + " are free");
      }
      for (const auto& en : entries) {
        if (!c.has(en.request)) {
          c.admit(en.request);
          p->admitted_here.push_back(en.request);
        }
        c.reserve(en.request, (int)en.tokens.size());
      }
    }
    for (const auto& en : entries) {
      M += (int64_t)en.tokens.size();
      n_want += (int64_t)en.want.size();
      p->requests.push_back(en.request);
      p->n_tokens.push_back((int)en.tokens.size());
    }
    // the pages are taken: whatever fails from here on (a part's plan, a buffer that cannot be had)
    // gives them back before the error leaves
    try {
      fill(*p, entries, starts, M, n_want, graph, capturing);
    } catch (...) {
      undo(*p);
      throw;
    }
    return p;
  }

  void fill(Prepared& prepared, const std::vector<StepEntry>& entries, const std::vector<int>& starts, int64_t M, int64_t n_want,
            Graph* graph, bool capturing) {
    Prepared* p = &prepared;
    CacheManager& c = *e.cache;
    const size_t R = entries.size();
    clear_slots();

    Workspace& work = graph ? graph->ws : ws;
    p->ctx.reset(new StepContext(e.ops, work, e.act_dtype));
    StepContext& ctx = *p->ctx;
    ctx.engine = &e;
    ctx.M = M;
    ctx.n_out = n_want;
    ctx.entries.reserve(R);
    bool decode_only = true;
    int row0 = 0, max_context = 0;
    for (size_t i = 0; i < R; ++i) {
      const auto& en = entries[i];
      const int n = (int)en.tokens.size();
      const int start = p->decode_fast ? starts[i] : c.length(en.request);
      ctx.entries.push_back({row0, n, start, c.slot(en.request)});
      decode_only = decode_only && n == 1;
      max_context = std::max(max_context, start + n);
      row0 += n;
    }
    ctx.decode_only = decode_only;
    ctx.max_context = max_context;

    // what the parts add to the step's metadata
    StepPlan& plan = p->plan;
    plan.entries_ = &ctx.entries;
    plan.M_ = M;
    plan.decode_only_ = decode_only;
    plan.max_seq_ = e.max_seq;
    plan.sized_for_longest_ = capturing;
    for (Part* part : parts) part->plan(plan);
    ctx.plan = &plan;

    // layout: tokens | positions | slots | out_rows | entries [R,4] | the parts' lists | tables
    const int W = c.table_width;
    const size_t o_tok = 0, o_pos = M, o_slot = 2 * M, o_out = 3 * M, o_ent = o_out + n_want;
    size_t off = o_ent + 4 * R;
    for (auto& kv : plan.lists_) {
      kv.second.offset = off;
      off += kv.second.n;
    }
    const size_t o_tab = off;
    const size_t total = o_tab + c.paged_groups().size() * R * W;
    int* host;
    int* dev;
    int my_turn = -1;
    meta_buffers(total);
    my_turn = turn;
    turn ^= 1;
    if (meta_used[my_turn]) hip_check(hipEventSynchronize(meta_event[my_turn]), "hipEventSynchronize");
    host = meta_host[my_turn];
    if (graph) {
      if (!graph->meta.data()) graph->meta = DeviceBuffer((total + 64) * 4);
      if (graph->meta.bytes() < total * 4) throw EngineError("the fixed metadata buffer is too small for this step");
      dev = (int*)graph->meta.data();
    } else {
      dev = (int*)meta_dev.data();
    }
    int* out_rows = host + o_out;
    size_t k = 0;
    for (size_t i = 0; i < R; ++i) {
      const auto& en = entries[i];
      const EntryRecord& rec = ctx.entries[i];
      memcpy(host + o_tok + rec.row0, en.tokens.data(), (size_t)rec.n_tokens * 4);
      for (int t = 0; t < rec.n_tokens; ++t) {
        host[o_pos + rec.row0 + t] = rec.start + t;
        host[o_slot + rec.row0 + t] = (int)i;
      }
      for (int w : en.want) out_rows[k++] = rec.row0 + w;
      memcpy(host + o_ent + 4 * i, &rec, 16);
    }
    for (const auto& kv : plan.lists_)
      if (kv.second.n) memcpy(host + kv.second.offset, kv.second.host.data(), kv.second.n * 4);
    size_t gi = 0;
    for (int g : c.paged_groups()) {
      int* base = host + o_tab + gi * R * W;
      for (size_t i = 0; i < R; ++i) memcpy(base + i * W, c.table_row(g, entries[i].request), (size_t)W * 4);
      ++gi;
    }
    hip_check(hipMemcpyAsync(dev, host, total * 4, hipMemcpyHostToDevice, stream), "hipMemcpyAsync(step metadata)");
    hip_check(hipEventRecord(meta_event[my_turn], stream), "hipEventRecord");
    meta_used[my_turn] = true;

    ctx.meta_dev = dev;
    ctx.tokens = dev + o_tok;
    ctx.fed_tokens = (const int*)feedback.data();
    ctx.n_fed_tokens = feedback_rows;
    ctx.positions = dev + o_pos;
    ctx.slots = dev + o_slot;
    ctx.out_rows = n_want ? dev + o_out : nullptr;
    ctx.entry_meta = dev + o_ent;
    ctx.views.assign(c.num_groups(), Ops::CacheView());
    gi = 0;
    for (int g : c.paged_groups()) {
      ctx.views[g].table = dev + o_tab + gi * R * W;
      ctx.views[g].table_width = W;
      ctx.views[g].page_size = e.page_size;
      ++gi;
    }
  }

  // The model over the step's tokens: embedding, the layers in run order, then final norm and
  // head on the wanted rows only.
  Tensor run(StepContext& ctx) {
    Model& m = *e.model;
    Tensor x = ctx.buf("x", DType::F32, {ctx.M, m.spec.hidden_size});
    m.embedding->forward(ctx, x);
    for (size_t r = 0; r < m.run_order.size(); ++r) {
      ctx.run = (int)r;
      BlockPart& b = *m.blocks[m.run_order[r]];
      if (!b.reads_through_ops()) ctx.ops.flush();
      b.forward(ctx, x);
    }
    if (!ctx.out_rows) {
      ctx.ops.flush();
      return Tensor();
    }
    if (!m.final_norm->reads_through_ops() || !m.head->reads_through_ops()) ctx.ops.flush();
    Rows h = m.final_norm->forward(ctx, x, ctx.out_rows, ctx.n_out, false);
    Tensor logits = m.head->forward(ctx, h);
    ctx.ops.flush();
    return logits;
  }

  void finish(Prepared& p) {
    if (p.decode_fast) {
      e.cache->commit_one_each(p.requests);
    } else {
      for (size_t i = 0; i < p.requests.size(); ++i) e.cache->commit(p.requests[i], p.n_tokens[i]);
    }
    ++e.steps_run;
  }

  // a step that failed after its reservation leaves the cache as it found it
  void undo(Prepared& p) {
    try {
      e.ops.flush();
    } catch (...) {
    }
    for (int64_t r : p.requests) e.cache->rollback(r);
    for (int64_t r : p.admitted_here)
      if (e.cache->has(r)) e.cache->release(r);
  }

  Tensor step(const std::vector<StepEntry>& entries) {
    auto p = prepare(entries, nullptr, false);
    Tensor logits;
    try {
      logits = run(*p->ctx);
    } catch (...) {
      undo(*p);
      throw;
    }
    finish(*p);
    return logits;
  }

  static std::string shape_key(const std::vector<StepEntry>& entries, bool& decode) {
    decode = true;
    for (const auto& en : entries) decode = decode && en.tokens.size() == 1 && en.want.size() == 1 && en.want[0] == 0;
    if (decode) return "d" + std::to_string(entries.size());
    std::string key = "s";
    for (const auto& en : entries) {
      key += std::to_string(en.tokens.size()) + ":";
      for (int w : en.want) key += std::to_string(w) + ",";
      key += ";";
    }
    return key;
  }

  Tensor capture(const std::vector<StepEntry>& entries, const std::string& key, bool decode) {
    std::unique_ptr<Graph> g(new Graph());
    auto p = prepare(entries, g.get(), true);
    try {
      // a first run outside the graph: it computes this step's result and makes every workspace
      // buffer the graph will use
      run(*p->ctx);
      hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
      if (!capture_stream) hip_check(hipStreamCreate(&capture_stream), "hipStreamCreate");
      g->ws.frozen = true;
      e.ops.set_stream(capture_stream);
      hipError_t err = hipStreamBeginCapture(capture_stream, hipStreamCaptureModeRelaxed);
      if (err == hipSuccess) {
        try {
          g->logits = run(*p->ctx);
        } catch (...) {
          hipGraph_t dead = nullptr;
          (void)hipStreamEndCapture(capture_stream, &dead);
          if (dead) (void)hipGraphDestroy(dead);
          e.ops.set_stream(stream);
          throw;
        }
        err = hipStreamEndCapture(capture_stream, &g->graph);
      }
      e.ops.set_stream(stream);
      hip_check(err, "capturing the step in a HIP graph");
      hip_check(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    } catch (...) {
      undo(*p);
      throw;
    }
    // capture records, it does not run: the first run above already wrote this step's keys, values
    // and logits, and a replay would write the same again
    finish(*p);
    Tensor logits = g->logits;
    if (!decode) {
      while (!shape_order.empty() && shape_order.size() >= max_step_graphs) {
        graphs.erase(shape_order.front());
        shape_order.pop_front();
      }
      shape_order.push_back(key);
    }
    graphs[key] = std::move(g);
    return logits;
  }

  Tensor step_graph(const std::vector<StepEntry>& entries) {
    if (foreign) return step(entries);      // parts outside the library launch on streams of their own
    bool decode = false;
    const std::string key = shape_key(entries, decode);
    auto it = graphs.find(key);
    if (it == graphs.end()) {
      if (!decode) {
        if (shapes_seen.size() > 4096) shapes_seen.clear();
        const int seen = ++shapes_seen[key];
        if (seen < STEP_GRAPH_AFTER) return step(entries);
        shapes_seen.erase(key);
      }
      return capture(entries, key, decode);
    }
    if (!decode) {
      shape_order.remove(key);
      shape_order.push_back(key);
    }
    Graph& g = *it->second;
    auto p = prepare(entries, &g, false);
    try {
      hip_check(hipGraphLaunch(g.exec, stream), "hipGraphLaunch");
    } catch (...) {
      undo(*p);
      throw;
    }
    finish(*p);
    return g.logits;
  }
};

// -------------------------------------------------------------------------------- the context
std::pair<int, int> StepContext::binding(const Part* part) const {
  if (!engine) throw EngineError("a part that keeps a cache cannot run outside an engine");
  const auto& b = engine->model->bindings[run];
  auto it = b.find(part);
  if (it == b.end()) throw EngineError("the part has no cache in this run of its layer");
  return it->second;
}
Tensor StepContext::kv_pool(int group, int layer) const {
  if (!engine) throw EngineError("no engine: no cache");
  return engine->kv_pool(group, layer);
}
Ops::CacheView StepContext::cache_view(int group) const { return views.at(group); }
Tensor StepContext::state(int group, int layer) const {
  if (!engine) throw EngineError("no engine: no state");
  return engine->state(group, layer);
}
const int* StepContext::planned(const std::string& key) const {
  if (!plan) return nullptr;
  auto it = plan->lists_.find(key);
  if (it == plan->lists_.end() || it->second.n == 0) return nullptr;
  return meta_dev + it->second.offset;
}
size_t StepContext::planned_size(const std::string& key) const {
  if (!plan) return 0;
  auto it = plan->lists_.find(key);
  return it == plan->lists_.end() ? 0 : it->second.n;
}
int64_t StepContext::value(const std::string& key, int64_t fallback) const {
  if (!plan) return fallback;
  auto it = plan->values_.find(key);
  return it == plan->values_.end() ? fallback : it->second;
}

// ------------------------------------------------------------------------------------- engine
static std::string engine_dtype(const Model& m, const EngineOptions& o) {
  const std::string dt = o.dtype.empty() ? m.dtype : o.dtype;
  if (dt.empty()) throw EngineError("the model has no weights yet: load them before making an engine");
  dtype_from_name(dt);
  if (!m.dtype.empty() && m.dtype != dt)
    throw EngineError("the model's weights were loaded as " + m.dtype + ", the engine is asked to run in " + dt);
  return dt;
}

Engine::Engine(std::shared_ptr<Model> model_, const EngineOptions& o)
    : model(std::move(model_)), ops(o.stream), act_dtype(dtype_from_name(engine_dtype(*model, o))),
      dtype(engine_dtype(*model, o)), page_size(o.page_size),
      max_seq([&] {
        if (o.page_size <= 0) throw EngineError("page_size must be positive");
        int64_t pages = o.num_pages;
        if (pages <= 0) {
          if (o.max_tokens <= 0) throw EngineError("give the cache pool a size: max_tokens or num_pages");
          pages = (o.max_tokens + o.page_size - 1) / o.page_size;
        }
        int64_t ms = o.max_seq;
        if (ms <= 0) {
          ms = pages * o.page_size;
          if (model->spec.max_position_embeddings > 0) ms = std::min(ms, model->spec.max_position_embeddings);
        }
        return (int)ms;
      }()),
      num_pages(o.num_pages > 0 ? o.num_pages : (o.max_tokens + o.page_size - 1) / o.page_size),
      impl_(new Impl(*this)) {
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev <= 0)
    throw EngineError("no GPU: this engine runs on an AMD GPU only (there is no CPU path)");
  impl_->stream = (hipStream_t)o.stream;
  impl_->max_step_graphs = (size_t)std::max(1, o.max_step_graphs);
  cache.reset(new CacheManager(model->cache_groups, page_size, (int)num_pages, o.max_requests, max_seq, o.page_scatter_window));
  // the tensors behind the cache manager.  Within a page the keys of a kv head lie [row][head_dim]
  // (a score sums over head_dim) and the values transposed, [head_dim][row] (the mix sums over
  // rows): each is contiguous along the dimension the matrix cores reduce over.
  for (const auto& g : model->cache_groups) {
    size_t per_layer;
    if (g.first.kind == CacheNeed::PagedKV) {
      per_layer = (size_t)num_pages * 2 * g.first.kv_heads * page_size * g.first.head_dim * dtype_size(act_dtype);
    } else if (g.first.kind == CacheNeed::PagedRows) {
      if (g.first.row_shape.empty() || g.first.row_shape.size() > 2)
        throw EngineError("a paged cache of rows needs a row shape of one or two dimensions");
      size_t n = 1;
      for (int64_t s : g.first.row_shape) n *= (size_t)s;
      per_layer = (size_t)num_pages * page_size * n * (g.first.rows_f32 ? 4 : dtype_size(act_dtype));
    } else {
      size_t n = 1;
      for (int64_t s : g.first.state_shape) n *= (size_t)s;
      per_layer = (size_t)o.max_requests * n * 4;
    }
    impl_->layer_bytes.push_back(per_layer);
    impl_->storage.emplace_back(per_layer * (size_t)g.second);
    if (g.first.kind == CacheNeed::State) ops.fill_zero(impl_->storage.back().data(), per_layer * (size_t)g.second);
  }
  model->walk([&](Part& p) {
    impl_->parts.push_back(&p);
    p.prepare(ops, max_seq);          // tables that depend on the longest sequence
  });
  impl_->foreign = model->has_foreign_parts();
  if (!impl_->foreign) {
    impl_->feedback_rows = cache->max_requests;
    impl_->feedback = DeviceBuffer((size_t)impl_->feedback_rows * 4);
    ops.fill_zero(impl_->feedback.data(), (size_t)impl_->feedback_rows * 4);
  }
  synchronize();
}

Engine::~Engine() {}

Tensor Engine::step(const std::vector<StepEntry>& entries) { return impl_->step(entries); }
Tensor Engine::step_graph(const std::vector<StepEntry>& entries) { return impl_->step_graph(entries); }
void Engine::release(int64_t request) { cache->release(request); }
int* Engine::token_feedback() { return (int*)impl_->feedback.data(); }
int Engine::feedback_rows() const { return impl_->feedback_rows; }
void Engine::synchronize() { hip_check(hipStreamSynchronize(impl_->stream), "hipStreamSynchronize"); }
void Engine::logits_to_host(const Tensor& logits, float* out) {
  if (!logits.defined()) return;
  hip_check(hipMemcpyAsync(out, logits.data, logits.bytes(), hipMemcpyDeviceToHost, impl_->stream), "hipMemcpyAsync");
  synchronize();
}
size_t Engine::num_graphs() const { return impl_->graphs.size(); }
std::vector<std::string> Engine::graph_keys() const {
  std::vector<std::string> keys;
  for (const auto& kv : impl_->graphs) keys.push_back(kv.first);
  return keys;
}
size_t Engine::cache_bytes() const {
  size_t n = 0;
  for (const auto& b : impl_->storage) n += b.bytes();
  return n;
}
Tensor Engine::kv_pool(int group, int layer) const {
  const auto& g = model->cache_groups.at(group);
  if (!g.first.paged()) throw EngineError("cache group " + std::to_string(group) + " has no pages");
  if (layer < 0 || layer >= g.second) throw EngineError("cache group " + std::to_string(group) + " has no layer " + std::to_string(layer));
  if (g.first.kind == CacheNeed::PagedRows) {
    std::vector<int64_t> shape = {num_pages, (int64_t)page_size};
    for (int64_t s : g.first.row_shape) shape.push_back(s);
    Tensor t((char*)impl_->storage[group].data() + (size_t)layer * impl_->layer_bytes[group],
             g.first.rows_f32 ? DType::F32 : act_dtype, {shape[0], shape[1], shape[2]});
    if (shape.size() == 4) t = Tensor(t.data, t.dtype, {shape[0], shape[1], shape[2], shape[3]});
    return t;
  }
  return Tensor((char*)impl_->storage[group].data() + (size_t)layer * impl_->layer_bytes[group], act_dtype,
                {num_pages, 2 * (int64_t)g.first.kv_heads, (int64_t)page_size, (int64_t)g.first.head_dim});
}
Tensor Engine::state(int group, int layer) const {
  const auto& g = model->cache_groups.at(group);
  if (g.first.kind != CacheNeed::State) throw EngineError("cache group " + std::to_string(group) + " holds no state");
  if (layer < 0 || layer >= g.second) throw EngineError("cache group " + std::to_string(group) + " has no layer " + std::to_string(layer));
  std::vector<int64_t> shape = {(int64_t)cache->max_requests};
  for (int64_t s : g.first.state_shape) shape.push_back(s);
  if (shape.size() > 4) throw EngineError("per-request state of more than three dimensions is not served");
  return Tensor((char*)impl_->storage[group].data() + (size_t)layer * impl_->layer_bytes[group], DType::F32, shape);
}

}  // namespace tinyinfer
