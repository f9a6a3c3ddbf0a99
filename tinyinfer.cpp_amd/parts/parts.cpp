// The parts a model is put together from, and their registry by family and kind.
//
//   embedding "table"     x[m, :] = float(E[tok[m], :]), no scaling (/root/reference/src/inference.cu:14-24)
//   norm      "rmsnorm"   y = x * rsqrt(mean(x^2) + eps) * w, eps inside the root, the weight multiplies
//                         directly (/root/reference/src/cuda/rms_norm.cu:15-25)
//   pos       "rope_neox" half-split rotation over the whole head: pair (k, k + hd/2) turns by
//                         pos * theta^(-2k/hd) (/root/reference/src/cuda/attention.cu:38,64-74; the
//                         adjacent-pair variant is the mistake listed in docs/report.md:91)
//   mixer     "attention" causal grouped-query attention over the paged cache: fused q/k/v product, per-head
//                         RMSNorm of q and k with a weight shared by all heads (before rotation; v is left
//                         alone), rotation, cache write, head h reads kv head h / (heads / kv_heads), scores
//                         scaled by 1/sqrt(hd), output projection added into the residual
//                         (/root/reference/src/inference.cu:41-55; src/cuda/attention.cu:12-87,107-198)
//   ffn       "swiglu"    y = silu(h Wg^T) * (h Wu^T); x += y Wd^T, gate and up rows held as one matrix
//                         (/root/reference/src/inference.cu:60-65,155-160; src/cuda/ffn.cu:13-15)
//   block     "pre_norm"  x += mixer(norm1(x)); x += ffn(norm2(x)) (/root/reference/src/inference.cu:35-66)
//   head      "linear"    logits = h E_out^T with E_out the embedding itself or a matrix of its own
//                         (/root/reference/src/cuda/lm_head.cu:5-10; the reference is always tied, src/model.h:42)
//
// A part gets every size and constant as a parameter and never looks at the model it sits in.
#include <algorithm>
#include <cmath>
#include <mutex>

#include "../include/inference.h"

namespace tinyinfer {

std::vector<std::string> Part::child_slots() const {
  std::vector<std::string> names;
  const size_t n = children().size();
  for (size_t i = 0; i < n; ++i) names.push_back(std::to_string(i));
  return names;
}

void Part::walk(const std::function<void(Part&)>& fn) {
  fn(*this);
  for (const auto& c : children()) c->walk(fn);
}

static std::string join(const std::string& prefix, const std::string& name) {
  if (prefix.empty()) return name;
  if (name.empty()) return prefix;
  return prefix + "." + name;
}

// ----------------------------------------------------------------------------------- registry
namespace {
struct Registered {
  PartFactory factory;
  std::vector<std::pair<std::string, std::string>> slots;
};
std::mutex g_parts_mutex;
std::map<std::pair<std::string, std::string>, Registered>& table() {
  static std::map<std::pair<std::string, std::string>, Registered> t;
  return t;
}
const char* FAMILIES[] = {"embedding", "norm", "pos", "mixer", "ffn", "block", "head"};
void register_builtin_parts();
void ensure_builtins() {
  static std::once_flag once;
  std::call_once(once, register_builtin_parts);
}
int64_t param_int(const Json& p, const char* key) {
  const Json* v = p.find(key);
  if (!v || !v->is_number()) throw ConfigError(std::string("part parameter '") + key + "' is missing or not a number");
  return v->as_int();
}
double param_float(const Json& p, const char* key) {
  const Json* v = p.find(key);
  if (!v || !v->is_number()) throw ConfigError(std::string("part parameter '") + key + "' is missing or not a number");
  return v->as_double();
}
}  // namespace

void register_part(const std::string& family, const std::string& kind, PartFactory factory,
                   std::vector<std::pair<std::string, std::string>> slots) {
  bool ok = false;
  for (const char* f : FAMILIES) ok = ok || family == f;
  if (!ok) throw ConfigError("unknown part family '" + family + "'");
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  table()[{family, kind}] = Registered{std::move(factory), std::move(slots)};
}

bool part_registered(const std::string& family, const std::string& kind) {
  ensure_builtins();
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  return table().count({family, kind}) != 0;
}

std::vector<std::string> registered_parts(const std::string& family) {
  ensure_builtins();
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  std::vector<std::string> kinds;
  for (const auto& kv : table())
    if (kv.first.first == family) kinds.push_back(kv.first.second);
  return kinds;
}

std::vector<std::pair<std::string, std::string>> block_slots(const std::string& kind) {
  ensure_builtins();
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  auto it = table().find({"block", kind});
  if (it == table().end()) throw ConfigError("no block arrangement of kind '" + kind + "'");
  return it->second.slots;
}

std::shared_ptr<Part> build_part(const std::string& family, const PartSpec& spec, const std::string& prefix,
                                 const PartChildren& children) {
  ensure_builtins();
  PartFactory factory;
  {
    std::lock_guard<std::mutex> lock(g_parts_mutex);
    auto it = table().find({family, spec.kind});
    if (it == table().end()) {
      std::string have;
      for (const auto& kv : table())
        if (kv.first.first == family) have += (have.empty() ? "'" : ", '") + kv.first.second + "'";
      throw ConfigError("no " + family + " part of kind '" + spec.kind + "'; registered: [" + have + "]");
    }
    factory = it->second.factory;
  }
  std::shared_ptr<Part> part = factory(prefix, spec.params, children);
  if (!part) throw ConfigError("the factory of " + family + " '" + spec.kind + "' returned no part");
  if (family != part->family())
    throw ConfigError("the factory of " + family + " '" + spec.kind + "' returned a part of family '" + part->family() + "'");
  if (part->built_kind.empty()) {
    part->built_kind = spec.kind;
    part->built_from = spec.params;
  }
  return part;
}

// ------------------------------------------------------------------------------- built-in parts
namespace {

class Embedding final : public EmbeddingPart {
 public:
  Embedding(const std::string& prefix, int64_t vocab, int64_t dim) : EmbeddingPart(prefix), vocab(vocab), dim(dim) {}
  const char* kind_name() const override { return "table"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    n.shape = {vocab, dim};
    return {{join(prefix, "weight"), n}};
  }
  void load(WeightSource& src) override { weight = src.fetch(join(prefix, "weight"), tensors()[0].second); }
  void forward(StepContext& ctx, const Tensor& x) override { ctx.ops.embed(weight, ctx.tokens, ctx.M, x, ctx.fed_tokens, ctx.n_fed_tokens); }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t vocab, dim;
  Tensor weight;
};

// `tied`: 1 reads `tied_to`; 0 reads its own `weight`; -1 takes its own weight if the checkpoint
// holds one and `tied_to` otherwise.
class LMHead final : public HeadPart {
 public:
  LMHead(const std::string& prefix, int64_t vocab, int64_t dim, int tied, std::string tied_to)
      : HeadPart(prefix), vocab(vocab), dim(dim), tied(tied), tied_to(std::move(tied_to)) {}
  const char* kind_name() const override { return "linear"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed must, may;
    must.shape = may.shape = {vocab, dim};
    may.optional = true;
    const std::string own = join(prefix, "weight");
    if (tied == 0) return {{own, must}};
    // a checkpoint that still carries the duplicate is accepted
    return {{tied_to, must}, {own, may}};
  }
  void load(WeightSource& src) override {
    const std::string own = join(prefix, "weight");
    TensorNeed n;
    n.shape = {vocab, dim};
    if (tied == 0 || (tied < 0 && src.has(own))) weight = src.fetch(own, n);
    else weight = src.fetch(tied_to, n);      // the source hands out one copy per name: the embedding's
  }
  Tensor forward(StepContext& ctx, const Rows& h) override {
    const Tensor& rows = h.materialize(ctx.ops);
    Tensor logits = ctx.buf("head.logits", DType::F32, {rows.shape[0], vocab});
    ctx.ops.linear(rows, weight, logits, Ops::Store);
    return logits;
  }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t vocab, dim;
  int tied;
  std::string tied_to;
  Tensor weight;
};

class RMSNorm final : public NormPart {
 public:
  RMSNorm(const std::string& prefix, int64_t dim, double eps) : NormPart(prefix), dim(dim), eps((float)eps) {}
  const char* kind_name() const override { return "rmsnorm"; }
  bool can_be_lazy() const override { return true; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    n.shape = {dim};
    n.role = TensorNeed::Vector;
    n.a = 1.0;
    n.b = 0.1;
    return {{join(prefix, "weight"), n}};
  }
  void load(WeightSource& src) override { weight = src.fetch(join(prefix, "weight"), tensors()[0].second); }
  // x: f32 [M, dim].  With `rows` only those rows of x are read, in that order.  `lazy`: the
  // consumer feeds the result to one product and nothing else, so where a kernel can take the
  // norm in, the rows come back not yet computed.
  Rows forward(StepContext& ctx, const Tensor& x, const int* rows, int64_t n_rows, bool lazy) override {
    const int64_t n = rows ? n_rows : x.shape[0];
    Rows r;
    r.t = ctx.buf("norm.out", ctx.act_dtype, {n, dim});
    if (lazy && !rows && ctx.ops.can_fuse_norm(n, r.t.dtype)) {
      r.lazy = true;
      r.x = x;
      r.weight = weight;
      r.eps = eps;
      return r;
    }
    ctx.ops.rmsnorm(x, weight, eps, r.t, rows, n_rows);
    return r;
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t dim;
  float eps;
  Tensor weight;
};

// The inverse frequencies are built once on the host in double precision and rounded to float.
// `prepare(n)` tabulates cosine and sine for positions below n, on the host, from the angle in double
// precision (rounded to float only at the end): a 32-bit angle pos * inv_freq[k] is pos * 2^-23 off, 6e-4
// five thousand tokens in, and differently at every position, so that not only distances would count.
// Positions beyond the table (none that an engine serves) have the angle and its sine and cosine in
// 32-bit on the device, as /root/reference/src/cuda/rope.cu:20-22 has them everywhere.
//
// A table never changes and is never freed while anything may read it: captured graphs hold its
// address in their kernel arguments.  Parts with the same head size and base share the longest table
// made so far; an engine that needs a longer one makes a new table, and every part keeps each table
// it has ever handed out until the part itself goes (its model outlives the engines on it).
struct RopeTable {
  int head_dim = 0;
  double theta = 0;
  DeviceBuffer inv_freq, table;
  int table_len = 0;
};
std::mutex g_rope_mutex;
std::map<std::pair<int, double>, std::weak_ptr<RopeTable>>& rope_tables() {
  static std::map<std::pair<int, double>, std::weak_ptr<RopeTable>> m;
  return m;
}

class RotaryNeox final : public PositionPart {
 public:
  RotaryNeox(const std::string& prefix, int64_t head_dim, double theta) : PositionPart(prefix), head_dim((int)head_dim), theta(theta) {
    if (head_dim % 2) throw ConfigError("rotary: head_dim " + std::to_string(head_dim) + " must be even");
  }
  const char* kind_name() const override { return "rope_neox"; }
  // the table this part reads now (null before the first use)
  std::shared_ptr<RopeTable> current() const {
    std::lock_guard<std::mutex> lock(g_rope_mutex);
    return kept.empty() ? nullptr : kept.back();
  }
  // a table of at least `len` positions (0: the frequencies alone will do)
  std::shared_ptr<RopeTable> table_for(int len) {
    std::lock_guard<std::mutex> lock(g_rope_mutex);
    if (!kept.empty() && kept.back()->table_len >= len) return kept.back();
    auto& slot = rope_tables()[{head_dim, theta}];
    std::shared_ptr<RopeTable> t = slot.lock();
    if (!t || t->table_len < len) {
      t = std::make_shared<RopeTable>();
      t->head_dim = head_dim;
      t->theta = theta;
      const int half = head_dim / 2;
      std::vector<double> inv(half);
      std::vector<float> inv32(half);
      for (int k = 0; k < half; ++k) {
        inv[k] = std::pow(theta, -2.0 * k / head_dim);
        inv32[k] = (float)inv[k];
      }
      t->inv_freq = DeviceBuffer((size_t)half * 4);
      upload(t->inv_freq.data(), inv32.data(), (size_t)half * 4);
      if (len > 0) {
        std::vector<float> host((size_t)len * half * 2);
        for (int p = 0; p < len; ++p)
          for (int k = 0; k < half; ++k) {
            const double angle = (double)p * inv[k];
            host[((size_t)p * half + k) * 2] = (float)std::cos(angle);
            host[((size_t)p * half + k) * 2 + 1] = (float)std::sin(angle);
          }
        t->table = DeviceBuffer(host.size() * 4);
        upload(t->table.data(), host.data(), host.size() * 4);
        t->table_len = len;
      }
      slot = t;
    }
    kept.push_back(t);
    return t;
  }
  void prepare(Ops&, int max_seq) override { table_for(max_seq); }
  bool fused(Ops::Rotation& rot) const override {
    const std::shared_ptr<RopeTable> t = current();
    if (!t) return false;
    rot.inv_freq = (const float*)t->inv_freq.data();
    rot.table = (const float*)t->table.data();
    rot.table_len = t->table_len;
    return true;
  }
  void apply(StepContext& ctx, const Tensor& q, const Tensor& k) override {
    const Tensor inv = inv_freq_tensor(ctx.ops);
    ctx.ops.rope_neox(q, ctx.positions, inv);
    if (k.defined()) ctx.ops.rope_neox(k, ctx.positions, inv);
  }
  Tensor inv_freq_tensor(Ops&) { return Tensor(table_for(0)->inv_freq.data(), DType::F32, {head_dim / 2}); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    const std::shared_ptr<RopeTable> t = current();
    if (!t) return {};
    const int half = head_dim / 2;
    std::vector<std::pair<std::string, Tensor>> h = {{"inv_freq", Tensor(t->inv_freq.data(), DType::F32, {half})}};
    if (t->table_len) h.emplace_back("table", Tensor(t->table.data(), DType::F32, {t->table_len, half, 2}));
    return h;
  }
  static void upload(void* dst, const void* src, size_t bytes);
  int head_dim;
  double theta;
  std::vector<std::shared_ptr<RopeTable>> kept;     // oldest first; the last one is read
};

class SwiGLU final : public FeedForwardPart {
 public:
  SwiGLU(const std::string& prefix, int64_t hidden, int64_t intermediate)
      : FeedForwardPart(prefix), hidden(hidden), intermediate(intermediate) {}
  const char* kind_name() const override { return "swiglu"; }
  bool takes_lazy_norm() const override { return true; }      // h goes into one product and nowhere else
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed up, down;
    up.shape = {intermediate, hidden};
    down.shape = {hidden, intermediate};
    return {{join(prefix, "gate_proj.weight"), up}, {join(prefix, "up_proj.weight"), up},
            {join(prefix, "down_proj.weight"), down}};
  }
  void load(WeightSource& src) override {
    // gate and up go straight into one matrix [2F, H]: one product yields both
    w_gate_up = src.alloc(src.matrix_dtype, {2 * intermediate, hidden});
    src.fill(join(prefix, "gate_proj.weight"), w_gate_up.rows(0, intermediate));
    src.fill(join(prefix, "up_proj.weight"), w_gate_up.rows(intermediate, intermediate));
    w_down = src.alloc(src.matrix_dtype, {hidden, intermediate});
    src.fill(join(prefix, "down_proj.weight"), w_down);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor y = ctx.buf("ffn.y", ctx.act_dtype, {h.t.shape[0], intermediate});
    ctx.ops.linear(h, w_gate_up, y, Ops::SwiGLU);
    ctx.ops.linear(y, w_down, x, Ops::Add, /*may_defer=*/true);
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w_gate_up", w_gate_up}, {"w_down", w_down}}; }
  int64_t hidden, intermediate;
  Tensor w_gate_up, w_down;
};

const int PREFILL_TILE_Q = 128;      // query rows per work item of the tiled attention kernels
const int PREFILL_TILE_SMALL = 64;   // and of the kernel that pairs a tile of many keys with one of few

class Attention final : public MixerPart {
 public:
  Attention(const std::string& prefix, const Json& p, const PartChildren& children) : MixerPart(prefix) {
    hidden = param_int(p, "hidden");
    heads = (int)param_int(p, "heads");
    kv_heads = (int)param_int(p, "kv_heads");
    head_dim = (int)param_int(p, "head_dim");
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
      throw ConfigError("attention: heads " + std::to_string(heads) + " not a multiple of kv_heads " + std::to_string(kv_heads));
    // every attention kernel's range (float32 and bfloat16 alike): refused when the part is built, not at its first step
    if (head_dim < 16 || head_dim % 16 || head_dim > 256)
      throw ConfigError("attention: head_dim " + std::to_string(head_dim) +
                        " is not served: the attention kernels take head sizes in steps of 16 up to 256");
    qk_norm = p.has("qk_norm") ? p.at("qk_norm").as_bool() : true;
    eps = (float)(p.has("eps") ? p.at("eps").as_double() : 1e-6);
    window = p.has("window") ? (int)p.at("window").as_int() : 0;
    scale = p.has("scale") ? (float)p.at("scale").as_double() : (float)(1.0 / std::sqrt((double)head_dim));
    shares_kv = p.has("shares_kv") && p.at("shares_kv").as_bool();
    for (const auto& c : children)
      if (c.first == "pos") pos = std::dynamic_pointer_cast<PositionPart>(c.second);
    if (!pos && p.has("pos")) pos = std::dynamic_pointer_cast<PositionPart>(build_part("pos", PartSpec::from_json(p.at("pos")), prefix));
    nq = (int64_t)heads * head_dim;
    nk = shares_kv ? 0 : (int64_t)kv_heads * head_dim;
  }
  const char* kind_name() const override { return "attention"; }
  bool takes_lazy_norm() const override { return true; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    if (pos) return {pos};
    return {};
  }
  std::vector<std::string> child_slots() const override {
    if (pos) return {"pos"};
    return {};
  }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    TensorNeed q, kv, o, nw;
    q.shape = {nq, hidden};
    kv.shape = {nk, hidden};
    o.shape = {hidden, nq};
    nw.shape = {head_dim};
    nw.role = TensorNeed::Vector;
    nw.a = 1.0;
    nw.b = 0.1;
    t.emplace_back(join(prefix, "q_proj.weight"), q);
    t.emplace_back(join(prefix, "o_proj.weight"), o);
    if (!shares_kv) {
      t.emplace_back(join(prefix, "k_proj.weight"), kv);
      t.emplace_back(join(prefix, "v_proj.weight"), kv);
    }
    if (qk_norm) {
      t.emplace_back(join(prefix, "q_norm.weight"), nw);
      if (!shares_kv) t.emplace_back(join(prefix, "k_norm.weight"), nw);
    }
    return t;
  }
  void load(WeightSource& src) override {
    // q, k and v go straight into the fused matrix (the reference builds its fused copy beside the
    // originals and keeps both: /root/reference/src/inference.cu:154-169)
    w_qkv = src.alloc(src.matrix_dtype, {nq + 2 * nk, hidden});
    src.fill(join(prefix, "q_proj.weight"), w_qkv.rows(0, nq));
    if (!shares_kv) {
      src.fill(join(prefix, "k_proj.weight"), w_qkv.rows(nq, nk));
      src.fill(join(prefix, "v_proj.weight"), w_qkv.rows(nq + nk, nk));
    }
    w_o = src.alloc(src.matrix_dtype, {hidden, nq});
    src.fill(join(prefix, "o_proj.weight"), w_o);
    if (qk_norm) {
      TensorNeed nw;
      nw.shape = {head_dim};
      nw.role = TensorNeed::Vector;
      q_norm_w = src.fetch(join(prefix, "q_norm.weight"), nw);
      if (!shares_kv) k_norm_w = src.fetch(join(prefix, "k_norm.weight"), nw);
    }
  }
  bool has_cache() const override { return true; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::PagedKV;
    n.kv_heads = kv_heads;
    n.head_dim = head_dim;
    n.window = window;
    return n;
  }

  // The work lists of the attention kernels for this step: query tiles of 128 rows in order,
  // tiles of 64 rows from the one whose last row sees the most keys to the one that sees the
  // fewest, and the rows of single-token entries.  Every attention part of a model asks for the
  // same lists; the first one builds them.
  void plan(StepPlan& plan) const override {
    if (plan.decode_only() || plan.has("attention.tiles")) return;
    const auto& entries = plan.entries();
    size_t n_tiles = 0, n_small = 0, n_dec = 0;
    for (const auto& e : entries) {
      if (e.n_tokens > 1) {
        n_tiles += (e.n_tokens + PREFILL_TILE_Q - 1) / PREFILL_TILE_Q;
        n_small += (e.n_tokens + PREFILL_TILE_SMALL - 1) / PREFILL_TILE_SMALL;
      } else {
        ++n_dec;
      }
    }
    int* tiles = plan.ints("attention.tiles", 2 * n_tiles);
    int* small = plan.ints("attention.tiles_small", 2 * n_small);
    int* dec = plan.ints("attention.decode_rows", n_dec);
    struct Small { int last, entry, row; };
    std::vector<Small> order;
    order.reserve(n_small);
    int portion_context = 0;
    size_t t = 0, d = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
      const auto& e = entries[i];
      if (e.n_tokens > 1) {
        for (int q0 = 0; q0 < e.n_tokens; q0 += PREFILL_TILE_Q) {
          tiles[t++] = (int)i;
          tiles[t++] = e.row0 + q0;
        }
        for (int q0 = 0; q0 < e.n_tokens; q0 += PREFILL_TILE_SMALL)
          order.push_back({e.start + std::min(q0 + PREFILL_TILE_SMALL, e.n_tokens) - 1, (int)i, e.row0 + q0});
        portion_context = std::max(portion_context, e.start + e.n_tokens);
      } else {
        dec[d++] = e.row0;
      }
    }
    std::stable_sort(order.begin(), order.end(), [](const Small& a, const Small& b) { return a.last > b.last; });
    for (size_t i = 0; i < order.size(); ++i) {
      small[2 * i] = order[i].entry;
      small[2 * i + 1] = order[i].row;
    }
    plan.set_value("attention.portion_context", portion_context);
  }

  AttentionWork work(const StepContext& ctx) const {
    AttentionWork w;
    w.M = ctx.M;
    w.positions = ctx.positions;
    w.slots = ctx.slots;
    w.entry_meta = ctx.entry_meta;
    w.decode_only = ctx.decode_only;
    w.slots_are_rows = ctx.decode_only;      // every entry is one row: a row's entry is the row itself
    w.max_context = ctx.max_context;
    w.split_context = ctx.max_context;
    if (!ctx.decode_only) {
      w.tiles = ctx.planned("attention.tiles");
      w.n_tiles = (int)(ctx.planned_size("attention.tiles") / 2);
      w.tiles_small = ctx.planned("attention.tiles_small");
      w.n_tiles_small = (int)(ctx.planned_size("attention.tiles_small") / 2);
      w.decode_rows = ctx.planned("attention.decode_rows");
      w.n_decode_rows = (int)ctx.planned_size("attention.decode_rows");
      w.portion_context = (int)ctx.value("attention.portion_context");
    }
    if (ctx.plan && ctx.plan->sized_for_longest()) {
      // a graph is being captured: what a replay launches must cover the longest sequence
      w.split_context = ctx.plan->max_seq();
      if (w.n_tiles) w.portion_context = std::max(w.portion_context, ctx.plan->max_seq() / 2);
    }
    return w;
  }

  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    const int64_t M = h.t.shape[0];
    const int64_t width = nq + 2 * nk;
    Tensor q = ctx.buf("attn.q", ctx.act_dtype, {M, nq});
    const auto bound = ctx.binding(this);
    const Tensor pool = ctx.kv_pool(bound.first, bound.second);
    const Ops::CacheView view = ctx.cache_view(bound.first);
    Ops::Rotation rot;
    const bool has_rot = pos && pos->fused(rot);
    Tensor a = ctx.buf("attn.out", ctx.act_dtype, {M, nq});
    const bool fusable = !pos || has_rot;       // a position encoding without a fused form needs the 32-bit projections
    const float* qw = q_norm_w.ptr<float>();
    const float* kw = k_norm_w.ptr<float>();
    const AttentionWork w = work(ctx);
    const int n_kv_written = shares_kv ? 0 : kv_heads;
    if (fusable && !ctx.decode_only &&
        ctx.ops.qkv_prepared(h, w_qkv, qw, kw, eps, rot, ctx.positions, ctx.slots, view, pool, q, heads, n_kv_written, head_dim)) {
      // a step of many tokens: the projection's epilogue prepared q and wrote the cache
      ctx.ops.attention(w, ctx.ws, view, q, pool, a, heads, kv_heads, head_dim, scale, window);
      ctx.ops.linear(a, w_o, x, Ops::Add, true);
      return;
    }
    Tensor qkv = ctx.buf("attn.qkv", DType::F32, {M, width});
    ctx.ops.linear(h, w_qkv, qkv, Ops::Store);
    if (fusable && ctx.ops.attention_from_projections(w, ctx.ws, view, qkv, qw, kw, eps, rot, pool, !shares_kv, a, heads,
                                                      kv_heads, head_dim, scale, window)) {
      // a step of single tokens: one kernel did it all
      ctx.ops.linear(a, w_o, x, Ops::Add, true);
      return;
    }
    if (pos && !has_rot) {
      // a position encoding without a fused form works on the 32-bit projections, after the per-head
      // norm (as in the fused order: norm, then position)
      if (qw || kw) {
        ctx.ops.qk_norm_inplace(qkv, qw, kw, eps, heads, n_kv_written, head_dim);
        qw = kw = nullptr;
      }
      Tensor qv = qkv.cols(0, nq);
      qv.ndim = 3;
      qv.shape[0] = M; qv.shape[1] = heads; qv.shape[2] = head_dim;
      qv.stride[0] = width; qv.stride[1] = head_dim; qv.stride[2] = 1;
      Tensor kv;
      if (!shares_kv) {
        kv = qkv.cols(nq, nk);
        kv.ndim = 3;
        kv.shape[0] = M; kv.shape[1] = kv_heads; kv.shape[2] = head_dim;
        kv.stride[0] = width; kv.stride[1] = head_dim; kv.stride[2] = 1;
      }
      ctx.ops.flush();
      pos->apply(ctx, qv, kv);
    }
    ctx.ops.qk_norm_rope_kv_write(qkv, qw, kw, eps, rot, ctx.positions, ctx.slots, view, pool, q, heads, n_kv_written, head_dim);
    ctx.ops.attention(w, ctx.ws, view, q, pool, a, heads, kv_heads, head_dim, scale, window);
    ctx.ops.linear(a, w_o, x, Ops::Add, true);
  }

  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_qkv", w_qkv}, {"w_o", w_o}, {"q_norm_w", q_norm_w}, {"k_norm_w", k_norm_w}};
  }
  int64_t hidden = 0, nq = 0, nk = 0;
  int heads = 0, kv_heads = 0, head_dim = 0, window = 0;
  bool qk_norm = true, shares_kv = false;
  float eps = 1e-6f, scale = 1.f;
  std::shared_ptr<PositionPart> pos;
  Tensor w_qkv, w_o, q_norm_w, k_norm_w;
};

// x += mixer(norm1(x)); x += ffn(norm2(x)).  The mixer and the feed-forward add into x
// themselves, so the residual sum happens in 32-bit in their last kernel.  That kernel may leave
// part of the sum to the norm that reads x next; before a part that does not read x through the
// kernels' own object, the sum is completed.
class PreNormBlock final : public BlockPart {
 public:
  PreNormBlock(const std::string& prefix, const PartChildren& c) : BlockPart(prefix) {
    for (const auto& kv : c) {
      if (kv.first == "norm1") norm1 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "mixer") mixer = std::dynamic_pointer_cast<MixerPart>(kv.second);
      if (kv.first == "norm2") norm2 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "ffn") ffn = std::dynamic_pointer_cast<FeedForwardPart>(kv.second);
    }
    if (!norm1 || !mixer || !norm2 || !ffn) throw ConfigError("block 'pre_norm' needs norm1, mixer, norm2 and ffn parts");
  }
  const char* kind_name() const override { return "pre_norm"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override { return {norm1, mixer, norm2, ffn}; }
  std::vector<std::string> child_slots() const override { return {"norm1", "mixer", "norm2", "ffn"}; }
  void forward(StepContext& ctx, const Tensor& x) override {
    if (!norm1->reads_through_ops()) ctx.ops.flush();
    Rows h = norm1->forward(ctx, x, nullptr, 0, mixer->takes_lazy_norm() && norm1->can_be_lazy());
    if (!mixer->reads_through_ops()) ctx.ops.flush();
    mixer->forward(ctx, h, x);
    if (!norm2->reads_through_ops()) ctx.ops.flush();
    h = norm2->forward(ctx, x, nullptr, 0, ffn->takes_lazy_norm() && norm2->can_be_lazy());
    if (!ffn->reads_through_ops()) ctx.ops.flush();
    ffn->forward(ctx, h, x);
  }
  std::shared_ptr<NormPart> norm1, norm2;
  std::shared_ptr<MixerPart> mixer;
  std::shared_ptr<FeedForwardPart> ffn;
};

void register_builtin_parts() {
  register_part("embedding", "table", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<Embedding>(prefix, param_int(p, "vocab"), param_int(p, "dim"));
  });
  register_part("head", "linear", [](const std::string& prefix, const Json& p, const PartChildren&) {
    const Json* t = p.find("tied");
    const int tied = (!t || t->is_null()) ? -1 : (t->as_bool() ? 1 : 0);
    return std::make_shared<LMHead>(prefix, param_int(p, "vocab"), param_int(p, "dim"), tied, p.at("tied_to").as_string());
  });
  register_part("norm", "rmsnorm", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<RMSNorm>(prefix, param_int(p, "dim"), param_float(p, "eps"));
  });
  register_part("pos", "rope_neox", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<RotaryNeox>(prefix, param_int(p, "head_dim"), param_float(p, "theta"));
  });
  register_part("ffn", "swiglu", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<SwiGLU>(prefix, param_int(p, "hidden"), param_int(p, "intermediate"));
  });
  register_part("mixer", "attention", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<Attention>(prefix, p, c);
  });
  register_part("block", "pre_norm",
                [](const std::string& prefix, const Json&, const PartChildren& c) { return std::make_shared<PreNormBlock>(prefix, c); },
                {{"norm1", "norm"}, {"mixer", "mixer"}, {"norm2", "norm"}, {"ffn", "ffn"}});
}

// --------------------------------------------------------------------------------- foreign parts
ForeignCalls g_foreign;
thread_local std::string g_foreign_error;

struct ForeignInfo {
  std::vector<std::pair<std::string, TensorNeed>> tensors;
  bool has_cache = false;
  CacheNeed cache;
  bool takes_lazy = false;
};

ForeignInfo read_description(const Json& d) {
  ForeignInfo info;
  if (const Json* ts = d.find("tensors"))
    for (const auto& kv : ts->members()) {
      TensorNeed n;
      for (const Json& s : kv.second.at("shape").items()) n.shape.push_back(s.as_int());
      const std::string role = kv.second.has("role") ? kv.second.at("role").as_string() : "matrix";
      n.role = role == "vector" ? TensorNeed::Vector : role == "table" ? TensorNeed::Table : TensorNeed::Matrix;
      if (kv.second.has("init")) n.init = kv.second.at("init").as_string();
      if (kv.second.has("a")) n.a = kv.second.at("a").as_double();
      if (kv.second.has("b")) n.b = kv.second.at("b").as_double();
      n.optional = kv.second.has("optional") && kv.second.at("optional").as_bool();
      info.tensors.emplace_back(kv.first, n);
    }
  if (d.has("cache_need")) {
    const Json& c = d.at("cache_need");
    info.has_cache = true;
    if (c.at("kind").as_string() == "state") {
      info.cache.kind = CacheNeed::State;
      for (const Json& s : c.at("shape").items()) info.cache.state_shape.push_back(s.as_int());
    } else if (c.at("kind").as_string() == "paged_rows") {
      info.cache.kind = CacheNeed::PagedRows;
      for (const Json& s : c.at("row_shape").items()) info.cache.row_shape.push_back(s.as_int());
      info.cache.rows_f32 = c.has("float32") && c.at("float32").as_bool();
      info.cache.window = (c.has("window") && !c.at("window").is_null()) ? (int)c.at("window").as_int() : 0;
    } else {
      info.cache.kind = CacheNeed::PagedKV;
      info.cache.kv_heads = (int)c.at("kv_heads").as_int();
      info.cache.head_dim = (int)c.at("head_dim").as_int();
      info.cache.window = c.has("window") ? (int)c.at("window").as_int() : 0;
    }
  }
  return info;
}

void foreign_call(uint64_t id, const char* op, StepContext* ctx, const Tensor* args, int n_args, const char* names,
                  Tensor* result) {
  if (!g_foreign.call) throw EngineError("a part implemented outside the library was called, but no call table is set");
  g_foreign_error.clear();
  if (ctx) ctx->ops.flush();        // whatever the part reads, it finds complete
  const int rc = g_foreign.call(id, op, ctx, args, n_args, names, result);
  if (rc != 0) throw EngineError(g_foreign_error.empty() ? std::string("a foreign part failed in '") + op + "'" : g_foreign_error);
}

// what all foreign parts share; Base is the family's interface
template <class Base> class Foreign : public Base {
 public:
  Foreign(uint64_t id, const std::string& prefix, const Json& description, const PartChildren& c)
      : Base(prefix), info(read_description(description)) {
    this->foreign_id = id;
    for (const auto& kv : c) {
      kids.push_back(kv.second);
      slots.push_back(kv.first);
    }
  }
  std::vector<std::string> child_slots() const override { return slots; }
  const char* kind_name() const override { return "foreign"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override { return info.tensors; }
  std::vector<std::shared_ptr<Part>> children() const override { return kids; }
  bool has_cache() const override { return info.has_cache; }
  CacheNeed cache_need() const override { return info.cache; }
  void load(WeightSource& src) override {
    std::vector<Tensor> ts;
    std::string names;
    for (const auto& kv : info.tensors) {
      if (!src.has(kv.first)) continue;
      ts.push_back(src.fetch(kv.first, kv.second));
      names += (names.empty() ? "" : "\n") + kv.first;
    }
    foreign_call(this->foreign_id, "load", nullptr, ts.data(), (int)ts.size(), names.c_str(), nullptr);
  }
  void prepare(Ops&, int max_seq) override {
    const std::string arg = std::to_string(max_seq);
    foreign_call(this->foreign_id, "prepare", nullptr, nullptr, 0, arg.c_str(), nullptr);
  }
  ForeignInfo info;
  std::vector<std::shared_ptr<Part>> kids;
  std::vector<std::string> slots;
};

class ForeignEmbedding final : public Foreign<EmbeddingPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Tensor& x) override { foreign_call(foreign_id, "forward", &ctx, &x, 1, "", nullptr); }
};
class ForeignNorm final : public Foreign<NormPart> {
 public:
  using Foreign::Foreign;
  Rows forward(StepContext& ctx, const Tensor& x, const int* rows, int64_t n_rows, bool) override {
    Tensor args[2] = {x, rows ? Tensor((void*)rows, DType::I32, {n_rows}) : Tensor()};
    Rows r;
    foreign_call(foreign_id, "forward", &ctx, args, 2, "", &r.t);
    return r;
  }
};
class ForeignPos final : public Foreign<PositionPart> {
 public:
  using Foreign::Foreign;
  void apply(StepContext& ctx, const Tensor& q, const Tensor& k) override {
    Tensor args[2] = {q, k};
    foreign_call(foreign_id, "apply", &ctx, args, 2, "", nullptr);
  }
};
class ForeignMixer final : public Foreign<MixerPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor args[2] = {h.materialize(ctx.ops), x};
    foreign_call(foreign_id, "forward", &ctx, args, 2, "", nullptr);
  }
};
class ForeignFFN final : public Foreign<FeedForwardPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor args[2] = {h.materialize(ctx.ops), x};
    foreign_call(foreign_id, "forward", &ctx, args, 2, "", nullptr);
  }
};
class ForeignBlock final : public Foreign<BlockPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Tensor& x) override { foreign_call(foreign_id, "forward", &ctx, &x, 1, "", nullptr); }
};
class ForeignHead final : public Foreign<HeadPart> {
 public:
  using Foreign::Foreign;
  Tensor forward(StepContext& ctx, const Rows& h) override {
    Tensor out;
    foreign_call(foreign_id, "forward", &ctx, &h.materialize(ctx.ops), 1, "", &out);
    return out;
  }
};
}  // namespace

void set_foreign_calls(const ForeignCalls& calls) { g_foreign = calls; }
void set_foreign_error(const std::string& message) { g_foreign_error = message; }
std::string take_foreign_error() {
  std::string m;
  m.swap(g_foreign_error);
  return m;
}

std::shared_ptr<Part> make_foreign_part(const std::string& family, uint64_t id, const std::string& prefix,
                                        const Json& description, const PartChildren& children) {
  if (family == "embedding") return std::make_shared<ForeignEmbedding>(id, prefix, description, children);
  if (family == "norm") return std::make_shared<ForeignNorm>(id, prefix, description, children);
  if (family == "pos") return std::make_shared<ForeignPos>(id, prefix, description, children);
  if (family == "mixer") return std::make_shared<ForeignMixer>(id, prefix, description, children);
  if (family == "ffn") return std::make_shared<ForeignFFN>(id, prefix, description, children);
  if (family == "block") return std::make_shared<ForeignBlock>(id, prefix, description, children);
  if (family == "head") return std::make_shared<ForeignHead>(id, prefix, description, children);
  throw ConfigError("unknown part family '" + family + "'");
}

}  // namespace tinyinfer

// small HIP helpers the rotary part needs (kept out of the class so that this file's other code
// does not depend on the HIP headers)
#include <hip/hip_runtime_api.h>
namespace tinyinfer {
namespace {
void RotaryNeox::upload(void* dst, const void* src, size_t bytes) {
  if (hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice) != hipSuccess) throw KernelError("rotary: copying the inverse frequencies failed");
}
}  // namespace
}  // namespace tinyinfer
