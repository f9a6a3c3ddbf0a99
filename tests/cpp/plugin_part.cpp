// A plugin: a feed-forward kind, its kernel library and an architecture that uses them, registered with
// the host library from outside it (tinyinfer::load_plugin).  Built by tests/test_plugin_gpu.py against
// include/inference.h; nothing under the framework's own folder knows of it.
//
//   ffn "toy_relu":  x += alpha * relu(h W1^T) W2^T      W1 [inner, hidden], W2 [hidden, inner]
//   "ToyCppLM":      embedding; layers of pre_norm(rmsnorm, attention with rotation, rmsnorm, toy_relu); norm; tied head
#include <hip/hip_runtime_api.h>

#include <cstdlib>

#include "inference.h"

using namespace tinyinfer;

namespace {
class ReluFFN final : public FeedForwardPart {
 public:
  ReluFFN(const std::string& prefix, int64_t hidden, int64_t inner, double alpha)
      : FeedForwardPart(prefix), hidden(hidden), inner(inner), alpha((float)alpha) {}
  const char* kind_name() const override { return "toy_relu"; }
  bool reads_through_ops() const override { return true; }       // x is touched through ctx.ops alone
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed up, down;
    up.shape = {inner, hidden};
    down.shape = {hidden, inner};
    up.b = down.b = 0.2;
    return {{prefix + ".w1", up}, {prefix + ".w2", down}};
  }
  void load(WeightSource& src) override {
    const auto needs = tensors();
    w1 = src.fetch(needs[0].first, needs[0].second);
    w2 = src.fetch(needs[1].first, needs[1].second);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    const Tensor& rows = h.materialize(ctx.ops);
    const int64_t M = rows.shape[0];
    Tensor u = ctx.buf("toy.u", DType::F32, {M, inner});
    Tensor y = ctx.buf("toy.y", ctx.act_dtype, {M, inner});
    ctx.ops.linear(rows, w1, u, Ops::Store);
    using Fn = int (*)(const float*, void*, long, float, int, hipStream_t);
    static Fn relu_scale = (Fn)kernel_symbol("toy_relu", "toy_relu_scale");
    if (relu_scale(u.ptr<float>(), y.data, (long)(M * inner), alpha, y.dtype == DType::BF16 ? 1 : 0, (hipStream_t)ctx.ops.stream()) != 0)
      throw KernelError("toy_relu_scale failed to launch");
    ctx.ops.linear(y, w2, x, Ops::Add, /*may_defer=*/true);
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w1", w1}, {"w2", w2}}; }
  int64_t hidden, inner;
  float alpha;
  Tensor w1, w2;
};

PartSpec part(const char* kind, const char* name) {
  PartSpec p;
  p.kind = kind;
  p.name = name;
  return p;
}

ModelSpec toy_spec(const Json& c) {
  const int64_t H = c.at("hidden").as_int(), V = c.at("vocab").as_int();
  ModelSpec s;
  s.architecture = "ToyCppLM";
  s.vocab_size = V;
  s.hidden_size = H;
  auto norm = [&](const char* name) {
    PartSpec p = part("rmsnorm", name);
    p.params.set("dim", H);
    p.params.set("eps", c.at("eps").as_double());
    return p;
  };
  for (int64_t i = 0; i < c.at("layers").as_int(); ++i) {
    LayerSpec l;
    l.prefix = "l." + std::to_string(i);
    l.block = part("pre_norm", "");
    PartSpec attn = part("attention", "attn");
    attn.params.set("hidden", H);
    attn.params.set("heads", c.at("heads").as_int());
    attn.params.set("kv_heads", c.at("kv_heads").as_int());
    attn.params.set("head_dim", c.at("head_dim").as_int());
    attn.params.set("eps", c.at("eps").as_double());
    PartSpec pos = part("rope_neox", "");
    pos.params.set("head_dim", c.at("head_dim").as_int());
    pos.params.set("theta", c.at("theta").as_double());
    attn.params.set("pos", pos.to_json());
    PartSpec ffn = part("toy_relu", "ffn");
    ffn.params.set("hidden", H);
    ffn.params.set("inner", c.at("inner").as_int());
    ffn.params.set("alpha", c.at("alpha").as_double());
    l.parts = {{"norm1", norm("n1")}, {"mixer", attn}, {"norm2", norm("n2")}, {"ffn", ffn}};
    s.layers.push_back(l);
  }
  s.embedding = part("table", "emb");
  s.embedding.params.set("vocab", V);
  s.embedding.params.set("dim", H);
  s.final_norm = norm("norm");
  s.lm_head = part("linear", "head");
  s.lm_head.params.set("vocab", V);
  s.lm_head.params.set("dim", H);
  s.lm_head.params.set("tied", true);
  s.lm_head.params.set("tied_to", "emb.weight");
  return s;
}
}  // namespace

extern "C" void tinyinfer_plugin_init() {
  if (const char* lib = getenv("TOY_RELU_LIB")) register_kernel_library("toy_relu", lib);
  register_part("ffn", "toy_relu", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<ReluFFN>(prefix, p.at("hidden").as_int(), p.at("inner").as_int(), p.at("alpha").as_double());
  });
  register_architecture({"ToyCppLM"}, toy_spec);
}
