// A program that uses the engine through its C++ interface alone: it includes inference.h and
// nothing else of the framework.  It loads a model folder, replays a trace of steps (the format of
// bin/trace_run: one JSON object a line) through Engine::step, writes the logits of every step
// that wants some, then runs a scheduled generation and prints the generated ids as JSON.
//
//   api_program MODEL_DIR DTYPE TRACE_FILE OUT_DIR MAX_TOKENS PAGE_SIZE 'PROMPTS_JSON' TEMPERATURE SEED CHUNK
//
// tests/test_cpp_api_gpu.py builds it, runs it and compares its output with the Python entry point's.
#include <cstdio>
#include <fstream>
#include <iostream>
#include <map>
#include <sstream>

#include "inference.h"

using namespace tinyinfer;

int main(int argc, char** argv) {
  if (argc < 11) {
    fprintf(stderr, "usage: %s MODEL_DIR DTYPE TRACE_FILE OUT_DIR MAX_TOKENS PAGE_SIZE PROMPTS_JSON TEMPERATURE SEED CHUNK\n", argv[0]);
    return 2;
  }
  try {
    const std::string dir = argv[1], dtype = argv[2], trace = argv[3], out_dir = argv[4];
    auto model = Model::from_folder(dir, dtype);
    EngineOptions opt;
    opt.page_size = atoi(argv[6]);
    opt.max_tokens = atol(argv[5]);
    opt.max_requests = 8;
    opt.max_seq = (int)opt.max_tokens;
    Engine engine(model, opt);

    // ---- the trace: steps of (request, tokens, wanted places), requests ended after a step
    std::map<std::string, int64_t> ids;
    auto id_of = [&](const std::string& name) {
      auto it = ids.find(name);
      if (it == ids.end()) it = ids.emplace(name, (int64_t)ids.size() + 1).first;
      return it->second;
    };
    std::ifstream in(trace);
    std::string line;
    const int64_t V = model->spec.vocab_size;
    while (std::getline(in, line)) {
      if (line.empty()) continue;
      const Json rec = Json::parse(line);
      std::vector<StepEntry> entries;
      for (const Json& e : rec.at("entries").items()) {
        StepEntry se;
        se.request = id_of(e.at("id").as_string());
        for (const Json& t : e.at("tokens").items()) se.tokens.push_back((int)t.as_int());
        if (e.has("want"))
          for (const Json& w : e.at("want").items()) se.want.push_back((int)w.as_int());
        entries.push_back(std::move(se));
      }
      if (!entries.empty()) {
        const Tensor logits = engine.step(entries);
        if (logits.defined()) {
          std::vector<float> host((size_t)logits.numel());
          engine.logits_to_host(logits, host.data());
          if (logits.shape[1] != V) throw Error("logits have the wrong width");
          const std::string path = out_dir + "/" + std::to_string(rec.at("step").as_int()) + ".f32";
          FILE* f = fopen(path.c_str(), "wb");
          if (!f || fwrite(host.data(), 4, host.size(), f) != host.size()) throw Error("cannot write " + path);
          fclose(f);
        } else {
          engine.synchronize();
        }
      }
      if (rec.has("end"))
        for (const Json& r : rec.at("end").items())
          if (engine.cache->has(id_of(r.as_string()))) engine.release(id_of(r.as_string()));
    }
    engine.cache->check();
    if (!engine.cache->live_requests().empty()) throw Error("the trace left requests in the cache");

    // ---- a scheduled generation: portions under a token budget beside decoding requests
    const Json prompts_json = Json::parse(argv[7]);
    std::vector<std::vector<int>> prompts;
    for (const Json& p : prompts_json.items()) {
      prompts.emplace_back();
      for (const Json& t : p.items()) prompts.back().push_back((int)t.as_int());
    }
    GenerateOptions go;
    go.max_new_tokens = 6;
    go.sampling.temperature = (float)atof(argv[8]);
    go.sampling.seed = (uint64_t)atoll(argv[9]);
    go.chunk_size = atoi(argv[10]);
    go.max_batched_tokens = 16;
    GenerationStats stats;
    const auto outs = generate(engine, prompts, go, &stats);
    Json result = Json::object();
    Json all = Json::array();
    for (const auto& o : outs) {
      Json a = Json::array();
      for (int t : o) a.push(t);
      all.push(a);
    }
    result.set("generated", all);
    result.set("steps", stats.steps);
    result.set("preemptions", stats.preemptions);
    result.set("free_pages", engine.cache->num_free_pages());
    std::cout << result.dump() << std::endl;
    return 0;
  } catch (const Error& e) {
    fprintf(stderr, "%s: %s\n", e.kind(), e.what());
    return 1;
  }
}
