// Trace replay: feeds given token ids through a model step by step and writes logits.  It samples
// nothing and has no forward pass, cache or loader of its own: it drives Engine::step of inference.h,
// the step function generation uses.
//
//   trace_run --model DIR --dtype bfloat16|float32 --out DIR (--max-tokens N | --num-pages N)
//             [--page-size P] [--max-requests R] [--max-seq S] [--random-weights --seed S] [--plugin LIB.so]...
//
// --plugin         a shared library that registers parts or architectures of its own (tinyinfer::load_plugin)
// --model          a folder with config.json and *.safetensors; with --random-weights config.json alone
//                  is enough and the weights are drawn on the device from --seed
// --max-tokens N   the most tokens live requests hold at any time, each request's count rounded up to a
//                  multiple of 64: the cache pool is made for this many
// --num-pages N    the pool's size in pages instead
//
// Steps come on standard input, one JSON object a line:
//   {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
// For a step in which something is wanted, OUT/<step>.f32 holds the logits at the wanted places
// ([wanted, vocab], little-endian float32, in the order of the entries and of `want`), and
// OUT/index.jsonl gets a line {"step", "request", "position", "file", "row"} for every row.  After every
// step a line `done <step>` is printed and flushed.  When the input ends the program exits with 0.
//
// The reference's tool of this kind writes the last token's logits of one prompt through another
// library (/root/reference/ref/ref_logits.cpp:13-19,59-67).
#include <cstdio>
#include <cstring>
#include <iostream>
#include <map>
#include <sys/stat.h>

#include "../include/inference.h"

using namespace tinyinfer;

namespace {
struct Args {
  std::string model, dtype, out;
  long max_tokens = 0, num_pages = 0;
  int page_size = 16, max_requests = 8, max_seq = 0;
  bool random_weights = false;
  unsigned long long seed = 0;
  std::vector<std::string> plugins;
};

int usage(const char* why) {
  fprintf(stderr,
          "trace_run: %s\n"
          "usage: trace_run --model DIR --dtype bfloat16|float32 --out DIR (--max-tokens N | --num-pages N)\n"
          "                 [--page-size P] [--max-requests R] [--max-seq S] [--random-weights --seed S]\n"
          "                 [--plugin LIB.so]...\n",
          why);
  return 2;
}

std::string json_string(const std::string& s) { return Json(s).dump(); }

void make_folders(const std::string& path) {
  for (size_t i = 1; i <= path.size(); ++i)
    if (i == path.size() || path[i] == '/') mkdir(path.substr(0, i).c_str(), 0777);
}
}  // namespace

int main(int argc, char** argv) {
  Args a;
  for (int i = 1; i < argc; ++i) {
    const std::string k = argv[i];
    auto value = [&]() -> const char* {
      if (i + 1 >= argc) {
        usage(("option " + k + " needs a value").c_str());
        exit(2);
      }
      return argv[++i];
    };
    if (k == "--model") a.model = value();
    else if (k == "--dtype") a.dtype = value();
    else if (k == "--out") a.out = value();
    else if (k == "--max-tokens") a.max_tokens = atol(value());
    else if (k == "--num-pages") a.num_pages = atol(value());
    else if (k == "--page-size") a.page_size = atoi(value());
    else if (k == "--max-requests") a.max_requests = atoi(value());
    else if (k == "--max-seq") a.max_seq = atoi(value());
    else if (k == "--seed") a.seed = strtoull(value(), nullptr, 10);
    else if (k == "--random-weights") a.random_weights = true;
    else if (k == "--plugin") a.plugins.push_back(value());
    else if (k == "-h" || k == "--help") return usage("feeds token ids through a model step by step and writes logits"), 0;
    else return usage(("unknown option " + k).c_str());
  }
  if (a.model.empty() || a.out.empty()) return usage("--model and --out are required");
  if (a.dtype != "bfloat16" && a.dtype != "float32") return usage("--dtype must be bfloat16 or float32");
  if (a.max_tokens <= 0 && a.num_pages <= 0) return usage("give the cache pool a size: --max-tokens or --num-pages");
  if (a.page_size <= 0 || (a.max_tokens > 0 && 64 % a.page_size)) return usage("--page-size must divide 64");
  if (a.max_requests <= 0) return usage("--max-requests must be positive");
  try {
    for (const auto& p : a.plugins) load_plugin(p);
    fprintf(stderr, "[trace_run] loading %s ...\n", a.model.c_str());
    std::shared_ptr<Model> model = a.random_weights ? Model::from_config(read_config_json(a.model), a.seed, a.dtype)
                                                    : Model::from_folder(a.model, a.dtype);
    EngineOptions opt;
    opt.page_size = a.page_size;
    opt.max_requests = a.max_requests;
    if (a.num_pages > 0) opt.num_pages = a.num_pages;
    else opt.max_tokens = a.max_tokens;
    const long pool_tokens = a.num_pages > 0 ? a.num_pages * a.page_size : a.max_tokens;
    opt.max_seq = a.max_seq > 0 ? a.max_seq : (int)pool_tokens;
    Engine engine(model, opt);
    make_folders(a.out);
    const std::string index_path = a.out + "/index.jsonl";
    FILE* index = fopen(index_path.c_str(), "w");
    if (!index) throw FileError("cannot write " + index_path);
    fprintf(stderr, "[trace_run] ready\n");

    std::map<std::string, int64_t> ids;
    auto id_of = [&](const Json& j) {
      const std::string name = j.type() == Json::String ? j.as_string() : j.dump();
      auto it = ids.find(name);
      if (it == ids.end()) it = ids.emplace(name, (int64_t)ids.size() + 1).first;
      return it->second;
    };
    const int64_t V = model->spec.vocab_size;
    std::vector<float> host;
    std::string line;
    while (std::getline(std::cin, line)) {
      if (line.find_first_not_of(" \t\r\n") == std::string::npos) continue;
      const Json rec = Json::parse(line);
      const int64_t step = rec.at("step").as_int();
      std::vector<StepEntry> entries;
      std::vector<std::string> names;
      if (rec.has("entries"))
        for (const Json& e : rec.at("entries").items()) {
          StepEntry se;
          se.request = id_of(e.at("id"));
          names.push_back(e.at("id").type() == Json::String ? e.at("id").as_string() : e.at("id").dump());
          for (const Json& t : e.at("tokens").items()) se.tokens.push_back((int)t.as_int());
          if (e.has("want"))
            for (const Json& w : e.at("want").items()) se.want.push_back((int)w.as_int());
          entries.push_back(std::move(se));
        }
      if (!entries.empty()) {
        std::vector<int> starts;
        for (const auto& e : entries) starts.push_back(engine.cache->has(e.request) ? engine.cache->length(e.request) : 0);
        const Tensor logits = engine.step(entries);
        if (logits.defined()) {
          if (logits.shape[1] != V) throw EngineError("the logits have the wrong width");
          host.resize((size_t)logits.numel());
          engine.logits_to_host(logits, host.data());
          const std::string file = std::to_string(step) + ".f32";
          const std::string path = a.out + "/" + file;
          FILE* f = fopen(path.c_str(), "wb");
          if (!f || fwrite(host.data(), 4, host.size(), f) != host.size()) throw FileError("cannot write " + path);
          fclose(f);
          int row = 0;
          for (size_t i = 0; i < entries.size(); ++i)
            for (int w : entries[i].want)
              fprintf(index, "{\"step\": %lld, \"request\": %s, \"position\": %d, \"file\": \"%s\", \"row\": %d}\n",
                      (long long)step, json_string(names[i]).c_str(), starts[i] + w, file.c_str(), row++);
          fflush(index);
        } else {
          engine.synchronize();
        }
      }
      if (rec.has("end"))
        for (const Json& r : rec.at("end").items())
          if (engine.cache->has(id_of(r))) engine.release(id_of(r));
      engine.cache->check();
      printf("done %lld\n", (long long)step);
      fflush(stdout);
    }
    fclose(index);
    return 0;
  } catch (const Error& e) {
    fprintf(stderr, "trace_run: %s: %s\n", e.kind(), e.what());
    return 1;
  } catch (const std::exception& e) {
    fprintf(stderr, "trace_run: %s\n", e.what());
    return 1;
  }
}
