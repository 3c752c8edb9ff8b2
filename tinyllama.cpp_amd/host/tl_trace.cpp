// tl_trace — replays recorded steps through a model and writes the logits asked for. It samples nothing: a scheduler's
// decisions (which tokens of which request run in which step) come from the input, the model work goes through
// tlhost::Session::forward, i.e. the same prefill and decode step that generate() uses.
//
//   tl_trace --model PATH --dtype bfloat16|float32 --out DIR [--max-tokens N] [--device D]
//
// PATH: anything Session opens (a checkpoint folder with config.json + model.safetensors, or a .gguf file).
// --dtype float32 makes the prompt-chunk matrix products FP32-grade (Session::set_exact); bfloat16 is the serving default.
// --max-tokens: the most tokens live requests hold at any time; sizes the cache.
// Standard input, one JSON object per line:
//   {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
// Each entry continues its request where earlier steps left it; `want` lists the token places of this step whose logits go
// to DIR/<step>.f32 (little-endian FP32, [wanted][vocab], in entry order); requests named in `end` give their cache back.
// After every step "done <step>" is printed and flushed. One request is live at a time (the single-sequence cache).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <iostream>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "tl_json.hpp"
#include "tl_session.hpp"

int main(int argc, char** argv) {
  std::string model, dtype = "bfloat16", out_dir;
  int max_tokens = 0, device = 0;
  for (int i = 1; i < argc; ++i) {
    const std::string k = argv[i];
    if (i + 1 >= argc) {
      fprintf(stderr, "tl_trace: option %s needs a value\n", k.c_str());
      return 2;
    }
    const char* v = argv[++i];
    if (k == "--model") model = v;
    else if (k == "--dtype") dtype = v;
    else if (k == "--out") out_dir = v;
    else if (k == "--max-tokens") max_tokens = atoi(v);
    else if (k == "--device") device = atoi(v);
    else {
      fprintf(stderr, "tl_trace: unknown option %s\n", k.c_str());
      return 2;
    }
  }
  if (model.empty() || out_dir.empty() || (dtype != "bfloat16" && dtype != "float32")) {
    fprintf(stderr, "usage: tl_trace --model PATH --dtype bfloat16|float32 --out DIR [--max-tokens N] [--device D]\n");
    return 2;
  }
  try {
    tlhost::Session session(model, device, max_tokens > 0 ? max_tokens : 0);
    session.set_exact(dtype == "float32");
    const size_t V = (size_t)session.get_config().vocab_size;
    std::map<std::string, int> fed;  // live requests -> tokens already in the cache
    std::string line;
    while (std::getline(std::cin, line)) {
      if (line.find_first_not_of(" \t\r\n") == std::string::npos) continue;
      const tlhost::Json step = tlhost::Json::parse(line);
      const long long n = step.at("step").as_int("step");
      std::vector<float> wanted;
      if (const tlhost::Json* entries = step.find("entries")) {
        for (const tlhost::Json& e : entries->arr) {
          const std::string& id = e.at("id").as_string("id");
          std::vector<int> tokens, want;
          for (const tlhost::Json& t : e.at("tokens").arr) tokens.push_back((int)t.as_int("token"));
          if (const tlhost::Json* w = e.find("want"))
            for (const tlhost::Json& t : w->arr) want.push_back((int)t.as_int("want"));
          if (tokens.empty()) continue;
          auto it = fed.find(id);
          if (it == fed.end()) {
            if (!fed.empty())
              throw std::runtime_error("request " + id + " starts while " + fed.begin()->first +
                                       " is live: this cache holds one sequence at a time");
            session.reset();
            it = fed.emplace(id, 0).first;
          }
          const std::vector<float> logits = session.forward(tokens, it->second, want);
          it->second += (int)tokens.size();
          wanted.insert(wanted.end(), logits.begin(), logits.end());
        }
      }
      if (const tlhost::Json* end = step.find("end"))
        for (const tlhost::Json& e : end->arr) fed.erase(e.as_string("end"));
      if (!wanted.empty()) {
        const std::string path = out_dir + "/" + std::to_string(n) + ".f32";
        FILE* f = fopen(path.c_str(), "wb");
        if (!f) throw std::runtime_error("cannot write " + path);
        const size_t wrote = fwrite(wanted.data(), sizeof(float), wanted.size(), f);
        if (fclose(f) != 0 || wrote != wanted.size()) throw std::runtime_error("short write to " + path);
        (void)V;
      }
      printf("done %lld\n", n);
      fflush(stdout);
    }
  } catch (const std::exception& e) {
    fprintf(stderr, "tl_trace: %s\n", e.what());
    return 1;
  }
  return 0;
}
