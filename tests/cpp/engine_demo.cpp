// A C++ program on the engine's library API: generates for several prompts at once.
//   engine_demo MODEL_DIR DTYPE "1,2,3;4,5" MAX_NEW_TOKENS [BLOCK_SIZE]
// prints one line of generated token ids per prompt.
#include <cstdio>
#include <cstdlib>
#include <sstream>
#include <string>
#include <vector>

#include "photon_engine.h"

int main(int argc, char** argv) {
  if (argc < 5) { std::fprintf(stderr, "usage: engine_demo MODEL_DIR DTYPE PROMPTS MAX_NEW_TOKENS [BLOCK_SIZE]\n"); return 2; }
  std::vector<std::vector<int>> prompts;
  std::stringstream all(argv[3]);
  for (std::string one; std::getline(all, one, ';');) {
    std::vector<int> ids;
    std::stringstream s(one);
    for (std::string t; std::getline(s, t, ',');) ids.push_back(std::atoi(t.c_str()));
    prompts.push_back(ids);
  }
  try {
    photon::EngineOptions opt;
    opt.dtype = argv[2];
    opt.max_batch = 4;
    opt.num_blocks = 128;
    if (argc > 5) opt.block_size = std::atoi(argv[5]);
    photon::Engine engine = photon::Engine::create(argv[1], opt);
    photon::SamplingParams params;
    params.max_new_tokens = std::atoi(argv[4]);
    params.ignore_eos = true;
    std::vector<long> ids;
    for (const auto& p : prompts) ids.push_back(engine.add_request(p, params));
    int steps = 0;
    while (engine.has_work()) { engine.step(); ++steps; }
    for (long id : ids) {
      if (!engine.finished(id)) { std::fprintf(stderr, "request %ld did not finish\n", id); return 1; }
      const std::vector<int> out = engine.get_result(id);
      for (size_t i = 0; i < out.size(); ++i) std::printf(i ? " %d" : "%d", out[i]);
      std::printf("\n");
    }
    std::fprintf(stderr, "steps: %d\n", steps);
  } catch (const photon::EngineError& e) {
    std::fprintf(stderr, "engine error: %s\n", e.what());
    return 3;
  }
  return 0;
}
