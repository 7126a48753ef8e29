// The engine for C and C++ programs.
//
// Reference: include/photon/scheduler/continuous_batch_engine.hpp (ContinuousBatchEngine with
// add_request(prompt, max_new_tokens) -> id, run_until_complete(), get_result(id)) and
// include/photon/arch/llama_model.hpp.  The names below follow it.
//
// The engine itself (scheduler, step function, kernels' dispatch) lives in the Python package;
// this library hosts an interpreter inside the calling process and drives that same engine, so
// a C++ program gets the same kernels, cache and scheduler as the command line.  Link against
// libphoton_api.so (built into photon_infer_amd/csrc/_build/ by
// `python -c "from photon_infer_amd.ops import build; build.build_module('api')"`).
//
// Threads: calls may come from any thread, one at a time per engine (each call takes the
// interpreter's lock).  Errors: functions return -1 / NULL and pi_engine_last_error() holds the
// text; the C++ class throws photon::EngineError.
#pragma once
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct pi_engine pi_engine;

// Zero / NULL fields keep the engine's defaults (EngineOptions in the Python package).
typedef struct pi_engine_options {
  const char* dtype;        // "bfloat16" | "float32"
  int block_size;           // tokens per cache page
  int num_blocks;           // pages per cache group
  int max_batch;            // most live requests
  int max_step_tokens;      // token budget of one step
  int chunk_size;           // largest prompt portion of one request in one step
  int max_model_len;        // most tokens a request may hold
} pi_engine_options;

pi_engine* pi_engine_create(const char* model_dir, const pi_engine_options* options);
void pi_engine_destroy(pi_engine* engine);
const char* pi_engine_last_error(void);

// Returns the request's id (>= 0).  seed < 0: the engine's own choice.
long pi_engine_add_request(pi_engine* engine, const int* prompt_tokens, int num_tokens, int max_new_tokens,
                           float temperature, long seed, int ignore_eos);
// One scheduled batch; returns how many requests finished during the call.
int pi_engine_step(pi_engine* engine);
int pi_engine_has_work(pi_engine* engine);
int pi_engine_run_until_complete(pi_engine* engine);
// Copies up to `capacity` generated tokens of request `id`; returns how many there are.
int pi_engine_result(pi_engine* engine, long id, int* tokens, int capacity);
// 1 once the request has finished, 0 before.
int pi_engine_finished(pi_engine* engine, long id);

#ifdef __cplusplus
}  // extern "C"

#include <stdexcept>
#include <string>
#include <vector>

namespace photon {

struct EngineError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct EngineOptions {
  std::string dtype;        // empty: default
  int block_size = 0, num_blocks = 0, max_batch = 0, max_step_tokens = 0, chunk_size = 0, max_model_len = 0;
};

struct SamplingParams {
  int max_new_tokens = 128;
  float temperature = 0.0f;   // 0: greedy
  long seed = -1;
  bool ignore_eos = false;
};

class Engine {
 public:
  static Engine create(const std::string& model_dir, const EngineOptions& o = EngineOptions()) {
    pi_engine_options c{};
    c.dtype = o.dtype.empty() ? nullptr : o.dtype.c_str();
    c.block_size = o.block_size; c.num_blocks = o.num_blocks; c.max_batch = o.max_batch;
    c.max_step_tokens = o.max_step_tokens; c.chunk_size = o.chunk_size; c.max_model_len = o.max_model_len;
    pi_engine* h = pi_engine_create(model_dir.c_str(), &c);
    if (!h) throw EngineError(pi_engine_last_error());
    return Engine(h);
  }
  Engine(Engine&& other) noexcept : h_(other.h_) { other.h_ = nullptr; }
  Engine& operator=(Engine&& other) noexcept {
    if (this != &other) { if (h_) pi_engine_destroy(h_); h_ = other.h_; other.h_ = nullptr; }
    return *this;
  }
  Engine(const Engine&) = delete;
  Engine& operator=(const Engine&) = delete;
  ~Engine() { if (h_) pi_engine_destroy(h_); }

  long add_request(const std::vector<int>& prompt_tokens, const SamplingParams& p = SamplingParams()) {
    return check(pi_engine_add_request(h_, prompt_tokens.data(), (int)prompt_tokens.size(), p.max_new_tokens, p.temperature,
                                       p.seed, p.ignore_eos));
  }
  int step() { return (int)check(pi_engine_step(h_)); }
  bool has_work() { return check(pi_engine_has_work(h_)) != 0; }
  void run_until_complete() { check(pi_engine_run_until_complete(h_)); }
  bool finished(long id) { return check(pi_engine_finished(h_, id)) != 0; }
  std::vector<int> get_result(long id) {
    int n = (int)check(pi_engine_result(h_, id, nullptr, 0));
    std::vector<int> out(n);
    if (n) check(pi_engine_result(h_, id, out.data(), n));
    return out;
  }

 private:
  explicit Engine(pi_engine* h) : h_(h) {}
  static long check(long v) {
    if (v < 0) throw EngineError(pi_engine_last_error());
    return v;
  }
  pi_engine* h_;
};

}  // namespace photon
#endif
