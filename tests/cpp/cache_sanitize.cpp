// A random workload on the host-side cache manager (csrc/runtime/cache.cpp), meant to be built
// together with it under -fsanitize=address,undefined and run on the CPU: requests are admitted,
// grow by portions and single tokens, and leave in random order, through the same C entry
// points the Python side calls, including calls that must be refused (out of pages, misuse).
// Exit status 0: every invariant held and every refusal left the state unchanged.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

extern "C" {
void* pi_cache_create(int n_groups, const int* windows, int page_size, const int* num_pages, int max_slots, int max_model_len);
void pi_cache_destroy(void* h);
const char* pi_cache_error(void* h);
int pi_cache_free_slots(void* h);
int pi_cache_free_pages(void* h, int g);
int pi_cache_admit(void* h);
int pi_cache_pages_needed(void* h, int slot, int new_tokens, int* out);
int pi_cache_reserve(void* h, int slot, int new_tokens);
int pi_cache_commit(void* h, int slot, int new_tokens);
int pi_cache_release(void* h, int slot);
int pi_cache_reserve_many(void* h, const int* slots, const int* new_tokens, int n);
int pi_cache_commit_many(void* h, const int* slots, const int* new_tokens, int n);
int pi_cache_check(void* h);
int32_t* pi_cache_lengths(void* h);
void* pi_pool_create(int num_pages);
void pi_pool_destroy(void* h);
int pi_pool_allocate(void* h, int n, int* out);
int pi_pool_free(void* h, const int* pages, int n);
int pi_pool_num_free(void* h);
}

#define REQUIRE(cond)                                                          \
  do {                                                                         \
    if (!(cond)) {                                                             \
      std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond);   \
      return 1;                                                                \
    }                                                                          \
  } while (0)

static int run(unsigned seed) {
  std::mt19937 rng(seed);
  auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (unsigned)(hi - lo + 1)); };
  const int groups = pick(1, 2);
  const int windows[2] = {-1, pick(4, 24)};            // all keys; a window of a few pages
  const int page = 1 << pick(1, 4);
  const int pages[2] = {pick(6, 40), pick(6, 40)};
  const int slots = pick(1, 6), max_len = pick(16, 200);
  void* c = pi_cache_create(groups, windows, page, pages, slots, max_len);
  REQUIRE(c != nullptr);
  std::vector<int> live;
  for (int step = 0; step < 400; ++step) {
    const int what = pick(0, 9);
    if (what < 2 && pi_cache_free_slots(c) > 0) {
      const int s = pi_cache_admit(c);
      REQUIRE(s >= 0 && s < slots);
      live.push_back(s);
    } else if (what < 3 && !live.empty()) {
      const int i = pick(0, (int)live.size() - 1);
      REQUIRE(pi_cache_release(c, live[i]) == 0);
      REQUIRE(pi_cache_release(c, live[i]) == 2);        // a second release is misuse and changes nothing
      live.erase(live.begin() + i);
    } else if (what < 8 && !live.empty()) {
      const int s = live[pick(0, (int)live.size() - 1)];
      const int n = pick(0, 3) ? 1 : pick(2, 3 * page);
      const int before = pi_cache_free_pages(c, 0);
      const int rc = pi_cache_reserve(c, s, n);
      REQUIRE(rc == 0 || rc == 1 || rc == 2);
      if (rc == 0) REQUIRE(pi_cache_commit(c, s, n) == 0);
      else REQUIRE(pi_cache_free_pages(c, 0) == before);  // refused: nothing was taken
    } else if (!live.empty()) {
      std::vector<int> ss(live), nn(live.size(), 1);      // a whole decode step, all or nothing
      const int before = pi_cache_free_pages(c, 0);
      const int rc = pi_cache_reserve_many(c, ss.data(), nn.data(), (int)ss.size());
      if (rc == 0) REQUIRE(pi_cache_commit_many(c, ss.data(), nn.data(), (int)ss.size()) == 0);
      else REQUIRE(pi_cache_free_pages(c, 0) == before);
    }
    REQUIRE(pi_cache_release(c, slots + 3) == 2 && pi_cache_reserve(c, -1, 1) == 2);   // ids outside the slots
    if (pi_cache_check(c) != 0) {
      std::fprintf(stderr, "seed %u step %d: %s\n", seed, step, pi_cache_error(c));
      return 1;
    }
  }
  for (int s : live) REQUIRE(pi_cache_release(c, s) == 0);
  for (int g = 0; g < groups; ++g) REQUIRE(pi_cache_free_pages(c, g) == pages[g]);
  REQUIRE(pi_cache_free_slots(c) == slots && pi_cache_check(c) == 0);
  pi_cache_destroy(c);

  void* p = pi_pool_create(9);
  int got[9], twice[2];
  REQUIRE(pi_pool_allocate(p, 9, got) == 0 && pi_pool_allocate(p, 1, twice) == 1);
  twice[0] = twice[1] = got[4];
  REQUIRE(pi_pool_free(p, twice, 2) == 2 && pi_pool_num_free(p) == 0);   // named twice in one call: refused whole
  REQUIRE(pi_pool_free(p, got, 9) == 0 && pi_pool_free(p, got, 1) == 2 && pi_pool_num_free(p) == 9);
  pi_pool_destroy(p);
  return 0;
}

int main(int argc, char** argv) {
  const int seeds = argc > 1 ? std::atoi(argv[1]) : 50;
  for (int s = 0; s < seeds; ++s)
    if (run(1000u + (unsigned)s)) return 1;
  std::printf("ok %d seeds\n", seeds);
  return 0;
}
