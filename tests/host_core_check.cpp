// The host core under the address and undefined-behaviour sanitizers: random orders of
// requests through the cache manager and the scheduler, with the bookkeeping checked after
// every operation.  Built and run by tests/test_host_sanitizers.py; no GPU.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "cache_manager.h"
#include "scheduler.h"

using namespace denno;

#define REQUIRE(c)                                                       \
  do {                                                                   \
    if (!(c)) {                                                          \
      std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, #c);       \
      std::exit(1);                                                      \
    }                                                                    \
  } while (0)

static void cache_random(unsigned seed, int window) {
  std::mt19937 rng(seed);
  CacheManager m({GroupSpec{kPaged, 24, 8, 0}, GroupSpec{kPaged, 12, 8, window}, GroupSpec{kState, 0, 1, 0}}, 5);
  std::vector<std::pair<int64_t, int>> live;
  int64_t next = 0;
  for (int it = 0; it < 3000; ++it) {
    int op = static_cast<int>(rng() % 100);
    if (op < 25 && live.size() < 5) {
      REQUIRE(m.add(next) >= 0);
      live.push_back({next++, 0});
    } else if (op < 80 && !live.empty()) {
      auto& r = live[rng() % live.size()];
      int n = r.second + 1 + static_cast<int>(rng() % 19);
      if (m.reserve(r.first, n) == kOk) {
        REQUIRE(m.commit(r.first, n) == kOk);
        r.second = n;
        std::vector<int32_t> tab(64);
        REQUIRE(m.block_table(r.first, 0, tab.data(), 64) == (n + 7) / 8);
      }
    } else if (op < 95 && !live.empty()) {
      size_t i = rng() % live.size();
      REQUIRE(m.release(live[i].first) == kOk);
      live.erase(live.begin() + static_cast<long>(i));
    } else {
      REQUIRE(m.release(next + 1000) == kUnknown);
    }
    REQUIRE(m.check() == kOk);
    int held = 0;
    for (auto& r : live) held += m.pages_held(r.first, 0);
    REQUIRE(held + m.free_pages(0) == 24);
  }
}

static void scheduler_random(unsigned seed, int policy) {
  std::mt19937 rng(seed);
  CacheManager cache({GroupSpec{kPaged, 20, 16, 0}}, 4);
  Scheduler s(&cache, 4, 48, 24, policy, 256);
  int64_t next = 0;
  int finished = 0, added = 0;
  for (int it = 0; it < 4000 && (finished < 60); ++it) {
    if (added < 60 && rng() % 3 == 0) {
      int prompt = 1 + static_cast<int>(rng() % 120), max_new = static_cast<int>(rng() % 40);
      int rc = s.add(next, prompt, max_new);
      REQUIRE(rc >= 0 || rc == kNeverFits);
      if (rc >= 0) ++added;
      else ++finished, ++added;
      ++next;
    }
    std::vector<StepEntry> plan;
    std::vector<int64_t> pre;
    s.schedule(&plan, &pre);
    REQUIRE(policy == kPreempt || pre.empty());
    int tokens = 0;
    for (auto& e : plan) {
      tokens += e.count;
      REQUIRE(e.start == s.computed(e.rid) && e.start + e.count <= s.known(e.rid));
      REQUIRE(s.step_done(e.rid, e.count) == kSchedOk);
    }
    REQUIRE(tokens <= 48);
    for (auto& e : plan) {
      if (!e.samples) continue;
      if (s.generated(e.rid) >= 0 && s.known(e.rid) - s.generated(e.rid) > 0) {
        int rc = s.token_sampled(e.rid);
        if (rc == kSchedBadState) {        // max_new was 0: the prompt is computed and that is all
          REQUIRE(s.finish(e.rid) == kSchedOk);
          ++finished;
        } else if (rc == 1 || rng() % 50 == 0) {   // its last token, or an end-of-sequence token
          REQUIRE(s.finish(e.rid) == kSchedOk);
          ++finished;
        }
      }
    }
    REQUIRE(cache.check() == kOk);
    REQUIRE(plan.size() > 0 || s.n_running() + s.n_waiting() == 0 || added < 60);
  }
  REQUIRE(finished == 60);
  REQUIRE(cache.live() == 0 && cache.free_pages(0) == 20);
}

int main() {
  for (unsigned seed = 0; seed < 6; ++seed) cache_random(seed, seed % 2 ? 20 : 0);
  for (unsigned seed = 0; seed < 6; ++seed) scheduler_random(seed, static_cast<int>(seed % 2));
  std::puts("host core ok");
  return 0;
}
