// A program that drives the cache manager and the scheduler with random requests, windows, small
// pools (so that requests are preempted and pages used again), aborts and end-of-sequence tokens,
// and checks the manager's invariants after every step.  Built with address and undefined-behaviour
// sanitizers (kernels/build.py, LYAPUNOV_AMD_SANITIZE=1) it is what runs the host runtime under
// them: a library loaded into an unsanitized interpreter cannot be.  The reference compiles its
// runtime with -Wall -Wextra only (setup.py:54).
//
//   runtime_selftest [rounds] [seed]        exit code 0: every check held
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <stdexcept>

#include "cache_manager.hpp"
#include "scheduler.hpp"

using namespace lyp;

#define EXPECT(cond, ...)                  \
  do {                                     \
    if (!(cond)) {                         \
      std::fprintf(stderr, "selftest: "); \
      std::fprintf(stderr, __VA_ARGS__);   \
      std::fprintf(stderr, "\n");         \
      return 1;                            \
    }                                      \
  } while (0)

static long long g_steps = 0, g_preemptions = 0, g_finished = 0, g_refused = 0, g_window_returns = 0;

static int one_round(std::mt19937& rng) {
  auto pick = [&](int lo, int hi) { return std::uniform_int_distribution<int>(lo, hi)(rng); };
  const int page = 1 << pick(0, 4);
  const int pages = pick(6, 40);
  const int window = pick(0, 2) == 0 ? pick(2, 3 * page) : 0;
  std::vector<GroupSpec> groups{{pages, page, 0}};
  if (window) groups.push_back({pages, page, window});
  CacheManager cache(groups, pick(2, 6));
  SchedulerConfig cfg;
  cfg.max_num_seqs = pick(1, 6);
  cfg.max_num_batched_tokens = pick(4, 64);
  cfg.max_model_len = pick(8, std::max(8, pages * page));
  cfg.max_chunk = pick(0, 1) ? pick(2, 16) : 0;
  cfg.eos_token_ids = {7};
  Scheduler sched(cfg, &cache);

  int64_t next_id = 0;
  int refused = 0, finished = 0;
  for (int step = 0; step < 400; ++step) {
    if (pick(0, 3) == 0) {
      std::vector<int32_t> prompt(pick(1, cfg.max_model_len + 2));
      for (auto& t : prompt) t = pick(8, 99);
      StopRule sp;
      sp.max_tokens = pick(1, 24);
      sp.ignore_eos = pick(0, 1) != 0;
      try {
        sched.add(next_id, prompt, sp);
      } catch (const std::exception&) {
        ++refused;  // too long for the model or for the pool: refused with a reason, nothing held
      }
      ++next_id;
    }
    if (next_id > 0 && pick(0, 15) == 0) {
      const int64_t victim = pick(0, static_cast<int>(next_id) - 1);
      if (sched.known(victim) && !sched.get(victim).finished()) {
        sched.abort(victim);
        sched.forget(victim);
      }
    }
    if (!sched.has_unfinished()) continue;
    const auto plan = sched.schedule();
    int tokens = 0, wanting = 0;
    for (const auto& e : plan) {
      EXPECT(e.count >= 1 && e.start == cache.length(e.id), "request %lld planned at %d, its cache holds %d",
             static_cast<long long>(e.id), e.start, cache.length(e.id));
      EXPECT(cache.capacity(e.id) >= e.start + e.count, "request %lld has no pages for its portion",
             static_cast<long long>(e.id));
      tokens += e.count;
      wanting += e.wants_logits ? 1 : 0;
    }
    EXPECT(tokens <= cfg.max_num_batched_tokens, "%d tokens in a step of at most %d", tokens, cfg.max_num_batched_tokens);
    EXPECT(static_cast<int>(plan.size()) <= cfg.max_num_seqs, "%zu requests in a step", plan.size());
    std::vector<int32_t> sampled(wanting);
    for (auto& t : sampled) t = pick(0, 40) == 0 ? 7 : pick(8, 99);
    sched.post_step(sampled);
    for (const auto& e : plan)
      if (sched.known(e.id) && sched.get(e.id).finished()) {
        EXPECT(!cache.has(e.id), "a finished request still holds pages");
        sched.forget(e.id);
        ++finished;
      }
    const std::string broken = cache.check();
    EXPECT(broken.empty(), "step %d: %s", step, broken.c_str());
  }
  // run dry: nothing new, everything ends, every page comes back
  // (portions of two tokens and a pool that forces recomputation make this take thousands of steps)
  for (int step = 0; step < 200000 && sched.has_unfinished(); ++step) {
    const auto plan = sched.schedule();
    int wanting = 0;
    for (const auto& e : plan) wanting += e.wants_logits ? 1 : 0;
    std::vector<int32_t> sampled(wanting, 9);
    sched.post_step(sampled);
  }
  EXPECT(!sched.has_unfinished(), "requests left after 200000 more steps");
  EXPECT(cache.num_requests() == 0, "%d requests still hold something", cache.num_requests());
  for (int g = 0; g < cache.num_groups(); ++g)
    EXPECT(cache.num_free_pages(g) == pages, "group %d: %d of %d pages came back", g, cache.num_free_pages(g), pages);
  EXPECT(cache.check().empty(), "%s", cache.check().c_str());
  g_steps += sched.counters().steps;
  g_preemptions += sched.counters().preemptions;
  g_finished += finished;
  g_refused += refused;
  g_window_returns += cache.counters().window_returns;
  return 0;
}

int main(int argc, char** argv) {
  const int rounds = argc > 1 ? std::atoi(argv[1]) : 50;
  std::mt19937 rng(argc > 2 ? std::atoi(argv[2]) : 1);
  for (int r = 0; r < rounds; ++r) {
    try {
      if (one_round(rng) != 0) {
        std::fprintf(stderr, "selftest: round %d failed\n", r);
        return 1;
      }
    } catch (const std::exception& e) {
      std::fprintf(stderr, "selftest: round %d threw: %s\n", r, e.what());
      return 1;
    }
  }
  std::printf("selftest: %d rounds, every check held (%lld steps, %lld requests finished, %lld preempted, %lld refused, "
              "%lld pages given back by windows)\n", rounds, g_steps, g_finished, g_preemptions, g_refused, g_window_returns);
  return 0;
}
