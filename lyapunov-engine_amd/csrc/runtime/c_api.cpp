// C interface of the host runtime (cache manager and scheduler), for ctypes.
// The reference binds the same two classes with pybind11
// (csrc/bindings.cpp:552-621).  Every function returns 0 (or a value >= 0) on
// success and a negative number on failure, with the message kept for
// lyp_rt_last_error().
#include <cstring>
#include <exception>
#include <string>

#include "cache_manager.hpp"
#include "scheduler.hpp"

namespace {
thread_local std::string g_error;

template <typename F>
int guarded(F&& f) {
  try {
    return f();
  } catch (const std::exception& e) {
    g_error = e.what();
    return -1;
  } catch (...) {
    g_error = "unknown error";
    return -1;
  }
}

int copy_out(const std::vector<int32_t>& v, int32_t* out, int cap) {
  const int n = static_cast<int>(v.size());
  if (out) std::memcpy(out, v.data(), sizeof(int32_t) * static_cast<size_t>(std::min(n, cap)));
  return n;
}
}  // namespace

using lyp::CacheManager;
using lyp::Scheduler;

extern "C" {

const char* lyp_rt_last_error() { return g_error.c_str(); }

// ------------------------------------------------------------- cache manager
void* lyp_cache_create(int num_groups, const int* num_pages, const int* page_size, const int* window,
                       int num_state_slots) {
  try {
    std::vector<lyp::GroupSpec> groups(num_groups);
    for (int g = 0; g < num_groups; ++g) groups[g] = {num_pages[g], page_size[g], window[g]};
    return new CacheManager(std::move(groups), num_state_slots);
  } catch (const std::exception& e) {
    g_error = e.what();
    return nullptr;
  }
}
void lyp_cache_destroy(void* h) { delete static_cast<CacheManager*>(h); }

int lyp_cache_add(void* h, int64_t id) {
  return guarded([&] { return static_cast<CacheManager*>(h)->add(id); });
}
int lyp_cache_has(void* h, int64_t id) { return static_cast<CacheManager*>(h)->has(id) ? 1 : 0; }
int lyp_cache_length(void* h, int64_t id) {
  return guarded([&] { return static_cast<CacheManager*>(h)->length(id); });
}
int lyp_cache_capacity(void* h, int64_t id) {
  return guarded([&] { return static_cast<CacheManager*>(h)->capacity(id); });
}
int lyp_cache_can_extend(void* h, int64_t id, int new_len) {
  return guarded([&] { return static_cast<CacheManager*>(h)->can_extend(id, new_len) ? 1 : 0; });
}
int lyp_cache_max_length(void* h, int64_t id) {
  return guarded([&] { return static_cast<CacheManager*>(h)->max_length(id); });
}
int lyp_cache_extend(void* h, int64_t id, int new_len) {
  return guarded([&] {
    static_cast<CacheManager*>(h)->extend(id, new_len);
    return 0;
  });
}
int lyp_cache_commit(void* h, int64_t id, int new_len) {
  return guarded([&] {
    static_cast<CacheManager*>(h)->commit(id, new_len);
    return 0;
  });
}
int lyp_cache_free(void* h, int64_t id) {
  return guarded([&] {
    static_cast<CacheManager*>(h)->free(id);
    return 0;
  });
}
int lyp_cache_reset(void* h) {
  return guarded([&] {
    static_cast<CacheManager*>(h)->reset();
    return 0;
  });
}
int lyp_cache_num_free_pages(void* h, int g) {
  return guarded([&] { return static_cast<CacheManager*>(h)->num_free_pages(g); });
}
int lyp_cache_num_free_slots(void* h) { return static_cast<CacheManager*>(h)->num_free_slots(); }
int lyp_cache_num_requests(void* h) { return static_cast<CacheManager*>(h)->num_requests(); }
int lyp_cache_state_slot(void* h, int64_t id) {
  return guarded([&] { return static_cast<CacheManager*>(h)->state_slot(id); });
}
// Copies up to `cap` entries; returns the table's length.
int lyp_cache_table(void* h, int64_t id, int g, int32_t* out, int cap) {
  return guarded([&] { return copy_out(static_cast<CacheManager*>(h)->table(id, g), out, cap); });
}
// For n requests at once: row b of `tables` (each `width` wide) receives the
// block table of ids[b] in group g, as far as it goes; `slots`, if given, the
// state slots.  Entries past a table's length are left alone.
int lyp_cache_export(void* h, const int64_t* ids, int n, int g, int32_t* tables, int width, int32_t* slots) {
  return guarded([&] {
    auto* m = static_cast<CacheManager*>(h);
    for (int b = 0; b < n; ++b) {
      const auto& t = m->table(ids[b], g);
      if (static_cast<int>(t.size()) > width) throw std::runtime_error("block table wider than the caller's rows");
      std::memcpy(tables + static_cast<size_t>(b) * width, t.data(), sizeof(int32_t) * t.size());
      if (slots) slots[b] = m->state_slot(ids[b]);
    }
    return 0;
  });
}
// The tables of one step.  Request ids[b] continues at position start[b] with
// count[b] new tokens: it must be known, hold exactly start[b] tokens and have
// pages for start[b] + count[b].  Row b of `tables` (`width` entries a row, at
// least as many as the longest request needs after the step) gets the block
// table in group g, -1 past its end; slot_map, for each new token in order, the
// page slot (page * page size + offset) its key and value go to; `slots`, if
// given, the state slots.
int lyp_cache_step_tables(void* h, const int64_t* ids, const int32_t* start, const int32_t* count, int n, int g,
                          int32_t* tables, int width, int32_t* slot_map, int32_t* slots) {
  return guarded([&] {
    auto* m = static_cast<CacheManager*>(h);
    const int ps = m->group(g).page_size;
    size_t at = 0;
    for (int b = 0; b < n; ++b) {
      const std::string who = "request " + std::to_string(ids[b]);
      if (!m->has(ids[b])) throw std::runtime_error(who + " is not known to the cache manager");
      if (count[b] < 1) throw std::runtime_error(who + " brings no tokens");
      if (start[b] != m->length(ids[b]))
        throw std::runtime_error(who + " continues at " + std::to_string(start[b]) + " but its cache holds " +
                                 std::to_string(m->length(ids[b])) + " tokens");
      const int end = start[b] + count[b];
      if (end > m->capacity(ids[b]))
        throw std::runtime_error(who + " has pages for " + std::to_string(m->capacity(ids[b])) +
                                 " tokens, the step needs " + std::to_string(end));
      const auto& t = m->table(ids[b], g);
      const int need = (end + ps - 1) / ps;
      if (need > width || need > static_cast<int>(t.size()))
        throw std::runtime_error(who + ": a block table row of " + std::to_string(width) + " entries for " +
                                 std::to_string(need) + " pages");
      int32_t* row = tables + static_cast<size_t>(b) * width;
      const int have = std::min(width, static_cast<int>(t.size()));
      std::memcpy(row, t.data(), sizeof(int32_t) * static_cast<size_t>(have));
      for (int i = have; i < width; ++i) row[i] = -1;
      for (int pos = start[b]; pos < end; ++pos) {
        const int32_t page = row[pos / ps];
        if (page < 0)
          throw std::runtime_error(who + " has no page for one of its new tokens in cache group " + std::to_string(g));
        slot_map[at++] = page * ps + pos % ps;
      }
      if (slots) slots[b] = m->state_slot(ids[b]);
    }
    return 0;
  });
}
// Pages for positions < new_lens[b] of every request ids[b], all or none: 1 if they are held now,
// 0 (and nothing taken) if some group lacks the pages.  For a caller that prepares the step after
// the one the scheduler planned.
int lyp_cache_reserve(void* h, const int64_t* ids, const int32_t* new_lens, int n) {
  return guarded([&] {
    auto* m = static_cast<CacheManager*>(h);
    for (int g = 0; g < m->num_groups(); ++g) {
      long long need = 0;
      for (int b = 0; b < n; ++b)
        if (new_lens[b] > m->capacity(ids[b])) need += m->pages_needed(ids[b], g, new_lens[b]);
      if (need > m->num_free_pages(g)) return 0;
    }
    for (int b = 0; b < n; ++b)
      if (new_lens[b] > m->capacity(ids[b])) m->extend(ids[b], new_lens[b]);
    return 1;
  });
}
int lyp_cache_ref_count(void* h, int g, int page) {
  return guarded([&] { return static_cast<CacheManager*>(h)->ref_count(g, page); });
}
// 0 if every invariant holds; else -1 and the description as the last error.
int lyp_cache_check(void* h) {
  const std::string what = static_cast<CacheManager*>(h)->check();
  if (what.empty()) return 0;
  g_error = what;
  return -1;
}
// out[0..3] = pages taken, pages returned, window returns, high-water mark.
void lyp_cache_counters(void* h, int64_t* out) {
  const auto& c = static_cast<CacheManager*>(h)->counters();
  out[0] = c.pages_taken;
  out[1] = c.pages_returned;
  out[2] = c.window_returns;
  out[3] = c.high_water;
}

// ------------------------------------------------------------------ scheduler
void* lyp_sched_create(void* cache, int max_num_seqs, int max_num_batched_tokens, int max_model_len, int max_chunk,
                       const int32_t* eos_ids, int n_eos) {
  try {
    lyp::SchedulerConfig cfg;
    cfg.max_num_seqs = max_num_seqs;
    cfg.max_num_batched_tokens = max_num_batched_tokens;
    cfg.max_model_len = max_model_len;
    cfg.max_chunk = max_chunk;
    cfg.eos_token_ids.assign(eos_ids, eos_ids + n_eos);
    return new Scheduler(std::move(cfg), static_cast<CacheManager*>(cache));
  } catch (const std::exception& e) {
    g_error = e.what();
    return nullptr;
  }
}
void lyp_sched_destroy(void* h) { delete static_cast<Scheduler*>(h); }

int lyp_sched_add(void* h, int64_t id, const int32_t* prompt, int n, int max_tokens, int ignore_eos) {
  return guarded([&] {
    lyp::StopRule rule;
    rule.max_tokens = max_tokens;
    rule.ignore_eos = ignore_eos != 0;
    static_cast<Scheduler*>(h)->add(id, std::vector<int32_t>(prompt, prompt + n), rule);
    return 0;
  });
}
int lyp_sched_abort(void* h, int64_t id) {
  return guarded([&] { return static_cast<Scheduler*>(h)->abort(id) ? 1 : 0; });
}
int lyp_sched_has_unfinished(void* h) { return static_cast<Scheduler*>(h)->has_unfinished() ? 1 : 0; }
int lyp_sched_num_waiting(void* h) { return static_cast<Scheduler*>(h)->num_waiting(); }
int lyp_sched_num_running(void* h) { return static_cast<Scheduler*>(h)->num_running(); }

// Plans a step.  Fills ids/start/count/wants (each with room for `cap`
// entries) and returns the number of entries, or -1.
int lyp_sched_schedule(void* h, int64_t* ids, int32_t* start, int32_t* count, int32_t* wants, int cap) {
  return guarded([&] {
    const auto plan = static_cast<Scheduler*>(h)->schedule();
    const int n = static_cast<int>(plan.size());
    if (n > cap) throw std::runtime_error("schedule: the plan has more entries than the caller's buffers");
    for (int i = 0; i < n; ++i) {
      ids[i] = plan[i].id;
      start[i] = plan[i].start;
      count[i] = plan[i].count;
      wants[i] = plan[i].wants_logits ? 1 : 0;
    }
    return n;
  });
}
int lyp_sched_post_step(void* h, const int32_t* sampled, int n) {
  return guarded([&] {
    static_cast<Scheduler*>(h)->post_step(std::vector<int32_t>(sampled, sampled + n));
    return 0;
  });
}
// As lyp_sched_post_step; also writes the status of every planned request
// after the step (in the order of the plan) into status_out.
int lyp_sched_post_step_status(void* h, const int32_t* sampled, int n, int32_t* status_out, int cap) {
  return guarded([&] {
    auto* s = static_cast<Scheduler*>(h);
    const auto plan = s->plan();
    if (static_cast<int>(plan.size()) > cap) throw std::runtime_error("post_step: status buffer too small");
    s->post_step(std::vector<int32_t>(sampled, sampled + n));
    for (size_t i = 0; i < plan.size(); ++i) status_out[i] = static_cast<int>(s->get(plan[i].id).status);
    return static_cast<int>(plan.size());
  });
}
// The tokens of the planned portions, one after the other; returns their number.
int lyp_sched_plan_tokens(void* h, int32_t* out, int cap) {
  return guarded([&] {
    auto* s = static_cast<Scheduler*>(h);
    int n = 0;
    for (const auto& e : s->plan()) {
      const auto& seq = s->get(e.id);
      if (n + e.count > cap) throw std::runtime_error("plan_tokens: buffer too small");
      std::memcpy(out + n, seq.tokens.data() + e.start, sizeof(int32_t) * static_cast<size_t>(e.count));
      n += e.count;
    }
    return n;
  });
}
int lyp_sched_last_preempted(void* h, int64_t* out, int cap) {
  const auto& v = static_cast<Scheduler*>(h)->last_preempted();
  const int n = static_cast<int>(v.size());
  for (int i = 0; i < std::min(n, cap); ++i) out[i] = v[i];
  return n;
}
// out = {prompt_len, total_len, num_computed, status, preemptions}
int lyp_sched_info(void* h, int64_t id, int32_t* out) {
  return guarded([&] {
    const auto& s = static_cast<Scheduler*>(h)->get(id);
    out[0] = s.prompt_len;
    out[1] = s.total_len();
    out[2] = s.num_computed;
    out[3] = static_cast<int>(s.status);
    out[4] = s.preemptions;
    return 0;
  });
}
// Copies tokens [from, from + cap) of the request; returns how many were copied.
int lyp_sched_tokens(void* h, int64_t id, int from, int32_t* out, int cap) {
  return guarded([&] {
    const auto& s = static_cast<Scheduler*>(h)->get(id);
    const int n = std::max(0, std::min(cap, s.total_len() - from));
    if (n > 0) std::memcpy(out, s.tokens.data() + from, sizeof(int32_t) * static_cast<size_t>(n));
    return n;
  });
}
int lyp_sched_forget(void* h, int64_t id) {
  return guarded([&] {
    static_cast<Scheduler*>(h)->forget(id);
    return 0;
  });
}
// out[0..3] = steps, scheduled tokens, preemptions, finished.
void lyp_sched_counters(void* h, int64_t* out) {
  const auto& c = static_cast<Scheduler*>(h)->counters();
  out[0] = c.steps;
  out[1] = c.scheduled_tokens;
  out[2] = c.preemptions;
  out[3] = c.finished;
}

}  // extern "C"
