// Iteration-level scheduler: which tokens of which requests the next step runs.
//
// After the reference's ContinuousScheduler (csrc/include/engine/scheduler.hpp:
// 12-53, csrc/engine/scheduler.cpp:7-138) and Sequence (sequence.hpp:11-88):
// a FIFO of waiting requests, a list of running ones, a budget of tokens and of
// requests per step, pages taken from the cache manager, finishing on an
// end-of-sequence token or on max_tokens, preemption by recomputation when the
// pages run out.  Differences, each on purpose:
//   * a step mixes single decoded tokens with portions of prompts, and new
//     requests are admitted while others run (the reference runs either all
//     prompts or all decodes, scheduler.cpp:43-70, 72-99);
//   * a prompt longer than the budget is cut into portions instead of blocking
//     the queue (scheduler.cpp:81-83);
//   * a preempted request recomputes its prompt and the tokens it has already
//     produced, and then goes on after them (the reference recomputes the
//     prompt only, scheduler.cpp:55-64);
//   * the victim of a preemption is the request admitted last;
//   * a request that can never fit is refused when it is added.
#pragma once

#include <cstdint>
#include <deque>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "cache_manager.hpp"

namespace lyp {

// The part of a request's sampling parameters (python/lyapunov_engine/engine/sampling.py:6-12,
// sequence.hpp:20-26) that decides when the request ends.  How a token is chosen (temperature,
// top-k, top-p, seed) is the sampler's business and never comes here.
struct StopRule {
  int max_tokens = 128;
  bool ignore_eos = false;
};

enum class Status : int {
  Waiting = 0,
  Running = 1,
  FinishedStopped = 2,       // an end-of-sequence token
  FinishedLengthCapped = 3,  // max_tokens or the model's length
  FinishedAborted = 4,
};

struct Sequence {
  int64_t id = 0;
  std::vector<int32_t> tokens;  // prompt, then what was generated
  int prompt_len = 0;
  int num_computed = 0;  // tokens whose keys are in the cache
  StopRule params;
  Status status = Status::Waiting;
  int preemptions = 0;

  int total_len() const { return static_cast<int>(tokens.size()); }
  int output_len() const { return total_len() - prompt_len; }
  bool finished() const { return static_cast<int>(status) >= static_cast<int>(Status::FinishedStopped); }
};

struct SchedulerConfig {
  int max_num_seqs = 256;
  int max_num_batched_tokens = 4096;
  int max_model_len = 4096;
  int max_chunk = 0;  // longest prompt portion in one step; 0: the budget alone decides
  std::vector<int32_t> eos_token_ids;
};

struct ScheduledEntry {
  int64_t id;
  int start;  // position of the first token of the portion
  int count;
  bool wants_logits;  // the portion ends the request's known tokens: sample after it
};

class Scheduler {
 public:
  Scheduler(SchedulerConfig config, CacheManager* cache);

  // Throws if the id is in use, the prompt is empty, it reaches the model's
  // length, or prompt + max_tokens could not fit in the page pools even alone.
  void add(int64_t id, const std::vector<int32_t>& prompt, const StopRule& params);
  bool abort(int64_t id);
  bool has_unfinished() const { return !waiting_.empty() || !running_.empty(); }
  int num_waiting() const { return static_cast<int>(waiting_.size()); }
  int num_running() const { return static_cast<int>(running_.size()); }

  // Plans the next step and takes its pages.  May preempt.
  std::vector<ScheduledEntry> schedule();
  // The planned step has run.  `sampled` holds one token for every entry that
  // wanted logits, in the order of the plan.
  void post_step(const std::vector<int32_t>& sampled);

  const Sequence& get(int64_t id) const { return *seqs_.at(id); }
  bool known(int64_t id) const { return seqs_.count(id) != 0; }
  void forget(int64_t id);  // drop a finished request's record
  const std::vector<int64_t>& last_preempted() const { return last_preempted_; }
  const std::vector<ScheduledEntry>& plan() const { return plan_; }

  struct Counters {
    int64_t steps = 0, scheduled_tokens = 0, preemptions = 0, finished = 0;
  };
  const Counters& counters() const { return counters_; }
  const SchedulerConfig& config() const { return config_; }

 private:
  using SeqPtr = std::shared_ptr<Sequence>;
  void preempt(const SeqPtr& seq);
  void finish(const SeqPtr& seq, Status status);
  bool is_eos(int32_t token) const;

  SchedulerConfig config_;
  CacheManager* cache_;
  std::deque<SeqPtr> waiting_;
  std::vector<SeqPtr> running_;  // in the order they were admitted
  std::unordered_map<int64_t, SeqPtr> seqs_;
  std::vector<ScheduledEntry> plan_;
  std::vector<int64_t> last_preempted_;
  Counters counters_;
};

}  // namespace lyp
