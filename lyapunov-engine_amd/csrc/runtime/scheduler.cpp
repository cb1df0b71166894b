#include "scheduler.hpp"

#include <algorithm>
#include <stdexcept>

namespace lyp {

Scheduler::Scheduler(SchedulerConfig config, CacheManager* cache) : config_(std::move(config)), cache_(cache) {
  if (!cache_) throw std::invalid_argument("scheduler needs a cache manager");
  if (config_.max_num_seqs <= 0 || config_.max_num_batched_tokens <= 0 || config_.max_model_len <= 0)
    throw std::invalid_argument("scheduler limits must be positive");
}

void Scheduler::add(int64_t id, const std::vector<int32_t>& prompt, const StopRule& params) {
  if (seqs_.count(id)) throw std::runtime_error("request id " + std::to_string(id) + " is in use");
  if (prompt.empty()) throw std::runtime_error("empty prompt");
  const int prompt_len = static_cast<int>(prompt.size());
  if (prompt_len >= config_.max_model_len)
    throw std::runtime_error("prompt of " + std::to_string(prompt_len) + " tokens leaves no room under max_model_len " +
                             std::to_string(config_.max_model_len));
  if (params.max_tokens <= 0) throw std::runtime_error("max_tokens must be positive");
  // A request that could not finish even with every page to itself would be
  // preempted for ever (the reference lets such a prompt block the queue,
  // csrc/engine/scheduler.cpp:81-83).
  const int64_t reach = std::min<int64_t>(static_cast<int64_t>(prompt_len) + params.max_tokens, config_.max_model_len);
  const int portion = config_.max_chunk > 0 ? std::min(config_.max_chunk, config_.max_num_batched_tokens)
                                            : config_.max_num_batched_tokens;
  for (int g = 0; g < cache_->num_groups(); ++g) {
    const int need = cache_->pages_held_at_most(g, static_cast<int>(reach), portion);
    if (need > cache_->group(g).num_pages)
      throw std::runtime_error("request needs " + std::to_string(need) + " pages of cache group " + std::to_string(g) +
                               ", which has " + std::to_string(cache_->group(g).num_pages));
  }
  auto seq = std::make_shared<Sequence>();
  seq->id = id;
  seq->tokens = prompt;
  seq->prompt_len = prompt_len;
  seq->params = params;
  seqs_[id] = seq;
  waiting_.push_back(seq);
}

bool Scheduler::abort(int64_t id) {
  auto it = seqs_.find(id);
  if (it == seqs_.end() || it->second->finished()) return false;
  SeqPtr seq = it->second;
  if (seq->status == Status::Running) {
    cache_->free(id);
    running_.erase(std::find(running_.begin(), running_.end(), seq));
  } else {
    waiting_.erase(std::find(waiting_.begin(), waiting_.end(), seq));
  }
  seq->status = Status::FinishedAborted;
  return true;
}

void Scheduler::forget(int64_t id) {
  auto it = seqs_.find(id);
  if (it != seqs_.end() && it->second->finished()) seqs_.erase(it);
}

void Scheduler::preempt(const SeqPtr& seq) {
  cache_->free(seq->id);
  running_.erase(std::find(running_.begin(), running_.end(), seq));
  seq->status = Status::Waiting;
  seq->num_computed = 0;
  ++seq->preemptions;
  ++counters_.preemptions;
  waiting_.push_front(seq);
  last_preempted_.push_back(seq->id);
}

void Scheduler::finish(const SeqPtr& seq, Status status) {
  cache_->free(seq->id);
  running_.erase(std::find(running_.begin(), running_.end(), seq));
  seq->status = status;
  ++counters_.finished;
}

bool Scheduler::is_eos(int32_t token) const {
  return std::find(config_.eos_token_ids.begin(), config_.eos_token_ids.end(), token) != config_.eos_token_ids.end();
}

std::vector<ScheduledEntry> Scheduler::schedule() {
  plan_.clear();
  last_preempted_.clear();
  int budget = config_.max_num_batched_tokens;
  auto portion_of = [&](const Sequence& s) {
    int n = std::min(s.total_len() - s.num_computed, budget);
    if (config_.max_chunk > 0) n = std::min(n, config_.max_chunk);
    return n;
  };

  // Running requests first, in the order they were admitted: a decoded token or
  // the next portion of a prompt each.  When pages run out, the request
  // admitted last is preempted; it is never one that already has its portion.
  size_t i = 0;
  while (i < running_.size()) {
    SeqPtr seq = running_[i];
    int n = portion_of(*seq);
    if (n <= 0) {
      ++i;
      continue;  // the budget is spent; the request keeps its pages and waits a step
    }
    bool placed = false;
    while (true) {
      if (cache_->can_extend(seq->id, seq->num_computed + n)) {
        placed = true;
        break;
      }
      if (running_.back() != seq) {
        preempt(running_.back());
        continue;
      }
      const int fit = cache_->max_length(seq->id) - seq->num_computed;
      if (fit >= 1 && fit < n) {
        n = fit;  // a shorter portion of the prompt
        continue;
      }
      preempt(seq);
      break;
    }
    if (!placed) break;  // seq was the last running request and is gone
    cache_->extend(seq->id, seq->num_computed + n);
    plan_.push_back({seq->id, seq->num_computed, n, seq->num_computed + n == seq->total_len()});
    budget -= n;
    ++i;
  }

  // Then new requests, oldest first, while requests, tokens and pages allow.
  // Nothing is admitted in a step that had to preempt.
  const int portion_cap = config_.max_chunk > 0 ? std::min(config_.max_chunk, config_.max_num_batched_tokens)
                                                : config_.max_num_batched_tokens;
  while (last_preempted_.empty() && !waiting_.empty() && static_cast<int>(running_.size()) < config_.max_num_seqs &&
         budget > 0) {
    SeqPtr seq = waiting_.front();
    bool room = cache_->num_free_slots() > 0;
    for (int g = 0; room && g < cache_->num_groups(); ++g)
      room = cache_->pages_held_at_most(g, seq->total_len(), portion_cap) <= cache_->num_free_pages(g);
    if (!room) break;
    const int n = portion_of(*seq);
    waiting_.pop_front();
    cache_->add(seq->id);
    cache_->extend(seq->id, n);
    seq->status = Status::Running;
    running_.push_back(seq);
    plan_.push_back({seq->id, 0, n, n == seq->total_len()});
    budget -= n;
  }

  ++counters_.steps;
  for (const auto& e : plan_) counters_.scheduled_tokens += e.count;
  return plan_;
}

void Scheduler::post_step(const std::vector<int32_t>& sampled) {
  size_t wanted = 0;
  for (const auto& e : plan_) wanted += e.wants_logits;
  // csrc/engine/scheduler.cpp:106-109
  if (wanted != sampled.size())
    throw std::runtime_error("the step planned " + std::to_string(wanted) + " sampled tokens and got " +
                             std::to_string(sampled.size()));
  size_t k = 0;
  for (const auto& e : plan_) {
    const int32_t token = e.wants_logits ? sampled[k++] : -1;
    SeqPtr seq = seqs_.at(e.id);
    if (seq->status != Status::Running) continue;  // aborted since the plan was made
    seq->num_computed += e.count;
    cache_->commit(seq->id, seq->num_computed);
    if (!e.wants_logits) continue;
    seq->tokens.push_back(token);
    // csrc/engine/scheduler.cpp:121-135
    if (!seq->params.ignore_eos && is_eos(token)) {
      finish(seq, Status::FinishedStopped);
    } else if (seq->output_len() >= seq->params.max_tokens || seq->total_len() >= config_.max_model_len) {
      finish(seq, Status::FinishedLengthCapped);
    }
  }
  plan_.clear();
}

}  // namespace lyp
