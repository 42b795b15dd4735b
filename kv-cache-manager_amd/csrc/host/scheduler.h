// Continuous batching, first come first served, with preemption by recomputation.
//
// A step is planned in three passes over one token budget:
//   room      every running request gets the page its next token needs; when the pool is empty the
//             youngest running request gives its pages back and waits again (its tokens stay, its
//             keys are computed again later);
//   running   requests that decode take one token each (all of them, before anything else is
//             counted against the budget); requests still inside their prompt take a portion;
//   waiting   the queue is admitted strictly in arrival order while sequences, tokens and pages
//             allow; a request that could never fit an empty pool is finished without a token.
// A portion is the part of a request's uncomputed tokens that runs in one step.  Its size is
// bounded by `prefill_chunk`; 0 means portions are never cut, and then a portion is everything that
// is left, a request enters a step only if all of it fits the budget (or the step is empty), and
// every plan equals the reference scheduler's (src/core/scheduler.cpp:25-105).  A portion that does
// not reach the request's last token samples nothing.
#pragma once
#include <algorithm>
#include <cstdint>
#include <deque>
#include <limits>
#include <memory>
#include <utility>
#include <vector>

#include "kv_manager.h"

namespace kvcm {

struct SchedulerConfig {
  int max_num_seqs = 256;         // most sequences running at once
  int max_batched_tokens = 4096;  // token budget of a step
  int prefill_chunk = 0;          // 0 = prompts are never cut
  int eos_id = -1;                // >= 0: a sampled token equal to it finishes the request
};

struct ScheduledSeq {
  Sequence* seq;
  int start;
  int num_tokens;
  bool is_prefill;  // the run covers tokens that were given (prompt, or all of them after a preemption)
  bool samples;     // the run reaches the last token, so a token is sampled from its last row
};

struct SchedulerCounters {
  int64_t steps = 0, preemptions = 0, admissions = 0, admission_blocked_steps = 0, rejected = 0;
  int64_t prefill_tokens = 0, decode_tokens = 0, prefill_tokens_saved = 0, batch_size_sum = 0;
  int max_running = 0;
};

class Scheduler {
 public:
  Scheduler(KVManager& kv, SchedulerConfig cfg) : kv_(kv), cfg_(cfg) {}

  void add(std::unique_ptr<Sequence> s) { waiting_.push_back(std::move(s)); }

  const std::vector<ScheduledSeq>& schedule(double now) {
    plan_.clear();
    make_room();
    int budget = cfg_.max_batched_tokens;
    plan_running(budget);
    if (admit_waiting(budget, now)) ++ctr_.admission_blocked_steps;
    ++ctr_.steps;
    ctr_.batch_size_sum += static_cast<int64_t>(running_.size());
    ctr_.max_running = std::max(ctr_.max_running, static_cast<int>(running_.size()));
    return plan_;
  }

  // next_tokens[i] belongs to plan entry i; it is ignored where that entry samples nothing.
  void update(const std::vector<int32_t>& next_tokens, double now) {
    if (next_tokens.size() < plan_.size()) throw std::invalid_argument("update: one token per plan entry");
    bool any_finished = false;
    for (size_t i = 0; i < plan_.size(); ++i) {
      const ScheduledSeq& run = plan_[i];
      Sequence& s = *run.seq;
      s.num_computed = run.start + run.num_tokens;
      kv_.commit(s);
      if (!run.samples) continue;
      s.in_prompt = false;
      s.tokens.push_back(next_tokens[i]);
      if (s.first_token < 0) s.first_token = now;
      const bool stop = s.done() || s.size() >= kv_.max_seq_len() || (cfg_.eos_id >= 0 && next_tokens[i] == cfg_.eos_id);
      if (stop) {
        s.finished = now;
        any_finished = true;
      }
    }
    if (any_finished) {
      std::deque<std::unique_ptr<Sequence>> still;
      for (auto& s : running_) {
        if (s->finished < 0) {
          still.push_back(std::move(s));
          continue;
        }
        kv_.release(*s);
        finished_.push_back(std::move(s));
      }
      running_.swap(still);
    }
    plan_.clear();
  }

  std::vector<std::unique_ptr<Sequence>> take_finished() { return std::exchange(finished_, {}); }

  bool idle() const { return waiting_.empty() && running_.empty(); }
  size_t num_waiting() const { return waiting_.size(); }
  size_t num_running() const { return running_.size(); }
  const std::deque<std::unique_ptr<Sequence>>& running() const { return running_; }
  const std::vector<ScheduledSeq>& plan() const { return plan_; }
  std::vector<const Sequence*> live() const {
    std::vector<const Sequence*> v;
    v.reserve(running_.size());
    for (const auto& s : running_) v.push_back(s.get());
    return v;
  }
  const SchedulerCounters& counters() const { return ctr_; }
  void reset_counters() { ctr_ = {}; }
  KVManager& kv() { return kv_; }
  const SchedulerConfig& config() const { return cfg_; }

 private:
  bool cuts_prompts() const { return cfg_.prefill_chunk > 0; }
  // The most tokens of one request a step takes, given what is left of the budget: a prompt that
  // may be cut shrinks to what is left (a new request always gets one token), one that may not is
  // taken whole.
  int portion_limit(int budget_left, int at_least) const {
    if (!cuts_prompts()) return std::numeric_limits<int>::max();
    return std::min(cfg_.prefill_chunk, std::max(budget_left, at_least));
  }
  static int uncomputed(const Sequence& s) { return s.size() - s.num_computed; }

  // Adds a run of `n` tokens of `s` to the plan and books it.
  void take(Sequence& s, int n, int& budget) {
    const bool given = s.in_prompt;   // tokens that were given to the engine, not sampled by it
    plan_.push_back({&s, s.num_computed, n, given, n == uncomputed(s)});
    budget -= n;
    if (given) {
      ctr_.prefill_tokens += n;
      s.prefill_tokens_computed += n;
    } else {
      ctr_.decode_tokens += n;
    }
  }

  // A page for the next token of every running request, oldest first.  The victim of an empty
  // pool is always the youngest; when that is the request asking, nothing younger is left to ask.
  void make_room() {
    size_t i = 0;
    while (i < running_.size()) {
      if (kv_.append_slot(*running_[i])) {
        ++i;
        continue;
      }
      const bool asked_for_itself = i + 1 == running_.size();
      std::unique_ptr<Sequence> victim = std::move(running_.back());
      running_.pop_back();
      kv_.release(*victim);
      ++victim->num_preemptions;
      ++ctr_.preemptions;
      waiting_.push_front(std::move(victim));
      if (asked_for_itself) break;
    }
  }

  // Running requests in admission order.  The tokens of decoding requests are set aside first, so
  // that a prompt's portion earlier in the order cannot starve them of budget.
  void plan_running(int& budget) {
    int decoding = 0;
    for (const auto& s : running_)
      if (!s->in_prompt) decoding += uncomputed(*s);
    int for_prompts = budget - decoding;
    for (auto& s : running_) {
      if (!s->in_prompt) {
        take(*s, uncomputed(*s), budget);
        continue;
      }
      const int n = std::min(uncomputed(*s), portion_limit(for_prompts, 0));
      if (n <= 0) continue;   // no budget left in this step: the request waits with its pages
      take(*s, n, budget);
      for_prompts -= n;
    }
  }

  // Returns true when the head of the queue was held back by the pool (not by the budget).
  bool admit_waiting(int& budget, double now) {
    while (!waiting_.empty() && static_cast<int>(running_.size()) < cfg_.max_num_seqs) {
      Sequence& head = *waiting_.front();
      // what the step must still have room for: one token of a prompt that may be cut, all of
      // one that may not; an empty step takes its first request whatever its size
      const int least = cuts_prompts() ? 1 : head.size();
      if (!plan_.empty() && budget < least) return false;
      if (!kv_.can_admit(head)) {
        if (!running_.empty()) return true;
        head.finished = now;  // it fits not even an empty pool: finished without a token
        ++ctr_.rejected;
        finished_.push_back(std::move(waiting_.front()));
        waiting_.pop_front();
        continue;
      }
      kv_.admit(head);  // pages for all its tokens; prefix hits move num_computed forward
      if (head.admitted < 0) head.admitted = now;
      head.in_prompt = true;
      ++ctr_.admissions;
      ctr_.prefill_tokens_saved += head.cached_tokens;
      take(head, std::min(uncomputed(head), portion_limit(budget, 1)), budget);
      running_.push_back(std::move(waiting_.front()));
      waiting_.pop_front();
    }
    return false;
  }

  KVManager& kv_;
  SchedulerConfig cfg_;
  std::deque<std::unique_ptr<Sequence>> waiting_;
  std::deque<std::unique_ptr<Sequence>> running_;  // admission order, back = youngest
  std::vector<std::unique_ptr<Sequence>> finished_;
  std::vector<ScheduledSeq> plan_;
  SchedulerCounters ctr_;
};

}  // namespace kvcm
