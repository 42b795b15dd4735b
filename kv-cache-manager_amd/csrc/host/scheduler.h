// Continuous batching, first come first served, with preemption by recomputation.
//
// A step is planned in three passes over one token budget:
//   pages     every active request gets the page its next token needs; when the pool is empty the
//             youngest active request gives its pages back and queues again at the front (its
//             tokens stay, its keys are computed again later);
//   active    requests that decode take one token each (all of them, before anything else is
//             counted against the budget); requests still inside their prompt take a portion;
//   queue     requests are admitted strictly in arrival order while sequences, tokens and pages
//             allow; a request that could never fit an empty pool is retired without a token.
// A portion is the part of a request's uncomputed tokens that runs in one step.  Its size is
// bounded by `prefill_chunk`; 0 means portions are never cut, and then a portion is everything that
// is left, a request enters a step only if all of it fits the budget (or the step is empty), and
// every plan equals the reference scheduler's (src/core/scheduler.cpp:25-105).  A portion that does
// not reach the request's last token samples nothing.
#pragma once
#include <cstdint>
#include <deque>
#include <limits>
#include <memory>
#include <stdexcept>
#include <utility>
#include <vector>

#include "kv_manager.h"

namespace kvcm {

struct SchedulerConfig {
  int max_num_seqs = 256, max_batched_tokens = 4096;   // most active requests; token budget of a step
  int prefill_chunk = 0;                               // 0 = prompts are never cut
  int eos_id = -1;                                     // >= 0: a sampled token equal to it ends the request
};

// What one step runs of one request: tokens [first, first + count).
struct PlannedRun {
  Sequence* request;
  int first, count;
  bool given;     // the tokens were given to the engine (prompt, or all of them after a preemption), not sampled by it
  bool samples;   // the run reaches the request's last token, so a token is sampled from its last row
};

struct SchedulerCounters {
  int64_t steps = 0, preemptions = 0, admissions = 0, admission_blocked_steps = 0, rejected = 0;
  int64_t prefill_tokens = 0, decode_tokens = 0, prefill_tokens_saved = 0, batch_size_sum = 0;
  int64_t max_running = 0;
};

class Scheduler {
 public:
  using Owned = std::unique_ptr<Sequence>;

  Scheduler(KVManager& pool, const SchedulerConfig& limits) : pool_(pool), limits_(limits) {}

  void add(Owned request) { queue_.push_back(std::move(request)); }

  const std::vector<PlannedRun>& schedule(double now) {
    runs_.clear();
    tokens_left_ = limits_.max_batched_tokens;
    secure_next_pages();
    plan_active();
    if (admit_from_queue(now) == Held::ByPool) tally_.admission_blocked_steps += 1;
    const int64_t n = static_cast<int64_t>(active_.size());
    tally_.steps += 1;
    tally_.batch_size_sum += n;
    if (n > tally_.max_running) tally_.max_running = n;
    return runs_;
  }

  // sampled[k] belongs to run k of the plan; it is ignored where that run samples nothing.
  void update(const std::vector<int32_t>& sampled, double now) {
    if (sampled.size() < runs_.size()) throw std::invalid_argument("update: one token per plan entry");
    bool some_ended = false;
    for (size_t k = 0; k < runs_.size(); ++k) {
      const PlannedRun& r = runs_[k];
      Sequence& q = *r.request;
      q.num_computed = r.first + r.count;
      pool_.commit(q);
      if (!r.samples) continue;
      const int32_t token = sampled[k];
      q.in_prompt = false;
      q.tokens.push_back(token);
      if (q.first_token < 0) q.first_token = now;
      if (q.done() || q.size() >= pool_.max_seq_len() || (limits_.eos_id >= 0 && token == limits_.eos_id)) {
        q.finished = now;
        some_ended = true;
      }
    }
    if (some_ended) retire_ended();
    runs_.clear();
  }

  std::vector<Owned> take_finished() { return std::exchange(retired_, {}); }

  bool idle() const { return queue_.empty() && active_.empty(); }
  size_t num_waiting() const { return queue_.size(); }
  size_t num_running() const { return active_.size(); }
  const std::vector<PlannedRun>& plan() const { return runs_; }
  // The requests that hold pages, in admission order.
  std::vector<const Sequence*> live() const {
    std::vector<const Sequence*> out(active_.size());
    for (size_t i = 0; i < active_.size(); ++i) out[i] = active_[i].get();
    return out;
  }
  const SchedulerCounters& counters() const { return tally_; }
  void reset_counters() { tally_ = SchedulerCounters{}; }
  const SchedulerConfig& config() const { return limits_; }

 private:
  enum class Held { No, ByPool };

  bool cuts_prompts() const { return limits_.prefill_chunk > 0; }
  // The most tokens of one request a step takes, given what is left of the budget: a prompt that
  // may be cut shrinks to what is left (a new request always gets one token), one that may not is
  // taken whole.
  int portion_limit(int left, int at_least) const {
    if (!cuts_prompts()) return std::numeric_limits<int>::max();
    const int room = left > at_least ? left : at_least;
    return room < limits_.prefill_chunk ? room : limits_.prefill_chunk;
  }
  static int uncomputed(const Sequence& q) { return q.size() - q.num_computed; }

  // Adds a run of `n` tokens of `q` to the plan and books it.
  void take(Sequence& q, int n) {
    runs_.push_back(PlannedRun{&q, q.num_computed, n, q.in_prompt, n == uncomputed(q)});
    tokens_left_ -= n;
    if (q.in_prompt) {
      tally_.prefill_tokens += n;
      q.prefill_tokens_computed += n;
    } else {
      tally_.decode_tokens += n;
    }
  }

  // A page for the next token of every active request, oldest first.  An empty pool takes the
  // pages of the youngest; when that is the request asking, nothing younger is left to ask.
  void secure_next_pages() {
    for (size_t at = 0; at < active_.size();) {
      if (pool_.append_slot(*active_[at])) {
        ++at;
        continue;
      }
      const bool was_asking = at + 1 == active_.size();
      Owned youngest = std::move(active_.back());
      active_.pop_back();
      pool_.release(*youngest);
      youngest->num_preemptions += 1;
      tally_.preemptions += 1;
      queue_.push_front(std::move(youngest));
      if (was_asking) return;
    }
  }

  // Active requests in admission order.  The tokens of decoding requests are set aside first, so
  // that a prompt's portion earlier in the order cannot starve them of budget.
  void plan_active() {
    int for_prompts = tokens_left_;
    for (const Owned& q : active_)
      if (!q->in_prompt) for_prompts -= uncomputed(*q);
    for (const Owned& q : active_) {
      const int open = uncomputed(*q);
      if (!q->in_prompt) {
        take(*q, open);
        continue;
      }
      const int cap = portion_limit(for_prompts, 0);
      const int n = open < cap ? open : cap;
      if (n <= 0) continue;   // no budget left in this step: the request waits with its pages
      take(*q, n);
      for_prompts -= n;
    }
  }

  // Admits from the front of the queue; says whether the front was held back by the pool (and not
  // by the budget or the limit of active requests).
  Held admit_from_queue(double now) {
    while (!queue_.empty() && static_cast<int>(active_.size()) < limits_.max_num_seqs) {
      Sequence& next = *queue_.front();
      // what the step must still have room for: one token of a prompt that may be cut, all of
      // one that may not; an empty step takes its first request whatever its size
      const int least = cuts_prompts() ? 1 : next.size();
      if (!runs_.empty() && tokens_left_ < least) return Held::No;
      if (!pool_.can_admit(next)) {
        if (!active_.empty()) return Held::ByPool;
        next.finished = now;   // it fits not even an empty pool: retired without a token
        tally_.rejected += 1;
        retired_.push_back(pop_queue());
        continue;
      }
      pool_.admit(next);   // pages for all its tokens; prefix hits move num_computed forward
      if (next.admitted < 0) next.admitted = now;
      next.in_prompt = true;
      tally_.admissions += 1;
      tally_.prefill_tokens_saved += next.cached_tokens;
      const int open = uncomputed(next), cap = portion_limit(tokens_left_, 1);
      take(next, open < cap ? open : cap);
      active_.push_back(pop_queue());
    }
    return Held::No;
  }

  Owned pop_queue() {
    Owned front = std::move(queue_.front());
    queue_.pop_front();
    return front;
  }

  // Requests whose `finished` time is set leave the active list (order kept) and give their pages back.
  void retire_ended() {
    size_t kept = 0;
    for (size_t i = 0; i < active_.size(); ++i) {
      if (active_[i]->finished >= 0) {
        pool_.release(*active_[i]);
        retired_.push_back(std::move(active_[i]));
      } else {
        if (kept != i) active_[kept] = std::move(active_[i]);
        ++kept;
      }
    }
    active_.resize(kept);
  }

  KVManager& pool_;
  SchedulerConfig limits_;
  std::deque<Owned> queue_;      // arrival order; a preempted request goes to the front
  std::vector<Owned> active_;    // admission order, back = youngest
  std::vector<Owned> retired_;
  std::vector<PlannedRun> runs_;
  int tokens_left_ = 0;
  SchedulerCounters tally_;
};

}  // namespace kvcm
