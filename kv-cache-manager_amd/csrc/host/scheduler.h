// Continuous batching, first come first served, with preemption by recomputation.
//
// With prefill_chunk == 0 every plan equals the reference scheduler's
// (src/core/scheduler.cpp:25-105): running sequences get their slot (the youngest is preempted
// when pages run out), each is planned whole, then the waiting queue is admitted strictly in
// order while tokens, sequences and pages allow.  With prefill_chunk > 0 a prompt is cut into
// portions of at most that many tokens and at most what is left of the step's token budget;
// decodes are served first, then unfinished prompts that already run (oldest first), then new
// admissions.  A portion that does not reach the sequence's last token samples nothing.
#pragma once
#include <algorithm>
#include <cstdint>
#include <deque>
#include <memory>
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
  bool is_prefill;
  bool samples;  // the run reaches the last token, so a token is sampled from its last row
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
    // 1) every running sequence needs room for all its tokens; when the pool is empty the
    //    youngest running sequence (possibly the one asking) loses its pages and waits again.
    for (size_t i = 0; i < running_.size();) {
      if (kv_.append_slot(*running_[i])) {
        ++i;
      } else {
        const bool self = i + 1 >= running_.size();
        preempt_youngest();
        if (self) break;
      }
    }
    int budget = cfg_.max_batched_tokens;
    const bool chunked = cfg_.prefill_chunk > 0;
    if (!chunked) {
      for (auto& s : running_) {
        const int n = s->size() - s->num_computed;
        plan_.push_back({s.get(), s->num_computed, n, false, true});
        budget -= n;
        ctr_.decode_tokens += n;
      }
    } else {
      for (auto& s : running_)
        if (s->size() - s->num_computed == 1) --budget;
      for (auto& s : running_) {
        const int rest = s->size() - s->num_computed;
        if (rest == 1) {
          plan_.push_back({s.get(), s->num_computed, 1, false, true});
          ++ctr_.decode_tokens;
        } else {
          const int n = std::min({rest, cfg_.prefill_chunk, std::max(budget, 0)});
          if (n <= 0) continue;
          plan_.push_back({s.get(), s->num_computed, n, true, n == rest});
          budget -= n;
          ctr_.prefill_tokens += n;
          s->prefill_tokens_computed += n;
        }
      }
    }

    // 2) admissions, strictly in arrival order
    bool blocked = false;
    while (!waiting_.empty() && static_cast<int>(running_.size()) < cfg_.max_num_seqs) {
      Sequence& head = *waiting_.front();
      const int len = head.size();
      if (!plan_.empty() && (chunked ? budget <= 0 : len > budget)) break;
      if (!kv_.can_admit(head)) {
        if (running_.empty()) {  // it can never fit: drop it, the next one may
          head.finished = now;
          ++ctr_.rejected;
          finished_.push_back(std::move(waiting_.front()));
          waiting_.pop_front();
          continue;
        }
        blocked = true;
        break;
      }
      kv_.admit(head);
      if (head.admitted < 0) head.admitted = now;
      const int rest = len - head.num_computed;
      const int n = chunked ? std::min({rest, cfg_.prefill_chunk, std::max(budget, 1)}) : rest;
      plan_.push_back({&head, head.num_computed, n, true, n == rest});
      budget -= n;
      ctr_.prefill_tokens += n;
      ctr_.prefill_tokens_saved += head.cached_tokens;
      head.prefill_tokens_computed += n;
      ++ctr_.admissions;
      running_.push_back(std::move(waiting_.front()));
      waiting_.pop_front();
    }
    if (blocked) ++ctr_.admission_blocked_steps;
    ++ctr_.steps;
    ctr_.batch_size_sum += static_cast<int64_t>(running_.size());
    ctr_.max_running = std::max(ctr_.max_running, static_cast<int>(running_.size()));
    return plan_;
  }

  // next_tokens[i] belongs to plan entry i; it is ignored where that entry samples nothing.
  void update(const std::vector<int32_t>& next_tokens, double now) {
    if (next_tokens.size() < plan_.size()) throw std::invalid_argument("update: one token per plan entry");
    for (size_t i = 0; i < plan_.size(); ++i) {
      Sequence& s = *plan_[i].seq;
      s.num_computed = plan_[i].start + plan_[i].num_tokens;
      kv_.commit(s);
      if (!plan_[i].samples) continue;
      s.tokens.push_back(next_tokens[i]);
      if (s.first_token < 0) s.first_token = now;
      const bool eos = cfg_.eos_id >= 0 && next_tokens[i] == cfg_.eos_id;
      if (s.done() || eos || s.size() >= kv_.max_seq_len()) s.finished = now;
    }
    for (auto it = running_.begin(); it != running_.end();) {
      if ((*it)->finished >= 0) {
        kv_.release(**it);
        finished_.push_back(std::move(*it));
        it = running_.erase(it);
      } else {
        ++it;
      }
    }
    plan_.clear();
  }

  std::vector<std::unique_ptr<Sequence>> take_finished() {
    std::vector<std::unique_ptr<Sequence>> out;
    out.swap(finished_);
    return out;
  }

  bool idle() const { return waiting_.empty() && running_.empty(); }
  size_t num_waiting() const { return waiting_.size(); }
  size_t num_running() const { return running_.size(); }
  const std::deque<std::unique_ptr<Sequence>>& running() const { return running_; }
  const std::vector<ScheduledSeq>& plan() const { return plan_; }
  std::vector<const Sequence*> live() const {
    std::vector<const Sequence*> v;
    for (const auto& s : running_) v.push_back(s.get());
    return v;
  }
  const SchedulerCounters& counters() const { return ctr_; }
  void reset_counters() { ctr_ = {}; }
  KVManager& kv() { return kv_; }
  const SchedulerConfig& config() const { return cfg_; }

 private:
  void preempt_youngest() {
    std::unique_ptr<Sequence> victim = std::move(running_.back());
    running_.pop_back();
    kv_.release(*victim);  // its tokens stay, its keys are computed again later
    ++victim->num_preemptions;
    ++ctr_.preemptions;
    waiting_.push_front(std::move(victim));
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
