// One request as the host side sees it.  `tokens` is prompt followed by generated tokens; keys
// and values of [0, num_computed) are in the cache; a step computes a run that starts at
// num_computed; a decode is the run of length one.  (Reference: src/core/sequence.h:10-30; the
// per-group tables, the state slot, the sampling fields and the window bookkeeping are additions.)
#pragma once
#include <cstdint>
#include <vector>

namespace kvcm {

struct Sequence {
  int64_t id = 0;
  std::vector<int32_t> tokens;              // prompt, then what was generated
  int prompt_len = 0, max_new_tokens = 0;
  int num_computed = 0;                     // keys and values of [0, num_computed) are in the cache
  // True from admission until a token has been sampled: the runs of that time cover tokens that
  // were given (the prompt, or everything after a preemption), and are booked as prefill.
  bool in_prompt = false;

  // One page table per cache group (empty for groups that hold fixed-size state).  Logical token
  // t of group g lives in page tables[g][t / B]; an entry of -1 is a page that a window has
  // passed and that was given back.
  std::vector<std::vector<int32_t>> tables;
  std::vector<int32_t> released_below;  // per group: pages [0, released_below) were given back
  int state_slot = -1;                  // index into every fixed-state group's slot array

  // Prefix cache: chain hashes of the leading full pages that are registered or were hit, and
  // the tokens skipped at the last admission thanks to hits.
  std::vector<uint64_t> page_hashes;
  int cached_tokens = 0;

  // Sampling (the reference samples greedily only).
  float temperature = 0.f;
  uint64_t sampler_seed = 0;

  // Clock values of the engine; -1 = has not happened.  first_token < 0 at finish = rejected.
  double arrival = 0;
  double admitted = -1, first_token = -1, finished = -1;
  int num_preemptions = 0;
  int64_t prefill_tokens_computed = 0, prefill_tokens_saved = 0;

  int size() const { return static_cast<int>(tokens.size()); }
  int num_generated() const { return size() - prompt_len; }
  bool done() const { return size() - prompt_len >= max_new_tokens; }
};

}  // namespace kvcm
