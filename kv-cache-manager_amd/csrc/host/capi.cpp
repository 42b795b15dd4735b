// C interface of the host core (allocator, prefix cache, cache managers, scheduler, batch
// builder) for the Python side.  Every function that can fail returns a negative value (or a
// null handle) and leaves a message for kvcm_last_error().
#include <cstring>
#include <string>
#include <unordered_map>

#include "batch_builder.h"
#include "block_allocator.h"
#include "kv_manager.h"
#include "scheduler.h"
#include "xxhash64.h"

using namespace kvcm;

namespace {

thread_local std::string g_error;

struct Core {
  std::unique_ptr<KVManager> kv;
  std::unique_ptr<Scheduler> sched;
  // sequences driven from outside (replay, tests); the scheduler owns its own
  std::unordered_map<int64_t, std::unique_ptr<Sequence>> loose;
  // sequences the scheduler owns, by id, while they wait or run
  std::unordered_map<int64_t, Sequence*> scheduled;
  std::vector<std::unique_ptr<Sequence>> finished;

  Sequence* find(int64_t id) {
    auto a = loose.find(id);
    if (a != loose.end()) return a->second.get();
    auto b = scheduled.find(id);
    if (b != scheduled.end()) return b->second;
    throw std::invalid_argument("unknown sequence id " + std::to_string(id));
  }
};

template <class F>
int64_t guarded(F&& f) {
  try {
    return f();
  } catch (const std::exception& e) {
    g_error = e.what();
    return -1;
  }
}

PagedManager* as_paged(Core* c) {
  auto* p = dynamic_cast<PagedManager*>(c->kv.get());
  if (!p) throw std::invalid_argument("this call needs the paged policy");
  return p;
}

}  // namespace

extern "C" {

const char* kvcm_last_error() { return g_error.c_str(); }

// ---------------------------------------------------------------------------------- hashing
uint64_t kvcm_xxh64(const void* data, uint64_t len, uint64_t seed) { return XXH64::digest(data, len, seed); }
uint64_t kvcm_chain_hash(uint64_t parent, const int32_t* tokens, int n) { return chain_hash(parent, tokens, n); }

// -------------------------------------------------------------------------------- allocator
void* kvcm_allocator_new(int n) { return new BlockAllocator(n); }
void kvcm_allocator_delete(void* a) { delete static_cast<BlockAllocator*>(a); }
int kvcm_allocator_allocate(void* a) { return static_cast<BlockAllocator*>(a)->allocate(); }
int kvcm_allocator_op(void* a, int op, int id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* al = static_cast<BlockAllocator*>(a);
    switch (op) {
      case 0: al->free(id); return 0;
      case 1: al->incref(id); return 0;
      case 2: return al->decref(id) ? 1 : 0;
      case 3: al->push_free(id); return 0;
      case 4: al->revive(id); return 0;
      default: throw std::invalid_argument("unknown allocator op");
    }
  }));
}
int kvcm_allocator_refcount(void* a, int id) { return static_cast<BlockAllocator*>(a)->refcount(id); }
int kvcm_allocator_num_free(void* a) { return static_cast<BlockAllocator*>(a)->num_free(); }

// ------------------------------------------------------------------------------------- core
void* kvcm_core_new(int policy, int num_groups, const int32_t* kinds, const int32_t* windows,
                    const int32_t* num_blocks, int block_size, int max_seq_len, int prefix_caching,
                    int watermark_blocks, double watermark_frac, int max_num_seqs, int max_batched_tokens,
                    int prefill_chunk, int eos_id) {
  try {
    KVManagerConfig kc;
    kc.policy = policy == 0 ? "paged" : policy == 1 ? "contiguous" : "?";
    for (int g = 0; g < num_groups; ++g)
      kc.groups.push_back({static_cast<GroupKind>(kinds[g]), windows[g], num_blocks[g]});
    kc.block_size = block_size;
    kc.max_seq_len = max_seq_len;
    kc.prefix_caching = prefix_caching != 0 && policy == 0;  // the contiguous policy never caches
    kc.watermark_blocks = watermark_blocks;
    kc.watermark_frac = watermark_frac;
    kc.max_slots = max_num_seqs;
    auto core = std::make_unique<Core>();
    core->kv = make_kv_manager(kc);
    SchedulerConfig sc;
    sc.max_num_seqs = max_num_seqs;
    sc.max_batched_tokens = max_batched_tokens;
    sc.prefill_chunk = prefill_chunk;
    sc.eos_id = eos_id;
    core->sched = std::make_unique<Scheduler>(*core->kv, sc);
    return core.release();
  } catch (const std::exception& e) {
    g_error = e.what();
    return nullptr;
  }
}
void kvcm_core_delete(void* c) { delete static_cast<Core*>(c); }

int kvcm_core_policy_name(void* c, char* out, int cap) {
  const std::string n = static_cast<Core*>(c)->kv->name();
  std::strncpy(out, n.c_str(), cap - 1);
  out[cap - 1] = 0;
  return static_cast<int>(n.size());
}

// ---------------------------------------------------------------- sequences driven by hand
int kvcm_seq_new(void* c, int64_t id, const int32_t* tokens, int n, int max_new_tokens) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    if (core->loose.count(id) || core->scheduled.count(id)) throw std::invalid_argument("sequence id in use");
    auto s = std::make_unique<Sequence>();
    s->id = id;
    s->tokens.assign(tokens, tokens + n);
    s->prompt_len = n;
    s->max_new_tokens = max_new_tokens;
    core->loose.emplace(id, std::move(s));
    return 0;
  }));
}
int kvcm_seq_delete(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    auto it = core->loose.find(id);
    if (it == core->loose.end()) throw std::invalid_argument("unknown sequence id");
    for (const auto& t : it->second->tables)
      if (!t.empty()) throw std::logic_error("delete: the sequence still holds pages");
    core->loose.erase(it);
    return 0;
  }));
}
int kvcm_seq_push_tokens(void* c, int64_t id, const int32_t* tokens, int n) {
  return static_cast<int>(guarded([&]() -> int64_t {
    Sequence* s = static_cast<Core*>(c)->find(id);
    s->tokens.insert(s->tokens.end(), tokens, tokens + n);
    return s->size();
  }));
}
int kvcm_seq_pop_token(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    Sequence* s = static_cast<Core*>(c)->find(id);
    if (s->tokens.empty()) throw std::logic_error("pop on an empty sequence");
    s->tokens.pop_back();
    return s->size();
  }));
}
int kvcm_seq_can_admit(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    return core->kv->can_admit(*core->find(id)) ? 1 : 0;
  }));
}
int kvcm_seq_admit(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    core->kv->admit(*core->find(id));
    return 0;
  }));
}
int kvcm_seq_append_slot(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    return core->kv->append_slot(*core->find(id)) ? 1 : 0;
  }));
}
int kvcm_seq_set_computed(void* c, int64_t id, int n) {
  return static_cast<int>(guarded([&]() -> int64_t {
    Sequence* s = static_cast<Core*>(c)->find(id);
    if (n < 0 || n > s->size()) throw std::invalid_argument("num_computed outside the sequence");
    s->num_computed = n;
    return 0;
  }));
}
int kvcm_seq_commit(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    core->kv->commit(*core->find(id));
    return 0;
  }));
}
int kvcm_seq_release(void* c, int64_t id) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    core->kv->release(*core->find(id));
    return 0;
  }));
}
// out: size, prompt_len, num_computed, cached_tokens, state_slot, num_preemptions, max_new_tokens,
//      num_hashes, prefill_tokens_computed, prefill_tokens_saved
int kvcm_seq_info(void* c, int64_t id, int64_t* out) {
  return static_cast<int>(guarded([&]() -> int64_t {
    const Sequence* s = static_cast<Core*>(c)->find(id);
    out[0] = s->size(); out[1] = s->prompt_len; out[2] = s->num_computed; out[3] = s->cached_tokens;
    out[4] = s->state_slot; out[5] = s->num_preemptions; out[6] = s->max_new_tokens;
    out[7] = static_cast<int64_t>(s->page_hashes.size());
    out[8] = s->prefill_tokens_computed; out[9] = s->prefill_tokens_saved;
    return 0;
  }));
}
int kvcm_seq_table(void* c, int64_t id, int g, int32_t* out, int cap) {
  return static_cast<int>(guarded([&]() -> int64_t {
    const Sequence* s = static_cast<Core*>(c)->find(id);
    if (g < 0 || g >= static_cast<int>(s->tables.size())) return 0;
    const auto& t = s->tables[g];
    const int n = std::min<int>(cap, static_cast<int>(t.size()));
    std::memcpy(out, t.data(), sizeof(int32_t) * n);
    return static_cast<int64_t>(t.size());
  }));
}
int kvcm_seq_tokens(void* c, int64_t id, int32_t* out, int cap) {
  return static_cast<int>(guarded([&]() -> int64_t {
    const Sequence* s = static_cast<Core*>(c)->find(id);
    const int n = std::min<int>(cap, s->size());
    std::memcpy(out, s->tokens.data(), sizeof(int32_t) * n);
    return s->size();
  }));
}

// ------------------------------------------------------------------------- manager queries
int kvcm_num_groups(void* c) { return static_cast<Core*>(c)->kv->num_groups(); }
int kvcm_block_size(void* c) { return static_cast<Core*>(c)->kv->block_size(); }
int kvcm_blocks_in_use(void* c, int g) { return static_cast<Core*>(c)->kv->blocks_in_use(g); }
int kvcm_blocks_cached_free(void* c, int g) { return static_cast<Core*>(c)->kv->blocks_cached_free(g); }
int kvcm_state_slots_free(void* c) { return static_cast<Core*>(c)->kv->slots().num_free(); }
int kvcm_num_free_pages(void* c, int g) {
  return static_cast<int>(guarded([&]() -> int64_t { return as_paged(static_cast<Core*>(c))->allocator(g).num_free(); }));
}
int kvcm_page_refcount(void* c, int g, int page) {
  return static_cast<int>(guarded([&]() -> int64_t { return as_paged(static_cast<Core*>(c))->allocator(g).refcount(page); }));
}
int kvcm_num_hashed(void* c, int g) {
  return static_cast<int>(guarded([&]() -> int64_t { return as_paged(static_cast<Core*>(c))->cache(g).num_hashed(); }));
}
int kvcm_lru_order(void* c, int g, int32_t* out, int cap) {
  return static_cast<int>(guarded([&]() -> int64_t {
    const auto order = as_paged(static_cast<Core*>(c))->cache(g).lru_order();
    for (size_t i = 0; i < order.size() && static_cast<int>(i) < cap; ++i) out[i] = order[i];
    return static_cast<int64_t>(order.size());
  }));
}
int kvcm_count_match(void* c, int g, const int32_t* tokens, int num_pages, int32_t* parked_hits) {
  return static_cast<int>(guarded([&]() -> int64_t {
    int parked = 0;
    const int hits = as_paged(static_cast<Core*>(c))->cache(g).count_match(tokens, num_pages, &parked);
    if (parked_hits) *parked_hits = parked;
    return hits;
  }));
}
int kvcm_num_free_extents(void* c, int g) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* m = dynamic_cast<ContiguousManager*>(static_cast<Core*>(c)->kv.get());
    if (!m) throw std::invalid_argument("this call needs the contiguous policy");
    return m->num_free_extents(g);
  }));
}
// out: queried, hits, inserted, evictions, duplicate inserts
int kvcm_prefix_stats(void* c, int g, int64_t* out) {
  const PrefixCacheStats s = static_cast<Core*>(c)->kv->prefix_stats(g);
  out[0] = s.queried_blocks; out[1] = s.hit_blocks; out[2] = s.inserted_blocks;
  out[3] = s.evictions; out[4] = s.duplicate_inserts;
  return 0;
}
// ids: live sequences (ids == null: the scheduler's running ones).
// out: num_blocks, block_size, in_use, cached_free, allocated, used, tail_waste, reserved_unused,
//      table_entries, num_seqs
int kvcm_kv_stats(void* c, int g, const int64_t* ids, int n, int64_t* out) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    std::vector<const Sequence*> live;
    if (ids) for (int i = 0; i < n; ++i) live.push_back(core->find(ids[i]));
    else live = core->sched->live();
    const KVStats s = core->kv->stats(live, g);
    out[0] = s.num_blocks; out[1] = s.block_size; out[2] = s.blocks_in_use; out[3] = s.blocks_cached_free;
    out[4] = s.allocated_slots; out[5] = s.used_slots; out[6] = s.tail_waste_slots;
    out[7] = s.reserved_unused_slots; out[8] = s.block_table_entries; out[9] = s.num_seqs;
    return 0;
  }));
}

// -------------------------------------------------------------------------------- scheduler
int kvcm_sched_add(void* c, int64_t id, const int32_t* tokens, int n, int max_new_tokens,
                   float temperature, uint64_t sampler_seed, double arrival) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    if (core->loose.count(id) || core->scheduled.count(id)) throw std::invalid_argument("sequence id in use");
    if (n <= 0) throw std::invalid_argument("a request needs at least one token");
    auto s = std::make_unique<Sequence>();
    s->id = id;
    s->tokens.assign(tokens, tokens + n);
    s->prompt_len = n;
    s->max_new_tokens = max_new_tokens;
    s->temperature = temperature;
    s->sampler_seed = sampler_seed;
    s->arrival = arrival;
    core->scheduled.emplace(id, s.get());
    core->sched->add(std::move(s));
    return 0;
  }));
}
int kvcm_sched_schedule(void* c, double now) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    const auto& plan = core->sched->schedule(now);
    // rejected requests are already in the scheduler's finished list; keep `scheduled` honest
    return static_cast<int64_t>(plan.size());
  }));
}
// Per plan entry: id, start, count, flags (bit0 prefill, bit1 samples), index of the token it
// would generate, temperature, sampler seed.
int kvcm_sched_plan(void* c, int64_t* ids, int32_t* start, int32_t* count, int32_t* flags,
                    int32_t* gen_index, float* temperature, uint64_t* seed, int cap) {
  return static_cast<int>(guarded([&]() -> int64_t {
    const auto& plan = static_cast<Core*>(c)->sched->plan();
    if (static_cast<int>(plan.size()) > cap) throw std::length_error("plan buffer too small");
    for (size_t i = 0; i < plan.size(); ++i) {
      ids[i] = plan[i].request->id;
      start[i] = plan[i].first;
      count[i] = plan[i].count;
      flags[i] = (plan[i].given ? 1 : 0) | (plan[i].samples ? 2 : 0);
      gen_index[i] = plan[i].request->num_generated();
      temperature[i] = plan[i].request->temperature;
      seed[i] = plan[i].request->sampler_seed;
    }
    return static_cast<int64_t>(plan.size());
  }));
}
// Runs the scheduler and says what it planned without handing the entries over:
// out[0..9] = {entries, prompt tokens, decoding sequences, entries that sample, 1 if every entry is a
// single token that samples (a decode-shaped step), the longest context a row of the step sees,
// rows in all, leading entries of one token, the longest run, 0}.
int kvcm_sched_schedule_summary(void* c, double now, int64_t* out) {
  return static_cast<int>(guarded([&]() -> int64_t {
    const auto& plan = static_cast<Core*>(c)->sched->schedule(now);
    int64_t prefill = 0, decode = 0, sampling = 0, single = 1, longest = 0, rows = 0, leading = 0, run = 0;
    bool still_leading = true;
    for (const auto& p : plan) {
      if (p.given) prefill += p.count; else ++decode;
      if (p.samples) ++sampling;
      if (p.count != 1 || !p.samples) single = 0;
      if (p.first + p.count > longest) longest = p.first + p.count;
      rows += p.count;
      if (p.count > run) run = p.count;
      if (p.count != 1) still_leading = false;
      if (still_leading) ++leading;
    }
    out[0] = static_cast<int64_t>(plan.size()); out[1] = prefill; out[2] = decode; out[3] = sampling;
    out[4] = plan.empty() ? 0 : single;
    out[5] = longest;   // the longest context any row of the step sees
    out[6] = rows; out[7] = leading; out[8] = run; out[9] = 0;
    return static_cast<int64_t>(plan.size());
  }));
}
// The step's sampled ids, in the order of the plan's sampling entries; entries that did not
// sample get none.
int kvcm_sched_update_sampled(void* c, const int32_t* ids, int n, double now) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    const auto& plan = core->sched->plan();
    std::vector<int32_t> next(plan.size(), -1);
    int k = 0;
    for (size_t i = 0; i < plan.size(); ++i)
      if (plan[i].samples) {
        if (k >= n) throw std::invalid_argument("update_sampled: fewer ids than sampling entries");
        next[i] = ids[k++];
      }
    if (k != n) throw std::invalid_argument("update_sampled: more ids than sampling entries");
    core->sched->update(next, now);
    return 0;
  }));
}
int kvcm_sched_update(void* c, const int32_t* next, int n, double now) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    core->sched->update(std::vector<int32_t>(next, next + n), now);
    return 0;
  }));
}
// Moves what the scheduler finished into the core's holding area; returns how many wait there.
int kvcm_sched_collect_finished(void* c) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    for (auto& s : core->sched->take_finished()) {
      core->scheduled.erase(s->id);
      core->finished.push_back(std::move(s));
    }
    return static_cast<int64_t>(core->finished.size());
  }));
}
// info: id, prompt_len, size, num_preemptions, prefill_tokens_computed, prefill_tokens_saved
// times: arrival, admitted, first_token, finished
int kvcm_finished_get(void* c, int i, int64_t* info, double* times, int32_t* tokens, int cap) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    if (i < 0 || i >= static_cast<int>(core->finished.size())) throw std::out_of_range("finished index");
    const Sequence& s = *core->finished[i];
    info[0] = s.id; info[1] = s.prompt_len; info[2] = s.size(); info[3] = s.num_preemptions;
    info[4] = s.prefill_tokens_computed; info[5] = s.prefill_tokens_saved;
    times[0] = s.arrival; times[1] = s.admitted; times[2] = s.first_token; times[3] = s.finished;
    const int n = std::min<int>(cap, s.size());
    if (tokens) std::memcpy(tokens, s.tokens.data(), sizeof(int32_t) * n);
    return s.size();
  }));
}
void kvcm_finished_clear(void* c) { static_cast<Core*>(c)->finished.clear(); }
int kvcm_sched_idle(void* c) { return static_cast<Core*>(c)->sched->idle() ? 1 : 0; }
int kvcm_sched_num_waiting(void* c) { return static_cast<int>(static_cast<Core*>(c)->sched->num_waiting()); }
int kvcm_sched_num_running(void* c) { return static_cast<int>(static_cast<Core*>(c)->sched->num_running()); }
// out: steps, preemptions, admissions, admission_blocked_steps, rejected, prefill_tokens,
//      decode_tokens, prefill_tokens_saved, batch_size_sum, max_running
int kvcm_sched_counters(void* c, int64_t* out) {
  const SchedulerCounters& k = static_cast<Core*>(c)->sched->counters();
  out[0] = k.steps; out[1] = k.preemptions; out[2] = k.admissions; out[3] = k.admission_blocked_steps;
  out[4] = k.rejected; out[5] = k.prefill_tokens; out[6] = k.decode_tokens;
  out[7] = k.prefill_tokens_saved; out[8] = k.batch_size_sum; out[9] = k.max_running;
  return 0;
}
void kvcm_sched_reset_counters(void* c) { static_cast<Core*>(c)->sched->reset_counters(); }

// ---------------------------------------------------------------------------- batch builder
int kvcm_batch_desc_len(void* c) { return batch_desc_len(static_cast<Core*>(c)->kv->num_groups()); }

// Entries given explicitly.  want_offsets has n+1 entries into `want`; a null want_offsets asks
// for the last row of every entry.
int kvcm_build_batch(void* c, int n, const int64_t* ids, const int32_t* start, const int32_t* count,
                     const int32_t* want_offsets, const int32_t* want, int pad_rows, int pad_seqs,
                     int pad_logit_rows, int table_stride, int32_t* out, int64_t cap, int32_t* desc) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    std::vector<BatchEntry> entries(n);
    for (int i = 0; i < n; ++i) {
      entries[i].seq = core->find(ids[i]);
      entries[i].start = start[i];
      entries[i].count = count[i];
      if (want_offsets) entries[i].want.assign(want + want_offsets[i], want + want_offsets[i + 1]);
      else entries[i].want = {count[i] - 1};
    }
    build_batch(*core->kv, entries, pad_rows, pad_seqs, pad_logit_rows, table_stride, out, cap, desc);
    return desc[kTotalInts];
  }));
}

// The scheduler's current plan; logits are wanted at the last row of every entry that samples.
static void plan_entries(Core* core, std::vector<BatchEntry>& entries) {
  for (const auto& p : core->sched->plan()) {
    BatchEntry e;
    e.seq = p.request;
    e.start = p.first;
    e.count = p.count;
    if (p.samples) e.want = {p.count - 1};
    e.temperature = p.request->temperature;
    e.sampler_seed = p.request->sampler_seed;
    e.request_id = p.request->id;
    e.token_index = p.request->num_generated();
    entries.push_back(std::move(e));
  }
}

// As kvcm_build_batch_from_plan, padded to a recorded step's shape: `pad_leading` single-row
// sequences first (see build_batch).
int kvcm_build_batch_from_plan_shaped(void* c, int pad_rows, int pad_seqs, int pad_logit_rows, int table_stride,
                                      int pad_leading, int32_t* out, int64_t cap, int32_t* desc) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    std::vector<BatchEntry> entries;
    plan_entries(core, entries);
    build_batch(*core->kv, entries, pad_rows, pad_seqs, pad_logit_rows, table_stride, out, cap, desc, pad_leading);
    return desc[kTotalInts];
  }));
}

int kvcm_build_batch_from_plan(void* c, int pad_rows, int pad_seqs, int pad_logit_rows, int table_stride,
                               int32_t* out, int64_t cap, int32_t* desc) {
  return static_cast<int>(guarded([&]() -> int64_t {
    auto* core = static_cast<Core*>(c);
    std::vector<BatchEntry> entries;
    for (const auto& p : core->sched->plan()) {
      BatchEntry e;
      e.seq = p.request;
      e.start = p.first;
      e.count = p.count;
      if (p.samples) e.want = {p.count - 1};
      e.temperature = p.request->temperature;
      e.sampler_seed = p.request->sampler_seed;
      e.request_id = p.request->id;
      e.token_index = p.request->num_generated();
      entries.push_back(std::move(e));
    }
    build_batch(*core->kv, entries, pad_rows, pad_seqs, pad_logit_rows, table_stride, out, cap, desc);
    return desc[kTotalInts];
  }));
}

}  // extern "C"
