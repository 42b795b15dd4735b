// The host core (allocator, managers, prefix cache, scheduler, batch builder) driven through its
// C interface by a random workload, built with -fsanitize=address,undefined and run on the CPU:
// a page held twice, freed twice or lost, a read past a table, or an overflow ends the run.
// The model is a fake: every sampled token is a hash of (request, position), as the reference's
// scheduler test uses a constant (tests/test_scheduler.cpp:19-39).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

extern "C" {
const char* kvcm_last_error();
void* kvcm_core_new(int policy, int num_groups, const int32_t* kinds, const int32_t* windows, const int32_t* num_blocks,
                    int block_size, int max_seq_len, int prefix_caching, int watermark_blocks, double watermark_frac,
                    int max_num_seqs, int max_batched_tokens, int prefill_chunk, int eos_id);
void kvcm_core_delete(void* c);
int kvcm_sched_add(void* c, int64_t id, const int32_t* tokens, int n, int max_new_tokens, float temperature,
                   uint64_t sampler_seed, double arrival);
int kvcm_sched_schedule_summary(void* c, double now, int64_t* out);
int kvcm_sched_update_sampled(void* c, const int32_t* ids, int n, double now);
int kvcm_sched_collect_finished(void* c);
void kvcm_finished_clear(void* c);
int kvcm_sched_idle(void* c);
int kvcm_sched_counters(void* c, int64_t* out);
int kvcm_batch_desc_len(void* c);
int kvcm_build_batch_from_plan(void* c, int pad_rows, int pad_seqs, int pad_logit_rows, int table_stride, int32_t* out,
                               int64_t cap, int32_t* desc);
int kvcm_blocks_in_use(void* c, int g);
int kvcm_state_slots_free(void* c);
}

#define CHECK(cond, ...)                                                      \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::fprintf(stderr, "FAILED %s:%d: ", __FILE__, __LINE__);             \
      std::fprintf(stderr, __VA_ARGS__);                                      \
      std::fprintf(stderr, " (last error: %s)\n", kvcm_last_error());         \
      std::exit(1);                                                           \
    }                                                                         \
  } while (0)

static int run(int policy, int groups, int block_size, int blocks, bool prefix, int chunk, uint64_t seed, int requests) {
  std::mt19937_64 rng(seed);
  std::vector<int32_t> kinds(groups), windows(groups), nblocks(groups);
  for (int g = 0; g < groups; ++g) {   // group 0 full keys; others: a window, then state
    kinds[g] = g == 0 ? 0 : (g == 1 ? 1 : 2);
    windows[g] = g == 1 ? 24 : 0;
    nblocks[g] = g == 2 ? 0 : blocks;
  }
  const int max_seq = 160, max_seqs = 12, budget = 96;
  void* core = kvcm_core_new(policy, groups, kinds.data(), windows.data(), nblocks.data(), block_size, max_seq, prefix,
                             -1, 0.01, max_seqs, budget, chunk, /*eos*/ 7);
  CHECK(core != nullptr, "core_new");
  const int desc_len = kvcm_batch_desc_len(core);
  std::vector<int32_t> desc(desc_len), meta(1 << 16);
  std::vector<int32_t> shared(40);
  for (auto& t : shared) t = 10 + int(rng() % 50);
  int64_t next_id = 0;
  int finished = 0, steps = 0;
  auto add = [&]() {
    std::vector<int32_t> toks;
    if (rng() % 2) toks.insert(toks.end(), shared.begin(), shared.begin() + 8 + rng() % 32);   // shared prefixes
    const int own = 1 + rng() % 60;
    for (int i = 0; i < own; ++i) toks.push_back(10 + int(rng() % 200));
    const int max_new = 1 + rng() % 40;
    CHECK(kvcm_sched_add(core, next_id++, toks.data(), int(toks.size()), max_new, 0.f, 0, double(steps)) == 0, "add");
  };
  for (int i = 0; i < 6; ++i) add();
  int added = 6;
  while (true) {
    if (added < requests && rng() % 3 == 0) { add(); ++added; }
    int64_t sum[10];
    const int n = kvcm_sched_schedule_summary(core, double(steps), sum);
    CHECK(n >= 0, "schedule");
    if (n == 0) {
      finished += kvcm_sched_collect_finished(core);
      kvcm_finished_clear(core);
      if (added >= requests && kvcm_sched_idle(core)) break;
      CHECK(!kvcm_sched_idle(core) || added < requests, "nothing scheduled while requests wait");
      if (kvcm_sched_idle(core)) { add(); ++added; }
      ++steps;
      CHECK(steps < 200000, "no progress");
      continue;
    }
    const int pad = rng() % 2 ? 16 : 0;
    const int64_t total = kvcm_build_batch_from_plan(core, pad, pad, pad, 0, meta.data(), int64_t(meta.size()), desc.data());
    CHECK(total > 0, "build_batch");
    CHECK(desc[0] == sum[1] + sum[2] || sum[1] + sum[2] <= desc[0], "rows %d vs planned %lld", desc[0], (long long)(sum[1] + sum[2]));
    // every real row's slot of a paged group lies inside the pool, no slot is used twice in a step
    for (int g = 0; g < groups; ++g) {
      if (kinds[g] == 2) continue;
      const int32_t* slots = meta.data() + desc[20 + 4 * g];
      std::vector<char> seen(size_t(blocks) * block_size, 0);
      for (int r = 0; r < desc[0]; ++r) {
        CHECK(slots[r] >= 0 && slots[r] < blocks * block_size, "slot %d out of the pool", slots[r]);
        CHECK(!seen[slots[r]], "slot %d given to two rows", slots[r]);
        seen[slots[r]] = 1;
      }
    }
    std::vector<int32_t> ids(sum[3]);
    for (auto& t : ids) t = int(rng() % 97 == 0 ? 7 : 10 + rng() % 200);   // now and then the end-of-sequence id
    CHECK(kvcm_sched_update_sampled(core, ids.data(), int(ids.size()), double(steps)) == 0, "update");
    finished += kvcm_sched_collect_finished(core);
    kvcm_finished_clear(core);
    ++steps;
    CHECK(steps < 200000, "no progress");
  }
  int64_t k[10];
  kvcm_sched_counters(core, k);
  for (int g = 0; g < groups; ++g) CHECK(kvcm_blocks_in_use(core, g) == 0, "group %d: %d pages still held", g, kvcm_blocks_in_use(core, g));
  CHECK(kvcm_state_slots_free(core) == max_seqs, "state slots lost");
  CHECK(finished == added, "%d of %d requests came back", finished, added);
  std::printf("policy %d groups %d B %d blocks %d prefix %d chunk %d: %d requests, %d steps, %lld preemptions, %lld rejected\n",
              policy, groups, block_size, blocks, int(prefix), chunk, added, steps, (long long)k[1], (long long)k[4]);
  kvcm_core_delete(core);
  return 0;
}

int main() {
  run(0, 1, 4, 40, true, 0, 1, 300);     // paged, prefix cache, whole prompts, pressure
  run(0, 1, 8, 24, false, 16, 2, 300);   // paged, portions of 16
  run(0, 1, 4, 64, true, 8, 3, 300);     // prefix cache with portions
  run(1, 1, 4, 60, false, 0, 4, 200);    // contiguous
  run(0, 3, 4, 48, false, 12, 5, 300);   // full + window + state groups
  std::puts("host core stress: ok");
  return 0;
}
