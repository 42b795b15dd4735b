// The engine's step loop, native: schedule -> packed batch metadata -> one upload -> the step's
// launches -> one download of the sampled ids -> update, as the reference's Engine::step does it
// (src/engine/engine.cpp:73-90), for every step whose shape has a recorded program
// (step_program.hip); decode-shaped shapes are additionally captured into a HIP graph.
//
// The scheduler, the cache manager and the batch builder live in the host core, a library of its
// own without any GPU dependency; this file reaches them through the addresses of nine of its C
// functions, handed over when the engine is made.  A step of a shape that has no program yet is
// not run here: the caller runs it once through the model's parts while recording, and registers
// the program.  Requests come in and finished ones go out through this object too (add, idle,
// take_finished as in src/engine/engine.h:29-52), so that a native caller serves without the
// interpreter for as long as the steps it meets have recorded shapes.
//
// Shapes.  A step is brought to a canonical shape so that programs are reused: its leading
// single-token runs (the scheduler puts decoding requests first) are padded to a bucket D with
// padding sequences of one padding row, the other sequences to a bucket P, their rows to a
// multiple of 64, the longest run to a multiple of 64, and the longest context to a class bound.
// Padding rows have context length 0 and slot -1: they store nothing and attend to nothing.
#include <chrono>
#include <cstring>
#include <map>
#include <memory>
#include <tuple>

#include "common.h"
#include "kvcm_hip.h"

namespace {

struct HostApi {
  int (*schedule_summary)(void* core, double now, int64_t* out);
  int (*build_batch_from_plan_shaped)(void* core, int pad_rows, int pad_seqs, int pad_logit_rows, int table_stride,
                                      int pad_leading, int32_t* out, int64_t cap, int32_t* desc);
  int (*update_sampled)(void* core, const int32_t* ids, int n, double now);
  const char* (*last_error)();
  int (*add)(void* core, int64_t id, const int32_t* tokens, int n, int max_new_tokens, float temperature,
             uint64_t sampler_seed, double arrival);
  int (*idle)(void* core);
  int (*collect_finished)(void* core);
  int (*finished_get)(void* core, int i, int64_t* info, double* times, int32_t* tokens, int cap);
  void (*finished_clear)(void* core);
};

struct Shape {
  int rows = 0, seqs = 0, leading = 0, logit_rows = 0, max_run = 0, context_bound = 0, table_stride = 0;
  auto key() const { return std::make_tuple(rows, seqs, leading, logit_rows, max_run, context_bound); }
};

struct Recorded {
  void* program = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  long long replays = 0;
  ~Recorded() {
    if (exec) hipGraphExecDestroy(exec);
    if (graph) hipGraphDestroy(graph);
    if (program) kvcm_program_delete(program);
  }
};

const int kRunBuckets[] = {1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256, 384, 512};
const int kSeqBuckets[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512};
const int kContextClasses[] = {1024, 2048, 4096, 8192, 16384, 32768};

template <size_t N>
int bucket(const int (&b)[N], int n, int limit) {
  for (int v : b)
    if (n <= v) return v < limit ? v : limit;
  return limit;
}
int round_up(int n, int m) { return (n + m - 1) / m * m; }

struct Engine {
  void* core = nullptr;
  HostApi host{};
  int32_t* meta_host = nullptr;   // pinned
  int32_t* meta_dev = nullptr;
  long long meta_ints = 0;
  int32_t* sampled_dev = nullptr;
  int32_t* sampled_host = nullptr;   // pinned
  int max_sampled = 0;
  int block_size = 16, max_context = 0, max_tokens = 0, max_seqs = 0, max_logit_rows = 0;
  int graph_rows = 256;   // decode-shaped steps up to this many rows replay a graph
  hipStream_t stream = nullptr;
  std::map<decltype(Shape().key()), std::unique_ptr<Recorded>> recorded;
  std::vector<int32_t> desc;
  int64_t summary[10] = {};
  int64_t last_plan[20] = {};   // what kvcm_engine_plan last reported
  int last_plan_entries = 0;
  Shape shape;   // of the current plan
  bool planned = false;
  long long steps_replayed = 0, steps_as_graph = 0;
  std::chrono::steady_clock::time_point t_plan;
};

// The canonical shape of the plan the scheduler just made; false when it fits no recorded form
// (beyond the engine's limits).
bool canonical(const Engine& e, const int64_t* s, Shape& out) {
  const int n = int(s[0]), sampling = int(s[3]), longest = int(s[5]), rows = int(s[6]), leading = int(s[7]), run = int(s[8]);
  const bool decode_shaped = s[4] != 0;
  (void)sampling;
  Shape sh;
  const int row_limit = e.max_tokens, seq_limit = e.max_seqs;
  if (decode_shaped) {
    sh.leading = sh.seqs = sh.rows = sh.logit_rows = bucket(kRunBuckets, n, seq_limit < row_limit ? seq_limit : row_limit);
    sh.max_run = 1;
    if (sh.rows < n) return false;
  } else {
    sh.leading = leading > 0 ? bucket(kRunBuckets, leading, seq_limit) : 0;
    const int others = n - leading;
    const int others_padded = bucket(kSeqBuckets, others, seq_limit);
    sh.seqs = sh.leading + others_padded;
    sh.rows = sh.leading + round_up(rows - leading, 64);
    sh.max_run = round_up(run, 64);
    sh.logit_rows = sh.seqs;
    if (sh.leading < leading || others_padded < others || sh.seqs > seq_limit || sh.rows > row_limit ||
        sh.logit_rows > e.max_logit_rows)
      return false;
  }
  sh.context_bound = e.max_context;
  for (int c : kContextClasses)
    if (longest <= c && c < e.max_context) {
      sh.context_bound = c;
      break;
    }
  if (longest > sh.context_bound) return false;
  sh.table_stride = (sh.context_bound + e.block_size - 1) / e.block_size;
  out = sh;
  return true;
}

}  // namespace

extern "C" {

// host_functions: addresses of kvcm_sched_schedule_summary, kvcm_build_batch_from_plan_shaped,
// kvcm_sched_update_sampled, kvcm_last_error, kvcm_sched_add, kvcm_sched_idle, kvcm_sched_collect_finished,
// kvcm_finished_get and kvcm_finished_clear of the host core library, in this order.
void* kvcm_engine_new(void* core, const uint64_t* host_functions, int32_t* meta_host, int32_t* meta_dev, long long meta_ints,
                      int32_t* sampled_dev, int32_t* sampled_host, int max_sampled, int num_groups, int block_size,
                      int max_context, int max_tokens, int max_seqs, int max_logit_rows, int graph_rows, hipStream_t stream) {
  if (!core || !host_functions || !meta_host || !meta_dev || !sampled_dev || !sampled_host || !stream) {
    kvcm::set_error("engine_new: null argument (the engine needs a stream of its own, not the default one)");
    return nullptr;
  }
  auto e = std::make_unique<Engine>();
  e->core = core;
  e->host.schedule_summary = reinterpret_cast<decltype(HostApi::schedule_summary)>(host_functions[0]);
  e->host.build_batch_from_plan_shaped = reinterpret_cast<decltype(HostApi::build_batch_from_plan_shaped)>(host_functions[1]);
  e->host.update_sampled = reinterpret_cast<decltype(HostApi::update_sampled)>(host_functions[2]);
  e->host.last_error = reinterpret_cast<decltype(HostApi::last_error)>(host_functions[3]);
  e->host.add = reinterpret_cast<decltype(HostApi::add)>(host_functions[4]);
  e->host.idle = reinterpret_cast<decltype(HostApi::idle)>(host_functions[5]);
  e->host.collect_finished = reinterpret_cast<decltype(HostApi::collect_finished)>(host_functions[6]);
  e->host.finished_get = reinterpret_cast<decltype(HostApi::finished_get)>(host_functions[7]);
  e->host.finished_clear = reinterpret_cast<decltype(HostApi::finished_clear)>(host_functions[8]);
  for (int i = 0; i < 9; ++i)
    if (!host_functions[i]) {
      kvcm::set_error("engine_new: host function %d is null", i);
      return nullptr;
    }
  e->meta_host = meta_host; e->meta_dev = meta_dev; e->meta_ints = meta_ints;
  e->sampled_dev = sampled_dev; e->sampled_host = sampled_host; e->max_sampled = max_sampled;
  e->block_size = block_size; e->max_context = max_context; e->max_tokens = max_tokens; e->max_seqs = max_seqs;
  e->max_logit_rows = max_logit_rows < max_sampled ? max_logit_rows : max_sampled;
  e->graph_rows = graph_rows;
  e->stream = stream;
  e->desc.assign(20 + 4 * num_groups, 0);
  return e.release();
}

void kvcm_engine_delete(void* engine) { delete static_cast<Engine*>(engine); }

// Runs the scheduler.  out[0..9]: the host core's summary (entries, prompt tokens, decoding
// sequences, sampling entries, decode-shaped, longest context, rows, leading single runs, longest
// run, 0); out[10..17]: 1 if the plan has a canonical shape, then that shape (rows, sequences,
// leading, logit rows, longest run, context bound, table stride); out[18]: 1 if a program for it is
// recorded, out[19]: 1 if such a step should be captured as a graph when recorded.
// Returns the number of plan entries, negative on failure.
int kvcm_engine_plan(void* engine, double now, int64_t* out) {
  auto* e = static_cast<Engine*>(engine);
  e->planned = false;
  e->t_plan = std::chrono::steady_clock::now();
  const int n = e->host.schedule_summary(e->core, now, e->summary);
  if (n < 0) {
    kvcm::set_error("engine_plan: %s", e->host.last_error());
    return -1;
  }
  std::memcpy(out, e->summary, sizeof(e->summary));
  for (int i = 10; i < 20; ++i) out[i] = 0;
  Shape sh;
  if (n > 0 && canonical(*e, e->summary, sh)) {
    e->shape = sh;
    e->planned = true;
    out[10] = 1; out[11] = sh.rows; out[12] = sh.seqs; out[13] = sh.leading; out[14] = sh.logit_rows;
    out[15] = sh.max_run; out[16] = sh.context_bound; out[17] = sh.table_stride;
    out[18] = e->recorded.count(sh.key()) ? 1 : 0;
    out[19] = (e->summary[4] != 0 && sh.rows <= e->graph_rows) ? 1 : 0;
  }
  std::memcpy(e->last_plan, out, sizeof(e->last_plan));
  e->last_plan_entries = n;
  return n;
}

// What the last kvcm_engine_plan (or kvcm_engine_step) reported, again, without running the scheduler:
// for the caller that records a step kvcm_engine_step could not run.  Returns that plan's entries.
int kvcm_engine_last_plan(void* engine, int64_t* out) {
  auto* e = static_cast<Engine*>(engine);
  std::memcpy(out, e->last_plan, sizeof(e->last_plan));
  if (e->planned) out[18] = e->recorded.count(e->shape.key()) ? 1 : 0;
  return e->last_plan_entries;
}

// Hands a recorded program for the current plan's shape to the engine (which owns it from now on).
// as_graph: capture it into a HIP graph (only launches of this library's kernels may be in it).
int kvcm_engine_register(void* engine, void* program, int as_graph) {
  auto* e = static_cast<Engine*>(engine);
  KVCM_REQUIRE(e->planned && program != nullptr, "engine_register: no planned step of a canonical shape");
  auto rec = std::make_unique<Recorded>();
  rec->program = program;
  if (as_graph) {
    hipError_t err = hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal);
    KVCM_REQUIRE(err == hipSuccess, "engine_register: begin capture: %s", hipGetErrorString(err));
    const int rc = kvcm_program_run(program, e->stream);
    err = hipStreamEndCapture(e->stream, &rec->graph);
    if (rc != 0) return rc;
    KVCM_REQUIRE(err == hipSuccess && rec->graph != nullptr, "engine_register: end capture: %s", hipGetErrorString(err));
    err = hipGraphInstantiate(&rec->exec, rec->graph, nullptr, nullptr, 0);
    KVCM_REQUIRE(err == hipSuccess, "engine_register: instantiate: %s", hipGetErrorString(err));
  }
  e->recorded[e->shape.key()] = std::move(rec);
  return 0;
}

// Runs the planned step from its recorded program: build, upload, launches, download, update.
// info[0..4]: rows, sequences, sampled ids, 1 if a graph was replayed, microseconds the host spent
// from the scheduler's call to the last launch (before it waits for the GPU).  Returns 1 when the step
// ran, 0 when its shape has no program (nothing was done: the caller runs and records it),
// negative on failure.  defer_update: stop before the update; the sampled ids lie in the pinned
// buffer the engine was given and the caller updates the scheduler itself (teacher forcing).
int kvcm_engine_run(void* engine, double now, int defer_update, int64_t* info) {
  auto* e = static_cast<Engine*>(engine);
  if (!e->planned) return 0;
  auto it = e->recorded.find(e->shape.key());
  if (it == e->recorded.end()) return 0;
  Recorded& rec = *it->second;
  const Shape& sh = e->shape;
  const int total = e->host.build_batch_from_plan_shaped(e->core, sh.rows, sh.seqs, sh.logit_rows, sh.table_stride, sh.leading,
                                                         e->meta_host, e->meta_ints, e->desc.data());
  if (total < 0) {
    kvcm::set_error("engine_run: %s", e->host.last_error());
    return -1;
  }
  // the recorded launches were made for exactly this padded shape
  KVCM_REQUIRE(e->desc[15] == sh.rows && e->desc[16] == sh.seqs && e->desc[17] == sh.logit_rows,
               "engine_run: the batch (%d rows, %d sequences, %d logit rows) does not have the recorded shape (%d, %d, %d)",
               e->desc[15], e->desc[16], e->desc[17], sh.rows, sh.seqs, sh.logit_rows);
  const int sampling = int(e->summary[3]);
  KVCM_REQUIRE(sampling <= e->max_sampled, "engine_run: %d sampling rows exceed the sampler's %d", sampling, e->max_sampled);
  hipError_t err = hipMemcpyAsync(e->meta_dev, e->meta_host, size_t(total) * 4, hipMemcpyHostToDevice, e->stream);
  KVCM_REQUIRE(err == hipSuccess, "engine_run: upload: %s", hipGetErrorString(err));
  if (rec.exec) {
    err = hipGraphLaunch(rec.exec, e->stream);
    KVCM_REQUIRE(err == hipSuccess, "engine_run: graph launch: %s", hipGetErrorString(err));
    ++e->steps_as_graph;
  } else {
    if (int rc = kvcm_program_run(rec.program, e->stream)) return rc;
  }
  if (sampling > 0) {
    err = hipMemcpyAsync(e->sampled_host, e->sampled_dev, size_t(sampling) * 4, hipMemcpyDeviceToHost, e->stream);
    KVCM_REQUIRE(err == hipSuccess, "engine_run: download: %s", hipGetErrorString(err));
  }
  const double issued = std::chrono::duration<double>(std::chrono::steady_clock::now() - e->t_plan).count();
  err = hipStreamSynchronize(e->stream);
  KVCM_REQUIRE(err == hipSuccess, "engine_run: %s", hipGetErrorString(err));
  const double spent = std::chrono::duration<double>(std::chrono::steady_clock::now() - e->t_plan).count();
  if (!defer_update && e->host.update_sampled(e->core, e->sampled_host, sampling, now + spent) < 0) {
    kvcm::set_error("engine_run: %s", e->host.last_error());
    return -1;
  }
  ++rec.replays;
  ++e->steps_replayed;
  e->planned = false;
  info[0] = e->desc[0]; info[1] = e->desc[1]; info[2] = sampling; info[3] = rec.exec ? 1 : 0;
  info[4] = static_cast<int64_t>(issued * 1e6);
  return 1;
}

// ---- requests in, finished requests out (src/engine/engine.h:29-52: add, idle, step, take_finished) ----
// A request: its prompt's token ids, how many tokens it may generate, its sampling temperature (0:
// greedy) and seed, and its arrival time on the caller's clock (the clock of `now` in plan / run / step).
int kvcm_engine_add(void* engine, long long id, const int32_t* tokens, int n, int max_new_tokens, float temperature,
                    uint64_t sampler_seed, double arrival) {
  auto* e = static_cast<Engine*>(engine);
  KVCM_REQUIRE(e != nullptr && tokens != nullptr && n > 0, "engine_add: a request needs at least one token");
  if (e->host.add(e->core, id, tokens, n, max_new_tokens, temperature, sampler_seed, arrival) < 0) {
    kvcm::set_error("engine_add: %s", e->host.last_error());
    return -1;
  }
  return 0;
}

// 1 when no request waits or runs.
int kvcm_engine_idle(void* engine) {
  auto* e = static_cast<Engine*>(engine);
  return e->host.idle(e->core);
}

// One step: plan, then run from the shape's recorded program.  Returns 1 when a step ran (info as
// kvcm_engine_run fills it), 2 when the scheduler planned nothing (idle, or every waiting request
// was rejected), 0 when the planned step's shape has no program yet: the plan stands, nothing ran,
// and the caller has the step recorded (the model's parts decide its launches) and registers it
// with kvcm_engine_register before it goes on.  Negative on failure.
int kvcm_engine_step(void* engine, double now, int64_t* info) {
  int64_t plan[20];
  const int n = kvcm_engine_plan(engine, now, plan);
  if (n < 0) return n;
  if (n == 0) return 2;
  return kvcm_engine_run(engine, now, 0, info);
}

// Moves what finished since the last call into a holding area and says how many requests wait there;
// kvcm_engine_finished_get reads entry i of it (info: id, prompt length, tokens in all, preemptions,
// prompt tokens computed, prompt tokens served from the prefix cache; times: arrival, admission, first
// token, finish; tokens: prompt and generated ids, at most cap of them; returns the number of tokens),
// kvcm_engine_finished_clear empties it.
int kvcm_engine_take_finished(void* engine) {
  auto* e = static_cast<Engine*>(engine);
  const int n = e->host.collect_finished(e->core);
  if (n < 0) kvcm::set_error("engine_take_finished: %s", e->host.last_error());
  return n;
}
int kvcm_engine_finished_get(void* engine, int i, int64_t* info, double* times, int32_t* tokens, int cap) {
  auto* e = static_cast<Engine*>(engine);
  const int n = e->host.finished_get(e->core, i, info, times, tokens, cap);
  if (n < 0) kvcm::set_error("engine_finished_get: %s", e->host.last_error());
  return n;
}
void kvcm_engine_finished_clear(void* engine) {
  auto* e = static_cast<Engine*>(engine);
  e->host.finished_clear(e->core);
}

// out: programs recorded, of them graphs, steps replayed, of them as graphs.
void kvcm_engine_stats(void* engine, int64_t* out) {
  auto* e = static_cast<Engine*>(engine);
  long long graphs = 0;
  for (const auto& kv : e->recorded) graphs += kv.second->exec ? 1 : 0;
  out[0] = static_cast<int64_t>(e->recorded.size()); out[1] = graphs; out[2] = e->steps_replayed; out[3] = e->steps_as_graph;
}

}  // extern "C"
