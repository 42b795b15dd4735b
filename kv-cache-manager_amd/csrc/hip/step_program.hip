// Recorded steps: the launches of one step as a list that is replayed natively.
//
// The reference's step function issues its kernels from C++ in a fixed order
// (src/model/llama.cpp:54-141).  Here the order comes from the parts a model is assembled from, so
// it is not known at compile time; it is recorded instead: while the parts run a step of some shape
// once, every launching entry point of this library that they call is noted with its arguments,
// and later steps of the same shape call the same entry points again from here, without the parts.
// Nothing else changes between two steps of one shape: the kernels read token ids, positions,
// page tables and sampling parameters from the step's metadata buffer in device memory.
#include <cstring>
#include <type_traits>
#include <utility>
#include <vector>

#include "common.h"
#include "kvcm_hip.h"

namespace {

union Slot {
  uint64_t u;
  void* p;
  long long ll;
  int i;
  float f;
};
static_assert(sizeof(Slot) == 8, "one 64-bit slot per argument");

template <class T> struct FromSlot;
template <class T> struct FromSlot<T*> {
  static T* get(const Slot& s) { return static_cast<T*>(s.p); }
};
template <> struct FromSlot<int> {
  static int get(const Slot& s) { return s.i; }
};
template <> struct FromSlot<float> {
  static float get(const Slot& s) { return s.f; }
};
template <> struct FromSlot<long long> {
  static long long get(const Slot& s) { return s.ll; }
};

// Argument I of N: the replay's stream in the last place, the recorded value elsewhere.
template <class A, size_t I, size_t N>
A pick(const Slot* s, hipStream_t stream) {
  if constexpr (I + 1 == N) {
    static_assert(std::is_same<A, hipStream_t>::value, "the last argument of a launching entry is its stream");
    return stream;
  } else {
    return FromSlot<A>::get(s[I]);
  }
}

template <class F, F fn> struct Thunk;
template <class... A, int (*fn)(A...)>
struct Thunk<int (*)(A...), fn> {
  static constexpr int arity = sizeof...(A);
  template <size_t... I>
  static int go(const Slot* s, hipStream_t stream, std::index_sequence<I...>) {
    return fn(pick<A, I, sizeof...(A)>(s, stream)...);
  }
  static int call(const Slot* s, hipStream_t stream) { return go(s, stream, std::index_sequence_for<A...>{}); }
};

struct Entry {
  const char* name;
  int arity;
  int (*call)(const Slot*, hipStream_t);
};

#define KVCM_ENTRY(fn) {#fn, Thunk<decltype(&fn), &fn>::arity, &Thunk<decltype(&fn), &fn>::call}
const Entry kEntries[] = {
    KVCM_ENTRY(kvcm_embed),
    KVCM_ENTRY(kvcm_rmsnorm),
    KVCM_ENTRY(kvcm_rope_cache),
    KVCM_ENTRY(kvcm_rope_table),
    KVCM_ENTRY(kvcm_swiglu),
    KVCM_ENTRY(kvcm_add_residual),
    KVCM_ENTRY(kvcm_gemm_skinny),
    KVCM_ENTRY(kvcm_reduce_store),
    KVCM_ENTRY(kvcm_gemm_skinny_swiglu),
    KVCM_ENTRY(kvcm_gemm_skinny_swiglu_normed),
    KVCM_ENTRY(kvcm_gemm_f32),
    KVCM_ENTRY(kvcm_gemm_bf16),
    KVCM_ENTRY(kvcm_gemm_library),
    KVCM_ENTRY(kvcm_gemm8),
    KVCM_ENTRY(kvcm_gemm8_residual_norm),
    KVCM_ENTRY(kvcm_attention_generic),
    KVCM_ENTRY(kvcm_attention_decode),
    KVCM_ENTRY(kvcm_attention_decode_fused),
    KVCM_ENTRY(kvcm_attention_prefill),
    KVCM_ENTRY(kvcm_sample),
};
#undef KVCM_ENTRY

constexpr int kMaxArgs = 28;

struct Launch {
  const Entry* entry;
  Slot args[kMaxArgs];
};

struct Program {
  std::vector<Launch> launches;
};

}  // namespace

extern "C" {

void* kvcm_program_new() { return new Program(); }
void kvcm_program_delete(void* program) { delete static_cast<Program*>(program); }
int kvcm_program_size(void* program) { return static_cast<int>(static_cast<Program*>(program)->launches.size()); }

int kvcm_program_add(void* program, const char* entry, const uint64_t* args, int num_args) {
  KVCM_REQUIRE(program != nullptr && entry != nullptr && args != nullptr, "program_add: null argument");
  for (const Entry& e : kEntries) {
    if (std::strcmp(e.name, entry) != 0) continue;
    KVCM_REQUIRE(num_args == e.arity, "program_add: %s takes %d arguments, %d were recorded", entry, e.arity, num_args);
    KVCM_REQUIRE(e.arity <= kMaxArgs, "program_add: %s has more arguments than a recorded launch holds", entry);
    Launch l{};
    l.entry = &e;
    for (int i = 0; i < num_args; ++i) l.args[i].u = args[i];
    static_cast<Program*>(program)->launches.push_back(l);
    return 0;
  }
  KVCM_REQUIRE(false, "program_add: %s is not a launching entry of this library", entry);
}

int kvcm_program_run(void* program, hipStream_t stream) {
  KVCM_REQUIRE(program != nullptr, "program_run: null program");
  const Program& p = *static_cast<Program*>(program);
  for (size_t k = 0; k < p.launches.size(); ++k) {
    const int rc = p.launches[k].entry->call(p.launches[k].args, stream);
    if (rc != 0) return rc;   // the entry left its message
  }
  return 0;
}

}  // extern "C"
