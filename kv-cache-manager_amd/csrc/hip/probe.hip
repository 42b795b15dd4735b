// Small kernels that measure the machine rather than the model: what a launch costs, how fast HBM
// streams, how fast the matrix cores multiply, and what it costs workgroups of one launch to depend on one
// another (a barrier across the launch, the last workgroup to arrive adding up the others' sums, a whole
// step as one launch of dependent phases).  bench.py prints the first figures beside the published
// peaks, bin/kvkernel --floor times chains of launches, bin/kvkernel --sync the dependencies inside one.
// The reference's kernel benchmark times its attention kernel only (src/main_kernel_bench.cpp:102-126).
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

__global__ void probe_empty_kernel() {}

// dst[i] = src[i] + 1 over 16-byte pieces: every byte is read and written once
__global__ void probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, long long n) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    uint4 v = src[i];
    v.x += 1u;
    dst[i] = v;
  }
}

// reads n 16-byte pieces, keeps nothing (the sum is stored only if it has a value it never has)
__global__ void probe_read_kernel(const uint4* __restrict__ src, long long n, unsigned* __restrict__ sink) {
  unsigned acc = 0;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    const uint4 v = src[i];
    acc += v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9E3779B9u) sink[threadIdx.x] = acc;
}

// The same with a workgroup's share of the bytes contiguous (as a product's workgroup streams its own weight
// rows) and a stated number of 16-byte loads on their way per lane: what a launch reads per microsecond
// as a function of how many CUs it covers and how many waves each has.
template <int INFLIGHT>
__global__ void probe_stream_kernel(const uint4* __restrict__ src, long long n, unsigned* __restrict__ sink) {
  const long long per = (n + gridDim.x - 1) / gridDim.x;
  const long long lo = blockIdx.x * per, hi = lo + per < n ? lo + per : n;
  unsigned acc = 0;
  for (long long i = lo + threadIdx.x; i < hi; i += (long long)blockDim.x * INFLIGHT) {
    uint4 v[INFLIGHT];
#pragma unroll
    for (int u = 0; u < INFLIGHT; ++u) {
      const long long j = i + (long long)u * blockDim.x;
      v[u] = src[j < hi ? j : hi - 1];
    }
#pragma unroll
    for (int u = 0; u < INFLIGHT; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9E3779B9u) sink[threadIdx.x] = acc;
}

// `iters` rounds of four independent 32x32x16 bfloat16 matrix instructions per wave: 4 * 32768 flops a round
__global__ void __launch_bounds__(256) probe_mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = static_cast<__bf16>(1.0f + threadIdx.x * 1e-3f); b[i] = static_cast<__bf16>(0.5f); }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int i = 0; i < iters; ++i) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  const float s = c0[0] + c1[1] + c2[2] + c3[3];
  if (s == 12345.678f) sink[threadIdx.x] = s;
}

// ---- dependencies between the workgroups of one launch -------------------------------------------------
// Data goes from one workgroup to another past the caches: stores and loads of agent scope (the L2 of one of
// the chip's eight parts is not coherent with the others'), a wait for the stores, then a counter.  Every wait
// is bounded: a workgroup that has polled spin_cap times raises flags[0] and leaves, and so does the launch.
typedef __attribute__((ext_vector_type(4))) float probe_f4;
typedef __attribute__((ext_vector_type(4))) unsigned probe_u4;
__device__ __forceinline__ void store_agent(float* p, probe_f4 v) { asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory"); }
__device__ __forceinline__ probe_f4 load_agent(const float* p) {
  probe_f4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1\n s_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ bool wait_for(const unsigned* counter, unsigned target, int spin_cap) {
  int it = 0;
  while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target && ++it < spin_cap) __builtin_amdgcn_s_sleep(1);
  return it < spin_cap;
}

// `rounds` times: every workgroup writes 1 KB, all meet at a counter, every workgroup reads another one's 1 KB
// and checks it (flags[1] counts wrong values).  fences: ordinary stores and loads with a release and an
// acquire fence of agent scope instead of stores and loads past the caches.  awaited: how many arrivals a round
// waits for (the launch's workgroups; a test of the bounded wait names one more, who never comes).
__global__ void __launch_bounds__(256) probe_barrier_kernel(float* data, unsigned* counter, unsigned* flags, int rounds, int spin_cap, int fences, int awaited) {
  const int G = gridDim.x, b = blockIdx.x, t = threadIdx.x;
  __shared__ int ok;
  unsigned errors = 0;
  for (int r = 0; r < rounds; ++r) {
    float* mine = data + (size_t(r & 1) * G + b) * 256;
    if (!fences) {
      if (t < 64) store_agent(mine + 4 * t, probe_f4{float(b), float(r), float(t), 1.f});
      wait_stores();
    } else {
      mine[t] = float(b + r);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    }
    __syncthreads();
    if (t == 0) {
      __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ok = wait_for(counter, unsigned(r) * G + awaited, spin_cap);
    }
    __syncthreads();
    if (!ok) {
      if (t == 0) atomicAdd(flags, 1u);
      return;
    }
    const int other = (b * 7 + 3 + r) % G;
    const float* theirs = data + (size_t(r & 1) * G + other) * 256;
    if (!fences) {
      if (t < 64) {
        const probe_f4 v = load_agent(theirs + 4 * t);
        errors += !(v.x == float(other) && v.y == float(r) && v.z == float(t));
      }
    } else {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      errors += theirs[t] != float(other + r);
    }
  }
  if (errors) atomicAdd(flags + 1, errors);
}

// S workgroups per tile write 4 KB of sums each; the last of a tile's to arrive adds them up in order
__global__ void __launch_bounds__(256) probe_last_arriver_kernel(float* partials, unsigned* counters, float* out, int S, unsigned* flags) {
  const int tile = blockIdx.x / S, s = blockIdx.x % S, t = threadIdx.x;
  store_agent(partials + (size_t(tile) * S + s) * 1024 + 4 * t, probe_f4{float(s + 1), float(tile), 1.f, 2.f});
  wait_stores();
  __shared__ unsigned last;
  __syncthreads();
  if (t == 0) last = __hip_atomic_fetch_add(counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == unsigned(S - 1);
  __syncthreads();
  if (!last) return;
  probe_f4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < S; k0 += 4) {   // four loads on their way at a time (a sum beyond S repeats the last and is not added)
    probe_f4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float* src = partials + (size_t(tile) * S + (k0 + j < S ? k0 + j : S - 1)) * 1024 + 4 * t;
      asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[j]) : "v"(src) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3])::"memory");
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (k0 + j < S) sum += v[j];
  }
  reinterpret_cast<probe_f4*>(out)[size_t(tile) * 256 + t] = sum;
  if (t == 0) counters[tile] = 0;   // for the next launch
  if (sum.x != float(S * (S + 1) / 2) || sum.y != float(S * tile)) atomicAdd(flags + 1, 1u);
}
__global__ void __launch_bounds__(256) probe_write_sums_kernel(float* partials, int S) {
  const int tile = blockIdx.x / S, s = blockIdx.x % S;
  reinterpret_cast<probe_f4*>(partials)[(size_t(tile) * S + s) * 256 + threadIdx.x] = probe_f4{float(s + 1), float(tile), 1.f, 2.f};
}
__global__ void __launch_bounds__(256) probe_add_sums_kernel(const float* partials, float* out, int S) {
  probe_f4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < S; ++k) sum += reinterpret_cast<const probe_f4*>(partials)[(size_t(blockIdx.x) * S + k) * 256 + threadIdx.x];
  reinterpret_cast<probe_f4*>(out)[size_t(blockIdx.x) * 256 + threadIdx.x] = sum;
}

// A decode step as ONE launch: `layers` times `phases` phases; in a phase a workgroup reads its share of the
// phase's bytes (the next phase's first pieces are asked for before the wait), waits until every workgroup
// has finished the phase before (a counter per sixteen workgroups, whose last arriver counts at a second
// one), reads 4 KB that the phase before left past the caches, and leaves 64 bytes of its own.
constexpr int kProbeMaxPhases = 8;
struct PhasePlan {
  long long start[kProbeMaxPhases + 1];   // in 16-byte pieces, inside one layer's bytes
  long long layer_pieces;
  int phases, layers, spin_cap;
};
__global__ void __launch_bounds__(1024) probe_phases_kernel(const probe_u4* weights, PhasePlan plan, unsigned* counters, float* act, unsigned* flags,
                                                            unsigned* sink) {
  constexpr int THREADS = 1024;
  const int G = gridDim.x, b = blockIdx.x, t = threadIdx.x;
  __shared__ int ok;
  probe_u4 acc = {0u, 0u, 0u, 0u};
  int step = 0;
  for (int layer = 0; layer < plan.layers; ++layer) {
    const probe_u4* wl = weights + (long long)(layer % 4) * plan.layer_pieces;   // four layers' bytes, so that no cache holds them
    for (int ph = 0; ph < plan.phases; ++ph, ++step) {
      const long long lo = plan.start[ph], n = plan.start[ph + 1] - lo, per = (n + G - 1) / G;
      const long long my_lo = lo + per * b, my_hi = my_lo + per < lo + n ? my_lo + per : lo + n;
      probe_u4 ahead[4];
      long long i = my_lo + t;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const long long j = i + (long long)k * THREADS;
        ahead[k] = wl[j < my_hi ? j : lo];
      }
      if (step > 0) {
        if (t == 0) ok = wait_for(counters + (long long)(step - 1) * 17 + 16, 16u, plan.spin_cap);
        __syncthreads();
        if (!ok) {
          if (t == 0) atomicAdd(flags, 1u);
          return;
        }
      }
      const probe_f4 a = load_agent(act + (step & 1) * 4096 + 4 * (t % 256));
      acc.x += __float_as_uint(a.x);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (i + (long long)k * THREADS < my_hi) acc ^= ahead[k];
      i += 4ll * THREADS;
      for (; i + 3ll * THREADS < my_hi; i += 4ll * THREADS) {
        const probe_u4 v0 = wl[i], v1 = wl[i + THREADS], v2 = wl[i + 2 * THREADS], v3 = wl[i + 3 * THREADS];
        acc ^= v0; acc ^= v1; acc ^= v2; acc ^= v3;
      }
      for (; i < my_hi; i += THREADS) acc ^= wl[i];
      if (t < 4) store_agent(act + ((step + 1) & 1) * 4096 + 4 * ((b * 4 + t) % 1024), probe_f4{float(acc.x & 7), 1.f, 2.f, 3.f});
      wait_stores();
      __syncthreads();
      if (t == 0) {
        const unsigned members = (G - (b % 16) + 15) / 16;
        if (__hip_atomic_fetch_add(counters + (long long)step * 17 + b % 16, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1)
          __hip_atomic_fetch_add(counters + (long long)step * 17 + 16, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (acc.x == 0x9E3779B9u) sink[t] = acc.y;
}

}  // namespace
}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_probe_empty(int grid, int block, hipStream_t s) {
  KVCM_REQUIRE(grid > 0 && block > 0 && block <= 1024, "probe_empty: bad launch %d x %d", grid, block);
  probe_empty_kernel<<<grid, block, 0, s>>>();
  return launch_status("probe_empty");
}

// dst = src + 1 over `bytes` bytes (a multiple of 16); bytes moved: 2 * bytes
int kvcm_probe_copy(const void* src, void* dst, long long bytes, int grid, hipStream_t s) {
  KVCM_REQUIRE(src && dst && bytes > 0 && bytes % 16 == 0 && grid > 0, "probe_copy: bad arguments");
  probe_copy_kernel<<<grid, 256, 0, s>>>(static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
  return launch_status("probe_copy");
}

int kvcm_probe_read(const void* src, long long bytes, void* sink, int grid, hipStream_t s) {
  KVCM_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && grid > 0, "probe_read: bad arguments");
  probe_read_kernel<<<grid, 256, 0, s>>>(static_cast<const uint4*>(src), bytes / 16, static_cast<unsigned*>(sink));
  return launch_status("probe_read");
}

// grid workgroups of `waves` waves, each workgroup an equal contiguous share of the bytes, `inflight` (4, 8 or
// 16) loads of 16 bytes on their way per lane
int kvcm_probe_stream(const void* src, long long bytes, void* sink, int grid, int waves, int inflight, hipStream_t s) {
  KVCM_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && grid > 0 && waves >= 1 && waves <= 16, "probe_stream: bad arguments");
  const uint4* p = static_cast<const uint4*>(src);
  unsigned* k = static_cast<unsigned*>(sink);
  if (inflight == 4) probe_stream_kernel<4><<<grid, waves * 64, 0, s>>>(p, bytes / 16, k);
  else if (inflight == 8) probe_stream_kernel<8><<<grid, waves * 64, 0, s>>>(p, bytes / 16, k);
  else if (inflight == 16) probe_stream_kernel<16><<<grid, waves * 64, 0, s>>>(p, bytes / 16, k);
  else KVCM_REQUIRE(false, "probe_stream: 4, 8 or 16 loads in flight");
  return launch_status("probe_stream");
}

// grid workgroups of four waves, each wave iters * 4 matrix instructions of 32768 flops
int kvcm_probe_mfma(int iters, void* sink, int grid, hipStream_t s) {
  KVCM_REQUIRE(iters > 0 && sink && grid > 0, "probe_mfma: bad arguments");
  probe_mfma_kernel<<<grid, 256, 0, s>>>(iters, static_cast<float*>(sink));
  return launch_status("probe_mfma");
}

// ---- dependencies inside one launch (bin/kvkernel --sync) ---------------------------------------------------
// Every workgroup must be resident at once for a wait to end: the callers keep G at the number of CUs (a
// workgroup that waits too long gives up, so a larger G costs time, not the GPU).  counter(s): zeroed by the
// caller before every launch; flags: [0] workgroups that gave up, [1] wrong values read.
// awaited: arrivals a round waits for, G in every measurement; G + 1 makes every wait run into its limit.
int kvcm_probe_barrier(float* data, unsigned* counter, unsigned* flags, int G, int rounds, int spin_cap, int fences, int awaited, hipStream_t s) {
  KVCM_REQUIRE(data && counter && flags && G > 0 && G <= 1024 && rounds > 0 && spin_cap > 0 && awaited >= G, "probe_barrier: bad arguments");
  probe_barrier_kernel<<<G, 256, 0, s>>>(data, counter, flags, rounds, spin_cap, fences, awaited);
  return launch_status("probe_barrier");
}

// last_arriver 1: one launch whose last workgroup per tile adds the tile's S sums; 0: two launches (write, add).
// partials: S * tiles * 4 KB; counters: tiles (zero before the first launch; a launch leaves them zero); out: tiles * 4 KB.
int kvcm_probe_sums(float* partials, unsigned* counters, float* out, int S, int tiles, int last_arriver, unsigned* flags, hipStream_t s) {
  KVCM_REQUIRE(partials && counters && out && flags && S > 0 && tiles > 0, "probe_sums: bad arguments");
  if (last_arriver) {
    probe_last_arriver_kernel<<<tiles * S, 256, 0, s>>>(partials, counters, out, S, flags);
  } else {
    probe_write_sums_kernel<<<tiles * S, 256, 0, s>>>(partials, S);
    probe_add_sums_kernel<<<tiles, 256, 0, s>>>(partials, out, S);
  }
  return launch_status("probe_sums");
}

// phase_bytes (host): bytes of each phase of a layer (multiples of 16).  weights: four times a layer's bytes.
// persistent 1: one launch of G workgroups of 1,024 threads (counters: layers * phases * 17, zeroed by the caller;
// act: 32 KB); 0: one launch per phase that reads the same bytes (a chain of layers * phases launches).
int kvcm_probe_phases(const void* weights, const long long* phase_bytes, int phases, int layers, int persistent, int G,
                      unsigned* counters, float* act, unsigned* flags, void* sink, int spin_cap, hipStream_t s) {
  KVCM_REQUIRE(weights && phase_bytes && phases > 0 && phases <= kProbeMaxPhases && layers > 0 && sink, "probe_phases: bad arguments");
  PhasePlan plan{};
  long long at = 0;
  for (int i = 0; i < phases; ++i) {
    KVCM_REQUIRE(phase_bytes[i] > 0 && phase_bytes[i] % 16 == 0, "probe_phases: a phase's bytes must be a positive multiple of 16");
    plan.start[i] = at;
    at += phase_bytes[i] / 16;
  }
  plan.start[phases] = at;
  plan.layer_pieces = at; plan.phases = phases; plan.layers = layers; plan.spin_cap = spin_cap;
  if (persistent) {
    KVCM_REQUIRE(counters && act && flags && G >= 16 && G <= 1024 && spin_cap > 0,
                 "probe_phases: the one launch needs counters, act, flags and 16 to 1,024 workgroups");
    probe_phases_kernel<<<G, 1024, 0, s>>>(static_cast<const probe_u4*>(weights), plan, counters, act, flags, static_cast<unsigned*>(sink));
    return launch_status("probe_phases");
  }
  for (int layer = 0; layer < layers; ++layer)
    for (int ph = 0; ph < phases; ++ph)
      probe_read_kernel<<<1024, 256, 0, s>>>(static_cast<const uint4*>(weights) + (layer % 4) * plan.layer_pieces + plan.start[ph],
                                             plan.start[ph + 1] - plan.start[ph], static_cast<unsigned*>(sink));
  return launch_status("probe_phases");
}

}  // extern "C"
