// Token choice from 32-bit logits: argmax (lowest index among equal maxima, as the reference's
// argmax, src/cuda/kernels.cu:90-119) and temperature sampling by the Gumbel-max rule,
//   id = argmax_j ( logit_j / T - log(-log u_j) ),
// where u_j is a pure function of (seed, request id, index of the generated token, j): the draw
// does not depend on what else is in the batch or on how the prompt was cut.  The reference
// samples greedily only; temperature 0 here is exactly that rule.
#include <cfloat>

#include "common.h"

namespace kvcm {

constexpr int kSampleThreads = 1024;  // one workgroup per row: its latency is the kernel's time

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__global__ void __launch_bounds__(kSampleThreads)
    sample_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ temperature,
                  const uint64_t* __restrict__ seeds, const long long* __restrict__ request_ids,
                  const int* __restrict__ token_index, int* __restrict__ out, int V) {
  const int r = blockIdx.x;
  const float* row = logits + size_t(r) * ld;
  const float temp = temperature ? temperature[r] : 0.f;
  uint64_t key = 0;
  if (temp > 0.f) {
    key = mix64(seeds[r] + 0x9E3779B97F4A7C15ull * (static_cast<uint64_t>(request_ids[r]) + 1ull));
    key = mix64(key ^ (static_cast<uint64_t>(token_index[r]) * 0xBF58476D1CE4E5B9ull));
  }
  float best = -INFINITY;
  int idx = 0x7fffffff;
  // 16 values per thread and trip, all requested before the first is looked at (an index beyond
  // the row reads its last element and is skipped afterwards): the row costs a few trips to
  // memory, not one per element
  constexpr int kBatch = 16;
  for (int j0 = threadIdx.x; j0 < V; j0 += kSampleThreads * kBatch) {
    float v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int j = j0 + u * kSampleThreads;
      v[u] = row[j < V ? j : V - 1];
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int j = j0 + u * kSampleThreads;
      float x = v[u];
      if (temp > 0.f) {
        const float r = (float(mix64(key + uint64_t(j)) >> 41) + 0.5f) * (1.0f / 8388608.0f);  // exact in 24 bits
        x = x / temp - logf(-logf(r));
      }
      if (j < V && (x > best || (x == best && j < idx))) { best = x; idx = j; }
    }
  }
  __shared__ float sv[kSampleThreads / kWave];
  __shared__ int si[kSampleThreads / kWave];
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, kWave);
    const int oi = __shfl_xor(idx, o, kWave);
    if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
  }
  if (threadIdx.x % kWave == 0) { sv[threadIdx.x / kWave] = best; si[threadIdx.x / kWave] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kSampleThreads / kWave; ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < idx)) { best = sv[w]; idx = si[w]; }
    out[r] = idx == 0x7fffffff ? 0 : idx;  // a row of NaNs falls back to id 0
  }
}

}  // namespace kvcm

using namespace kvcm;

// temperature == null (or an entry <= 0): argmax.  seeds, request_ids, token_index may be null
// only when temperature is.
extern "C" int kvcm_sample(const float* logits, int ld, const float* temperature, const uint64_t* seeds,
                           const long long* request_ids, const int* token_index, int* out, int R, int V,
                           hipStream_t s) {
  if (R == 0) return 0;
  KVCM_REQUIRE(R > 0 && V > 0 && ld >= V, "sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
  KVCM_REQUIRE(!temperature || (seeds && request_ids && token_index), "sample: temperature needs seeds and ids");
  sample_kernel<<<R, kSampleThreads, 0, s>>>(logits, ld, temperature, seeds, request_ids, token_index, out, V);
  return launch_status("sample");
}
