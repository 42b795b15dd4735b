// Random weights on the device: out[i] = mean + std * n_i with n_i a standard normal value that
// depends on (key, i) alone, so that a tensor's values depend neither on the order in which tensors
// are made nor on where (the host makes the same values from the same rule, weights/random_init.py).
// The reference has no random-weights mode (src/main_bench.cpp:6-7 loads real weights).
//
// The rule, all in 64-bit integers and double precision:
//   mix(z)  = the SplitMix64 output function
//   z1      = mix(key + (i + 1) * 0x9E3779B97F4A7C15),  z2 = mix(z1)
//   u1      = ((z1 >> 12) + 0.5) / 2^52  in (0, 1),     u2 = (z2 >> 12) / 2^52  in [0, 1)
//   n_i     = sqrt(-2 ln u1) * cos(2 pi u2)                                  (Box-Muller)
// and out[i] = float(mean + std * float(n_i)) rounded to the storage type.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {
namespace {

__host__ __device__ inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ inline float normal_at(uint64_t key, uint64_t i) {
  const uint64_t z1 = mix64(key + (i + 1) * 0x9E3779B97F4A7C15ull);
  const uint64_t z2 = mix64(z1);
  const double u1 = (double(z1 >> 12) + 0.5) * (1.0 / 4503599627370496.0);
  const double u2 = double(z2 >> 12) * (1.0 / 4503599627370496.0);
  return float(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2));
}

template <class T>
__global__ void fill_normal_kernel(T* __restrict__ out, long long n, uint64_t key, float mean, float std) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    // product and sum are rounded one after the other, as the host does it: the empty statement keeps
    // the compiler from contracting them into one fused operation
    float scaled = std * normal_at(key, uint64_t(i));
    asm volatile("" : "+v"(scaled));
    store_f(out + i, mean + scaled);
  }
}

__global__ void fill_index_kernel(int* __restrict__ out, long long n, uint64_t key, int modulus) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
    out[i] = int(mix64(key + (uint64_t(i) + 1) * 0x9E3779B97F4A7C15ull) % uint64_t(modulus));
}

}  // namespace
}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_fill_normal(void* out, int dtype, long long n, uint64_t key, float mean, float std, hipStream_t s) {
  if (n == 0) return 0;
  KVCM_REQUIRE(out != nullptr && n > 0, "fill_normal: bad arguments");
  const unsigned blocks = static_cast<unsigned>(n / 256 + 1 < 8192 ? n / 256 + 1 : 8192);
  if (dtype == kF32) fill_normal_kernel<float><<<blocks, 256, 0, s>>>(static_cast<float*>(out), n, key, mean, std);
  else if (dtype == kBF16) fill_normal_kernel<bf16_t><<<blocks, 256, 0, s>>>(static_cast<bf16_t*>(out), n, key, mean, std);
  else KVCM_REQUIRE(false, "fill_normal: unknown dtype %d", dtype);
  return launch_status("fill_normal");
}

// Integer tables: out[i] = mix(key + (i + 1) * 0x9E3779B97F4A7C15) mod modulus, as int32.
int kvcm_fill_index(int* out, long long n, uint64_t key, int modulus, hipStream_t s) {
  if (n == 0) return 0;
  KVCM_REQUIRE(out != nullptr && n > 0 && modulus > 0, "fill_index: bad arguments");
  const unsigned blocks = static_cast<unsigned>(n / 256 + 1 < 8192 ? n / 256 + 1 : 8192);
  fill_index_kernel<<<blocks, 256, 0, s>>>(out, n, key, modulus);
  return launch_status("fill_index");
}

}  // extern "C"
