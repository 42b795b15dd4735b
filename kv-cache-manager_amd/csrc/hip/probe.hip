// Small kernels that measure the machine rather than the model: what a launch costs, how fast HBM
// streams, how fast the matrix cores multiply.  bench.py prints their figures beside the published
// peaks, bin/kvkernel --floor times chains of them.  The reference's kernel benchmark times its
// attention kernel only (src/main_kernel_bench.cpp:102-126).
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

// grid workgroups of four waves, each wave iters * 4 matrix instructions of 32768 flops
int kvcm_probe_mfma(int iters, void* sink, int grid, hipStream_t s) {
  KVCM_REQUIRE(iters > 0 && sink && grid > 0, "probe_mfma: bad arguments");
  probe_mfma_kernel<<<grid, 256, 0, s>>>(iters, static_cast<float*>(sink));
  return launch_status("probe_mfma");
}

}  // extern "C"
