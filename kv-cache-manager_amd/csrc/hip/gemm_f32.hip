// Y[M,N] = X[M,K] * W[N,K]^T in true 32-bit: plain FMA, no matrix-core mode of lower precision.
// Every output element is one chain of fused multiply-adds over k = 0 .. K-1 in ascending order,
// whatever M, the tile shape or the position of the element in its tile: a row's result does not
// depend on which other rows share the launch.  (The reference has no 32-bit path; its GEMMs are
// cuBLAS calls with this same operand layout, src/model/llama.cpp:45-52.)
#include "common.h"

namespace kvcm {

constexpr int kBN = 64, kBK = 16;

template <int BM>  // 64 (TM = 4 rows per thread) or 16 (TM = 1)
__global__ void __launch_bounds__(256)
    gemm_f32_kernel(const float* __restrict__ X, const float* __restrict__ W, float* __restrict__ Y, int M, int N,
                    int K, int ldx, int ldw, int ldy) {
  constexpr int TM = BM / 16;
  __shared__ float Xs[kBK][BM + 4];
  __shared__ float Ws[kBK][kBN + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * kBN;
  float acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += kBK) {
    // stage X[m0 .. m0+BM) x [k0 .. k0+16) and W[n0 .. n0+64) x [k0 .. k0+16), zero outside
    for (int e = threadIdx.x; e < BM * kBK; e += 256) {
      const int r = e / kBK, c = e % kBK;
      const int m = m0 + r, k = k0 + c;
      Xs[c][r] = (m < M && k < K) ? X[size_t(m) * ldx + k] : 0.f;
    }
    for (int e = threadIdx.x; e < kBN * kBK; e += 256) {
      const int r = e / kBK, c = e % kBK;
      const int n = n0 + r, k = k0 + c;
      Ws[c][r] = (n < N && k < K) ? W[size_t(n) * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kBK; ++k) {
      float a[TM], b[4];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = Xs[k][ty * TM + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) Y[size_t(m) * ldy + n] = acc[i][j];
    }
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" int kvcm_gemm_f32(const float* X, const float* W, float* Y, int M, int N, int K, int ldx, int ldw,
                             int ldy, hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  KVCM_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm_f32: leading dimensions too small");
  if (M <= 32) {
    const dim3 grid((N + kBN - 1) / kBN, (M + 15) / 16);
    gemm_f32_kernel<16><<<grid, 256, 0, s>>>(X, W, Y, M, N, K, ldx, ldw, ldy);
  } else {
    const dim3 grid((N + kBN - 1) / kBN, (M + 63) / 64);
    gemm_f32_kernel<64><<<grid, 256, 0, s>>>(X, W, Y, M, N, K, ldx, ldw, ldy);
  }
  return launch_status("gemm_f32");
}
