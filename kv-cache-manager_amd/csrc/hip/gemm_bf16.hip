// Y[M,N] = X[M,K] * W[N,K]^T with bfloat16 operands on the matrix cores
// (v_mfma_f32_16x16x32_bf16), 32-bit accumulation, bfloat16 or 32-bit output.  The reference's
// five GEMM call sites (QKV, O, gate/up, down, LM head; src/model/llama.cpp:45-52,108-128) all
// have this shape: activations row-major [rows, in], weights row-major [out, in].
//
// Tile: 64 x 64 outputs per workgroup of four waves, each wave a 32 x 32 quadrant (2 x 2 MFMA
// tiles), K advanced 32 at a time through LDS.  Any M, N, K: rows and columns outside the matrix
// are staged as zeros and never stored.
#include "common.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kTile = 64, kStepK = 32, kPitch = kStepK + 8;  // pitch 80 bytes keeps 16-byte alignment

__device__ __forceinline__ uint4 load_row_piece(const uint16_t* base, int row, int rows, int k, int K, int ld,
                                                bool vec_ok) {
  uint4 v = {0u, 0u, 0u, 0u};
  if (row >= rows || k >= K) return v;
  const uint16_t* p = base + size_t(row) * ld + k;
  if (vec_ok && k + 8 <= K) return *reinterpret_cast<const uint4*>(p);
  uint16_t tmp[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) tmp[i] = (k + i < K) ? p[i] : uint16_t(0);
  v.x = tmp[0] | (uint32_t(tmp[1]) << 16);
  v.y = tmp[2] | (uint32_t(tmp[3]) << 16);
  v.z = tmp[4] | (uint32_t(tmp[5]) << 16);
  v.w = tmp[6] | (uint32_t(tmp[7]) << 16);
  return v;
}

template <class TO>
__global__ void __launch_bounds__(256)
    gemm_bf16_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W, TO* __restrict__ Y, int M, int N,
                     int K, int ldx, int ldw, int ldy, int vec_ok) {
  __shared__ __attribute__((aligned(16))) uint16_t Xs[kTile][kPitch];
  __shared__ __attribute__((aligned(16))) uint16_t Ws[kTile][kPitch];
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  const int ld_row = tid / 4, ld_k = (tid % 4) * 8;
  const int frag_row = lane % 16, frag_k = (lane / 16) * 8;

  f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int k0 = 0; k0 < K; k0 += kStepK) {
    const uint4 xv = load_row_piece(X, m0 + ld_row, M, k0 + ld_k, K, ldx, vec_ok);
    const uint4 wv = load_row_piece(W, n0 + ld_row, N, k0 + ld_k, K, ldw, vec_ok);
    *reinterpret_cast<uint4*>(&Xs[ld_row][ld_k]) = xv;
    *reinterpret_cast<uint4*>(&Ws[ld_row][ld_k]) = wv;
    __syncthreads();
    bf16x8 a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = *reinterpret_cast<const bf16x8*>(&Xs[wm * 32 + i * 16 + frag_row][frag_k]);
#pragma unroll
    for (int j = 0; j < 2; ++j) b[j] = *reinterpret_cast<const bf16x8*>(&Ws[wn * 32 + j * 16 + frag_row][frag_k]);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    __syncthreads();
  }

  // accumulator layout: lane holds column (lane % 16), rows 4 * (lane / 16) + r
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 32 + j * 16 + lane % 16;
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + wm * 32 + i * 16 + (lane / 16) * 4 + r;
        if (m < M) store_f(Y + size_t(m) * ldy + n, acc[i][j][r]);
      }
    }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" int kvcm_gemm_bf16(const void* X, const void* W, void* Y, int out_dtype, int M, int N, int K, int ldx,
                              int ldw, int ldy, hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  KVCM_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm_bf16: leading dimensions too small");
  const int vec_ok = (ldx % 8 == 0) && (ldw % 8 == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0) &&
                     (reinterpret_cast<uintptr_t>(W) % 16 == 0);
  const dim3 grid((N + kTile - 1) / kTile, (M + kTile - 1) / kTile);
  KVCM_REQUIRE(grid.y <= 65535, "gemm_bf16: too many rows for one launch (%d)", M);
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const uint16_t* w = static_cast<const uint16_t*>(W);
  if (out_dtype == kBF16)
    gemm_bf16_kernel<bf16_t><<<grid, 256, 0, s>>>(x, w, static_cast<bf16_t*>(Y), M, N, K, ldx, ldw, ldy, vec_ok);
  else if (out_dtype == kF32)
    gemm_bf16_kernel<float><<<grid, 256, 0, s>>>(x, w, static_cast<float*>(Y), M, N, K, ldx, ldw, ldy, vec_ok);
  else KVCM_REQUIRE(false, "gemm_bf16: unknown output dtype %d", out_dtype);
  return launch_status("gemm_bf16");
}
