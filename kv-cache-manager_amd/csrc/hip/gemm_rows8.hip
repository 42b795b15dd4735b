// Products for decode steps of at most 8 rows, Y[M,N] = X[M,K] * W[N,K]^T (bfloat16), made so that a
// layer needs no launch of its own for its two RMS norms.  The reference runs norm, product,
// residual add as separate kernels (src/model/llama.cpp:104-124, src/cuda/kernels.cu:34-49,84-88);
// at these sizes a launch costs more than the bytes it moves, so here the norm is split in two and
// folded into the products around it:
//
//   producer (O and down projections, kvcm_gemm8_residual_norm): adds its rounded result to the
//     32-bit residual stream x, and leaves for the norm that follows  xg = round(g * round(x))
//     and, per row and 8-column tile, the sum of x^2;
//   consumer (QKV and gate/up projections, kvcm_gemm8 with `ss_in`): multiplies W with xg and scales
//     its 32-bit sums by rstd = rsqrt(mean x^2 + eps), which it adds up from the tiles' sums in a
//     fixed order, before it rounds (and, for gate/up, applies SwiGLU).
//
// Rounding.  The reference rounds x * rstd to 16 bits, then multiplies by g and rounds again.  rstd
// is not known while x is being made, so here x itself is rounded, multiplied by g and rounded, and
// rstd multiplies the finished sum in 32 bits: the same number of roundings of the same relative
// size at another place, not bit-identical.  The 32-bit path does not use these kernels.
//
// Shape of the work.  A workgroup (4 waves) owns 8 output columns per row group (RG = 1 or 2) and all
// of K; no partial sums leave it.  With at most 8 rows a 16x16x32 matrix instruction has half its
// rows idle, so each instruction serves two halves of the wave's K range at once: operand rows 0..7
// are the 8 batch rows (weight columns) over the first half, rows 8..15 the same over the second
// half; of the 16x16 result only the two diagonal 8x8 blocks mean anything and are added.  Every lane
// asks for all its weight bytes of a trip at once (32 contiguous bytes per row and unit, four lanes
// one 128-byte line), two trips in flight.  The waves' sums meet in LDS in a fixed order.
//
// More rows than 8 go through the shared-rows product with norms of their own (gemm_skinny.hip): every
// workgroup here reads all of X, M x K per 8 or 16 output columns, from L2, which at 8 rows is as many
// bytes as the weights themselves (a 16-row variant of this kernel lost to the shared-rows path at every
// size measured: TinyLlama sizes batch 16 1.26 -> 1.17 ms, Llama-3-8B sizes 4.82 -> 4.05 ms).
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

namespace {

constexpr int kUnit = 64;   // k elements per unit: 4 lanes x 16 elements = one 128-byte line per row
constexpr int kCols = 8;    // output columns per row group

union Frag {
  uint4 u;
  bf16x8 v;
};

enum Epilogue : int { kStore = 0, kSwiglu = 1, kResidualNorm = 2 };

struct Gemm8Args {
  const uint16_t* X; int ldx;
  const uint16_t* W; int ldw;
  int M, N, K;
  const float* ss_in; int tiles_in; float inv_width, eps;   // SCALED
  void* out; int ldo;                                       // kStore, kSwiglu
  float* resid; const void* g; int g_f32; uint16_t* xg; float* ss_out;   // kResidualNorm (width N)
};

// One trip: UT units of this lane's weight rows (RG groups) and of its batch row.
template <int RG, int UT>
struct Trip {
  Frag w[RG][UT][2];
  Frag x[UT][2];
};

template <int NW, int RG, int UT, bool SCALED, int EPI, class TO>
__global__ void __launch_bounds__(NW * kWave) gemm8_kernel(const Gemm8Args a) {
  static_assert(NW == 4 || NW == 8, "four or eight waves share a tile's K");
  constexpr int kSlots = 2 * NW, kRowsPerWave = 8 / NW;
  __shared__ f32x4 red[NW][RG][kWave];
  __shared__ float rstd_s[8];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int r = lane % 16, kq = lane / 16;
  const int half = r / 8, c = r % 8;
  const int n0 = blockIdx.x * (kCols * RG);   // kSwiglu: N is the width of the result, RG == 2 means gate and up
  const int units = a.K / kUnit;
  // this lane's slice of K: slot = 2 * wave + half of 2 * NW
  const int slot = 2 * wave + half;
  const int u_lo = units * slot / kSlots, u_hi = units * (slot + 1) / kSlots;
  const int cnt = u_hi - u_lo;
  const int other = units * (slot ^ 1) / kSlots;
  const int cnt_other = units * ((slot ^ 1) + 1) / kSlots - other;
  const int n_main = cnt < cnt_other ? cnt : cnt_other, n_max = cnt > cnt_other ? cnt : cnt_other;

  const uint16_t* wrow[RG];
#pragma unroll
  for (int g = 0; g < RG; ++g) {
    // kSwiglu: group 0 holds gate rows, group 1 the up rows of the same columns (W is [gate | up])
    const int row = EPI == kSwiglu ? (g == 0 ? n0 / 2 + c : a.N + n0 / 2 + c) : n0 + g * kCols + c;
    wrow[g] = a.W + size_t(row) * a.ldw + kq * 16;
  }
  const uint16_t* xrow = a.X + size_t(c < a.M ? c : 0) * a.ldx + kq * 16;

  f32x4 acc[RG];
#pragma unroll
  for (int g = 0; g < RG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto fetch = [&](int j0, Trip<RG, UT>& t) {
#pragma unroll
    for (int d = 0; d < UT; ++d) {
      int j = j0 + d;
      j = j < cnt ? j : (cnt > 0 ? cnt - 1 : 0);   // beyond the slice: repeat its last unit, not multiplied
      const size_t off = size_t(u_lo + j < units ? u_lo + j : 0) * kUnit;
#pragma unroll
      for (int g = 0; g < RG; ++g) {
        t.w[g][d][0].u = *reinterpret_cast<const uint4*>(wrow[g] + off);
        t.w[g][d][1].u = *reinterpret_cast<const uint4*>(wrow[g] + off + 8);
      }
      t.x[d][0].u = *reinterpret_cast<const uint4*>(xrow + off);
      t.x[d][1].u = *reinterpret_cast<const uint4*>(xrow + off + 8);
    }
  };
  auto multiply = [&](int j0, const Trip<RG, UT>& t) {
#pragma unroll
    for (int d = 0; d < UT; ++d) {
      const int j = j0 + d;
      if (j >= n_max) break;                      // uniform over the wave
      Frag x0 = t.x[d][0], x1 = t.x[d][1];
      if (j >= n_main && j >= cnt) {              // this half of the wave has run out: its rows add nothing
        x0.u = uint4{0u, 0u, 0u, 0u};
        x1.u = uint4{0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int g = 0; g < RG; ++g) {
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x0.v, t.w[g][d][0].v, acc[g], 0, 0, 0);
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x1.v, t.w[g][d][1].v, acc[g], 0, 0, 0);
      }
    }
  };
  // What the epilogue needs from memory is asked for ahead of the weights and used behind their
  // requests, so that it is worked on while the weights are on their way: the tiles' sums of squares
  // of up to two rows per wave (SCALED; added up in a fixed order), and this thread's element of the
  // residual stream and of the norm's weight (kResidualNorm; threads of the first wave).
  constexpr int kSsRegs = 4;   // tiles per lane kept in registers: widths up to 8 * 64 * 4 = 2048; wider rows add the rest directly
  float ssv[kRowsPerWave][kSsRegs];
  float ss_more[kRowsPerWave] = {};
  const int em = threadIdx.x / 8, en = threadIdx.x % 8;   // the epilogue's (row, column) of the first 64 threads
  float resid_in = 0.f, g_in = 0.f;
  auto ask_epilogue = [&]() {
    if constexpr (SCALED) {
#pragma unroll
      for (int i = 0; i < kRowsPerWave; ++i) {
        const int m = wave + NW * i;
        const float* p = a.ss_in + size_t(m < a.M ? m : 0) * a.tiles_in;
#pragma unroll
        for (int q = 0; q < kSsRegs; ++q) {
          const int t = lane + q * kWave;
          ssv[i][q] = p[t < a.tiles_in ? t : 0];
        }
        for (int t = lane + kSsRegs * kWave; t < a.tiles_in; t += kWave) ss_more[i] += p[t];
      }
    }
    if constexpr (EPI == kResidualNorm) {
      if (threadIdx.x < kWave) {
        const int col = n0 + en;
        resid_in = a.resid[size_t(em < a.M ? em : 0) * a.N + col];
        g_in = a.g_f32 ? static_cast<const float*>(a.g)[col] : load_f(static_cast<const bf16_t*>(a.g) + col);
      }
    }
  };
  auto rstd_to_lds = [&]() {
    if constexpr (SCALED) {
#pragma unroll
      for (int i = 0; i < kRowsPerWave; ++i) {
        float part = ss_more[i];
#pragma unroll
        for (int q = 0; q < kSsRegs; ++q) part += (lane + q * kWave < a.tiles_in) ? ssv[i][q] : 0.f;
        const float s = wave_sum(part);
        if (lane == 0) rstd_s[wave + NW * i] = rsqrtf(s * a.inv_width + a.eps);
      }
    }
  };
  ask_epilogue();
  if (n_max > 0) {
    Trip<RG, UT> ta, tb;
    fetch(0, ta);
    if (UT < n_max) fetch(UT, tb);
    rstd_to_lds();
    for (int j0 = 0; j0 < n_max; j0 += 2 * UT) {
      multiply(j0, ta);
      if (j0 + UT >= n_max) break;
      if (j0 + 2 * UT < n_max) fetch(j0 + 2 * UT, ta);
      multiply(j0 + UT, tb);
      if (j0 + 3 * UT < n_max) fetch(j0 + 3 * UT, tb);
    }
  } else {
    rstd_to_lds();
  }

#pragma unroll
  for (int g = 0; g < RG; ++g) red[wave][g][lane] = acc[g];
  __syncthreads();
  if (threadIdx.x >= kWave) return;

  // thread -> (row m, column n of a group): the two diagonal blocks of every wave's result
  const int m = em, n = en;
  float v[RG];
#pragma unroll
  for (int g = 0; g < RG; ++g) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      s += red[w][g][(m / 4) * 16 + n][m % 4];
      s += red[w][g][(2 + m / 4) * 16 + n + 8][m % 4];
    }
    v[g] = SCALED ? s * rstd_s[m] : s;
  }
  const bool live = m < a.M;
  if constexpr (EPI == kStore) {
    if (live) {
#pragma unroll
      for (int g = 0; g < RG; ++g) store_f(static_cast<TO*>(a.out) + size_t(m) * a.ldo + n0 + g * kCols + n, v[g]);
    }
  } else if constexpr (EPI == kSwiglu) {
    static_assert(EPI != kSwiglu || RG == 2, "gate and up are the two row groups");
    if (live) {
      const float gate = round_to<TO>(v[0]);
      const float act = silu<TO>(gate);
      store_f(static_cast<TO*>(a.out) + size_t(m) * a.ldo + n0 / 2 + n, round_to<TO>(act) * round_to<TO>(v[RG - 1]));
    }
  } else {
    static_assert(EPI != kResidualNorm || RG == 1, "one 8-column tile per workgroup leaves one sum of squares");
    const int col = n0 + n;
    float xn = 0.f;
    if (live) {
      xn = resid_in + round_to<bf16_t>(v[0]);
      a.resid[size_t(m) * a.N + col] = xn;
      a.xg[size_t(m) * a.N + col] = float_to_bf16_bits(g_in * round_to<bf16_t>(xn));
    }
    float sq = xn * xn;
    sq += __shfl_xor(sq, 1, kWave);
    sq += __shfl_xor(sq, 2, kWave);
    sq += __shfl_xor(sq, 4, kWave);
    if (live && n == 0) a.ss_out[size_t(m) * (a.N / kCols) + blockIdx.x] = sq;
  }
}

bool operands_ok(const Gemm8Args& a) {
  return a.ldx % 8 == 0 && a.ldw % 8 == 0 && reinterpret_cast<uintptr_t>(a.X) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(a.W) % 16 == 0 && a.ldx >= a.K && a.ldw >= a.K;
}

}  // namespace
}  // namespace kvcm

using namespace kvcm;

extern "C" {

// Shapes these kernels take: at most 8 rows with whole 8-column tiles; whole 64-element units of K.
int kvcm_gemm8_supported(int M, int N, int K) {
  return M >= 1 && M <= 8 && K >= kUnit && K % kUnit == 0 && N >= 8 && N % 8 == 0;
}

// out[M, N] = (X * W^T) (* rstd per row when ss_in is given: X is then xg of a producer, ss_in its
// [M][tiles_in] sums of squares over a width of 8 * tiles_in, eps the norm's).  swiglu != 0: W is
// [gate (N rows) | up (N rows)] and out[M, N] = round(silu(round(gate))) * round(up).
int kvcm_gemm8(const void* X, int ldx, const void* W, int ldw, int M, int N, int K, const float* ss_in, int tiles_in,
               float eps, void* out, int out_dtype, int ldo, int swiglu, hipStream_t st) {
  KVCM_REQUIRE(kvcm_gemm8_supported(M, N, K), "gemm8: unsupported shape M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "gemm8: unknown output dtype %d", out_dtype);
  KVCM_REQUIRE(out != nullptr && ldo >= N, "gemm8: missing output or leading dimension below N");
  KVCM_REQUIRE(ss_in == nullptr || tiles_in > 0, "gemm8: sums of squares without their count");
  Gemm8Args a{};
  a.X = static_cast<const uint16_t*>(X); a.ldx = ldx; a.W = static_cast<const uint16_t*>(W); a.ldw = ldw;
  a.M = M; a.N = N; a.K = K; a.ss_in = ss_in; a.tiles_in = tiles_in;
  a.inv_width = tiles_in > 0 ? 1.0f / float(tiles_in * kCols) : 0.f; a.eps = eps; a.out = out; a.ldo = ldo;
  KVCM_REQUIRE(operands_ok(a), "gemm8: operands must be 16-byte aligned with leading dimensions that are multiples of 8 and at least K");
  const bool scaled = ss_in != nullptr;
  // longer trips where two trips of UT units per half would not have a tile's whole K on its way at once
#define KVCM_G8(RG, UT, SC, EP, TO)                                                         \
  do {                                                                                      \
    if (K / kUnit > 8 * 2 * UT) gemm8_kernel<4, RG, UT + UT / 2, SC, EP, TO><<<grid, 256, 0, st>>>(a); \
    else gemm8_kernel<4, RG, UT, SC, EP, TO><<<grid, 256, 0, st>>>(a);                      \
  } while (0)
  if (swiglu) {
    const dim3 grid(N / kCols);
    if (out_dtype == kBF16) { if (scaled) KVCM_G8(2, 2, true, kSwiglu, bf16_t); else KVCM_G8(2, 2, false, kSwiglu, bf16_t); }
    else { if (scaled) KVCM_G8(2, 2, true, kSwiglu, float); else KVCM_G8(2, 2, false, kSwiglu, float); }
    return launch_status("gemm8_swiglu");
  }
  // two row groups per workgroup once a single one would give more than about four workgroups per CU
  // (measured in whole decode steps: the head and the QKV product of a 7B model), and also where that leaves no CU
  // with more columns than it has with one (TinyLlama's QKV product: 320 tiles are two workgroups on 64 of the
  // 256 CUs either way, and 160 workgroups of two groups start and end faster: batch 8 1.027 -> 1.008 ms; at 768
  // tiles, a width of 4,096 with 8 KV heads, two groups give some CUs four tiles instead of three and are slower)
  constexpr int kCUs = 256;
  const int tiles = N / kCols;
  const bool two_fit = tiles > kCUs && 2 * ((tiles / 2 + kCUs - 1) / kCUs) <= (tiles + kCUs - 1) / kCUs;
  if (N % (2 * kCols) == 0 && (tiles > 1024 || two_fit)) {
    const dim3 grid(N / (2 * kCols));
    if (out_dtype == kBF16) { if (scaled) KVCM_G8(2, 2, true, kStore, bf16_t); else KVCM_G8(2, 2, false, kStore, bf16_t); }
    else { if (scaled) KVCM_G8(2, 2, true, kStore, float); else KVCM_G8(2, 2, false, kStore, float); }
  } else {
    const dim3 grid(N / kCols);
    if (out_dtype == kBF16) { if (scaled) KVCM_G8(1, 4, true, kStore, bf16_t); else KVCM_G8(1, 4, false, kStore, bf16_t); }
    else { if (scaled) KVCM_G8(1, 4, true, kStore, float); else KVCM_G8(1, 4, false, kStore, float); }
  }
  return launch_status("gemm8");
}

// resid[M, N] += round(X * W^T); xg[M, N] = round(g * round(resid)); ss_out[M][N / 8] = sums of resid^2
// per 8-column tile.  g: the following norm's weight, float32 or bfloat16.
int kvcm_gemm8_residual_norm(const void* X, int ldx, const void* W, int ldw, int M, int N, int K, float* resid,
                             const void* g, int g_dtype, void* xg, float* ss_out, hipStream_t st) {
  KVCM_REQUIRE(kvcm_gemm8_supported(M, N, K), "gemm8_residual_norm: unsupported shape M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(resid != nullptr && g != nullptr && xg != nullptr && ss_out != nullptr, "gemm8_residual_norm: null operand");
  KVCM_REQUIRE(g_dtype == kBF16 || g_dtype == kF32, "gemm8_residual_norm: unknown weight dtype %d", g_dtype);
  Gemm8Args a{};
  a.X = static_cast<const uint16_t*>(X); a.ldx = ldx; a.W = static_cast<const uint16_t*>(W); a.ldw = ldw;
  a.M = M; a.N = N; a.K = K; a.resid = resid; a.g = g; a.g_f32 = g_dtype == kF32; a.xg = static_cast<uint16_t*>(xg);
  a.ss_out = ss_out;
  KVCM_REQUIRE(operands_ok(a), "gemm8_residual_norm: operands must be 16-byte aligned with leading dimensions that are multiples of 8 and at least K");
  const dim3 grid(N / kCols);
  if (K / kUnit > 8 * 2 * 4) gemm8_kernel<4, 1, 6, false, kResidualNorm, bf16_t><<<grid, 256, 0, st>>>(a);
  else gemm8_kernel<4, 1, 4, false, kResidualNorm, bf16_t><<<grid, 256, 0, st>>>(a);
  return launch_status("gemm8_residual_norm");
}

}  // extern "C"
