// Decode-shaped products: Y[M,N] = X[M,K] * W[N,K]^T with few rows (M <= 64) and a weight matrix
// that has to be streamed from HBM once.  The reference leaves these to cuBLAS
// (src/model/llama.cpp:45-52); here the point is to keep enough weight bytes in flight on 256 CUs.
//
// One workgroup (4 waves) owns 16 output columns and one slice of K ("split"); its waves divide
// the slice among themselves, each streaming its rows of W straight from global memory into
// MFMA operand registers (every lane 32 contiguous bytes, four lanes one 128-byte line) and
// multiplying with the matching pieces of X (v_mfma_f32_16x16x32_bf16).  The four waves' sums
// are added through LDS in a fixed order.  With one split the result is stored; with S splits the
// 32-bit partial sums go to scratch [S][M][N] and the consumer adds them in split order:
// reduce_store below, or the fused consumers (residual add + RMS norm, SwiGLU, rotary + cache
// write) in elementwise.hip.  No atomics: the result is the same on every run.
//
// SWIGLU variant: W is a fused [gate (I rows) | up (I rows)] matrix; a workgroup takes 8 gate rows
// and the 8 up rows of the same columns, and stores act = round(round(silu(g)) * u) [M, I]
// directly (g, u rounded to the storage type first, exactly what the separate SwiGLU kernel
// computes from the stored product).  Unsplit only.
#include "common.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kUnit = 64;  // k elements per unit: 4 lanes x 16 elements = one 128-byte line per row

union Frag {
  uint4 u;
  bf16x8 v;
};

template <int MT, class TO, bool SWIGLU>
__global__ void __launch_bounds__(256)
    gemm_skinny_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W, float* __restrict__ partials,
                       TO* __restrict__ out, int M, int N, int K, int ldx, int ldw, int ldo, int S) {
  __shared__ f32x4 red[4][MT][kWave];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int r = lane % 16, kq = lane / 16;
  const int n0 = blockIdx.x * (SWIGLU ? 8 : 16);   // SWIGLU: N is I, the width of the result
  const int s = blockIdx.y;
  const int units = K / kUnit;
  const int u_lo = int((long long)units * s / S), u_hi = int((long long)units * (s + 1) / S);
  const int span = u_hi - u_lo;
  const int w_lo = u_lo + span * wave / 4, w_hi = u_lo + span * (wave + 1) / 4;

  const uint16_t* wrow = W + size_t(SWIGLU ? (r < 8 ? n0 + r : N + n0 + r - 8) : n0 + r) * ldw + kq * 16;
  const uint16_t* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    xrow[t] = X + size_t(m < M ? m : 0) * ldx + kq * 16;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  int u = w_lo;
  for (; u + 2 <= w_hi; u += 2) {  // two units per trip: four weight loads in flight per lane
    Frag b[4];
    const uint16_t* p = wrow + size_t(u) * kUnit;
    b[0].u = *reinterpret_cast<const uint4*>(p);
    b[1].u = *reinterpret_cast<const uint4*>(p + 8);
    b[2].u = *reinterpret_cast<const uint4*>(p + kUnit);
    b[3].u = *reinterpret_cast<const uint4*>(p + kUnit + 8);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      // rows beyond M read row 0 (always there) and are dropped at the store: no branch
      // around a load, which would make the compiler wait for it on the spot
      Frag a[4];
      const uint16_t* q = xrow[t] + size_t(u) * kUnit;
      a[0].u = *reinterpret_cast<const uint4*>(q);
      a[1].u = *reinterpret_cast<const uint4*>(q + 8);
      a[2].u = *reinterpret_cast<const uint4*>(q + kUnit);
      a[3].u = *reinterpret_cast<const uint4*>(q + kUnit + 8);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, b[i].v, acc[t], 0, 0, 0);
    }
  }
  for (; u < w_hi; ++u) {
    Frag b[2];
    const uint16_t* p = wrow + size_t(u) * kUnit;
    b[0].u = *reinterpret_cast<const uint4*>(p);
    b[1].u = *reinterpret_cast<const uint4*>(p + 8);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      Frag a[2];
      const uint16_t* q = xrow[t] + size_t(u) * kUnit;
      a[0].u = *reinterpret_cast<const uint4*>(q);
      a[1].u = *reinterpret_cast<const uint4*>(q + 8);
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, b[i].v, acc[t], 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  if constexpr (SWIGLU) {
    for (int item = threadIdx.x; item < MT * kWave; item += 256) {
      const int t = item / kWave, l = item % kWave;
      if (l % 16 >= 8) continue;
      f32x4 g = red[0][t][l], up = red[0][t][l + 8];
#pragma unroll
      for (int w = 1; w < 4; ++w) {
        const f32x4 a = red[w][t][l], b = red[w][t][l + 8];
        g[0] += a[0]; g[1] += a[1]; g[2] += a[2]; g[3] += a[3];
        up[0] += b[0]; up[1] += b[1]; up[2] += b[2]; up[3] += b[3];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = t * 16 + (l / 16) * 4 + i;
        if (m >= M) continue;
        const float x = round_to<TO>(g[i]);
        const float act = x / (1.0f + expf(-x));
        store_f(out + size_t(m) * ldo + n0 + l % 16, round_to<TO>(act) * round_to<TO>(up[i]));
      }
    }
    return;
  }
  for (int item = threadIdx.x; item < MT * kWave; item += 256) {
    const int t = item / kWave, l = item % kWave;
    f32x4 v = red[0][t][l];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const f32x4 o = red[w][t][l];
      v[0] += o[0]; v[1] += o[1]; v[2] += o[2]; v[3] += o[3];
    }
    const int n = n0 + l % 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = t * 16 + (l / 16) * 4 + i;
      if (m >= M) continue;
      if (S > 1) partials[(size_t(s) * M + m) * N + n] = v[i];
      else store_f(out + size_t(m) * ldo + n, v[i]);
    }
  }
}

// The same product for 17 .. 64 rows.  With that many rows X is no longer small: every 16-column
// tile needs all of it, and re-reading it from L2 per tile would cost four times the weights'
// bytes.  Here a workgroup owns 64 columns (one 16-column tile per wave) and a slice of K, and
// its waves share X through LDS: per step of 64 k the workgroup stages X[rows][64] once
// (double-buffered, the next step's global loads are issued before the current step's products),
// every wave streams its own 16 weight rows from HBM and multiplies them with the staged rows.
// No reduction between waves; split-K partial sums as above.  SWIGLU: a wave's tile is 8 gate + 8
// up rows, the workgroup stores 32 activation columns.
constexpr int kXPad = 8;    // bfloat16 of padding per staged row, so that rows spread over the banks
constexpr int kDepth = 4;   // units of 64 k per trip: what a lane has in flight is 4 x (32 B of W + 32 B of X)

// KH = 2: eight waves, the second four take the second half of the workgroup's K slice with X
// buffers of their own, and the halves are added through LDS at the end (first half + second
// half).  For launches with far fewer workgroups than CUs (a product that may not be split and
// has few columns): twice the waves at work per CU.
template <int MT, int KH, class TO, bool SWIGLU>
__global__ void __launch_bounds__(256 * KH)
    gemm_rows64_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W, float* __restrict__ partials,
                       TO* __restrict__ out, int M, int N, int K, int ldx, int ldw, int ldo, int S) {
  __shared__ __attribute__((aligned(16))) uint16_t xs[KH][2][MT * 16][kDepth * kUnit + kXPad];
  const int kh = threadIdx.x / 256, tid = threadIdx.x % 256;
  const int wave = tid / kWave, lane = tid % kWave;
  const int r = lane % 16, kq = lane / 16;
  constexpr int kCols = SWIGLU ? 8 : 16;
  const int c0 = blockIdx.x * (4 * kCols) + wave * kCols;   // this wave's first output column
  const int s = blockIdx.y;
  const int units = K / kUnit;
  const int s_lo = int((long long)units * s / S), s_hi = int((long long)units * (s + 1) / S);
  const int u_lo = s_lo + (s_hi - s_lo) * kh / KH, u_hi = s_lo + (s_hi - s_lo) * (kh + 1) / KH;
  // every wave of the workgroup runs the same number of trips (and barriers): that of the longer half
  const int trips = ((s_hi - s_lo + KH - 1) / KH + kDepth - 1) / kDepth;

  const uint16_t* wrow = W + size_t(SWIGLU ? (r < 8 ? c0 + r : N + c0 + r - 8) : c0 + r) * ldw + kq * 16;
  // staging: thread -> (row tid / 4, 16 elements at (tid % 4) * 16 of every unit); rows beyond M
  // read row 0 and are dropped at the store
  const int srow = tid / 4, sseg = (tid % 4) * 16;
  const bool stages = srow < MT * 16;                         // uniform per wave
  const uint16_t* xsrc = X + size_t(srow < M ? srow : 0) * ldx + sseg;

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // A trip's operands: kDepth units of this wave's weight rows and of this thread's piece of X.
  // Units beyond the slice repeat its last unit (no load behind a branch) and are not multiplied.
  struct Trip {
    Frag b[kDepth][2];
    uint4 x[kDepth][2];
  };
  // Workgroups walk their slice from different starting points (and wrap around): if all of them
  // read the same k at the same time, their rows, a multiple of 4 KB apart, would queue up at the
  // same few memory channels.
  const int span = u_hi - u_lo > 0 ? u_hi - u_lo : 1;   // (an empty half cannot happen: a slice has at least KH units)
  const int phase = (blockIdx.x * 5) % span;   // the same for all waves that share staged X
  auto fetch = [&](int j0, Trip& tr) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int j = j0 + d < span ? j0 + d : span - 1;
      const int u = u_lo + (j + phase) % span;
      const uint16_t* p = wrow + size_t(u) * kUnit;
      tr.b[d][0].u = *reinterpret_cast<const uint4*>(p);
      tr.b[d][1].u = *reinterpret_cast<const uint4*>(p + 8);
      const uint16_t* q = xsrc + size_t(u) * kUnit;
      tr.x[d][0] = *reinterpret_cast<const uint4*>(q);
      tr.x[d][1] = *reinterpret_cast<const uint4*>(q + 8);
    }
  };
  auto stage = [&](int buf, const Trip& tr) {
    if (stages) {
#pragma unroll
      for (int d = 0; d < kDepth; ++d) {
        *reinterpret_cast<uint4*>(&xs[kh][buf][srow][d * kUnit + sseg]) = tr.x[d][0];
        *reinterpret_cast<uint4*>(&xs[kh][buf][srow][d * kUnit + sseg + 8]) = tr.x[d][1];
      }
    }
  };
  auto multiply = [&](int buf, int j0, const Trip& tr) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      if (j0 + d >= span) break;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        Frag a0, a1;
        a0.u = *reinterpret_cast<const uint4*>(&xs[kh][buf][t * 16 + r][d * kUnit + kq * 16]);
        a1.u = *reinterpret_cast<const uint4*>(&xs[kh][buf][t * 16 + r][d * kUnit + kq * 16 + 8]);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, tr.b[d][0].v, acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, tr.b[d][1].v, acc[t], 0, 0, 0);
      }
    }
  };
  // Two trips in registers: while one is multiplied, the next one's loads are on their way.  LDS
  // buffer i holds the X of the trip in register set i; a buffer is written one barrier after its
  // last read.
  {
    Trip ta, tb;
    fetch(0, ta);
    for (int i = 0; i < trips; i += 2) {
      const int j0 = i * kDepth;
      fetch(j0 + kDepth, tb);
      stage(0, ta);
      __syncthreads();
      multiply(0, j0, ta);
      if (i + 1 >= trips) break;
      fetch(j0 + 2 * kDepth, ta);
      stage(1, tb);
      __syncthreads();
      multiply(1, j0 + kDepth, tb);
    }
  }
  if constexpr (KH == 2) {   // second half -> LDS -> first half
    __syncthreads();         // nobody reads staged X any more
    f32x4* red = reinterpret_cast<f32x4*>(&xs[0][0][0][0]);
    if (kh == 1) {
#pragma unroll
      for (int t = 0; t < MT; ++t) red[(wave * MT + t) * kWave + lane] = acc[t];
    }
    __syncthreads();
    if (kh == 1) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const f32x4 o = red[(wave * MT + t) * kWave + lane];
      acc[t][0] += o[0]; acc[t][1] += o[1]; acc[t][2] += o[2]; acc[t][3] += o[3];
    }
  }
  // accumulator: column = r of the wave's tile, rows = 4 kq + i
  if constexpr (SWIGLU) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      f32x4 up;
#pragma unroll
      for (int i = 0; i < 4; ++i) up[i] = __shfl(acc[t][i], (lane & ~15) | ((r + 8) & 15), kWave);
      if (r >= 8) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = t * 16 + kq * 4 + i;
        if (m >= M) continue;
        const float x = round_to<TO>(acc[t][i]);
        const float act = x / (1.0f + expf(-x));
        store_f(out + size_t(m) * ldo + c0 + r, round_to<TO>(act) * round_to<TO>(up[i]));
      }
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = t * 16 + kq * 4 + i;
      if (m >= M) continue;
      if (S > 1) partials[(size_t(s) * M + m) * N + c0 + r] = acc[t][i];
      else store_f(out + size_t(m) * ldo + c0 + r, acc[t][i]);
    }
}

// out[m][n] = sum over splits, in split order.
template <class TO>
__global__ void reduce_store_kernel(const float* __restrict__ partials, TO* __restrict__ out, int M, int N, int ldo, int S) {
  const size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x;
  if (i >= size_t(M) * N) return;
  float v = 0.f;
  for (int s = 0; s < S; ++s) v += partials[size_t(s) * M * N + i];
  store_f(out + (i / N) * ldo + i % N, v);
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// More than 16 rows and whole groups of 64 columns: the kernel whose waves share X through LDS.
static bool shares_rows(int M, int N) { return M > 16 && N % 64 == 0; }

// How many splits of K a launch of this shape uses (0: the shape is not supported by this kernel).
int kvcm_gemm_skinny_splits(int M, int N, int K) {
  if (M <= 0 || M > 64 || N % 16 != 0 || K % kUnit != 0 || N <= 0 || K <= 0) return 0;
  if (shares_rows(M, N)) {
    const int groups = N / 64, units = K / kUnit;
    if (groups >= 256) return 1;
    int S = (512 + groups - 1) / groups;       // aim at two workgroups per CU ...
    if (S > units / 4) S = units / 4;          // ... of at least four steps each ...
    if (S > 8) S = 8;                          // ... and partial sums that stay small beside the weights
    return S < 1 ? 1 : S;
  }
  const int tiles = N / 16, units = K / kUnit;
  int S = (640 + tiles - 1) / tiles;           // aim at >= 640 workgroups (2.5 per CU)
  if (S > units / 2) S = units / 2;            // at least two units per split ...
  if (S < 1) S = 1;
  if (S > 16) S = 16;
  return S;
}

// S == 1: the result is stored to `out` (bfloat16 or float32).  S > 1: partial sums are written to
// `partials` [S][M][N]; `out` is not touched (pass S from kvcm_gemm_skinny_splits).
int kvcm_gemm_skinny(const void* X, const void* W, float* partials, void* out, int out_dtype, int M, int N, int K,
                     int ldx, int ldw, int ldo, int S, hipStream_t st) {
  KVCM_REQUIRE(kvcm_gemm_skinny_splits(M, N, K) > 0, "gemm_skinny: unsupported shape M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(S >= 1 && S <= K / kUnit, "gemm_skinny: bad split count %d", S);
  KVCM_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && reinterpret_cast<uintptr_t>(X) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(W) % 16 == 0,
               "gemm_skinny: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
  KVCM_REQUIRE(ldx >= K && ldw >= K, "gemm_skinny: leading dimensions too small");
  KVCM_REQUIRE(S == 1 ? (out != nullptr && ldo >= N) : partials != nullptr, "gemm_skinny: missing output buffer");
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const uint16_t* w = static_cast<const uint16_t*>(W);
  const int mt = (M + 15) / 16;
  if (shares_rows(M, N)) {
    const dim3 grid64(N / 64, S);
    const bool two_halves = (N / 64) * S < 128 && K / kUnit / S >= 4 * kDepth;   // far fewer workgroups than CUs
#define KVCM_ROWS64(MT, TO) \
  do {                                                                                                             \
    if (two_halves)                                                                                                \
      gemm_rows64_kernel<MT, 2, TO, false><<<grid64, 512, 0, st>>>(x, w, partials, static_cast<TO*>(out), M, N, K, ldx, ldw, ldo, S); \
    else                                                                                                           \
      gemm_rows64_kernel<MT, 1, TO, false><<<grid64, 256, 0, st>>>(x, w, partials, static_cast<TO*>(out), M, N, K, ldx, ldw, ldo, S); \
  } while (0)
    if (out_dtype == kBF16) {
      if (mt == 2) KVCM_ROWS64(2, bf16_t); else if (mt == 3) KVCM_ROWS64(3, bf16_t); else KVCM_ROWS64(4, bf16_t);
    } else if (out_dtype == kF32) {
      if (mt == 2) KVCM_ROWS64(2, float); else if (mt == 3) KVCM_ROWS64(3, float); else KVCM_ROWS64(4, float);
    } else {
      KVCM_REQUIRE(false, "gemm_skinny: unknown output dtype %d", out_dtype);
    }
#undef KVCM_ROWS64
    return launch_status("gemm_rows64");
  }
  const dim3 grid(N / 16, S);
#define KVCM_SKINNY(MT, TO) \
  gemm_skinny_kernel<MT, TO, false><<<grid, 256, 0, st>>>(x, w, partials, static_cast<TO*>(out), M, N, K, ldx, ldw, ldo, S)
  if (out_dtype == kBF16) {
    if (mt == 1) KVCM_SKINNY(1, bf16_t); else if (mt == 2) KVCM_SKINNY(2, bf16_t); else if (mt == 3) KVCM_SKINNY(3, bf16_t); else KVCM_SKINNY(4, bf16_t);
  } else if (out_dtype == kF32) {
    if (mt == 1) KVCM_SKINNY(1, float); else if (mt == 2) KVCM_SKINNY(2, float); else if (mt == 3) KVCM_SKINNY(3, float); else KVCM_SKINNY(4, float);
  } else {
    KVCM_REQUIRE(false, "gemm_skinny: unknown output dtype %d", out_dtype);
  }
#undef KVCM_SKINNY
  return launch_status("gemm_skinny");
}

// May act = swiglu(X * [gate | up]^T) be computed in one launch?  I is the width of the result.
int kvcm_gemm_skinny_swiglu_supported(int M, int I, int K) {
  if (!(M > 0 && M <= 64 && I > 0 && I % 8 == 0 && K > 0 && K % kUnit == 0)) return 0;
  // with too few workgroups a split product fills the chip better than this unsplit one
  if (M > 16 && I % 32 == 0) return I / 32 >= 160;
  return I / 8 >= 320;
}

// W [2 I, K] (gate rows, then up rows); out [M, I].
int kvcm_gemm_skinny_swiglu(const void* X, const void* W, void* out, int out_dtype, int M, int I, int K, int ldx,
                            int ldw, int ldo, hipStream_t st) {
  KVCM_REQUIRE(kvcm_gemm_skinny_swiglu_supported(M, I, K), "gemm_skinny_swiglu: unsupported shape M=%d I=%d K=%d", M, I, K);
  KVCM_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && reinterpret_cast<uintptr_t>(X) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(W) % 16 == 0,
               "gemm_skinny_swiglu: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
  KVCM_REQUIRE(ldx >= K && ldw >= K && out != nullptr && ldo >= I, "gemm_skinny_swiglu: leading dimensions too small");
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const uint16_t* w = static_cast<const uint16_t*>(W);
  const int mt = (M + 15) / 16;
  if (M > 16 && I % 32 == 0) {
    const dim3 grid32(I / 32, 1);
    const bool two_halves = I / 32 < 128 && K / kUnit >= 4 * kDepth;   // far fewer workgroups than CUs
#define KVCM_ROWS64(MT, TO) \
  do {                                                                                                             \
    if (two_halves)                                                                                                \
      gemm_rows64_kernel<MT, 2, TO, true><<<grid32, 512, 0, st>>>(x, w, nullptr, static_cast<TO*>(out), M, I, K, ldx, ldw, ldo, 1); \
    else                                                                                                           \
      gemm_rows64_kernel<MT, 1, TO, true><<<grid32, 256, 0, st>>>(x, w, nullptr, static_cast<TO*>(out), M, I, K, ldx, ldw, ldo, 1); \
  } while (0)
    if (out_dtype == kBF16) {
      if (mt == 2) KVCM_ROWS64(2, bf16_t); else if (mt == 3) KVCM_ROWS64(3, bf16_t); else KVCM_ROWS64(4, bf16_t);
    } else if (out_dtype == kF32) {
      if (mt == 2) KVCM_ROWS64(2, float); else if (mt == 3) KVCM_ROWS64(3, float); else KVCM_ROWS64(4, float);
    } else {
      KVCM_REQUIRE(false, "gemm_skinny_swiglu: unknown output dtype %d", out_dtype);
    }
#undef KVCM_ROWS64
    return launch_status("gemm_rows64_swiglu");
  }
  const dim3 grid(I / 8, 1);
#define KVCM_SKINNY(MT, TO) \
  gemm_skinny_kernel<MT, TO, true><<<grid, 256, 0, st>>>(x, w, nullptr, static_cast<TO*>(out), M, I, K, ldx, ldw, ldo, 1)
  if (out_dtype == kBF16) {
    if (mt == 1) KVCM_SKINNY(1, bf16_t); else if (mt == 2) KVCM_SKINNY(2, bf16_t); else if (mt == 3) KVCM_SKINNY(3, bf16_t); else KVCM_SKINNY(4, bf16_t);
  } else if (out_dtype == kF32) {
    if (mt == 1) KVCM_SKINNY(1, float); else if (mt == 2) KVCM_SKINNY(2, float); else if (mt == 3) KVCM_SKINNY(3, float); else KVCM_SKINNY(4, float);
  } else {
    KVCM_REQUIRE(false, "gemm_skinny_swiglu: unknown output dtype %d", out_dtype);
  }
#undef KVCM_SKINNY
  return launch_status("gemm_skinny_swiglu");
}

int kvcm_reduce_store(const float* partials, void* out, int out_dtype, int M, int N, int ldo, int S, hipStream_t st) {
  if (M == 0 || N == 0) return 0;
  KVCM_REQUIRE(M > 0 && N > 0 && S >= 1 && ldo >= N, "reduce_store: bad sizes");
  const size_t n = size_t(M) * N;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  if (out_dtype == kBF16) reduce_store_kernel<bf16_t><<<blocks, 256, 0, st>>>(partials, static_cast<bf16_t*>(out), M, N, ldo, S);
  else if (out_dtype == kF32) reduce_store_kernel<float><<<blocks, 256, 0, st>>>(partials, static_cast<float*>(out), M, N, ldo, S);
  else KVCM_REQUIRE(false, "reduce_store: unknown output dtype %d", out_dtype);
  return launch_status("reduce_store");
}

}  // extern "C"
