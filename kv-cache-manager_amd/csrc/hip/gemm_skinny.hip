// Decode-shaped products: Y[M,N] = X[M,K] * W[N,K]^T with few rows and a weight matrix that has to be
// streamed from HBM once.  The reference leaves these to cuBLAS (src/model/llama.cpp:45-52); here the
// point is to keep enough weight bytes in flight on 256 CUs.  Two kernels: the first for up to 64 rows
// and any width that is a multiple of 16, each tile reading the rows from L2 itself; the second, further
// down, for up to 512 rows and widths that are multiples of 64, a workgroup's waves sharing the rows
// through LDS.  Shapes both take go to the second.
//
// First kernel: one workgroup (4 waves) owns 16 output columns and one slice of K ("split"); its waves divide
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
#include <mutex>

#include "common.h"
#include "kvcm_hip.h"

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
  if constexpr (MT == 1) {
    for (; u + 8 <= w_hi; u += 8) {  // long slices: eight units per trip
      Frag b[16], a[16];
      const uint16_t* p = wrow + size_t(u) * kUnit;
      const uint16_t* q = xrow[0] + size_t(u) * kUnit;
#pragma unroll
      for (int i = 0; i < 16; ++i) b[i].u = *reinterpret_cast<const uint4*>(p + (i / 2) * kUnit + (i % 2) * 8);
#pragma unroll
      for (int i = 0; i < 16; ++i) a[i].u = *reinterpret_cast<const uint4*>(q + (i / 2) * kUnit + (i % 2) * 8);
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, b[i].v, acc[0], 0, 0, 0);
    }
    for (; u + 4 <= w_hi; u += 4) {  // few rows leave registers for four units per trip: eight weight loads in flight per lane
      Frag b[8], a[8];
      const uint16_t* p = wrow + size_t(u) * kUnit;
      const uint16_t* q = xrow[0] + size_t(u) * kUnit;
#pragma unroll
      for (int i = 0; i < 8; ++i) b[i].u = *reinterpret_cast<const uint4*>(p + (i / 2) * kUnit + (i % 2) * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) a[i].u = *reinterpret_cast<const uint4*>(q + (i / 2) * kUnit + (i % 2) * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, b[i].v, acc[0], 0, 0, 0);
    }
  }
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
        const float act = silu<TO>(x);
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

// The same product with the rows shared by a workgroup's waves: the kernel every unfolded product of up
// to 512 rows takes when its width is a multiple of 64 (the one above serves the other widths).  X is
// not small beside the weights: every 16-column tile needs all of it, and re-reading it from L2 per tile
// costs as many bytes as the weights from 8 rows on.  Here a workgroup of NWV waves owns NWV column tiles (one 16-column tile per wave;
// the last workgroup may have fewer tiles than waves), up to 128 rows and a slice of K, and its waves
// share X through LDS: per trip of DEPTH x 64 k the workgroup stages X[rows][DEPTH * 64] once
// (double-buffered; the next trip's global loads are issued before the current trip's products), every
// wave streams its own 16 weight rows from HBM and multiplies them with the staged rows.  No reduction
// between waves; split-K partial sums as above.  More than 128 rows run as row blocks of 128
// (blockIdx.z), each streaming the weights again.
// SWIGLU: a wave's tile is 8 gate + 8 up rows, it stores 8 activation columns.
constexpr int kXPad = 8;    // bfloat16 of padding per staged row, so that rows spread over the banks
constexpr int kRowBlock = 128;

template <int MT, int DEPTH, class TO, bool SWIGLU, int NWV>
__global__ void __launch_bounds__(NWV * kWave)
    gemm_rows_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W, float* __restrict__ partials,
                     TO* __restrict__ out, int M, int N, int K, int ldx, int ldw, int ldo, int S,
                     const float* __restrict__ ss_in, int tiles_in, float eps) {
  constexpr int kPassRows = NWV * kWave / 4;                      // rows the workgroup's threads stage at a time (x 64 k)
  constexpr int RP = (MT * 16 + kPassRows - 1) / kPassRows;       // staging passes
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][MT * 16][DEPTH * kUnit + kXPad];
  __shared__ float rstd_s[MT * 16];   // ss_in: every row's 1 / sqrt(mean x^2 + eps), which the unsplit result is scaled by
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int r = lane % 16, kq = lane / 16;
  constexpr int kCols = SWIGLU ? 8 : 16;
  const int c0 = blockIdx.x * (NWV * kCols) + wave * kCols;   // this wave's first output column
  const bool col_on = c0 < N;                                   // the last workgroup may have fewer tiles than waves
  const int s = blockIdx.y;
  const int row_base = blockIdx.z * kRowBlock;
  const int units = K / kUnit;
  const int u_lo = int((long long)units * s / S), u_hi = int((long long)units * (s + 1) / S);
  const int trips = (u_hi - u_lo + DEPTH - 1) / DEPTH;

  const int cw = col_on ? c0 : 0;   // a wave without a tile reads the first tile's rows and drops them
  const uint16_t* wrow = W + size_t(SWIGLU ? (r < 8 ? cw + r : N + cw + r - 8) : cw + r) * ldw + kq * 16;
  // staging: thread -> (row tid / 4 + kPassRows p, 16 elements at (tid % 4) * 16 of every unit); rows
  // beyond M read the block's first row and are dropped at the store
  const int srow = threadIdx.x / 4, sseg = (threadIdx.x % 4) * 16;
  const uint16_t* xsrc[RP];
#pragma unroll
  for (int p = 0; p < RP; ++p) {
    const int m = row_base + srow + kPassRows * p;
    xsrc[p] = X + size_t(m < M ? m : row_base) * ldx + sseg;
  }

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // A trip's operands: DEPTH units of this wave's weight rows and of this thread's pieces of X.
  // Units beyond the slice repeat its last unit (no load behind a branch) and are not multiplied.
  struct Trip {
    Frag b[DEPTH][2];
    uint4 x[DEPTH][RP][2];
  };
  // Workgroups walk their slice from different starting points (and wrap around): if all of them
  // read the same k at the same time, their rows, a multiple of 4 KB apart, would queue up at the
  // same few memory channels.
  const int span = u_hi - u_lo > 0 ? u_hi - u_lo : 1;
  const int phase = (blockIdx.x * 5) % span;   // the same for all waves: they share staged X
  auto fetch = [&](int j0, Trip& tr) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int j = j0 + d < span ? j0 + d : span - 1;
      const int u = u_lo + (j + phase) % span;
      const uint16_t* p = wrow + size_t(u) * kUnit;
      tr.b[d][0].u = *reinterpret_cast<const uint4*>(p);
      tr.b[d][1].u = *reinterpret_cast<const uint4*>(p + 8);
#pragma unroll
      for (int q = 0; q < RP; ++q) {
        const uint16_t* xp = xsrc[q] + size_t(u) * kUnit;
        tr.x[d][q][0] = *reinterpret_cast<const uint4*>(xp);
        tr.x[d][q][1] = *reinterpret_cast<const uint4*>(xp + 8);
      }
    }
  };
  auto stage = [&](int buf, const Trip& tr) {
#pragma unroll
    for (int q = 0; q < RP; ++q) {
      if (srow + kPassRows * q < MT * 16) {   // uniform per wave
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
          *reinterpret_cast<uint4*>(&xs[buf][srow + kPassRows * q][d * kUnit + sseg]) = tr.x[d][q][0];
          *reinterpret_cast<uint4*>(&xs[buf][srow + kPassRows * q][d * kUnit + sseg + 8]) = tr.x[d][q][1];
        }
      }
    }
  };
  auto multiply = [&](int buf, int j0, const Trip& tr) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (j0 + d >= span) break;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        Frag a0, a1;
        a0.u = *reinterpret_cast<const uint4*>(&xs[buf][t * 16 + r][d * kUnit + kq * 16]);
        a1.u = *reinterpret_cast<const uint4*>(&xs[buf][t * 16 + r][d * kUnit + kq * 16 + 8]);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, tr.b[d][0].v, acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, tr.b[d][1].v, acc[t], 0, 0, 0);
      }
    }
  };
  // Two trips in registers: while one is multiplied, the next one's loads are on their way.  LDS
  // buffer i holds the X of the trip in register set i; a buffer is written one barrier after its
  // last read.
  // X = round(g round(x)) of a norm folded into this product (gemm_rows8.hip): the rows' scales from their
  // tiles' sums of squares, a wave per row, added in a fixed order while the first loads are on their way
  auto scales = [&]() {
    if (ss_in == nullptr) return;
    for (int m = wave; m < MT * 16; m += NWV) {
      if (row_base + m >= M) {   // a row the block does not have: its sums are dropped at the store
        if (lane == 0) rstd_s[m] = 1.f;
        continue;
      }
      const float* p = ss_in + size_t(row_base + m) * tiles_in;
      float part[4] = {0.f, 0.f, 0.f, 0.f};   // four loads on their way per lane
      int t = lane;
      for (; t + 3 * kWave < tiles_in; t += 4 * kWave) {
#pragma unroll
        for (int q = 0; q < 4; ++q) part[q] += p[t + q * kWave];
      }
      for (; t < tiles_in; t += kWave) part[0] += p[t];
      const float sum = wave_sum((part[0] + part[1]) + (part[2] + part[3]));
      if (lane == 0) rstd_s[m] = rsqrtf(sum / float(tiles_in * 8) + eps);
    }
  };
  if (u_lo < u_hi) {
    Trip ta, tb;
    fetch(0, ta);
    scales();
    for (int i = 0; i < trips; i += 2) {
      const int j0 = i * DEPTH;
      fetch(j0 + DEPTH, tb);
      stage(0, ta);
      __syncthreads();
      multiply(0, j0, ta);
      if (i + 1 >= trips) break;
      fetch(j0 + 2 * DEPTH, ta);
      stage(1, tb);
      __syncthreads();
      multiply(1, j0 + DEPTH, tb);
    }
  } else {
    scales();
  }
  if (ss_in != nullptr) {   // (the same for the whole workgroup)
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[t][i] *= rstd_s[t * 16 + kq * 4 + i];
  }
  if (!col_on) return;
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
        const int m = row_base + t * 16 + kq * 4 + i;
        if (m >= M) continue;
        const float x = round_to<TO>(acc[t][i]);
        const float act = silu<TO>(x);
        store_f(out + size_t(m) * ldo + c0 + r, round_to<TO>(act) * round_to<TO>(up[i]));
      }
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = row_base + t * 16 + kq * 4 + i;
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

constexpr int kMaxSharedRows = 512;

// Whole groups of 64 columns: the kernel whose waves share X through LDS.
static bool shares_rows(int M, int N) { return M > 0 && M <= kMaxSharedRows && N % 64 == 0; }
static int row_blocks(int M) { return (M + kRowBlock - 1) / kRowBlock; }
// The SwiGLU form (I: the activation's width) is unsplit: with too few workgroups a split product and a
// launch for SwiGLU fill the chip better.
static bool swiglu_shares_rows(int M, int I) {
  return M > 0 && M <= kMaxSharedRows && I % 32 == 0 && (I / 32) * row_blocks(M) >= 160;
}

// Waves per workgroup (each takes one column tile) so that tiles x splits x row blocks make about one
// workgroup per CU and none is left out: what this kernel streams per microsecond grows with the CUs it
// covers, not with the waves on each (measured:
// gate/up at TinyLlama sizes, 704 tiles, 32 rows: 176 workgroups of four waves 16.5 us, 235 of three
// 13.2 us; at Llama-3-8B sizes, 1,792 tiles, 64 rows: 448 of four 63 us, 256 of seven 51 us).  One wave
// more where that saves a staging pass (the workgroup's threads stage 16 rows per wave at a time: 64 rows
// are two passes for three waves, one for four).
constexpr int kRowsCUs = 256;
static int rows_waves(long long units, int mt) {
  const long long want = (units + kRowsCUs - 1) / kRowsCUs;
  int w = want < 2 ? 2 : want > 8 ? 8 : static_cast<int>(want);
  if (w < 8 && (mt + w) / (w + 1) < (mt + w - 1) / w) ++w;
  return w;
}
static int rows_tiles_m(int M) { return M > kRowBlock ? kRowBlock / 16 : (M + 15) / 16; }

// Splits of K of a plain shared-rows product: eight where there are few column tiles, or where K is long
// against the rows (the partial sums, S*M*N floats that the next kernel reads, are small against the
// weights then), else four; as long as every slice has a trip of its own and the partial sums stay below
// the weights' bytes; halved while more than eight waves a workgroup would be needed to get down to one
// workgroup per CU.  Measured at 17 to 128 rows over the projections of TinyLlama and Llama-3-8B sizes,
// alone and in whole decode steps.
static int rows_splits(int M, int N, int K) {
  const long long tiles = static_cast<long long>(N / 16) * row_blocks(M);
  const int units = K / kUnit;
  if (tiles >= 4 * kRowsCUs) return 1;
  int S = tiles <= 128 || (M > 48 && K >= 112 * M) ? 8 : 4;
  const int trip = M <= 64 ? 4 : 2;   // units per trip (the launch's choice below)
  const int cap = units / trip < K / (2 * M) ? units / trip : K / (2 * M);
  while (S > 1 && S > cap) S >>= 1;
  while (S > 1 && tiles * S > 8 * kRowsCUs) S >>= 1;
  return S;
}

// One launch of the shared-rows kernel: MT row tiles per block (8 for every block when there are
// several), two k-depths: four units per trip up to 64 rows, two beyond (LDS holds rows x depth).
template <class TO, bool SWIGLU, int NWV>
static void launch_rows_n(hipStream_t st, const uint16_t* x, const uint16_t* w, float* partials, TO* out, int M, int N,
                          int K, int ldx, int ldw, int ldo, int S, const float* ss_in, int tiles_in, float eps) {
  const int mt = rows_tiles_m(M);
  const int tiles = N / (SWIGLU ? 8 : 16);
  const dim3 grid((tiles + NWV - 1) / NWV, S, row_blocks(M));
#define KVCM_ROWS(MT, DEPTH) \
  gemm_rows_kernel<MT, DEPTH, TO, SWIGLU, NWV><<<grid, NWV * kWave, 0, st>>>(x, w, partials, out, M, N, K, ldx, ldw, ldo, S, \
                                                                             ss_in, tiles_in, eps)
  switch (mt) {
    case 1: KVCM_ROWS(1, 4); break;
    case 2: KVCM_ROWS(2, 4); break;
    case 3: KVCM_ROWS(3, 4); break;
    case 4: KVCM_ROWS(4, 4); break;
    case 5: case 6: KVCM_ROWS(6, 2); break;
    default: KVCM_ROWS(8, 2); break;
  }
#undef KVCM_ROWS
}

// N: the result's width (SWIGLU: the activation's).  A 32-bit result (the head's logits, thousands of
// tiles) keeps four waves.
template <class TO, bool SWIGLU>
static void launch_rows(hipStream_t st, const uint16_t* x, const uint16_t* w, float* partials, TO* out, int M, int N, int K,
                        int ldx, int ldw, int ldo, int S, const float* ss_in = nullptr, int tiles_in = 0, float eps = 0.f) {
  const long long units = static_cast<long long>(N / (SWIGLU ? 8 : 16)) * row_blocks(M) * S;
  const int waves = sizeof(TO) == 4 || (S == 1 && !SWIGLU) ? 4 : rows_waves(units, rows_tiles_m(M));
#define KVCM_WAVES(NWV) launch_rows_n<TO, SWIGLU, NWV>(st, x, w, partials, out, M, N, K, ldx, ldw, ldo, S, ss_in, tiles_in, eps)
  if constexpr (sizeof(TO) == 4) {
    KVCM_WAVES(4);
  } else {
    switch (waves) {
      case 2: KVCM_WAVES(2); break;
      case 3: KVCM_WAVES(3); break;
      case 4: KVCM_WAVES(4); break;
      case 5: KVCM_WAVES(5); break;
      case 6: KVCM_WAVES(6); break;
      case 7: KVCM_WAVES(7); break;
      default: KVCM_WAVES(8); break;
    }
  }
#undef KVCM_WAVES
}


extern "C" {

// How many splits of K a launch of this shape uses (0: the shape is not supported by this kernel).
int kvcm_gemm_skinny_splits(int M, int N, int K) {
  if (M <= 0 || N % 16 != 0 || K % kUnit != 0 || N <= 0 || K <= 0) return 0;
  if (shares_rows(M, N)) return rows_splits(M, N, K);
  if (M > 64) return 0;
  const int tiles = N / 16, units = K / kUnit;
  int S = (640 + tiles - 1) / tiles;           // aim at >= 640 workgroups (2.5 per CU) ...
  if (S >= 5) S = 8;                           // ... five to seven slices lose to eight in whole decode steps (measured)
  while (S > 1 && S > units / 2) --S;          // at least two units per slice
  return S;
}

// Waves per workgroup that the shared-rows kernel runs a bfloat16 product of this shape with (0: another
// kernel takes the shape).  swiglu: N is the activation's width, S is 1.
int kvcm_gemm_skinny_waves(int M, int N, int K, int S, int swiglu) {
  if (swiglu ? !swiglu_shares_rows(M, N) : !shares_rows(M, N)) return 0;
  if (K <= 0 || K % kUnit != 0 || S < 1) return 0;
  if (!swiglu && S == 1) return 4;
  return rows_waves(static_cast<long long>(N / (swiglu ? 8 : 16)) * row_blocks(M) * S, rows_tiles_m(M));
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
  KVCM_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "gemm_skinny: unknown output dtype %d", out_dtype);
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const uint16_t* w = static_cast<const uint16_t*>(W);
  const int mt = (M + 15) / 16;
  if (shares_rows(M, N)) {
    if (out_dtype == kBF16) launch_rows<bf16_t, false>(st, x, w, partials, static_cast<bf16_t*>(out), M, N, K, ldx, ldw, ldo, S);
    else launch_rows<float, false>(st, x, w, partials, static_cast<float*>(out), M, N, K, ldx, ldw, ldo, S);
    return launch_status("gemm_rows");
  }
  const dim3 grid(N / 16, S);
#define KVCM_SKINNY(MT, TO) \
  gemm_skinny_kernel<MT, TO, false><<<grid, 256, 0, st>>>(x, w, partials, static_cast<TO*>(out), M, N, K, ldx, ldw, ldo, S)
  if (out_dtype == kBF16) {
    if (mt == 1) KVCM_SKINNY(1, bf16_t); else if (mt == 2) KVCM_SKINNY(2, bf16_t); else if (mt == 3) KVCM_SKINNY(3, bf16_t); else KVCM_SKINNY(4, bf16_t);
  } else {
    if (mt == 1) KVCM_SKINNY(1, float); else if (mt == 2) KVCM_SKINNY(2, float); else if (mt == 3) KVCM_SKINNY(3, float); else KVCM_SKINNY(4, float);
  }
#undef KVCM_SKINNY
  return launch_status("gemm_skinny");
}

// May act = swiglu(X * [gate | up]^T) be computed in one launch?  I is the width of the result.
int kvcm_gemm_skinny_swiglu_supported(int M, int I, int K) {
  if (!(M > 0 && I > 0 && I % 8 == 0 && K > 0 && K % kUnit == 0)) return 0;
  if (swiglu_shares_rows(M, I)) return 1;
  // with too few workgroups a split product fills the chip better than an unsplit one; the kernel whose
  // every tile reads the rows from L2 serves a few rows, or widths that are no multiple of 32
  if (I % 32 == 0 && M > 16) return 0;
  return M <= 64 && I / 8 >= 320;
}

// W [2 I, K] (gate rows, then up rows); out [M, I].
int kvcm_gemm_skinny_swiglu(const void* X, const void* W, void* out, int out_dtype, int M, int I, int K, int ldx,
                            int ldw, int ldo, hipStream_t st) {
  KVCM_REQUIRE(kvcm_gemm_skinny_swiglu_supported(M, I, K), "gemm_skinny_swiglu: unsupported shape M=%d I=%d K=%d", M, I, K);
  KVCM_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && reinterpret_cast<uintptr_t>(X) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(W) % 16 == 0,
               "gemm_skinny_swiglu: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
  KVCM_REQUIRE(ldx >= K && ldw >= K && out != nullptr && ldo >= I, "gemm_skinny_swiglu: leading dimensions too small");
  KVCM_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "gemm_skinny_swiglu: unknown output dtype %d", out_dtype);
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const uint16_t* w = static_cast<const uint16_t*>(W);
  const int mt = (M + 15) / 16;
  if (swiglu_shares_rows(M, I)) {
    if (out_dtype == kBF16) launch_rows<bf16_t, true>(st, x, w, nullptr, static_cast<bf16_t*>(out), M, I, K, ldx, ldw, ldo, 1);
    else launch_rows<float, true>(st, x, w, nullptr, static_cast<float*>(out), M, I, K, ldx, ldw, ldo, 1);
    return launch_status("gemm_rows_swiglu");
  }
  const dim3 grid(I / 8, 1);
#define KVCM_SKINNY(MT, TO) \
  gemm_skinny_kernel<MT, TO, true><<<grid, 256, 0, st>>>(x, w, nullptr, static_cast<TO*>(out), M, I, K, ldx, ldw, ldo, 1)
  if (out_dtype == kBF16) {
    if (mt == 1) KVCM_SKINNY(1, bf16_t); else if (mt == 2) KVCM_SKINNY(2, bf16_t); else if (mt == 3) KVCM_SKINNY(3, bf16_t); else KVCM_SKINNY(4, bf16_t);
  } else {
    if (mt == 1) KVCM_SKINNY(1, float); else if (mt == 2) KVCM_SKINNY(2, float); else if (mt == 3) KVCM_SKINNY(3, float); else KVCM_SKINNY(4, float);
  }
#undef KVCM_SKINNY
  return launch_status("gemm_skinny_swiglu");
}

// The same with a folded RMS norm in front (gemm_rows8.hip): X is xg = round(g round(x)) of the norm's producer,
// ss_in its [M][tiles_in] sums of x^2 per 8-column tile, eps the norm's; the sums are scaled by
// rsqrt(mean x^2 + eps) before they are rounded.  For the widths at which this kernel's few long-lived
// workgroups stream the gate/up matrix faster than the 8-row kernel's many short ones (from 1,024 tiles on:
// Llama-3-8B sizes, one row: 50.8 against 43.9 us).
int kvcm_gemm_skinny_swiglu_normed_preferred(int M, int I, int K) {
  return K > 0 && K % kUnit == 0 && swiglu_shares_rows(M, I) && I / 8 >= 4 * kRowsCUs;
}
int kvcm_gemm_skinny_swiglu_normed(const void* X, const void* W, const float* ss_in, int tiles_in, float eps, void* out,
                                   int M, int I, int K, int ldx, int ldw, int ldo, hipStream_t st) {
  KVCM_REQUIRE(K > 0 && K % kUnit == 0 && swiglu_shares_rows(M, I), "gemm_skinny_swiglu_normed: unsupported shape M=%d I=%d K=%d", M, I, K);
  KVCM_REQUIRE(ss_in != nullptr && tiles_in > 0 && tiles_in * 8 == K, "gemm_skinny_swiglu_normed: %d tiles of sums for a width of %d", tiles_in, K);
  KVCM_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && reinterpret_cast<uintptr_t>(X) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0,
               "gemm_skinny_swiglu_normed: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
  KVCM_REQUIRE(ldx >= K && ldw >= K && out != nullptr && ldo >= I, "gemm_skinny_swiglu_normed: leading dimensions too small");
  launch_rows<bf16_t, true>(st, static_cast<const uint16_t*>(X), static_cast<const uint16_t*>(W), nullptr, static_cast<bf16_t*>(out),
                            M, I, K, ldx, ldw, ldo, 1, ss_in, tiles_in, eps);
  return launch_status("gemm_rows_swiglu_normed");
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

// ---- the product for callers that cannot allocate -------------------------------------------
// Partial sums of a split product, for kvcm_gemm_skinny_noalloc: part of the library's device
// image, one copy per GPU at that GPU's own address.  Host code never passes the array's name to a
// kernel (on the host it is a stand-in, not a device address): it passes the address that
// hipGetSymbolAddress gave for the current device.
constexpr long long kNoAllocFloats = 2ll << 20;
static __device__ __align__(256) float scratch[kNoAllocFloats];

constexpr int kMaxDevices = 64;
static float* g_noalloc_ptr[kMaxDevices];
static std::mutex g_noalloc_lock;

// The current device's copy of the array; looked up once per device, with that device current.
static int noalloc_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("gemm_skinny_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    return -2;
  }
  KVCM_REQUIRE(dev >= 0 && dev < kMaxDevices, "gemm_skinny_noalloc: device %d beyond the %d this library keeps track of", dev, kMaxDevices);
  std::lock_guard<std::mutex> hold(g_noalloc_lock);
  if (g_noalloc_ptr[dev] == nullptr) {
    float* p = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("gemm_skinny_noalloc: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
      return -2;
    }
    g_noalloc_ptr[dev] = p;
  }
  *out = g_noalloc_ptr[dev];
  return 0;
}

long long kvcm_gemm_skinny_noalloc_capacity() { return kNoAllocFloats; }

int kvcm_gemm_skinny_noalloc(const void* X, const void* W, void* out, int out_dtype, int M, int N, int K, int ldx,
                             int ldw, int ldo, hipStream_t st) {
  const int S = kvcm_gemm_skinny_splits(M, N, K);
  KVCM_REQUIRE(S > 0, "gemm_skinny_noalloc: unsupported shape M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(out != nullptr && ldo >= N, "gemm_skinny_noalloc: missing output buffer or leading dimension below N");
  if (S == 1) return kvcm_gemm_skinny(X, W, nullptr, out, out_dtype, M, N, K, ldx, ldw, ldo, 1, st);
  const long long need = (long long)S * M * N;
  KVCM_REQUIRE(need <= kNoAllocFloats,
               "gemm_skinny_noalloc: M=%d N=%d K=%d needs %lld floats of partial sums (%d slices), the built-in array holds %lld",
               M, N, K, need, S, kNoAllocFloats);
  float* partials = nullptr;
  if (int rc = noalloc_scratch(&partials)) return rc;
  if (int rc = kvcm_gemm_skinny(X, W, partials, out, out_dtype, M, N, K, ldx, ldw, ldo, S, st)) return rc;
  return kvcm_reduce_store(partials, out, out_dtype, M, N, ldo, S, st);
}

}  // extern "C"
