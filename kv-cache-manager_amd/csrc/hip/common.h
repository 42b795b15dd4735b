// Shared device helpers for the gfx950 kernels: storage types, conversions, wave64 reductions,
// and the error channel of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kvcm {

constexpr int kWave = 64;

// Storage types.  bf16 is kept as raw bits so that loads can be vectorised freely.
struct bf16_t { uint16_t bits; };

enum DType : int { kF32 = 0, kBF16 = 1 };

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }
// Round to nearest, ties to even; a NaN stays a quiet NaN.  gfx950 converts in one instruction
// (v_cvt_pk_bf16_f32); written out in integer operations it costs six and a branch, which epilogues
// that round a dozen values per lane pay in microseconds.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

template <class T> __device__ __forceinline__ float load_f(const T* p);
template <> __device__ __forceinline__ float load_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_f<bf16_t>(const bf16_t* p) { return bf16_bits_to_float(p->bits); }

template <class T> __device__ __forceinline__ void store_f(T* p, float v);
template <> __device__ __forceinline__ void store_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_f<bf16_t>(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// Value after one trip through the storage type (identity for float).
template <class T> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<bf16_t>(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }

// silu(x) = x / (1 + exp(-x)) for a result stored as T.  A bfloat16 result keeps 8 bits of it: the
// hardware's exp2 and reciprocal (about 1 ulp of float each) take a tenth of the instructions of the
// exact functions, which in a product's epilogue is microseconds (a 64-lane wave spends 4 cycles
// per instruction).  A float result takes the exact functions.  One definition for every kernel
// that applies it, so that all of them give the same bits.
template <class T> __device__ __forceinline__ float silu(float x);
template <> __device__ __forceinline__ float silu<float>(float x) { return x / (1.0f + expf(-x)); }
template <> __device__ __forceinline__ float silu<bf16_t>(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * x));
}

// (a, b) rotated by the angle whose cosine and sine are given.  One explicit sequence of
// operations, shared by every kernel that rotates, so that all of them give the same bits.
__device__ __forceinline__ void rotate_pair(float& a, float& b, float cs, float sn) {
  const float ra = __fmaf_rn(a, cs, -__fmul_rn(b, sn));
  const float rb = __fmaf_rn(b, cs, __fmul_rn(a, sn));
  a = ra;
  b = rb;
}

// A 16-byte piece of 8 bfloat16 with only its first n (0..8) kept, the others zero.  Value pieces that
// reach past a context's end hold whatever the page's previous owner left there; their probabilities
// are zero, but zero times a stale Inf or NaN would not be: such pieces are cut before they are multiplied.
__device__ __forceinline__ uint4 keep_first_bf16(uint4 v, int n) {
  auto word = [n](int j) -> uint32_t { return n >= 2 * j + 2 ? 0xFFFFFFFFu : (n == 2 * j + 1 ? 0x0000FFFFu : 0u); };
  return uint4{v.x & word(0), v.y & word(1), v.z & word(2), v.w & word(3)};
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of THREADS threads (a multiple of 64); every thread gets the result.  The
// order of additions depends on THREADS only.
template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* scratch /* THREADS/64 + 1 floats */) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < THREADS / kWave; ++w) s += scratch[w];
    scratch[THREADS / kWave] = s;
  }
  __syncthreads();
  const float r = scratch[THREADS / kWave];
  __syncthreads();
  return r;
}

// ---- host side ------------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int launch_status(const char* what);

}  // namespace kvcm

#define KVCM_REQUIRE(cond, ...)          \
  do {                                   \
    if (!(cond)) {                       \
      kvcm::set_error(__VA_ARGS__);      \
      return -1;                         \
    }                                    \
  } while (0)
