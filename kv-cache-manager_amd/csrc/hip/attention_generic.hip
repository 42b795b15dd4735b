// Attention of query rows over the paged cache, one wave per (row, query head).
//
// The same arithmetic as the reference kernel (src/cuda/paged_attention.cu:50-183): q is scaled
// in 32-bit before the dot product, a row with context length c sees keys 0 .. c-1 of its own
// sequence through the block table (causality is nothing but c = position + 1), query head h
// reads KV head h / (heads / kv_heads), softmax and the P*V sums are 32-bit and the result is
// divided by the sum once.  Differences: keys are taken 64 at a time with a running maximum
// (no score buffer that grows with the context), any head_dim that is a multiple of 8 up to 256
// and any group size work, storage is float or bfloat16, and an optional window hides keys with
// position <= row position - window.
//
// A row's result is a fixed sequence of operations on its own keys: chunks start at absolute
// multiples of 64, lanes map to keys and dims the same way every time.  It therefore does not
// depend on which other rows are in the launch, nor on which physical pages hold the keys.
#include <cfloat>

#include "common.h"

namespace kvcm {

constexpr int kAttnWaves = 4;
constexpr int kMaxHeadDim = 256;

template <class T> struct Vec;
template <> struct Vec<float> { static constexpr int N = 4; };
template <> struct Vec<bf16_t> { static constexpr int N = 8; };

template <class T>
__device__ __forceinline__ float dot_piece(const float* q, const T* k);
template <>
__device__ __forceinline__ float dot_piece<float>(const float* q, const float* k) {
  const float4 v = *reinterpret_cast<const float4*>(k);
  float s = q[0] * v.x;
  s = fmaf(q[1], v.y, s);
  s = fmaf(q[2], v.z, s);
  return fmaf(q[3], v.w, s);
}
template <>
__device__ __forceinline__ float dot_piece<bf16_t>(const float* q, const bf16_t* k) {
  const uint4 v = *reinterpret_cast<const uint4*>(k);
  float s = q[0] * bf16_bits_to_float(v.x & 0xffffu);
  s = fmaf(q[1], bf16_bits_to_float(v.x >> 16), s);
  s = fmaf(q[2], bf16_bits_to_float(v.y & 0xffffu), s);
  s = fmaf(q[3], bf16_bits_to_float(v.y >> 16), s);
  s = fmaf(q[4], bf16_bits_to_float(v.z & 0xffffu), s);
  s = fmaf(q[5], bf16_bits_to_float(v.z >> 16), s);
  s = fmaf(q[6], bf16_bits_to_float(v.w & 0xffffu), s);
  return fmaf(q[7], bf16_bits_to_float(v.w >> 16), s);
}

template <class T>
__global__ void __launch_bounds__(kAttnWaves* kWave)
    attention_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                             const T* __restrict__ kcache, const T* __restrict__ vcache,
                             const int* __restrict__ tables, int table_stride, const int* __restrict__ row_seq,
                             const int* __restrict__ ctx_lens, long long items, int nh, int nkv, int hd, int B,
                             float scale, int window) {
  extern __shared__ float q_lds[];  // [waves][hd], q * scale
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const long long item = static_cast<long long>(blockIdx.x) * kAttnWaves + wave;
  const bool active = item < items;
  const int row = active ? static_cast<int>(item / nh) : 0;
  const int head = active ? static_cast<int>(item % nh) : 0;
  float* qs = q_lds + wave * hd;
  if (active)
    for (int d = lane; d < hd; d += kWave) qs[d] = load_f(q + size_t(row) * q_stride + size_t(head) * hd + d) * scale;
  __syncthreads();
  if (!active) return;

  const int kvh = head / (nh / nkv);
  const int ctx = ctx_lens[row];
  T* orow = out + size_t(row) * out_stride + size_t(head) * hd;
  if (ctx <= 0) {
    for (int d = lane; d < hd; d += kWave) store_f(orow + d, 0.f);
    return;
  }
  const int first = (window > 0 && ctx > window) ? ctx - window : 0;
  const int* table = tables + size_t(row_seq[row]) * table_stride;
  const size_t head_stride = size_t(B) * hd, page_stride = head_stride * nkv;

  float m = -INFINITY, l = 0.f;
  float o[kMaxHeadDim / kWave] = {0.f, 0.f, 0.f, 0.f};
  for (int c0 = (first / kWave) * kWave; c0 < ctx; c0 += kWave) {
    const int t = c0 + lane;
    const bool valid = t >= first && t < ctx;
    float s = -INFINITY;
    if (valid) {
      const T* kp = kcache + size_t(table[t / B]) * page_stride + kvh * head_stride + size_t(t % B) * hd;
      s = 0.f;
      for (int d = 0; d < hd; d += Vec<T>::N) s += dot_piece<T>(qs + d, kp + d);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < kMaxHeadDim / kWave; ++i) o[i] *= alpha;
    const int j_lo = first > c0 ? first - c0 : 0;
    const int j_hi = ctx - c0 < kWave ? ctx - c0 : kWave;
    for (int j = j_lo; j < j_hi; ++j) {
      const float pj = __shfl(p, j, kWave);
      const int tj = c0 + j;
      const T* vp = vcache + size_t(table[tj / B]) * page_stride + kvh * head_stride + tj % B;  // [dim][slot]
#pragma unroll
      for (int i = 0; i < kMaxHeadDim / kWave; ++i) {
        const int d = lane + i * kWave;
        if (d < hd) o[i] = fmaf(pj, load_f(vp + size_t(d) * B), o[i]);
      }
    }
    m = m_new;
  }
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / kWave; ++i) {
    const int d = lane + i * kWave;
    if (d < hd) store_f(orow + d, o[i] / l);
  }
}

}  // namespace kvcm

using namespace kvcm;

// out = {vector registers per lane, bytes of LDS per workgroup, workgroups that fit on one CU,
// threads per workgroup} of the bfloat16 kernel at this head size.
extern "C" int kvcm_attention_generic_info(int hd, int* out) {
  hipFuncAttributes a;
  const size_t lds = sizeof(float) * kAttnWaves * hd;
  int per_cu = 0;
  KVCM_REQUIRE(hipFuncGetAttributes(&a, reinterpret_cast<const void*>(&attention_generic_kernel<bf16_t>)) == hipSuccess &&
                   hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attention_generic_kernel<bf16_t>,
                                                                kAttnWaves * kWave, lds) == hipSuccess,
               "attention_generic_info: the runtime gave no attributes");
  out[0] = a.numRegs; out[1] = static_cast<int>(a.sharedSizeBytes + lds); out[2] = per_cu; out[3] = kAttnWaves * kWave;
  return 0;
}

extern "C" int kvcm_attention_generic(const void* q, int dtype, int q_stride, void* out, int out_stride,
                                      const void* kcache, const void* vcache, const int* tables, int table_stride,
                                      const int* row_seq, const int* ctx_lens, int T, int nh, int nkv, int hd,
                                      int B, float scale, int window, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && B > 0, "attention: bad sizes T=%d heads=%d kv_heads=%d B=%d", T, nh, nkv, B);
  KVCM_REQUIRE(nh % nkv == 0, "attention: %d query heads are not a multiple of %d kv heads", nh, nkv);
  KVCM_REQUIRE(hd % 8 == 0 && hd > 0 && hd <= kMaxHeadDim,
               "attention: head_dim %d is not supported (multiples of 8 up to %d are)", hd, kMaxHeadDim);
  KVCM_REQUIRE(q_stride >= nh * hd && out_stride >= nh * hd, "attention: row strides too small");
  KVCM_REQUIRE(window >= 0, "attention: negative window");
  const long long items = static_cast<long long>(T) * nh;
  const long long blocks = (items + kAttnWaves - 1) / kAttnWaves;
  KVCM_REQUIRE(blocks < (1ll << 31), "attention: too many rows");
  const size_t lds = sizeof(float) * kAttnWaves * hd;
  if (dtype == kF32)
    attention_generic_kernel<float><<<dim3(static_cast<unsigned>(blocks)), kAttnWaves * kWave, lds, s>>>(
        static_cast<const float*>(q), q_stride, static_cast<float*>(out), out_stride,
        static_cast<const float*>(kcache), static_cast<const float*>(vcache), tables, table_stride, row_seq,
        ctx_lens, items, nh, nkv, hd, B, scale, window);
  else if (dtype == kBF16)
    attention_generic_kernel<bf16_t><<<dim3(static_cast<unsigned>(blocks)), kAttnWaves * kWave, lds, s>>>(
        static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), out_stride,
        static_cast<const bf16_t*>(kcache), static_cast<const bf16_t*>(vcache), tables, table_stride, row_seq,
        ctx_lens, items, nh, nkv, hd, B, scale, window);
  else KVCM_REQUIRE(false, "attention: unknown dtype %d", dtype);
  return launch_status("attention_generic");
}
