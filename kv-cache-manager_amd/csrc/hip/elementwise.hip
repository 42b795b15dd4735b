// Row-wise kernels of the decoder: embedding gather, RMS norm (optionally fused with the residual
// add and a row gather), rotary positions fused with the cache write, SwiGLU, residual add.
// Each follows the arithmetic of the reference's kernel of the same purpose
// (src/cuda/kernels.cu:27-88, src/cuda/kv_cache.cu:19-38); sums, angles and the residual stream
// are 32-bit in both storage modes.
#include <cstdarg>
#include <cstdio>
#include <string>

#include "common.h"

namespace kvcm {

static thread_local std::string g_hip_error;

void set_error(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_hip_error = buf;
}

int launch_status(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  set_error("%s: %s", what, hipGetErrorString(e));
  return -2;
}

// ------------------------------------------------------------------------------- embedding
template <class TW>
__global__ void embed_kernel(const int* __restrict__ ids, const TW* __restrict__ table, float* __restrict__ x,
                             int H, int V) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* dst = x + size_t(t) * H;
  if (id < 0 || id >= V) {  // the host refuses such ids; never read outside the table
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = 0.f;
    return;
  }
  const TW* src = table + size_t(id) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = load_f(src + i);
}

// -------------------------------------------------------------------------------- RMS norm
// v = x[src] (+ add[src]); optionally x[src] = v; out[r] = w * round(v * inv)  with
// inv = 1/sqrt(mean(v^2) + eps).  src = rows ? rows[r] : r.  The added term is a tensor, or the
// split-K partial sums of the product that made it ([S][T][H] floats, added in split order and
// rounded to the storage type as the stored product would have been).
constexpr int kNormThreads = 256;
template <class TA, class TW, class TO>
__global__ void __launch_bounds__(kNormThreads)
    rmsnorm_kernel(float* __restrict__ x, const TA* __restrict__ add, const float* __restrict__ partials, int S,
                   int T, const int* __restrict__ rows, const TW* __restrict__ w, TO* __restrict__ out, int H,
                   float eps, int write_back) {
  __shared__ float scratch[kNormThreads / kWave + 1];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + size_t(src) * H;
  const TA* ar = add ? add + size_t(src) * H : nullptr;
  const float* pr = partials ? partials + size_t(src) * H : nullptr;
  const size_t pstride = size_t(T) * H;
  const bool adds = ar || pr;
  auto added = [&](int i) {
    if (ar) return load_f(ar + i);
    float a = 0.f;
    for (int s = 0; s < S; ++s) a += pr[s * pstride + i];
    return round_to<TO>(a);
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += kNormThreads) {
    float v = xr[i];
    if (adds) {
      v += added(i);
      if (write_back) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum<kNormThreads>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / float(H) + eps);
  TO* o = out + size_t(r) * H;
  for (int i = threadIdx.x; i < H; i += kNormThreads) {
    float v = xr[i];
    if (adds && !write_back) v += added(i);
    store_f(o + i, load_f(w + i) * round_to<TO>(v * inv));
  }
}

// The same computation for rows whose length is a multiple of 4 and at most 1024 * VPT: every
// thread keeps its VPT groups of four values in registers and asks for all of its inputs at once,
// so the row costs one round trip to memory instead of one per element.  Its sum of squares adds
// in another order than the kernel above, so the two may differ in the last bit; which of them
// runs depends on the row length and on alignment only, never on the batch.
template <class T> __device__ __forceinline__ void load4(const T* p, float* f);
template <> __device__ __forceinline__ void load4<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
template <> __device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float* f) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  f[0] = bf16_bits_to_float(v.x & 0xffffu); f[1] = bf16_bits_to_float(v.x >> 16);
  f[2] = bf16_bits_to_float(v.y & 0xffffu); f[3] = bf16_bits_to_float(v.y >> 16);
}
template <class T> __device__ __forceinline__ void store4(T* p, const float* f);
template <> __device__ __forceinline__ void store4<float>(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = float4{f[0], f[1], f[2], f[3]};
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, const float* f) {
  uint2 v;
  v.x = float_to_bf16_bits(f[0]) | (uint32_t(float_to_bf16_bits(f[1])) << 16);
  v.y = float_to_bf16_bits(f[2]) | (uint32_t(float_to_bf16_bits(f[3])) << 16);
  *reinterpret_cast<uint2*>(p) = v;
}

template <class TA, class TW, class TO, int VPT>
__global__ void __launch_bounds__(kNormThreads)
    rmsnorm_rows4_kernel(float* __restrict__ x, const TA* __restrict__ add, const float* __restrict__ partials, int S,
                         int T, const int* __restrict__ rows, const TW* __restrict__ w, TO* __restrict__ out, int H,
                         float eps, int write_back) {
  __shared__ float scratch[kNormThreads / kWave + 1];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + size_t(src) * H;
  const size_t pstride = size_t(T) * H;
  float v[VPT][4], wv[VPT][4];
  bool on[VPT];
  int at[VPT];
  // thread t owns elements 4 * (t + 256 k) .. + 3.  Every load is unconditional (a thread beyond
  // the row reads the row's last four elements and its values are zeroed afterwards): a branch
  // around a load makes the compiler wait for that load on the spot, one memory latency each.
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = 4 * (threadIdx.x + k * kNormThreads);
    on[k] = i < H;
    at[k] = on[k] ? i : H - 4;
    load4<float>(xr + at[k], v[k]);
    load4<TW>(w + at[k], wv[k]);
  }
  if (add) {
    const TA* ar = add + size_t(src) * H;
    float a[VPT][4];
#pragma unroll
    for (int k = 0; k < VPT; ++k) load4<TA>(ar + at[k], a[k]);
#pragma unroll
    for (int k = 0; k < VPT; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) v[k][e] += a[k][e];
  } else if (partials) {
    const float* pr = partials + size_t(src) * H;
    float a[VPT][4];
#pragma unroll
    for (int k = 0; k < VPT; ++k) a[k][0] = a[k][1] = a[k][2] = a[k][3] = 0.f;
    // eight splits per trip (four for wide rows, whose pieces would not fit the registers), all their loads
    // requested before the first sum; a split beyond S reads split S - 1 again and adds nothing, so the
    // order of the sums is that of the splits
    constexpr int TRIP = VPT <= 2 ? 8 : 4;
    for (int s0 = 0; s0 < S; s0 += TRIP) {
      float p[TRIP][VPT][4];
#pragma unroll
      for (int j = 0; j < TRIP; ++j) {
        const int sj = s0 + j < S ? s0 + j : S - 1;
#pragma unroll
        for (int k = 0; k < VPT; ++k) load4<float>(pr + sj * pstride + at[k], p[j][k]);
      }
#pragma unroll
      for (int j = 0; j < TRIP; ++j) {
        const bool keep = s0 + j < S;
#pragma unroll
        for (int k = 0; k < VPT; ++k)
#pragma unroll
          for (int e = 0; e < 4; ++e) a[k][e] += keep ? p[j][k][e] : 0.f;
      }
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) v[k][e] += round_to<TO>(a[k][e]);
  }
#pragma unroll
  for (int k = 0; k < VPT; ++k)
    if (!on[k]) v[k][0] = v[k][1] = v[k][2] = v[k][3] = 0.f;
  if ((add || partials) && write_back) {
#pragma unroll
    for (int k = 0; k < VPT; ++k)
      if (on[k]) store4<float>(xr + 4 * (threadIdx.x + k * kNormThreads), v[k]);
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k)
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += v[k][e] * v[k][e];
  ss = block_sum<kNormThreads>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / float(H) + eps);
  TO* o = out + size_t(r) * H;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    if (!on[k]) continue;
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = wv[k][e] * round_to<TO>(v[k][e] * inv);
    store4<TO>(o + 4 * (threadIdx.x + k * kNormThreads), y);
  }
}

// --------------------------------------------------------- rotary positions + cache write
// One block per token row of the fused [q | k | v] buffer.  q and k heads are rotated in place
// (pairs (j, j + hd/2), angle = float(pos) * inv_freq[j] in 32-bit); rotated k and plain v are
// copied to the paged cache at slot = page * B + offset; keys [page][kv_head][B][hd], values
// transposed inside the page [page][kv_head][hd][B].
// inv_freq == null: no rotation.  slots == null or slot < 0: no cache write.
// partials != null: the fused rows do not exist yet; they are the split-K sums [S][rows][width]
// of the projection that makes them (added in split order, rounded to the storage type), and only
// what a later kernel reads is stored: q to the fused rows, k and v to the cache.
template <class T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, const int* __restrict__ slots,
                                  T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv, int hd, int B,
                                  const float* __restrict__ partials, int S, const float2* __restrict__ cos_sin,
                                  int first_head) {
  // one workgroup per (row, head): q heads, then k heads, then v heads (from first_head on: the
  // q heads are left alone when the attention kernel rotates them as it reads them)
  const int t = blockIdx.x, h = blockIdx.y + first_head;
  T* row = qkv + size_t(t) * row_stride;
  const int half = hd / 2;
  const int width = (nh + 2 * nkv) * hd;
  const float* prow = partials ? partials + size_t(t) * width : nullptr;
  const size_t pstride = size_t(gridDim.x) * width;
  auto value = [&](int c) {
    if (!prow) return load_f(row + c);
    float a = 0.f;
    for (int s0 = 0; s0 < S; s0 += 4) {   // four loads requested together; a split beyond S adds nothing
      float p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) p[j] = prow[(s0 + j < S ? s0 + j : S - 1) * pstride + c];
#pragma unroll
      for (int j = 0; j < 4; ++j) a += s0 + j < S ? p[j] : 0.f;
    }
    return round_to<T>(a);
  };
  const int slot = slots ? slots[t] : -1;
  const size_t page = slot >= 0 ? slot / B : 0;
  const int off = slot >= 0 ? slot % B : 0;
  const bool is_q = h < nh, is_k = !is_q && h < nh + nkv;
  if (is_q || is_k) {
    T* cache_row = (is_k && slot >= 0) ? kcache + ((page * nkv + (h - nh)) * B + off) * hd : nullptr;
    if (inv_freq || cos_sin) {
      const float pos = cos_sin ? 0.f : float(positions[t]);
      for (int j = threadIdx.x; j < half; j += blockDim.x) {
        float sn, cs;
        if (cos_sin) {   // computed once per step by rope_table_kernel, the same values
          const float2 t2 = cos_sin[size_t(t) * half + j];
          cs = t2.x;
          sn = t2.y;
        } else {
          sincosf(pos * inv_freq[j], &sn, &cs);
        }
        const int c = h * hd + j;
        float ra = value(c), rb = value(c + half);
        rotate_pair(ra, rb, cs, sn);
        if (!prow || is_q) {
          store_f(row + c, ra);
          store_f(row + c + half, rb);
        }
        if (cache_row) {
          store_f(cache_row + j, ra);
          store_f(cache_row + j + half, rb);
        }
      }
    } else {
      for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        const float a = value(h * hd + d);
        if (prow && is_q) store_f(row + h * hd + d, a);
        if (cache_row) store_f(cache_row + d, a);
      }
    }
    return;
  }
  if (slot < 0) return;
  // values are stored transposed inside the page: [page][kv_head][dim][slot]
  T* cache_head = vcache + (page * nkv + (h - nh - nkv)) * size_t(hd) * B + off;
  for (int d = threadIdx.x; d < hd; d += blockDim.x) store_f(cache_head + size_t(d) * B, value(h * hd + d));
}

// Values of whole fused rows to their transposed pages ([page][kv_head][dim][slot]): a thread takes
// one dim of one kv head for a group of 8 rows.  Lanes are neighbours in dim, so a wave reads
// contiguous pieces of each row; where the group's slots are 8 consecutive ones that start at a
// multiple of 8 (the rows of a prompt portion) the thread stores them as one vector, which makes the
// page rows whole again, otherwise slot by slot.  Groups are counted from the first row whose slot
// is a multiple of 8, so that a portion which starts anywhere in its sequence is still stored in
// vectors (rows before it form a short group of their own).
constexpr int kVGroup = 8;
template <class T>
__device__ __forceinline__ void v_page_item(const T* __restrict__ qkv, int row_stride, const int* __restrict__ slots,
                                            T* __restrict__ vcache, int nh, int nkv, int hd, int B, int rows, long long item) {
  const int d = int(item % hd), kvh = int((item / hd) % nkv), g = int(item / (static_cast<long long>(hd) * nkv));
  const int s_first = slots[0];
  const int shift = s_first >= 0 ? (kVGroup - s_first % kVGroup) % kVGroup : 0;
  const int lo = shift - kVGroup + g * kVGroup;
  const T* src = qkv + size_t(nh + nkv + kvh) * hd + d;
  bool whole = lo >= 0 && lo + kVGroup <= rows && B % kVGroup == 0;
  int s0 = -1;
  if (whole) {
    s0 = slots[lo];
    whole = s0 >= 0 && s0 % kVGroup == 0;
#pragma unroll
    for (int k = 1; k < kVGroup; ++k) whole = whole && slots[lo + k] == s0 + k;
  }
  if (whole) {
    float v[kVGroup];
#pragma unroll
    for (int k = 0; k < kVGroup; ++k) v[k] = load_f(src + size_t(lo + k) * row_stride);
    T* dst = vcache + ((size_t(s0 / B) * nkv + kvh) * hd + d) * B + s0 % B;
    store4<T>(dst, v);
    store4<T>(dst + 4, v + 4);
    return;
  }
  for (int t = lo < 0 ? 0 : lo; t < lo + kVGroup && t < rows; ++t) {
    const int slot = slots[t];
    if (slot >= 0) store_f(vcache + ((size_t(slot / B) * nkv + kvh) * hd + d) * B + slot % B, load_f(src + size_t(t) * row_stride));
  }
}

// The same for whole fused rows (no partial sums) whose head size is a multiple of 16: a thread
// takes 8 pairs of a q or k head with vector loads and stores (items below qk_items), or one dim of
// a v head for 8 rows (the items after them), so a prompt's rows move at memory speed.  Same
// formulas, same values as the kernel above.
template <class T>
__global__ void __launch_bounds__(256)
    rope_cache_vec_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                          const float* __restrict__ inv_freq, const int* __restrict__ slots, T* __restrict__ kcache,
                          T* __restrict__ vcache, int nh, int nkv, int hd, int B, const float2* __restrict__ cos_sin,
                          int rows, long long qk_items, long long items, int first_head) {
  const long long item = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x;
  if (item >= items) return;
  if (item >= qk_items) {
    v_page_item<T>(qkv, row_stride, slots, vcache, nh, nkv, hd, B, rows, item - qk_items);
    return;
  }
  const int cph = hd / 16, heads = nh + nkv - first_head, half = hd / 2;   // first_head = nh: the k heads only
  const int c = int(item % cph), h = first_head + int((item / cph) % heads), t = int(item / (static_cast<long long>(cph) * heads));
  T* row = qkv + size_t(t) * row_stride + size_t(h) * hd;
  const int slot = slots ? slots[t] : -1;
  const size_t page = slot >= 0 ? slot / B : 0;
  const int off = slot >= 0 ? slot % B : 0;
  const bool is_k = h >= nh;
  T* cache_row = (is_k && slot >= 0) ? kcache + ((page * nkv + (h - nh)) * B + off) * hd : nullptr;
  const int j0 = c * 8;
  float a[8], b[8];
  load4<T>(row + j0, a); load4<T>(row + j0 + 4, a + 4);
  load4<T>(row + half + j0, b); load4<T>(row + half + j0 + 4, b + 4);
  if (inv_freq || cos_sin) {
    float cs[8], sn[8];
    if (cos_sin) {
      const float4* tab = reinterpret_cast<const float4*>(cos_sin + size_t(t) * half + j0);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float4 v = tab[k];
        cs[2 * k] = v.x; sn[2 * k] = v.y; cs[2 * k + 1] = v.z; sn[2 * k + 1] = v.w;
      }
    } else {
      const float pos = float(positions[t]);
#pragma unroll
      for (int e = 0; e < 8; ++e) sincosf(pos * inv_freq[j0 + e], &sn[e], &cs[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) rotate_pair(a[e], b[e], cs[e], sn[e]);
    store4<T>(row + j0, a); store4<T>(row + j0 + 4, a + 4);
    store4<T>(row + half + j0, b); store4<T>(row + half + j0 + 4, b + 4);
  }
  if (cache_row) {
    store4<T>(cache_row + j0, a); store4<T>(cache_row + j0 + 4, a + 4);
    store4<T>(cache_row + half + j0, b); store4<T>(cache_row + half + j0 + 4, b + 4);
  }
}

// cos and sin of float(pos) * inv_freq[j] for every row of a step: the angles depend on the row
// only, so a step computes them once and every layer's rotation reads them.
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float2* __restrict__ cos_sin, int half) {
  const int t = blockIdx.x;
  const float pos = float(positions[t]);
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float sn, cs;
    sincosf(pos * inv_freq[j], &sn, &cs);
    cos_sin[size_t(t) * half + j] = float2{cs, sn};
  }
}

// ---------------------------------------------------------------------------------- SwiGLU
// act = round( round(silu(g)) * u ), row = [gate (I) | up (I)], silu(g) = g / (1 + exp(-g)).
template <class T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const T* g = gu + size_t(t) * 2 * I;
  const T* u = g + I;
  T* o = out + size_t(t) * I;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < I) {
    const float x = load_f(g + i);
    store_f(o + i, round_to<T>(silu<T>(x)) * load_f(u + i));
  }
}

template <class T>
__global__ void __launch_bounds__(256) swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int i = 8 * (blockIdx.x * blockDim.x + threadIdx.x);
  if (i >= I) return;
  const T* g = gu + size_t(t) * 2 * I + i;
  float x[8], u[8], y[8];
  load4<T>(g, x); load4<T>(g + 4, x + 4);
  load4<T>(g + I, u); load4<T>(g + I + 4, u + 4);
#pragma unroll
  for (int e = 0; e < 8; ++e) y[e] = round_to<T>(silu<T>(x[e])) * u[e];
  T* o = out + size_t(t) * I + i;
  store4<T>(o, y); store4<T>(o + 4, y + 4);
}

// ------------------------------------------------------------------------------- residual
template <class T>
__global__ void add_residual_kernel(float* __restrict__ x, const T* __restrict__ y, size_t n) {
  for (size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x; i < n; i += size_t(gridDim.x) * blockDim.x)
    x[i] += load_f(y + i);
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

const char* kvcm_hip_last_error() { return g_hip_error.c_str(); }

int kvcm_embed(const int* ids, const void* table, int table_dtype, float* x, int T, int H, int V, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
  if (table_dtype == kF32) embed_kernel<float><<<T, 256, 0, s>>>(ids, static_cast<const float*>(table), x, H, V);
  else if (table_dtype == kBF16) embed_kernel<bf16_t><<<T, 256, 0, s>>>(ids, static_cast<const bf16_t*>(table), x, H, V);
  else KVCM_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
  return launch_status("embed");
}

// add: a tensor of x's shape, or null.  partials: split-K sums [S][T][H] (T = rows of x), or null.
int kvcm_rmsnorm(float* x, const void* add, int add_dtype, const float* partials, int S, int T, const int* rows,
                 const void* w, int w_dtype, void* out, int out_dtype, int R, int H, float eps, int write_back,
                 hipStream_t s) {
  if (R == 0) return 0;
  KVCM_REQUIRE(R > 0 && H > 0, "rmsnorm: bad sizes R=%d H=%d", R, H);
  KVCM_REQUIRE(!(rows && (add || partials) && write_back), "rmsnorm: a gathered add cannot write back");
  KVCM_REQUIRE(!(add && partials), "rmsnorm: the added term is a tensor or partial sums, not both");
  KVCM_REQUIRE(!partials || (S >= 1 && T >= 1), "rmsnorm: partial sums need their split count and row count");
  const bool rows4 = H % 4 == 0 && H <= 8 * 1024 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(add) % 16 == 0 && reinterpret_cast<uintptr_t>(partials) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int vpt = (H + 1023) / 1024;
#define KVCM_NORM4(TA, TW, TO, VPT)                                                                                  \
  rmsnorm_rows4_kernel<TA, TW, TO, VPT><<<R, kNormThreads, 0, s>>>(x, static_cast<const TA*>(add), partials, S, T, rows, \
                                                                   static_cast<const TW*>(w), static_cast<TO*>(out), H, eps, write_back)
#define KVCM_NORM(TA, TW, TO)                                                                                 \
  do {                                                                                                        \
    if (!rows4)                                                                                               \
      rmsnorm_kernel<TA, TW, TO><<<R, kNormThreads, 0, s>>>(x, static_cast<const TA*>(add), partials, S, T, rows, \
                                                            static_cast<const TW*>(w), static_cast<TO*>(out), H, eps, write_back); \
    else if (vpt <= 1) KVCM_NORM4(TA, TW, TO, 1);                                                             \
    else if (vpt <= 2) KVCM_NORM4(TA, TW, TO, 2);                                                             \
    else if (vpt <= 4) KVCM_NORM4(TA, TW, TO, 4);                                                             \
    else KVCM_NORM4(TA, TW, TO, 8);                                                                           \
  } while (0)
  const int key = ((add ? add_dtype : out_dtype) << 2) | (w_dtype << 1) | out_dtype;
  switch (key) {
    case 0b000: KVCM_NORM(float, float, float); break;
    case 0b111: KVCM_NORM(bf16_t, bf16_t, bf16_t); break;
    case 0b101: KVCM_NORM(bf16_t, float, bf16_t); break;
    case 0b001: KVCM_NORM(float, float, bf16_t); break;
    case 0b011: KVCM_NORM(float, bf16_t, bf16_t); break;
    default: KVCM_REQUIRE(false, "rmsnorm: unsupported dtypes add=%d w=%d out=%d", add_dtype, w_dtype, out_dtype);
  }
#undef KVCM_NORM
#undef KVCM_NORM4
  return launch_status("rmsnorm");
}

int kvcm_rope_cache(void* qkv, int dtype, int row_stride, const int* positions, const float* inv_freq,
                    const int* slots, void* kcache, void* vcache, int T, int nh, int nkv, int hd, int B,
                    const float* partials, int S, const float* cos_sin, int skip_q, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(hd > 0 && hd % 2 == 0, "rope: head_dim %d must be even", hd);
  KVCM_REQUIRE(!skip_q || !partials, "rope: the q heads of un-added partial sums cannot be left alone");
  const int first_head = skip_q ? nh : 0;
  if (nh + 2 * nkv - first_head == 0) return 0;
  KVCM_REQUIRE(nh >= 0 && nkv >= 0 && row_stride >= (nh + 2 * nkv) * hd, "rope: row stride %d too small", row_stride);
  KVCM_REQUIRE(!slots || (kcache && vcache && B > 0), "rope: cache write without a cache");
  KVCM_REQUIRE(!inv_freq || positions || cos_sin, "rope: rotation without positions");
  KVCM_REQUIRE(!partials || S >= 1, "rope: partial sums need their split count");
  KVCM_REQUIRE(nh + 2 * nkv <= 65535 && nh + 2 * nkv > 0, "rope: too many heads");
  const bool aligned = reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(kcache) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(vcache) % 16 == 0 && reinterpret_cast<uintptr_t>(cos_sin) % 16 == 0 &&
                       row_stride % 4 == 0;
  if (!partials && hd % 16 == 0 && aligned) {
    // q and k heads: 8 pairs per item; v heads (only when there is a cache to store them to): one
    // dim of 8 rows per item, one group more than the rows fill because groups start at a slot
    // that is a multiple of 8
    const long long qk_items = static_cast<long long>(T) * (nh + nkv - first_head) * (hd / 16);
    const long long v_items = slots ? static_cast<long long>((T + kVGroup - 1) / kVGroup + 1) * nkv * hd : 0;
    const long long items = qk_items + v_items;
    const long long blocks = (items + 255) / 256;
    KVCM_REQUIRE(blocks < (1ll << 31), "rope: too many rows");
    if (blocks == 0) return 0;
    if (dtype == kF32)
      rope_cache_vec_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, s>>>(
          static_cast<float*>(qkv), row_stride, positions, inv_freq, slots, static_cast<float*>(kcache),
          static_cast<float*>(vcache), nh, nkv, hd, B, reinterpret_cast<const float2*>(cos_sin), T, qk_items, items, first_head);
    else if (dtype == kBF16)
      rope_cache_vec_kernel<bf16_t><<<static_cast<unsigned>(blocks), 256, 0, s>>>(
          static_cast<bf16_t*>(qkv), row_stride, positions, inv_freq, slots, static_cast<bf16_t*>(kcache),
          static_cast<bf16_t*>(vcache), nh, nkv, hd, B, reinterpret_cast<const float2*>(cos_sin), T, qk_items, items, first_head);
    else KVCM_REQUIRE(false, "rope: unknown dtype %d", dtype);
    return launch_status("rope_cache");
  }
  const dim3 grid(T, nh + 2 * nkv - first_head);
  const int threads = 64;
  if (dtype == kF32)
    rope_cache_kernel<float><<<grid, threads, 0, s>>>(static_cast<float*>(qkv), row_stride, positions, inv_freq, slots,
                                                  static_cast<float*>(kcache), static_cast<float*>(vcache), nh, nkv, hd, B,
                                                  partials, S, reinterpret_cast<const float2*>(cos_sin), first_head);
  else if (dtype == kBF16)
    rope_cache_kernel<bf16_t><<<grid, threads, 0, s>>>(static_cast<bf16_t*>(qkv), row_stride, positions, inv_freq, slots,
                                                   static_cast<bf16_t*>(kcache), static_cast<bf16_t*>(vcache), nh, nkv, hd, B,
                                                   partials, S, reinterpret_cast<const float2*>(cos_sin), first_head);
  else KVCM_REQUIRE(false, "rope: unknown dtype %d", dtype);
  return launch_status("rope_cache");
}

// cos_sin [T][half][2] floats
int kvcm_rope_table(const int* positions, const float* inv_freq, float* cos_sin, int T, int half, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && half > 0, "rope_table: bad sizes T=%d half=%d", T, half);
  rope_table_kernel<<<T, 64, 0, s>>>(positions, inv_freq, reinterpret_cast<float2*>(cos_sin), half);
  return launch_status("rope_table");
}

int kvcm_swiglu(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  KVCM_REQUIRE(T <= 65535, "swiglu: too many rows for one launch (%d)", T);
  if (I % 8 == 0 && reinterpret_cast<uintptr_t>(gate_up) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const dim3 vgrid((I / 8 + 255) / 256, T);
    if (dtype == kF32) swiglu_vec_kernel<float><<<vgrid, 256, 0, s>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), I);
    else if (dtype == kBF16) swiglu_vec_kernel<bf16_t><<<vgrid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), I);
    else KVCM_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
    return launch_status("swiglu");
  }
  const dim3 grid((I + 255) / 256, T);
  if (dtype == kF32) swiglu_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), I);
  else if (dtype == kBF16) swiglu_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), I);
  else KVCM_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
  return launch_status("swiglu");
}

int kvcm_add_residual(float* x, const void* y, int dtype, long long n, hipStream_t s) {
  if (n == 0) return 0;
  KVCM_REQUIRE(n > 0, "add_residual: bad size");
  const int blocks = static_cast<int>(n / 256 + 1 < 8192 ? n / 256 + 1 : 8192);
  if (dtype == kF32) add_residual_kernel<float><<<blocks, 256, 0, s>>>(x, static_cast<const float*>(y), size_t(n));
  else if (dtype == kBF16) add_residual_kernel<bf16_t><<<blocks, 256, 0, s>>>(x, static_cast<const bf16_t*>(y), size_t(n));
  else KVCM_REQUIRE(false, "add_residual: unknown dtype %d", dtype);
  return launch_status("add_residual");
}

}  // extern "C"
