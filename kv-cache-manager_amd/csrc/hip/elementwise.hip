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

// --------------------------------------------------------- rotary positions + cache write
// One block per token row of the fused [q | k | v] buffer.  q and k heads are rotated in place
// (pairs (j, j + hd/2), angle = float(pos) * inv_freq[j] in 32-bit); rotated k and plain v are
// copied to the paged cache at slot = page * B + offset, layout [page][kv_head][B][hd].
// inv_freq == null: no rotation.  slots == null or slot < 0: no cache write.
// partials != null: the fused rows do not exist yet; they are the split-K sums [S][rows][width]
// of the projection that makes them (added in split order, rounded to the storage type), and only
// what a later kernel reads is stored: q to the fused rows, k and v to the cache.
template <class T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, const int* __restrict__ slots,
                                  T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv, int hd, int B,
                                  const float* __restrict__ partials, int S) {
  const int t = blockIdx.x;
  T* row = qkv + size_t(t) * row_stride;
  const int half = hd / 2;
  const int width = (nh + 2 * nkv) * hd;
  const float* prow = partials ? partials + size_t(t) * width : nullptr;
  const size_t pstride = size_t(gridDim.x) * width;
  auto value = [&](int c) {
    if (!prow) return load_f(row + c);
    float a = 0.f;
    for (int s = 0; s < S; ++s) a += prow[s * pstride + c];
    return round_to<T>(a);
  };
  const int slot = slots ? slots[t] : -1;
  const size_t page = slot >= 0 ? slot / B : 0;
  const int off = slot >= 0 ? slot % B : 0;
  if (inv_freq) {
    const float pos = float(positions[t]);
    const int pairs = (nh + nkv) * half;
    for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
      const int h = i / half, j = i % half;
      float sn, cs;
      sincosf(pos * inv_freq[j], &sn, &cs);
      const int c = h * hd + j;
      const float a = value(c), b = value(c + half);
      const float ra = a * cs - b * sn, rb = b * cs + a * sn;
      if (!prow || h < nh) {
        store_f(row + c, ra);
        store_f(row + c + half, rb);
      }
      if (slot >= 0 && h >= nh) {
        T* dst = kcache + ((page * nkv + (h - nh)) * B + off) * hd;
        store_f(dst + j, ra);
        store_f(dst + j + half, rb);
      }
    }
  } else if (prow) {
    for (int i = threadIdx.x; i < nh * hd; i += blockDim.x) store_f(row + i, value(i));
  }
  if (slot < 0) return;
  const int koff = nh * hd, voff = (nh + nkv) * hd;
  for (int i = threadIdx.x; i < nkv * hd; i += blockDim.x) {
    const int h = i / hd, d = i % hd;
    const size_t dst = ((page * nkv + h) * B + off) * hd + d;
    if (!inv_freq) store_f(kcache + dst, value(koff + i));
    store_f(vcache + dst, value(voff + i));
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
    const float s = x / (1.0f + expf(-x));
    store_f(o + i, round_to<T>(s) * load_f(u + i));
  }
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
#define KVCM_NORM(TA, TW, TO)                                                                              \
  rmsnorm_kernel<TA, TW, TO><<<R, kNormThreads, 0, s>>>(x, static_cast<const TA*>(add), partials, S, T, rows, \
                                                        static_cast<const TW*>(w), static_cast<TO*>(out), H, eps, write_back)
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
  return launch_status("rmsnorm");
}

int kvcm_rope_cache(void* qkv, int dtype, int row_stride, const int* positions, const float* inv_freq,
                    const int* slots, void* kcache, void* vcache, int T, int nh, int nkv, int hd, int B,
                    const float* partials, int S, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(hd > 0 && hd % 2 == 0, "rope: head_dim %d must be even", hd);
  KVCM_REQUIRE(nh >= 0 && nkv >= 0 && row_stride >= (nh + 2 * nkv) * hd, "rope: row stride %d too small", row_stride);
  KVCM_REQUIRE(!slots || (kcache && vcache && B > 0), "rope: cache write without a cache");
  KVCM_REQUIRE(!inv_freq || positions, "rope: rotation without positions");
  KVCM_REQUIRE(!partials || S >= 1, "rope: partial sums need their split count");
  const int work = (nh + nkv) * hd / 2;
  const int threads = work >= 256 ? 256 : work >= 128 ? 128 : 64;
  if (dtype == kF32)
    rope_cache_kernel<float><<<T, threads, 0, s>>>(static_cast<float*>(qkv), row_stride, positions, inv_freq, slots,
                                                  static_cast<float*>(kcache), static_cast<float*>(vcache), nh, nkv, hd, B,
                                                  partials, S);
  else if (dtype == kBF16)
    rope_cache_kernel<bf16_t><<<T, threads, 0, s>>>(static_cast<bf16_t*>(qkv), row_stride, positions, inv_freq, slots,
                                                   static_cast<bf16_t*>(kcache), static_cast<bf16_t*>(vcache), nh, nkv, hd, B,
                                                   partials, S);
  else KVCM_REQUIRE(false, "rope: unknown dtype %d", dtype);
  return launch_status("rope_cache");
}

int kvcm_swiglu(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
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
