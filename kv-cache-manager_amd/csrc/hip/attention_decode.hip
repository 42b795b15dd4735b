// Decode attention over the paged bfloat16 cache: few query rows, long contexts, the context of
// every row cut into fixed partitions that run in parallel and are merged afterwards.
//
// The structure follows the reference's kernels (src/cuda/paged_attention.cu:50-203): one
// workgroup per (kv head, row, partition) serves all GROUP query heads of that kv head, so that
// every key and value read from the cache is used GROUP times; pass 1 writes scaled scores to LDS,
// pass 2 turns them into exp(s - max) per head, pass 3 accumulates P*V in registers; a second
// kernel merges the partitions by their maxima and sums.  Rebuilt for CDNA4: scores come from the
// matrix cores with the cache's own layout as operand, all of a partition's keys and values are
// requested before the first use, partitions are 256 tokens, and any group size from 1 to 8 and
// head sizes 64 and 128 are compiled (other shapes take the generic kernel).  Partition
// boundaries are absolute multiples of 256: a row's result does not depend on the batch around it.
#include <cfloat>

#include "common.h"

namespace kvcm {

constexpr int kDecWaves = 4;
constexpr int kDecPart = 256;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
union Frag8 {
  uint4 u;
  bf16x8 v;
};

// partial results per (row, head, partition): HD floats of o / sum, then max, then sum
//
// Both products run on the matrix cores with the cache's own layouts as the B operand, 16 bytes
// per lane straight from global memory: for the scores a lane reads 8 dims of one token (keys are
// [slot][dim]), for P*V it reads 8 tokens of one dim (values are [dim][slot]).  The group's query
// heads are the rows of the A operand (rows beyond GROUP are zero).  Each wave takes every fourth
// 16-token tile for the scores and a quarter of the partition's tokens for P*V; the only
// reduction left is over the four waves.
template <int HD, int GROUP>
__global__ void __launch_bounds__(kDecWaves* kWave)
    attention_decode_kernel(const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ kcache,
                            const uint16_t* __restrict__ vcache, const int* __restrict__ tables, int table_stride,
                            const int* __restrict__ row_seq, const int* __restrict__ ctx_lens, int nh, int nkv, int B,
                            float scale, int num_parts, float* __restrict__ scratch) {
  constexpr int KSTEPS = HD / 32;                    // matrix instructions per 16-token tile of scores
  constexpr int TILES = kDecPart / 16 / kDecWaves;   // score tiles per wave
  constexpr int DT = HD / 16;                        // 16-dim tiles of the output
  constexpr int VSTEPS = kDecPart / 32 / kDecWaves;  // 32-token steps of P*V per wave
  const int kvh = blockIdx.x, row = blockIdx.y, part = blockIdx.z;
  const int ctx = ctx_lens[row];
  const int start = part * kDecPart;
  if (start >= ctx) return;
  const int end = min(ctx, start + kDecPart);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;

  __shared__ __attribute__((aligned(16))) float scores[GROUP][kDecPart];
  __shared__ __attribute__((aligned(16))) float red[kDecWaves][16][HD + 4];
  __shared__ float s_max[GROUP], s_sum[GROUP];

  const int* table = tables + size_t(row_seq[row]) * table_stride;
  const size_t head_elems = size_t(B) * HD, page_elems = head_elems * nkv;

  // Where each token of the partition lives, one table lookup per thread, shared through LDS:
  // for keys the offset of the token's row, for values the offset of the token's slot in dim 0,
  // both inside this kv head's part of the cache and in units of 8 elements.  Tokens beyond the
  // context point at the last valid token (keys) or the last valid group of 8 (values), so that
  // every load below is unconditional (a branch around a load makes the compiler wait for it at
  // once); what is loaded for them is never used: no score is stored, their probability is zero.
  __shared__ uint32_t where_k[kDecPart];
  __shared__ uint32_t where_v[kDecPart / 8];
  {
    const int t = min(start + int(threadIdx.x), end - 1);
    const size_t head0 = size_t(table[t / B]) * page_elems + kvh * head_elems;
    where_k[threadIdx.x] = uint32_t((head0 + size_t(t % B) * HD) / 8);
    if (threadIdx.x % 8 == 0) {
      const int tv = min(start + int(threadIdx.x), (end - 1) & ~7);
      where_v[threadIdx.x / 8] = uint32_t((size_t(table[tv / B]) * page_elems + kvh * head_elems + tv % B) / 8);
    }
  }
  __syncthreads();

  // ---- requests first: this wave's keys and values
  const int n16 = lane % 16, kq = lane / 16;
  Frag8 kf[TILES][KSTEPS];
#pragma unroll
  for (int i = 0; i < TILES; ++i) {
    const int tok = (wave + i * kDecWaves) * 16 + n16;
    const uint16_t* kp = kcache + (size_t(where_k[tok]) << 3) + kq * 8;
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c) kf[i][c].u = *reinterpret_cast<const uint4*>(kp + c * 32);
  }
  Frag8 vf[VSTEPS][DT];
#pragma unroll
  for (int j = 0; j < VSTEPS; ++j) {
    const int tok8 = (wave * VSTEPS + j) * 4 + kq;      // which group of 8 tokens this lane reads
    const uint16_t* vp = vcache + (size_t(where_v[tok8]) << 3) + size_t(n16) * B;
#pragma unroll
    for (int d = 0; d < DT; ++d) vf[j][d].u = *reinterpret_cast<const uint4*>(vp + size_t(d) * 16 * B);
  }
  Frag8 qf[KSTEPS];
  const int qhead = kvh * GROUP + (n16 < GROUP ? n16 : 0);
#pragma unroll
  for (int c = 0; c < KSTEPS; ++c) {
    qf[c].u = *reinterpret_cast<const uint4*>(q + size_t(row) * q_stride + size_t(qhead) * HD + c * 32 + kq * 8);
    if (n16 >= GROUP) qf[c].u = uint4{0u, 0u, 0u, 0u};
  }
  // keep every request above ahead of the first use below: the point of this kernel is that a
  // partition costs one trip to memory, not one per token
  __builtin_amdgcn_sched_barrier(0);

  // ---- pass 1: scores[head][token] = scale * q . k
#pragma unroll
  for (int i = 0; i < TILES; ++i) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c].v, kf[i][c].v, acc, 0, 0, 0);
    const int tok = (wave + i * kDecWaves) * 16 + n16;       // accumulator: column = token, rows = heads 4*kq..+3
    if (start + tok < end) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int g = kq * 4 + r;
        if (g < GROUP) scores[g][tok] = acc[r] * scale;
      }
    }
  }
  __syncthreads();

  // ---- pass 2: exp(s - max) and its sum, one wave per head at a time
  const int n = end - start;
  for (int g = wave; g < GROUP; g += kDecWaves) {
    float m = -FLT_MAX;
    for (int i = lane; i < n; i += kWave) m = fmaxf(m, scores[g][i]);
    m = wave_max(m);
    float sum = 0.f;
    for (int i = lane; i < kDecPart; i += kWave) {
      const float e = i < n ? expf(scores[g][i] - m) : 0.f;   // zero beyond the context: pass 3 reads whole quarters
      scores[g][i] = e;
      sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) { s_max[g] = m; s_sum[g] = sum; }
  }
  __syncthreads();

  // ---- pass 3: out[head][dim] += P[head][token] * V[token][dim].  The probabilities stay 32-bit values as in the
  // reference (src/cuda/paged_attention.cu:150-183); a matrix instruction takes bfloat16 operands, so p goes in as two
  // of them, p rounded and what the rounding took away, and the product runs twice.
  f32x4 o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < VSTEPS; ++j) {
    Frag8 pf, pl;
    pf.u = uint4{0u, 0u, 0u, 0u};
    pl.u = uint4{0u, 0u, 0u, 0u};
    if (n16 < GROUP) {
      const float* pr = &scores[n16][(wave * VSTEPS + j) * 32 + kq * 8];
      const float4 a = *reinterpret_cast<const float4*>(pr), b = *reinterpret_cast<const float4*>(pr + 4);
      const float p[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      uint32_t hi[4], lo[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t h0 = float_to_bf16_bits(p[2 * e]), h1 = float_to_bf16_bits(p[2 * e + 1]);
        hi[e] = h0 | (h1 << 16);
        lo[e] = uint32_t(float_to_bf16_bits(p[2 * e] - __uint_as_float(h0 << 16))) |
                (uint32_t(float_to_bf16_bits(p[2 * e + 1] - __uint_as_float(h1 << 16))) << 16);
      }
      pf.u = uint4{hi[0], hi[1], hi[2], hi[3]};
      pl.u = uint4{lo[0], lo[1], lo[2], lo[3]};
    }
    // value slots past the context's end hold stale data, which zero probabilities do not cancel if it is Inf or NaN
    const int left = end - (start + (wave * VSTEPS + j) * 32 + kq * 8);
#pragma unroll
    for (int d = 0; d < DT; ++d) {
      Frag8 v = vf[j][d];
      if (left < 8) v.u = keep_first_bf16(v.u, left);
      o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf.v, v.v, o[d], 0, 0, 0);
      o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl.v, v.v, o[d], 0, 0, 0);
    }
  }
  // accumulator: column = dim n16 of tile d, rows = heads 4*kq..+3
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][kq * 4 + r][d * 16 + n16] = o[d][r];
  __syncthreads();
  for (int i = threadIdx.x; i < GROUP * HD; i += kDecWaves * kWave) {
    const int g = i / HD, d = i % HD;
    float s = red[0][g][d];
#pragma unroll
    for (int w = 1; w < kDecWaves; ++w) s += red[w][g][d];
    const size_t idx = (size_t(row) * nh + kvh * GROUP + g) * num_parts + part;
    float* dst = scratch + idx * (HD + 2);
    dst[d] = s / s_sum[g];
    if (d == 0) { dst[HD] = s_max[g]; dst[HD + 1] = s_sum[g]; }
  }
}

// out = sum_p w_p o_p / sum_p w_p with w_p = sum_p * exp(max_p - max)   (paged_attention.cu:186-203)
// One workgroup of 256 threads per (head, row): the maximum is found by all threads together,
// then 256 / HD groups of HD threads each take every (256 / HD)-th partition and their sums meet
// in LDS, so that a long context (hundreds of partitions) costs a few trips to memory, not one
// per partition.
constexpr int kMergeThreads = 256;
constexpr int kMergeFew = 8;       // parts up to which a thread merges its element alone

template <int HD>
__global__ void __launch_bounds__(kMergeThreads)
attention_decode_merge_kernel(const float* __restrict__ scratch, const int* __restrict__ ctx_lens,
                              uint16_t* __restrict__ out, int out_stride, int nh, int num_parts, int part_tokens) {
  constexpr int GROUPS = kMergeThreads / HD;
  static_assert(GROUPS >= 1 && kMergeThreads % HD == 0, "head_dim must divide the merge workgroup");
  __shared__ float wave_top[kMergeThreads / kWave];
  __shared__ float sums[GROUPS][HD + 1];
  const int head = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
  const int g = tid / HD, d = tid % HD;
  const int ctx = ctx_lens[row];
  uint16_t* o = out + size_t(row) * out_stride + size_t(head) * HD + d;
  if (ctx <= 0) {                                   // the whole workgroup leaves together
    if (g == 0) *o = 0;
    return;
  }
  const int np = (ctx + part_tokens - 1) / part_tokens;
  const float* base = scratch + (size_t(row) * nh + head) * num_parts * (HD + 2);
  if (np <= kMergeFew) {
    // a few parts: every thread of the first group asks for all it needs at once (one trip to memory, no barrier)
    if (g != 0) return;
    float pm[kMergeFew], pl[kMergeFew], po[kMergeFew];
#pragma unroll
    for (int i = 0; i < kMergeFew; ++i) {
      const float* part = base + size_t(i < np ? i : 0) * (HD + 2);
      pm[i] = part[HD]; pl[i] = part[HD + 1]; po[i] = part[d];
    }
    float top = -FLT_MAX;
#pragma unroll
    for (int i = 0; i < kMergeFew; ++i) top = i < np ? fmaxf(top, pm[i]) : top;
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int i = 0; i < kMergeFew; ++i) {
      const float w = i < np ? pl[i] * expf(pm[i] - top) : 0.f;
      num = fmaf(w, po[i], num);
      den += w;
    }
    *o = float_to_bf16_bits(num / den);
    return;
  }
  float m = -FLT_MAX;
  for (int i = tid; i < np; i += kMergeThreads) m = fmaxf(m, base[i * (HD + 2) + HD]);
  m = wave_max(m);
  if (tid % kWave == 0) wave_top[tid / kWave] = m;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kMergeThreads / kWave; ++w) m = fmaxf(m, wave_top[w]);
  float num = 0.f, den = 0.f;
#pragma unroll 4
  for (int i = g; i < np; i += GROUPS) {
    const float* part = base + size_t(i) * (HD + 2);
    const float w = part[HD + 1] * expf(part[HD] - m);
    num = fmaf(w, part[d], num);
    den += w;
  }
  sums[g][d] = num;
  if (d == 0) sums[g][HD] = den;
  __syncthreads();
  if (g == 0) {
#pragma unroll
    for (int k = 1; k < GROUPS; ++k) {
      num += sums[k][d];
      den += sums[k][HD];
    }
    *o = float_to_bf16_bits(num / den);
  }
}

template <int HD, int GROUP>
int launch_decode(const void* q, int q_stride, void* out, int out_stride, const void* kc, const void* vc,
                  const int* tables, int table_stride, const int* row_seq, const int* ctx_lens, int T, int nh, int nkv,
                  int B, float scale, int num_parts, float* scratch, hipStream_t s) {
  attention_decode_kernel<HD, GROUP><<<dim3(nkv, T, num_parts), kDecWaves * kWave, 0, s>>>(
      static_cast<const uint16_t*>(q), q_stride, static_cast<const uint16_t*>(kc), static_cast<const uint16_t*>(vc),
      tables, table_stride, row_seq, ctx_lens, nh, nkv, B, scale, num_parts, scratch);
  attention_decode_merge_kernel<HD><<<dim3(nh, T), kMergeThreads, 0, s>>>(scratch, ctx_lens, static_cast<uint16_t*>(out),
                                                               out_stride, nh, num_parts, kDecPart);
  return 0;
}

// The merge alone, for the one-launch decode kernel when it cuts long contexts into parts.
int launch_decode_merge(const float* scratch, const int* ctx_lens, void* out, int out_stride, int nh, int T, int hd,
                        int num_parts, int part_tokens, hipStream_t s) {
  if (hd == 64)
    attention_decode_merge_kernel<64><<<dim3(nh, T), kMergeThreads, 0, s>>>(scratch, ctx_lens, static_cast<uint16_t*>(out),
                                                                   out_stride, nh, num_parts, part_tokens);
  else if (hd == 128)
    attention_decode_merge_kernel<128><<<dim3(nh, T), kMergeThreads, 0, s>>>(scratch, ctx_lens, static_cast<uint16_t*>(out),
                                                                    out_stride, nh, num_parts, part_tokens);
  else
    return -1;
  return 0;
}

template <int HD, int GROUP>
int decode_kernel_info(int* out) {
  hipFuncAttributes a;
  if (hipFuncGetAttributes(&a, reinterpret_cast<const void*>(&attention_decode_kernel<HD, GROUP>)) != hipSuccess) return -1;
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attention_decode_kernel<HD, GROUP>, kDecWaves * kWave, 0) != hipSuccess) return -1;
  out[0] = a.numRegs; out[1] = static_cast<int>(a.sharedSizeBytes); out[2] = per_cu; out[3] = kDecWaves * kWave;
  return 0;
}

template <int HD>
int dispatch_info(int group, int* out) {
  switch (group) {
    case 1: return decode_kernel_info<HD, 1>(out); case 2: return decode_kernel_info<HD, 2>(out);
    case 3: return decode_kernel_info<HD, 3>(out); case 4: return decode_kernel_info<HD, 4>(out);
    case 5: return decode_kernel_info<HD, 5>(out); case 6: return decode_kernel_info<HD, 6>(out);
    case 7: return decode_kernel_info<HD, 7>(out); case 8: return decode_kernel_info<HD, 8>(out);
    default: return -1;
  }
}

template <int HD>
int dispatch_group(int group, const void* q, int q_stride, void* out, int out_stride, const void* kc, const void* vc,
                   const int* tables, int table_stride, const int* row_seq, const int* ctx_lens, int T, int nh,
                   int nkv, int B, float scale, int num_parts, float* scratch, hipStream_t s) {
#define KVCM_DEC(G) \
  case G: return launch_decode<HD, G>(q, q_stride, out, out_stride, kc, vc, tables, table_stride, row_seq, ctx_lens, T, nh, nkv, B, scale, num_parts, scratch, s)
  switch (group) {
    KVCM_DEC(1); KVCM_DEC(2); KVCM_DEC(3); KVCM_DEC(4); KVCM_DEC(5); KVCM_DEC(6); KVCM_DEC(7); KVCM_DEC(8);
    default: return -1;
  }
#undef KVCM_DEC
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// 1 when this kernel takes the shape (bfloat16 only), else 0 (use the generic kernel).
int kvcm_attention_decode_supported(int nh, int nkv, int hd, int B) {
  if (nkv <= 0 || nh % nkv || B <= 0 || B % 8) return 0;
  const int g = nh / nkv;
  return (hd == 64 || hd == 128) && g >= 1 && g <= 8;
}

// What the compiled kernel for this shape uses: out = {vector registers per lane, bytes of LDS
// per workgroup, workgroups that fit on one CU, threads per workgroup}.
int kvcm_attention_decode_info(int nh, int nkv, int hd, int* out) {
  KVCM_REQUIRE(kvcm_attention_decode_supported(nh, nkv, hd, 8), "attention_decode_info: unsupported shape");
  const int rc = hd == 64 ? dispatch_info<64>(nh / nkv, out) : dispatch_info<128>(nh / nkv, out);
  KVCM_REQUIRE(rc == 0, "attention_decode_info: the runtime gave no attributes");
  return 0;
}

// Floats of scratch a launch needs: rows * heads * partitions * (head_dim + 2).
long long kvcm_attention_decode_scratch(int T, int nh, int hd, int max_context) {
  const long long parts = (max_context + kDecPart - 1) / kDecPart;
  return static_cast<long long>(T) * nh * (parts > 0 ? parts : 1) * (hd + 2);
}

// max_context: an upper bound of every row's context length (it fixes the number of partitions
// launched; rows with shorter contexts leave the surplus workgroups at once).
int kvcm_attention_decode(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                          const void* vcache, const int* tables, int table_stride, const int* row_seq,
                          const int* ctx_lens, int T, int nh, int nkv, int hd, int B, float scale, int max_context,
                          float* scratch, long long scratch_floats, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(kvcm_attention_decode_supported(nh, nkv, hd, B), "attention_decode: unsupported shape heads=%d kv_heads=%d head_dim=%d page=%d", nh, nkv, hd, B);
  KVCM_REQUIRE(T > 0 && B > 0 && max_context > 0, "attention_decode: bad sizes T=%d B=%d max_context=%d", T, B, max_context);
  KVCM_REQUIRE(B % 8 == 0, "attention_decode: the page size %d is not a multiple of 8", B);
  KVCM_REQUIRE(q_stride >= nh * hd && out_stride >= nh * hd && q_stride % 8 == 0, "attention_decode: bad row strides");
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(kcache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(vcache) % 16 == 0, "attention_decode: operands must be 16-byte aligned");
  KVCM_REQUIRE(scratch && scratch_floats >= kvcm_attention_decode_scratch(T, nh, hd, max_context),
               "attention_decode: scratch too small");
  KVCM_REQUIRE(T <= 65535, "attention_decode: too many rows (%d)", T);
  const int num_parts = (max_context + kDecPart - 1) / kDecPart;
  KVCM_REQUIRE(num_parts <= 65535, "attention_decode: context too long");
  const int group = nh / nkv;
  int rc;
  if (hd == 64)
    rc = dispatch_group<64>(group, q, q_stride, out, out_stride, kcache, vcache, tables, table_stride, row_seq, ctx_lens,
                            T, nh, nkv, B, scale, num_parts, scratch, s);
  else
    rc = dispatch_group<128>(group, q, q_stride, out, out_stride, kcache, vcache, tables, table_stride, row_seq, ctx_lens,
                             T, nh, nkv, B, scale, num_parts, scratch, s);
  KVCM_REQUIRE(rc == 0, "attention_decode: no kernel for group size %d", group);
  return launch_status("attention_decode");
}

}  // extern "C"
