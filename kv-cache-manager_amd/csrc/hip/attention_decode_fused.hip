// One launch for what a decode row needs between the QKV projection and the output projection:
// sum the projection's split-K partial sums, rotate q and k, store the new k and v to their page,
// and attend over the whole context.  The reference runs these as separate kernels
// (src/model/llama.cpp:108-116: rope, reshape_and_cache, paged_attention); on this chip a
// decode step is bound by the number of dependent launches, not by bytes, so they are one here.
//
// One workgroup per (kv head, row) serves the row's whole query group.  After a common prologue
// (q to LDS, new key and value to their page) its waves work on their own: the context is walked
// in chunks of 256 tokens; with head_dim 64 there are eight waves, wave w takes tokens
// 64 (w % 4) .. + 63 of every second chunk (starting at chunk w / 4), with head_dim 128 (registers)
// and in launches of many workgroups four waves take every chunk.  A wave keeps its own running
// maximum, sum and output, and asks for the keys and values of its next chunk before it computes
// the current one.  No barrier inside the loop; the waves' partial results are merged through LDS
// at the end, always in wave order.
//
// Both products run on the matrix cores, transposed: S^T = K Q^T puts one query head in each
// accumulator column, so a lane's softmax concerns one head only and its eight probabilities of a
// 32-token group are, packed to bfloat16, exactly the B operand of O^T += V^T P^T.  Scores never
// touch LDS.  The row -> token assignment of the two key tiles of a group is chosen so that those
// eight tokens are consecutive, which is what the transposed value pages ([dim][slot]) offer as
// 16-byte fragments.
// Only steps whose rows all belong to different sequences may use it: a row's new key is written
// by its own workgroup and read by nobody else.
//
// A few rows with long contexts cannot fill the chip with one workgroup per (kv head, row): then
// the context is cut into parts of whole chunks (blockIdx.z), every part repeats the small
// prologue for q, the part that holds the row's newest token stores it, each part leaves
// (o / l, maximum, l) in scratch and the merge kernel of the partitioned attention adds them up.
#include <cfloat>

#include "common.h"

namespace kvcm {

// attention_decode.hip: out = sum_p w_p o_p / sum_p w_p over parts of part_tokens tokens
int launch_decode_merge(const float* scratch, const int* ctx_lens, void* out, int out_stride, int nh, int T, int hd,
                        int num_parts, int part_tokens, hipStream_t s);

template <int HD> struct FusWaves { static constexpr int N = HD == 64 ? 8 : 4; };
constexpr int kFusChunk = 256;
constexpr float kFusNone = -1.0e30f;   // "no score yet": finite, so that differences stay finite

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2v;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
union FragF {
  uint4 u;
  bf16x8 v;
};
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
  union { bf16x2v v; uint32_t u; } r;
  r.v = __builtin_convertvector(f32x2v{a, b}, bf16x2v);   // one v_cvt_pk_bf16_f32, round to nearest even
  return r.u;
}

template <int HD, int GROUP, int WAVES>
__global__ void __launch_bounds__(WAVES* kWave, HD == 64 ? 8 / WAVES : 1)
    attention_decode_fused_kernel(const float* __restrict__ partials, int S, size_t pstride,
                                  const uint16_t* __restrict__ qkv, int qkv_stride,
                                  const float2* __restrict__ cos_sin, const int* __restrict__ slots,
                                  uint16_t* __restrict__ kcache, uint16_t* __restrict__ vcache,
                                  const int* __restrict__ tables, int table_stride, const int* __restrict__ row_seq,
                                  const int* __restrict__ ctx_lens, int nh, int nkv, int B, float scale,
                                  uint16_t* __restrict__ out, int out_stride, int part_chunks, int num_parts,
                                  float* __restrict__ scratch) {
  constexpr int KSTEPS = HD / 32;   // matrix instructions per 16-token tile of scores
  constexpr int DT = HD / 16;       // 16-dim tiles of the output
  constexpr int HALF = HD / 2;
  constexpr int kFusWaves = WAVES;
  constexpr int STRIDE = kFusWaves / 4;   // a wave takes every STRIDE-th chunk
  const int kvh = blockIdx.x, row = blockIdx.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wq = wave % 4, wfirst = wave / 4;   // which quarter of a chunk, and the first chunk, are this wave's

  __shared__ __attribute__((aligned(16))) uint16_t q_lds[GROUP][HD];
  __shared__ __attribute__((aligned(16))) float red[kFusWaves][16][HD + 4];
  __shared__ float w_max[kFusWaves][16], w_sum[kFusWaves][16];

  // ---- prologue, part one: this row's q (GROUP heads), k and v (one kv head) come from the
  // projection, a pair (j, j + HD/2) of one head per item.  The loads of every thread's first item
  // go out before anything else is waited for (they need the row's number only, and every row of
  // the launch, a padding row too, has its row in these arrays); the pages' numbers and the first
  // keys and values are requested behind them, and only then are the items finished, so that the
  // three trips to memory overlap instead of following one another.
  constexpr int kItems = (GROUP + 2) * HALF, kThreads = kFusWaves * kWave;
  const int width = (nh + 2 * nkv) * HD;
  const float* prow = partials ? partials + size_t(row) * width : nullptr;
  const uint16_t* rrow = qkv + size_t(row) * qkv_stride;
  struct Item { float a[4], b[4]; float2 rot; };
  auto item_col = [&](int item) {
    const int h = item / HALF, j = item % HALF;   // 0..GROUP-1: q heads, GROUP: k, GROUP+1: v
    return (h < GROUP ? (kvh * GROUP + h) * HD : h == GROUP ? (nh + kvh) * HD : (nh + nkv + kvh) * HD) + j;
  };
  auto item_request = [&](int item, Item& it) {
    const int col = item_col(item);
    if (prow) {   // the first four split-K sums (a split beyond S repeats the last and adds nothing)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const size_t o = size_t(j < S ? j : S - 1) * pstride + col;
        it.a[j] = prow[o];
        it.b[j] = prow[o + HALF];
      }
    } else {
      it.a[0] = bf16_bits_to_float(rrow[col]);
      it.b[0] = bf16_bits_to_float(rrow[col + HALF]);
    }
    it.rot = cos_sin && item / HALF <= GROUP ? cos_sin[size_t(row) * HALF + item % HALF] : float2{1.0f, 0.0f};
  };
  constexpr int kPer = (kItems + kThreads - 1) / kThreads;   // items per thread (past the last: item 0 again, dropped)
  Item mine_items[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int item = threadIdx.x + i * kThreads;
    item_request(item < kItems ? item : 0, mine_items[i]);
  }

  const int ctx = ctx_lens[row];
  if (ctx <= 0) {   // a padding row: zeros (from the merge when there are parts), nothing read or stored
    if (num_parts == 1)
      for (int i = threadIdx.x; i < GROUP * HD; i += kThreads)
        out[size_t(row) * out_stride + size_t(kvh) * GROUP * HD + i] = 0;
    return;
  }
  const int* table = tables + size_t(row_seq[row]) * table_stride;
  const size_t head_elems = size_t(B) * HD, page_elems = head_elems * nkv;
  const int nchunks = (ctx + kFusChunk - 1) / kFusChunk;
  const int last = nchunks - 1;
  // this workgroup's chunks: [c_lo, c_hi); the part that reaches the row's end stores its new token
  const int c_lo = num_parts == 1 ? 0 : int(blockIdx.z) * part_chunks;
  if (c_lo >= nchunks) return;   // the row ends before this part (the same for the whole workgroup)
  const int c_hi = num_parts == 1 ? nchunks : min(nchunks, c_lo + part_chunks);
  const int n_local = c_hi - c_lo;
  const bool stores = c_hi == nchunks;

  // Where this wave's 64 tokens of chunk c live: lane l looks up token 64 w + l, the offset of its
  // key row and of its group of 8 value slots, both inside this kv head's part of the cache and in
  // units of 8 elements.  Tokens beyond the context point at the last valid token (keys) or the
  // last valid group of 8 (values), so that every load below is unconditional; what they bring is
  // masked out.  The lanes that need an offset get it by a shuffle.
  struct Where { uint32_t k, v; };
  auto lookup = [&](int c) {
    const int t0 = c * kFusChunk + wq * 64 + lane;
    const int t = min(t0, ctx - 1), tv = min(t0, (ctx - 1) & ~7);
    const int pk = table[t / B], pv = table[tv / B];
    Where w;
    w.k = uint32_t((size_t(pk) * page_elems + kvh * head_elems + size_t(t % B) * HD) / 8);
    w.v = uint32_t((size_t(pv) * page_elems + kvh * head_elems + tv % B) / 8);
    return w;
  };
  // this wave's chunks: wfirst, wfirst + STRIDE, ...; lookups run two of them ahead of the
  // computation, so that their trip to memory is never waited for
  const int mine = n_local > wfirst ? (n_local - wfirst + STRIDE - 1) / STRIDE : 0;
  const int my_last = c_lo + wfirst + STRIDE * (mine > 0 ? mine - 1 : 0);
  auto nth = [&](int i) { return min(c_lo + wfirst + STRIDE * i, my_last); };   // past the last: the last again, never used
  Where wha = lookup(min(nth(0), last)), whb = lookup(min(nth(1), last));

  const int n16 = lane % 16, kq = lane / 16;
  // A chunk's operands for this wave: two groups of 32 tokens; a group's keys as two 16-row tiles
  // whose row r holds token 8 (r / 4) + 4 tile + r % 4 of the group, its values as [dim][8 tokens].
  struct Chunk {
    FragF k[2][2][KSTEPS];
    FragF v[2][DT];
  };
  auto request = [&](const Where& wh, Chunk& ch) {
#pragma unroll
    for (int g = 0; g < 2; ++g) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int tok = g * 32 + 8 * (n16 / 4) + 4 * t + n16 % 4;
        const uint16_t* kp = kcache + (size_t(__shfl(wh.k, tok, kWave)) << 3) + kq * 8;
#pragma unroll
        for (int c = 0; c < KSTEPS; ++c) ch.k[g][t][c].u = *reinterpret_cast<const uint4*>(kp + c * 32);
      }
      const uint16_t* vp = vcache + (size_t(__shfl(wh.v, g * 32 + 8 * kq, kWave)) << 3) + size_t(n16) * B;
#pragma unroll
      for (int d = 0; d < DT; ++d) ch.v[g][d].u = *reinterpret_cast<const uint4*>(vp + size_t(d) * 16 * B);
    }
  };
  // The wave's first chunk is requested now unless it holds the token that this workgroup is about
  // to store (then after the barrier below).  No load sits behind a branch: a wave that must wait
  // requests the cache's first bytes instead, every lane the same, and drops them.
  const int slot = slots ? slots[row] : -1;
  const bool ahead = mine > 0 && !(stores && slot >= 0 && nth(0) == last);
  Chunk cha, chb;
  {
    Where early = wha;
    if (!ahead) early.k = early.v = 0u;
    request(early, cha);
  }

  // ---- prologue, part two: sum, rotate, round; q to LDS, the new key and value to their page
  const size_t page = slot >= 0 ? slot / B : 0;
  const int off = slot >= 0 ? slot % B : 0;
  auto item_finish = [&](int item, const Item& it) {
    const int h = item / HALF, j = item % HALF;
    if (h >= GROUP && !(stores && slot >= 0)) return;
    float a = it.a[0], b = it.b[0];
    if (prow) {
      const int col = item_col(item);
      a = 0.f;
      b = 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        a += k < S ? it.a[k] : 0.f;
        b += k < S ? it.b[k] : 0.f;
      }
      for (int s0 = 4; s0 < S; s0 += 4) {   // four loads requested together
        float pa[4], pb[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const size_t o = size_t(s0 + k < S ? s0 + k : S - 1) * pstride + col;
          pa[k] = prow[o];
          pb[k] = prow[o + HALF];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          a += s0 + k < S ? pa[k] : 0.f;
          b += s0 + k < S ? pb[k] : 0.f;
        }
      }
      a = bf16_bits_to_float(float_to_bf16_bits(a));   // the projection's result is a bfloat16 value
      b = bf16_bits_to_float(float_to_bf16_bits(b));
    }
    if (h <= GROUP && cos_sin) rotate_pair(a, b, it.rot.x, it.rot.y);
    const uint16_t ab = float_to_bf16_bits(a), bb = float_to_bf16_bits(b);
    if (h < GROUP) {
      q_lds[h][j] = ab;
      q_lds[h][j + HALF] = bb;
    } else if (h == GROUP) {
      uint16_t* kr = kcache + ((page * nkv + kvh) * B + off) * HD;
      kr[j] = ab;
      kr[j + HALF] = bb;
    } else {   // values lie transposed inside the page: [dim][slot]
      uint16_t* vr = vcache + (page * nkv + kvh) * size_t(HD) * B + off;
      vr[size_t(j) * B] = ab;
      vr[size_t(j + HALF) * B] = bb;
    }
  };
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int item = threadIdx.x + i * kThreads;
    if (item < kItems) item_finish(item, mine_items[i]);
  }
  __syncthreads();   // q in LDS; the new key and value are stored before any wave of this workgroup loads them

  // B operand of S^T = K Q^T: lane = (query head n16, dims 8 kq .. + 7 of every 32); heads beyond the group are zero
  FragF qf[KSTEPS];
#pragma unroll
  for (int c = 0; c < KSTEPS; ++c) {
    qf[c].u = *reinterpret_cast<const uint4*>(&q_lds[n16 < GROUP ? n16 : 0][c * 32 + kq * 8]);
    if (n16 >= GROUP) qf[c].u = uint4{0u, 0u, 0u, 0u};
  }

  // running state of this lane's head (n16): maximum (log2 domain), this lane's share of the sum,
  // and O^T (column = head, rows = dims 16 d + 4 kq + i)
  float m_run = kFusNone, l_run = 0.f;
  f32x4 o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float scale2 = scale * 1.4426950408889634f;

  auto compute = [&](int c, const Chunk& ch) {
    const int base = c * kFusChunk + wq * 64 + 8 * kq;   // this lane's first token of group 0
    float s[2][8];
    float mx = kFusNone;
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < KSTEPS; ++k) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ch.k[g][t][k].v, qf[k].v, acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {   // accumulator row 4 kq + i of tile t = token 8 kq + 4 t + i of the group
          const bool valid = base + g * 32 + 4 * t + i < ctx;
          s[g][4 * t + i] = valid ? acc[i] * scale2 : kFusNone;
          mx = fmaxf(mx, s[g][4 * t + i]);
        }
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = exp2f(m_run - m_new);
    m_run = m_new;
    float sum = 0.f;
    // The probabilities stay 32-bit values as in the reference (src/cuda/paged_attention.cu:150-183 multiplies
    // 32-bit probabilities with the stored values): a matrix instruction takes bfloat16 operands, so p goes in
    // as two of them, p rounded and what the rounding took away (16 bits of mantissa in all), and the product
    // with the values runs twice.  The instruction count of a decode row does not show in its time.
    FragF pf[2], pl[2];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      float p[8];
      uint32_t hi[4], lo[4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        p[j] = s[g][j] > 0.5f * kFusNone ? exp2f(s[g][j] - m_new) : 0.f;
        sum += p[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        hi[j] = pack2_bf16(p[2 * j], p[2 * j + 1]);
        lo[j] = pack2_bf16(p[2 * j] - __uint_as_float(hi[j] << 16), p[2 * j + 1] - __uint_as_float(hi[j] & 0xffff0000u));
      }
      pf[g].u = uint4{hi[0], hi[1], hi[2], hi[3]};
      pl[g].u = uint4{lo[0], lo[1], lo[2], lo[3]};
    }
    l_run = l_run * alpha + sum;
    // this lane's 8 value slots of a group that reach past the context hold stale data: cut them
    // (only the chunk with the context's end has such slots)
    const bool cut = base + 40 > ctx;
#pragma unroll
    for (int d = 0; d < DT; ++d) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[d][i] *= alpha;
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        FragF vf = ch.v[g][d];
        if (cut) vf.u = keep_first_bf16(vf.u, ctx - (base + g * 32));
        o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[g].v, o[d], 0, 0, 0);
        o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pl[g].v, o[d], 0, 0, 0);
      }
    }
  };

  // The chunk after the last repeats the last one, so that no load sits behind a branch; what it
  // brings is never used.
  if (mine > 0) {
    if (!ahead) request(wha, cha);
    wha = lookup(nth(2));
    for (int i = 0; i < mine; i += 2) {
      request(whb, chb);                 // this wave's chunk i + 1
      whb = lookup(nth(i + 3));
      __builtin_amdgcn_sched_barrier(0);
      compute(c_lo + wfirst + STRIDE * i, cha);
      if (i + 1 >= mine) break;
      request(wha, cha);                 // chunk i + 2
      wha = lookup(nth(i + 4));
      __builtin_amdgcn_sched_barrier(0);
      compute(c_lo + wfirst + STRIDE * (i + 1), chb);
    }
  }

  // ---- the waves' results, merged in wave order: out = sum_w e_w o_w / sum_w e_w l_w, e_w = 2^(m_w - m)
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);
  if (kq == 0) { w_max[wave][n16] = m_run; w_sum[wave][n16] = l_run; }
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][n16][d * 16 + 4 * kq + i] = o[d][i];
  __syncthreads();
  for (int i = threadIdx.x; i < GROUP * HD; i += kFusWaves * kWave) {
    const int g = i / HD, d = i % HD;
    float m = w_max[0][g];
#pragma unroll
    for (int w = 1; w < kFusWaves; ++w) m = fmaxf(m, w_max[w][g]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < kFusWaves; ++w) {
      const float e = exp2f(w_max[w][g] - m);
      num = fmaf(e, red[w][g][d], num);
      den = fmaf(e, w_sum[w][g], den);
    }
    if (num_parts == 1) {
      out[size_t(row) * out_stride + size_t(kvh * GROUP + g) * HD + d] = float_to_bf16_bits(num / den);
    } else {   // (o / l, maximum in natural units, l) of this part, as the merge kernel reads them
      float* dst = scratch + ((size_t(row) * nh + kvh * GROUP + g) * num_parts + blockIdx.z) * (HD + 2);
      dst[d] = num / den;
      if (d == 0) {
        dst[HD] = m * 0.6931471805599453f;
        dst[HD + 1] = den;
      }
    }
  }
}

template <int HD, int GROUP>
int fused_kernel_info(int* out) {
  hipFuncAttributes a;
  int per_cu = 0;
  constexpr int W = FusWaves<HD>::N;
  if (hipFuncGetAttributes(&a, reinterpret_cast<const void*>(&attention_decode_fused_kernel<HD, GROUP, W>)) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attention_decode_fused_kernel<HD, GROUP, W>, W * kWave, 0) != hipSuccess)
    return -1;
  out[0] = a.numRegs; out[1] = static_cast<int>(a.sharedSizeBytes); out[2] = per_cu; out[3] = FusWaves<HD>::N * kWave;
  return 0;
}

template <int HD>
int dispatch_fused_info(int group, int* out) {
  switch (group) {
    case 1: return fused_kernel_info<HD, 1>(out); case 2: return fused_kernel_info<HD, 2>(out);
    case 3: return fused_kernel_info<HD, 3>(out); case 4: return fused_kernel_info<HD, 4>(out);
    case 5: return fused_kernel_info<HD, 5>(out); case 6: return fused_kernel_info<HD, 6>(out);
    case 7: return fused_kernel_info<HD, 7>(out); case 8: return fused_kernel_info<HD, 8>(out);
    default: return -1;
  }
}

template <int HD, int WAVES>
int dispatch_fused(int group, dim3 grid, hipStream_t s, const float* partials, int S, size_t pstride, const uint16_t* qkv,
                   int qkv_stride, const float2* cos_sin, const int* slots, uint16_t* kc, uint16_t* vc,
                   const int* tables, int table_stride, const int* row_seq, const int* ctx_lens, int nh, int nkv, int B,
                   float scale, uint16_t* out, int out_stride, int part_chunks, int num_parts, float* scratch) {
#define KVCM_FUSED(G)                                                                                                   \
  case G:                                                                                                               \
    attention_decode_fused_kernel<HD, G, WAVES><<<grid, WAVES * kWave, 0, s>>>(partials, S, pstride, qkv, qkv_stride,         \
                                                                           cos_sin, slots, kc, vc, tables, table_stride, \
                                                                           row_seq, ctx_lens, nh, nkv, B, scale, out,   \
                                                                           out_stride, part_chunks, num_parts, scratch); \
    return 0
  switch (group) {
    KVCM_FUSED(1); KVCM_FUSED(2); KVCM_FUSED(3); KVCM_FUSED(4); KVCM_FUSED(5); KVCM_FUSED(6); KVCM_FUSED(7); KVCM_FUSED(8);
    default: return -1;
  }
#undef KVCM_FUSED
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// 1 when this kernel takes the shape (bfloat16 only), else 0.
int kvcm_attention_decode_fused_supported(int nh, int nkv, int hd, int B) {
  if (nkv <= 0 || nh % nkv || B <= 0 || B % 8) return 0;
  const int g = nh / nkv;
  return (hd == 64 || hd == 128) && g >= 1 && g <= 8;
}

// What the compiled kernel for this shape uses: out = {vector registers per lane, bytes of LDS
// per workgroup, workgroups that fit on one CU, threads per workgroup}.
int kvcm_attention_decode_fused_info(int nh, int nkv, int hd, int* out) {
  KVCM_REQUIRE(kvcm_attention_decode_fused_supported(nh, nkv, hd, 8), "attention_decode_fused_info: unsupported shape");
  const int rc = hd == 64 ? dispatch_fused_info<64>(nh / nkv, out) : dispatch_fused_info<128>(nh / nkv, out);
  KVCM_REQUIRE(rc == 0, "attention_decode_fused_info: the runtime gave no attributes");
  return 0;
}

// How a launch for T rows with contexts of at most max_context cuts them: one workgroup per
// (kv head, row) while that fills the chip or contexts are short; else parts of whole chunks, about
// one workgroup per CU in all.  Returns the number of parts, *part_chunks chunks of 256 tokens each.
constexpr int kFusSingleMax = 1024;   // contexts up to this run as one part, unless few workgroups read much each (below)
constexpr int kFusTargetWorkgroups = 256;
// A workgroup of eight waves has a CU to itself (registers).  From two workgroups per CU on, a
// launch at head_dim 64 takes workgroups of four waves, each of which walks every chunk: two of
// them share a CU, and one's trips to memory in the prologue and its merge overlap the other's
// walk.  Measured inside decode steps of 512-token prompts: 128 rows 2.26 -> 2.16 ms, 256 rows
// 3.45 -> 3.22 ms, 64 rows (256 workgroups) 1.61 -> 1.63 ms, hence the limit.
constexpr long long kFusHalfFrom = 512;
// A workgroup reads its context through one CU, which has only so many requests on their way: with few
// workgroups and more than kFusFewBytes of keys and values each (512 tokens at head_dim 128), parts on CUs of
// their own are worth the second launch that merges them (Llama-3-8B sizes, 512-token prompts, batch 1 / 4 / 8:
// 3.86 / 3.95 / 3.96 -> 3.76 / 3.88 / 3.91 ms; batch 16, 128 workgroups: 4.01 -> 4.06, hence the limit; at
// head_dim 64 the same cut at 512 to 768 tokens gained nothing: 0.905 -> 0.911 ms).
constexpr int kFusFewWorkgroups = 64;
constexpr int kFusFewBytes = 256 << 10;
static int fused_parts(int T, int nkv, int hd, int max_context, int* part_chunks) {
  const int nchunks = max_context > 0 ? (max_context + kFusChunk - 1) / kFusChunk : 1;
  long long parts = 1;
  const long long wgs = static_cast<long long>(T) * nkv;
  const bool few = wgs <= kFusFewWorkgroups && static_cast<long long>(max_context) * hd * 4 > kFusFewBytes;
  if (max_context > kFusSingleMax || few) {
    parts = (kFusTargetWorkgroups + wgs - 1) / wgs;
    if (parts > nchunks) parts = nchunks;
    if (parts < 1) parts = 1;
  }
  int pc = static_cast<int>((nchunks + parts - 1) / parts);
  const int n = (nchunks + pc - 1) / pc;
  *part_chunks = n == 1 ? (1 << 20) : pc;
  return n;
}

// Floats of scratch a launch of these sizes needs (0: contexts are not cut).
long long kvcm_attention_decode_fused_scratch(int T, int nh, int nkv, int hd, int max_context) {
  int pc;
  const int parts = fused_parts(T, nkv, hd, max_context, &pc);
  return parts <= 1 ? 0 : static_cast<long long>(T) * nh * parts * (hd + 2);
}

// Rows of T different sequences.  The projection's result is either `partials` (split-K sums
// [S][T][width], width = (nh + 2 nkv) * hd, added in split order) or, when partials is null, the
// bfloat16 rows `qkv`.  cos_sin [T][hd/2] (cos, sin) rotates q and k by pairs (j, j + hd/2); null:
// no rotation.  slots [T]: where the row's key and value go (page * B + offset; negative or a
// null array: nothing is stored and the context is read as it is).  ctx_lens[t] includes the
// row's own token.  max_context: an upper bound of every row's context length (0: unknown, contexts
// are never cut into parts); scratch: kvcm_attention_decode_fused_scratch floats when that is not 0.
int kvcm_attention_decode_fused(const float* partials, int S, const void* qkv, int qkv_stride, const float* cos_sin,
                                const int* slots, void* kcache, void* vcache, const int* tables, int table_stride,
                                const int* row_seq, const int* ctx_lens, int T, int nh, int nkv, int hd, int B,
                                float scale, void* out, int out_stride, int max_context, float* scratch,
                                long long scratch_floats, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(kvcm_attention_decode_fused_supported(nh, nkv, hd, B),
               "attention_decode_fused: unsupported shape heads=%d kv_heads=%d head_dim=%d page=%d", nh, nkv, hd, B);
  KVCM_REQUIRE(T > 0 && T <= 65535 && nkv <= 65535, "attention_decode_fused: bad row count %d", T);
  KVCM_REQUIRE(partials ? (S >= 1 && S <= 64) : (qkv != nullptr && qkv_stride >= (nh + 2 * nkv) * hd),
               "attention_decode_fused: no projection result (splits %d, row stride %d)", S, qkv_stride);
  KVCM_REQUIRE(out_stride >= nh * hd, "attention_decode_fused: output rows too short");
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(kcache) % 16 == 0 && reinterpret_cast<uintptr_t>(vcache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(cos_sin) % 8 == 0,
               "attention_decode_fused: operands must be 16-byte aligned");
  const size_t pstride = size_t(T) * (nh + 2 * nkv) * hd;
  int part_chunks;
  const int parts = fused_parts(T, nkv, hd, max_context, &part_chunks);
  KVCM_REQUIRE(parts <= 65535, "attention_decode_fused: context too long");
  const long long need = kvcm_attention_decode_fused_scratch(T, nh, nkv, hd, max_context);
  KVCM_REQUIRE(need == 0 || (scratch != nullptr && scratch_floats >= need),
               "attention_decode_fused: scratch too small (%lld floats needed)", need);
  const dim3 grid(nkv, T, parts);
  int rc;
#define KVCM_FUSED_ARGS                                                                                                  \
  nh / nkv, grid, s, partials, S, pstride, static_cast<const uint16_t*>(qkv), qkv_stride,                                \
      reinterpret_cast<const float2*>(cos_sin), slots, static_cast<uint16_t*>(kcache), static_cast<uint16_t*>(vcache),   \
      tables, table_stride, row_seq, ctx_lens, nh, nkv, B, scale, static_cast<uint16_t*>(out), out_stride, part_chunks,  \
      parts, scratch
  if (hd == 128)
    rc = dispatch_fused<128, 4>(KVCM_FUSED_ARGS);
  else if (static_cast<long long>(nkv) * T * parts >= kFusHalfFrom)
    rc = dispatch_fused<64, 4>(KVCM_FUSED_ARGS);
  else
    rc = dispatch_fused<64, 8>(KVCM_FUSED_ARGS);
#undef KVCM_FUSED_ARGS
  KVCM_REQUIRE(rc == 0, "attention_decode_fused: no kernel for group size %d", nh / nkv);
  if (parts > 1) launch_decode_merge(scratch, ctx_lens, out, out_stride, nh, T, hd, parts, part_chunks * kFusChunk, s);
  return launch_status("attention_decode_fused");
}

}  // extern "C"
