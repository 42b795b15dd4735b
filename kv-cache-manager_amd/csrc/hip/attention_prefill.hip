// Prefill attention over the paged bfloat16 cache: runs of consecutive query positions of one
// sequence (a whole prompt, or a portion that starts anywhere) against every key the sequence has
// in the cache, its own included.  The reference runs its decode kernel row by row for this
// (src/cuda/paged_attention.cu:50-183, docs/design.md:113-114): every row re-reads all its keys.
// Here a workgroup takes 64 query rows of one head, each of its four waves 16 of them, and walks
// the keys 64 at a time with a running maximum (no score buffer), so keys are read once per 64
// rows; Q*K^T and P*V run on the matrix cores (v_mfma_f32_16x16x32_bf16) with the cache's own
// layouts as B operands, 16 bytes per lane straight from global memory: keys [slot][dim] give 8
// dims of one token, values [dim][slot] give 8 tokens of one dim.  Probabilities pass through LDS
// once, as bfloat16, to change from the accumulator layout to the A-operand layout.
//
// The only mask is causal: a row at position p sees tokens t <= p.  Rows of different sequences
// never share a workgroup.  Head sizes 64 and 128, pages that hold a multiple of 8 tokens.
#include <cfloat>

#include "common.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
union PFrag {
  uint4 u;
  bf16x8 v;
};

constexpr int kPfWaves = 4;
constexpr int kPfRows = 16 * kPfWaves;  // query rows per workgroup
constexpr int kPfChunk = 64;            // keys per trip
constexpr int kPfPitch = kPfChunk + 8;  // LDS row pitch of the probability tile, in bfloat16

__device__ __forceinline__ float row16_max(float v) {
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

template <int HD>
__global__ void __launch_bounds__(kPfWaves* kWave)
    attention_prefill_kernel(const uint16_t* __restrict__ q, int q_stride, uint16_t* __restrict__ out, int out_stride,
                             const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                             const int* __restrict__ tables, int table_stride, const int* __restrict__ run_start,
                             const int* __restrict__ seq_start, int nh, int nkv, int B, float scale) {
  constexpr int KSTEPS = HD / 32;  // matrix instructions per 16-token tile of scores
  constexpr int DT = HD / 16;      // 16-dim tiles of the output
  const int tile = blockIdx.x, seq = blockIdx.y, head = blockIdx.z;
  const int row0 = run_start[seq], n_rows = run_start[seq + 1] - row0;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int first = tile * kPfRows + wave * 16;  // first row of this wave inside the run
  if (first >= n_rows) return;                   // whole waves leave; nothing below synchronises across waves
  const int n16 = lane % 16, kq = lane / 16;
  const int pos0 = seq_start[seq];
  const int kvh = head / (nh / nkv);
  const int* table = tables + size_t(seq) * table_stride;
  const size_t head_elems = size_t(B) * HD, page_elems = head_elems * nkv;
  const uint16_t* kbase = kcache + kvh * head_elems;
  const uint16_t* vbase = vcache + kvh * head_elems;

  __shared__ __attribute__((aligned(16))) uint16_t p_lds[kPfWaves][16][kPfPitch];

  // A operand of the scores: lane holds 8 dims of query row n16 (rows past the run repeat its last row)
  PFrag qf[KSTEPS];
  {
    const int r = row0 + min(first + n16, n_rows - 1);
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c)
      qf[c].u = *reinterpret_cast<const uint4*>(q + size_t(r) * q_stride + size_t(head) * HD + c * 32 + kq * 8);
  }
  // accumulator rows of this lane: 4*kq + i; their positions decide what they may see
  int pos[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) pos[i] = pos0 + min(first + 4 * kq + i, n_rows - 1);
  const int last_pos = pos0 + min(first + 15, n_rows - 1);  // the wave's last row

  float m[4], l[4];
  f32x4 o[DT];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m[i] = -FLT_MAX; l[i] = 0.f; }
#pragma unroll
  for (int d = 0; d < DT; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int c0 = 0; c0 <= last_pos; c0 += kPfChunk) {
    // ---- requests: keys of four 16-token tiles, values of two 32-token steps.  Tokens past the
    // wave's last position point at that position: loads stay unconditional, the mask removes them.
    PFrag kf[4][KSTEPS], vf[2][DT];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = min(c0 + j * 16 + n16, last_pos);
      const uint16_t* kp = kbase + size_t(table[t / B]) * page_elems + size_t(t % B) * HD + kq * 8;
#pragma unroll
      for (int c = 0; c < KSTEPS; ++c) kf[j][c].u = *reinterpret_cast<const uint4*>(kp + c * 32);
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int t = min(c0 + c * 32 + kq * 8, last_pos & ~7);
      const uint16_t* vp = vbase + size_t(table[t / B]) * page_elems + t % B + size_t(n16) * B;
#pragma unroll
      for (int d = 0; d < DT; ++d) vf[c][d].u = *reinterpret_cast<const uint4*>(vp + size_t(d) * 16 * B);
    }

    // ---- scores: s[j][i] = scale * q[row 4kq+i] . k[token c0 + 16j + n16]
    f32x4 s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KSTEPS; ++c) s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c].v, kf[j][c].v, s[j], 0, 0, 0);
    }
    float mx[4], alpha[4], sum[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      mx[i] = -FLT_MAX;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int t = c0 + j * 16 + n16;
        s[j][i] = t <= pos[i] ? s[j][i] * scale : -FLT_MAX;
        mx[i] = fmaxf(mx[i], s[j][i]);
      }
      mx[i] = row16_max(mx[i]);
      const float m_new = fmaxf(m[i], mx[i]);   // finite from the first trip on: token 0 is visible to every row
      alpha[i] = expf(m[i] - m_new);
      m[i] = m_new;
      sum[i] = 0.f;
    }
    // ---- probabilities, to LDS in the accumulator layout (row 4kq+i, column 16j+n16)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = s[j][i] > -FLT_MAX ? expf(s[j][i] - m[i]) : 0.f;
        sum[i] += p;
        p_lds[wave][4 * kq + i][j * 16 + n16] = float_to_bf16_bits(p);
      }
#pragma unroll
    for (int i = 0; i < 4; ++i) l[i] = l[i] * alpha[i] + row16_sum(sum[i]);
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[d][i] *= alpha[i];
    __builtin_amdgcn_wave_barrier();  // the wave's own LDS traffic stays in program order
    // ---- out += P * V, P read back in the A-operand layout (row n16, 8 tokens kq*8..)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      PFrag pf;
      pf.u = *reinterpret_cast<const uint4*>(&p_lds[wave][n16][c * 32 + kq * 8]);
#pragma unroll
      for (int d = 0; d < DT; ++d) o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf.v, vf[c][d].v, o[d], 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = first + 4 * kq + i;
    if (r >= n_rows) continue;
    uint16_t* orow = out + size_t(row0 + r) * out_stride + size_t(head) * HD + n16;
    const float inv = 1.0f / l[i];
#pragma unroll
    for (int d = 0; d < DT; ++d) orow[d * 16] = float_to_bf16_bits(o[d][i] * inv);
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_attention_prefill_supported(int nh, int nkv, int hd, int B) {
  return nkv > 0 && nh % nkv == 0 && (hd == 64 || hd == 128) && B > 0 && B % 8 == 0;
}

// run_start [S+1]: first row of each sequence's run of consecutive positions (rows of a run are
// consecutive); seq_start [S]: position of a run's first row; tables [S][table_stride];
// max_run: the longest run (it sizes the launch).
int kvcm_attention_prefill(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                           const void* vcache, const int* tables, int table_stride, const int* run_start,
                           const int* seq_start, int S, int max_run, int nh, int nkv, int hd, int B, float scale,
                           hipStream_t s) {
  if (S == 0 || max_run == 0) return 0;
  KVCM_REQUIRE(kvcm_attention_prefill_supported(nh, nkv, hd, B),
               "attention_prefill: unsupported shape heads=%d kv_heads=%d head_dim=%d page=%d", nh, nkv, hd, B);
  KVCM_REQUIRE(S > 0 && max_run > 0 && S <= 65535 && nh <= 65535, "attention_prefill: bad sizes S=%d max_run=%d", S, max_run);
  KVCM_REQUIRE(q_stride >= nh * hd && out_stride >= nh * hd && q_stride % 8 == 0, "attention_prefill: bad row strides");
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(kcache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(vcache) % 16 == 0, "attention_prefill: operands must be 16-byte aligned");
  const dim3 grid((max_run + kPfRows - 1) / kPfRows, S, nh);
  const uint16_t *qq = static_cast<const uint16_t*>(q), *kc = static_cast<const uint16_t*>(kcache),
                 *vc = static_cast<const uint16_t*>(vcache);
  if (hd == 64)
    attention_prefill_kernel<64><<<grid, kPfWaves * kWave, 0, s>>>(qq, q_stride, static_cast<uint16_t*>(out), out_stride, kc, vc,
                                                                  tables, table_stride, run_start, seq_start, nh, nkv, B, scale);
  else
    attention_prefill_kernel<128><<<grid, kPfWaves * kWave, 0, s>>>(qq, q_stride, static_cast<uint16_t*>(out), out_stride, kc, vc,
                                                                   tables, table_stride, run_start, seq_start, nh, nkv, B, scale);
  return launch_status("attention_prefill");
}

}  // extern "C"
