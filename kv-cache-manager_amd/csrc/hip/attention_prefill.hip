// Prefill attention over the paged bfloat16 cache: runs of consecutive query positions of one
// sequence (a whole prompt, or a portion that starts anywhere) against every key the sequence has
// in the cache, its own included.  The reference runs its decode kernel row by row for this
// (src/cuda/paged_attention.cu:50-183, docs/design.md:113-114): every row re-reads all its keys.
//
// Here a workgroup takes 128 query rows of one head, each of its four waves 32 of them (two
// 16-row tiles), and walks the keys 64 at a time with a running maximum (no score buffer).  A
// chunk of keys and values is staged in LDS once per workgroup, double-buffered: the next chunk's
// global loads are in flight while the current one is multiplied.
//
// A launch ends when its longest walk does, and a wave needs about a microsecond for a chunk
// whatever else the chip does.  Launches of little work at head_dim 64 take 64 rows per workgroup
// (one tile per wave: twice the workgroups, each with fewer registers), and those that leave CUs
// without a full set of waves (a prompt of up to 1,024 tokens: 512 workgroups) eight waves: four
// groups of 16 rows times two halves of a 128-key trip, so that the longest walk is half as many
// trips; the halves' running maxima, sums and outputs meet in LDS at the end (1,024 tokens: 17.1 ->
// 14.7 us; where every CU has work for all its waves anyway the eight waves are slower: 2,048 tokens
// 43.5 against 37.3 us, eight portions of 300 tokens 23.9 against 19.9 us).
//
// Both products run on the matrix cores (v_mfma_f32_16x16x32_bf16), transposed:
//   S^T[token][row] = K[token][dim] * Q^T[dim][row]      A = keys as they lie ([slot][dim]),  B = Q
//   O^T[dim][row]  += V^T[dim][token] * P^T[token][row]  A = values as they lie ([dim][slot]), B = P
// In the accumulator of S^T a lane holds, for ONE query row (lane % 16), four tokens of each
// 16-token tile; after exp those registers, rounded to bfloat16 and packed, ARE the B operand of
// the second product (the order of the reduction index inside a matrix instruction is free as long
// as both operands agree, so the values are kept in LDS in that same token order: staging puts
// token 16 a + 4 q + e of a group of 32 at place 8 q + 4 a + e, and a lane's 8 tokens of a step are one
// 16-byte read; as two 8-byte reads of tokens as they lie they collided in the LDS banks).  The
// probabilities never touch LDS, a row's maximum lives in one lane, its sum comes from a third
// product (ones * P^T: the sum of the probabilities as the second product sees them), and the
// output is stored four dims at a time.
//
// The only mask is causal: a row at position p sees tokens t <= p.  Rows of different sequences
// never share a workgroup.  Head sizes 64 and 128; pages of 8, 16, 32, ... tokens (a power of two).
//
// While tiles x heads x sequences give fewer than two workgroups per CU, contexts are cut into
// segments of keys (multiples of 512, at absolute multiples of their length) that run as workgroups
// of their own: without that a short portion behind a long context leaves most of the chip idle.
// A tile whose rows see one segment stores its result; otherwise every segment leaves
// (o / l, m, l) per row in scratch and a second kernel merges them in segment order.
#include <cfloat>

#include "common.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
// 16 bytes on their way from the cache to LDS.  A native vector, not HIP's uint4: arrays of that
// struct type are not split into registers by the compiler, they went through scratch memory, and
// every load was waited for at once instead of two chunks later.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
union PFrag {
  uint4 u;
  bf16x8 v;
};

constexpr int kPfWaves = 4;                      // row groups of a workgroup (waves, or pairs of waves that halve a trip's keys)
constexpr int kPfGroupThreads = kPfWaves * kWave;
// A wave takes RT tiles of 16 query rows, a workgroup 64 RT rows: two tiles (128 rows) by default, one
// (64 rows) for launches of little work at head_dim 64, where twice the workgroups, each with fewer
// registers (four to a CU instead of two), hide one another's waits better than a workgroup's
// larger share of every staged chunk saves.
constexpr int kPfMaxRT = 2;
constexpr int kPfSmallWork = 35 * 256;           // 128-row workgroup chunks (about 35 per CU) up to which hd 64 takes 64-row tiles
constexpr long long kPfFewGroups = 512;           // workgroups (two per CU) up to which a 64-row tile takes eight waves (two halves of a 128-key trip)
constexpr int kPfChunk = 64;                     // keys a wave multiplies per trip (a trip stages KH chunks)
constexpr int kPfSeg = 512;                      // keys per segment: a multiple of this, chosen per launch
constexpr int kPfSegMax = 16384;                 // at most (its page ids lie in LDS)
constexpr long long kPfFill = 512;               // workgroups a launch should have before segments grow (two per CU)

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  union { bf16x2_t v; uint32_t u; } r;
  r.v = __builtin_convertvector(float2_t{a, b}, bf16x2_t);   // one v_cvt_pk_bf16_f32
  return r.u;
}
// all-reduce over the four lanes that share lane % 16 (lanes l, l^16, l^32, l^48)
__device__ __forceinline__ float quad_rows_max(float v) {
  // v_permlane16_swap / v_permlane32_swap with both operands the same register leave one half of
  // each lane pair in the first result and the other half in the second
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// Two waves per SIMD at least: with that bound the compiler keeps the accumulators of the matrix
// instructions in ordinary registers (no copies to and from the accumulation registers around the softmax).
// At head_dim 64 the kernel fits three (two tiles a wave: 168 registers) or four (one tile); the bound
// keeps it there, since one register more than 168 costs a third of the waves.
template <int HD, int RT, int KH>
__global__ void __launch_bounds__(kPfGroupThreads * KH, HD == 64 ? (RT == 1 ? 4 : 3) : 2)
    attention_prefill_kernel(const uint16_t* __restrict__ q, int q_stride, uint16_t* __restrict__ out, int out_stride,
                             const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                             const int* __restrict__ tables, int table_stride, const int* __restrict__ run_start,
                             const int* __restrict__ seq_start, int nh, int nkv, int B, int b_shift, float scale,
                             int seg_len, int max_segs, float* __restrict__ scratch, const float2* __restrict__ cos_sin) {
  constexpr int kPfRT = RT, kPfWaveRows = 16 * RT, kPfRows = kPfWaveRows * kPfWaves;   // tiles per wave, rows per wave and workgroup
  constexpr int KSTEPS = HD / 32;                          // matrix instructions per 16-token tile of scores
  constexpr int DT = HD / 16;                              // 16-dim tiles of the output
  constexpr int kPfThreads = kPfGroupThreads * KH, TRIP = kPfChunk * KH;   // threads, and keys staged per trip
  constexpr int PIECES = TRIP * HD / 8 / kPfThreads;       // 16-byte pieces of a trip per thread (keys; as many of values)
  // LDS rows are unpadded; the 16-byte columns of a row are permuted instead: column c of row r lies at
  // c ^ (r mod columns).  A wave's 16-byte reads (16 rows x 4 columns) then take the 8 cycles that 1 KiB
  // costs at 128 bytes a cycle; with rows padded by 16 bytes they took 12 (measured: 12.9 against 8.8
  // cycles per instruction and CU), and the counters showed 38 % of the LDS cycles as bank conflicts.
  constexpr int KPITCH = HD, VPITCH = TRIP;
  constexpr int KCOLS = HD / 8, VCOLS = TRIP / 8;   // 16-byte columns per row (the permutation uses the low three bits)
  // Workgroups are handed out in the order of blockIdx.x, round-robin over the chip's eight parts:
  // neighbours in that order are the heads of one (tile, segment), so that every part gets the
  // same mix of long and short walks.
  const int head = blockIdx.x % nh, seq = blockIdx.y;
  // The first half of the launch takes the longest walks, longest first, the second half the
  // shortest, shortest first: when two workgroups at a time fit a CU, a long walk shares it with a
  // short one and every CU gets about the same number of chunks (32 + 2, 30 + 4, ... for one prompt).
  const int n_units = gridDim.x / nh, turn = blockIdx.x / nh, top = (n_units + 1) / 2;
  const int unit = turn < top ? n_units - 1 - turn : turn - top;
  const int tile = unit / max_segs, seg = unit % max_segs;
  const int row0 = run_start[seq], n_rows = run_start[seq + 1] - row0;
  const int block_first = tile * kPfRows;
  if (block_first >= n_rows) return;
  const int wave_id = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int wave = wave_id % kPfWaves, half = wave_id / kPfWaves;   // row group, and which chunk of a trip
  const int n16 = lane % 16, kq = lane / 16;
  const int pos0 = seq_start[seq];
  const int kvh = head / (nh / nkv);
  const int* table = tables + size_t(seq) * table_stride;
  const size_t head_elems = size_t(B) * HD, page_elems = head_elems * nkv;
  const uint16_t* kbase = kcache + kvh * head_elems;
  const uint16_t* vbase = vcache + kvh * head_elems;
  const int tile_last_pos = pos0 + min(block_first + kPfRows, n_rows) - 1;
  const int seg_first = seg * seg_len;
  if (seg_first > tile_last_pos) return;
  const int n_segs = tile_last_pos / seg_len + 1;
  const int block_last_pos = min(tile_last_pos, seg_first + seg_len - 1);   // the last key this workgroup reads
  const int first = block_first + wave * kPfWaveRows;   // first row of this wave inside the run
  const bool wave_on = first < n_rows;
  const int wave_last_pos = pos0 + min(first + kPfWaveRows, n_rows) - 1;
  const int wave_first_pos = pos0 + min(first, n_rows - 1);
  const float scale_log2 = scale * 1.4426950408889634f;   // scores are kept in units of log2: exp(x) = exp2(x log2 e)
  const int b_mask = B - 1;

  // LDS: keys [2][TRIP][HD], values [2][HD][TRIP], then the sequence's page ids up to the workgroup's
  // last position (the address of a piece is one LDS read away instead of one more trip to global memory)
  extern __shared__ __attribute__((aligned(16))) unsigned char pf_lds[];
  uint16_t (*k_lds)[TRIP][KPITCH] = reinterpret_cast<uint16_t (*)[TRIP][KPITCH]>(pf_lds);
  uint16_t (*v_lds)[HD][VPITCH] = reinterpret_cast<uint16_t (*)[HD][VPITCH]>(pf_lds + sizeof(uint16_t) * 2 * TRIP * KPITCH);
  int* page_lds = reinterpret_cast<int*>(pf_lds + sizeof(uint16_t) * 4 * TRIP * HD);
  // Entries past the last page the workgroup may read repeat that page: a chunk's pieces beyond the
  // last position then come from valid memory without a clamp per piece (the mask keeps them out).
  const int page_lo = seg_first >> b_shift, page_hi = block_last_pos >> b_shift;
  const int page_slots = (((block_last_pos | (TRIP - 1)) >> b_shift) - page_lo) + 1;   // through the last trip's end
  for (int i = threadIdx.x; i < page_slots; i += kPfThreads) page_lds[i] = table[min(page_lo + i, page_hi)];

  // B operand of the scores: lane holds 8 dims of query row n16 of each tile (rows past the run
  // repeat its last row; they are never stored).  That row's position is what the lane may see.
  PFrag qf[kPfRT][KSTEPS];
  int pos[kPfRT];
#pragma unroll
  for (int rt = 0; rt < kPfRT; ++rt) {
    const int r = min(first + rt * 16 + n16, n_rows - 1);
    pos[rt] = pos0 + r;
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c)
      qf[rt][c].u = *reinterpret_cast<const uint4*>(q + size_t(row0 + r) * q_stride + size_t(head) * HD + c * 32 + kq * 8);
    if (cos_sin) {
      // q as the projection left it: rotated here by pairs (j, j + HD / 2), which one lane holds in its
      // fragments c and c + KSTEPS / 2, with the step's table of cos and sin ([row][HD / 2]), in 32-bit,
      // rounded to bfloat16 as the rotation kernel stores it
      const float2* tab = cos_sin + size_t(row0 + r) * (HD / 2) + kq * 8;
#pragma unroll
      for (int c = 0; c < KSTEPS / 2; ++c) {
        uint32_t* lo = reinterpret_cast<uint32_t*>(&qf[rt][c].u);
        uint32_t* hi = reinterpret_cast<uint32_t*>(&qf[rt][c + KSTEPS / 2].u);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float4 t2 = *reinterpret_cast<const float4*>(tab + c * 32 + 2 * w);   // cos, sin of two dims
          float a0 = bf16_bits_to_float(lo[w] & 0xFFFFu), a1 = bf16_bits_to_float(lo[w] >> 16);
          float b0 = bf16_bits_to_float(hi[w] & 0xFFFFu), b1 = bf16_bits_to_float(hi[w] >> 16);
          rotate_pair(a0, b0, t2.x, t2.y);
          rotate_pair(a1, b1, t2.z, t2.w);
          lo[w] = pack_bf16(a0, a1);
          hi[w] = pack_bf16(b0, b1);
        }
      }
    }
  }
  float m[kPfRT];
  f32x4 l[kPfRT];   // every element: the sum of the lane's query row (a product with a matrix of ones)
  PFrag ones;
  ones.u = uint4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  f32x4 o[kPfRT][DT];   // O^T: column = query row n16, rows = dims 16 d + 4 kq + i
#pragma unroll
  for (int rt = 0; rt < kPfRT; ++rt) {
    m[rt] = -FLT_MAX;
    l[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < DT; ++d) o[rt][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  __syncthreads();   // page_lds is filled

  // What this thread moves from the cache to LDS for a chunk that starts at token c0: PIECES
  // pieces of keys (8 dims of one token) and as many of values (8 tokens of one dim).  Tokens past
  // the workgroup's last position are read from that position's place instead (always valid
  // memory); the mask keeps them out.
  // A thread's key pieces are the same 8 dims of PIECES consecutive tokens (an aligned group, so one
  // page), its value pieces the same 8 tokens of dims 32 apart: one page lookup each per chunk, the
  // other pieces lie a constant away.
  struct Pieces { u32x4 k[PIECES], v[PIECES]; };
  constexpr int KTPR = HD / 8;   // threads per key row
  const int k_p = threadIdx.x / KTPR, k_col = threadIdx.x % KTPR;
  const int v_g = threadIdx.x % VCOLS, v_d = threadIdx.x / VCOLS;
  const int last_chunk = block_last_pos & ~(TRIP - 1);   // the last trip's first key
  const uint16_t* k_thread = kbase + k_col * 8;          // this thread's 8 dims of a key
  const uint16_t* v_thread = vbase + size_t(v_d) * B;    // this thread's first dim row of a page's values
  const int* pages = page_lds - page_lo;
  auto request = [&](int c0, Pieces& pc) {
    c0 = min(c0, last_chunk);   // past the last chunk: the last chunk again (no load behind a branch)
    const int tk = c0 + k_p * PIECES;
    const uint16_t* kp = k_thread + size_t(pages[tk >> b_shift]) * page_elems + size_t(tk & b_mask) * HD;
#pragma unroll
    for (int i = 0; i < PIECES; ++i) pc.k[i] = *reinterpret_cast<const u32x4*>(kp + i * HD);
    const int tv = c0 + v_g * 8;
    const uint16_t* vp = v_thread + size_t(pages[tv >> b_shift]) * page_elems + (tv & b_mask);
#pragma unroll
    for (int i = 0; i < PIECES; ++i) pc.v[i] = *reinterpret_cast<const u32x4*>(vp + size_t(i) * (kPfThreads / VCOLS) * B);
  };
  // c0: the chunk the pieces belong to.  Only in the workgroup's last chunk can value slots lie past
  // the last position; they hold stale data there, and probabilities of zero do not cancel a stale
  // Inf or NaN, so they are cut out.
  auto stage = [&](int buf, const Pieces& pc, int c0) {
    const bool tail = c0 >= last_chunk;                                // the same for every thread: a jump, no selects
    const int v_left = block_last_pos + 1 - (last_chunk + v_g * 8);    // n <= 0 keeps nothing, n >= 8 everything
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      *reinterpret_cast<u32x4*>(&k_lds[buf][k_p * PIECES + i][(k_col ^ ((k_p * PIECES + i) & (KCOLS - 1))) * 8]) = pc.k[i];
      // tokens 8 g .. 8 g + 7 of the chunk: inside their group of 32 tokens, token 16 a + 4 q + e goes to
      // place 8 q + 4 a + e, so that the 8 tokens a lane multiplies in one step lie together
      {
        const int r0 = (v_g * 8) % 32, grp = (v_g * 8) / 32;
        const int a = r0 / 16, q0 = (r0 % 16) / 4;
        uint16_t* row = &v_lds[buf][v_d + (kPfThreads / VCOLS) * i][4 * a];
        const int col = grp * 4 + q0, swz = v_d & 7;   // (v_d + rows-per-pass * i) mod 8
        uint4 piece{pc.v[i][0], pc.v[i][1], pc.v[i][2], pc.v[i][3]};
        if (tail) piece = keep_first_bf16(piece, v_left);
        *reinterpret_cast<uint2*>(row + 8 * (col ^ swz)) = uint2{piece.x, piece.y};
        *reinterpret_cast<uint2*>(row + 8 * ((col + 1) ^ swz)) = uint2{piece.z, piece.w};
      }
    }
  };

  auto compute = [&](int t0, int buf) {
    const int c0 = t0 + half * kPfChunk;   // this wave's chunk of the trip
    if (wave_on && c0 <= wave_last_pos && c0 <= block_last_pos) {
      // ---- S^T: s[rt][j][i] = k[token c0 + 16 j + 4 kq + i] . q[row n16 of tile rt]
      f32x4 s[kPfRT][4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        PFrag kf[KSTEPS];
#pragma unroll
        for (int c = 0; c < KSTEPS; ++c)
          kf[c].u = *reinterpret_cast<const uint4*>(&k_lds[buf][half * kPfChunk + j * 16 + n16][((c * 4 + kq) ^ (n16 & (KCOLS - 1))) * 8]);
#pragma unroll
        for (int rt = 0; rt < kPfRT; ++rt) {
          s[rt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KSTEPS; ++c)
            s[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[c].v, qf[rt][c].v, s[rt][j], 0, 0, 0);
        }
      }
      // ---- running maximum and sum of the lane's query row; probabilities stay in registers.
      // Scores stay raw: the scale (in units of log2) goes into the exponent's multiply-add, the
      // maximum is taken of raw scores (the scale is positive).  Only a chunk that some row of the
      // wave cannot see completely is masked.
      const bool diagonal = c0 + kPfChunk - 1 > wave_first_pos;
      PFrag pf[kPfRT][2];   // B operands of the two 32-token steps
#pragma unroll
      for (int rt = 0; rt < kPfRT; ++rt) {
        float mx = -FLT_MAX;
        if (diagonal) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int t = c0 + j * 16 + 4 * kq + i;
              s[rt][j][i] = t <= pos[rt] ? s[rt][j][i] : -FLT_MAX;
              mx = fmaxf(mx, s[rt][j][i]);
            }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[rt][j][i]);
        }
        mx = quad_rows_max(mx);
        // m is finite once the row has seen a key; a row that starts before this segment's first
        // key has seen none of it yet (m_new = -FLT_MAX): its probabilities are zero
        const float m_new = fmaxf(m[rt], mx);
        const bool seen = m_new > -0.5f * FLT_MAX;
        const float shift = seen ? -m_new * scale_log2 : -FLT_MAX;       // exp2(s * scale + shift)
        const float alpha = seen ? __builtin_amdgcn_exp2f((m[rt] - m_new) * scale_log2) : 1.0f;
        m[rt] = m_new;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i)   // masked scores are -FLT_MAX: the product overflows to -inf, exp2 gives 0
            s[rt][j][i] = __builtin_amdgcn_exp2f(fmaf(s[rt][j][i], scale_log2, shift));
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {   // the maximum moves in few chunks
#pragma unroll
          for (int i = 0; i < 4; ++i) l[rt][i] *= alpha;
#pragma unroll
          for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[rt][d][i] *= alpha;
        }
        // step c covers tiles 2c and 2c+1: reduction index e < 4 -> token 16(2c) + 4kq + e, e >= 4 -> 16(2c+1) + 4kq + e-4
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          pf[rt][c].u.x = pack_bf16(s[rt][2 * c][0], s[rt][2 * c][1]);
          pf[rt][c].u.y = pack_bf16(s[rt][2 * c][2], s[rt][2 * c][3]);
          pf[rt][c].u.z = pack_bf16(s[rt][2 * c + 1][0], s[rt][2 * c + 1][1]);
          pf[rt][c].u.w = pack_bf16(s[rt][2 * c + 1][2], s[rt][2 * c + 1][3]);
        }
      }
      // ---- the rows' sums, of the probabilities as the product below sees them: ones * P^T
#pragma unroll
      for (int rt = 0; rt < kPfRT; ++rt)
#pragma unroll
        for (int c = 0; c < 2; ++c) l[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pf[rt][c].v, l[rt], 0, 0, 0);
      // ---- O^T += V^T * P^T, values read in the same token order
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int d = 0; d < DT; ++d) {
          PFrag vf;
          vf.u = *reinterpret_cast<const uint4*>(&v_lds[buf][d * 16 + n16][((half * 8 + c * 4 + kq) ^ (n16 & 7)) * 8]);
#pragma unroll
          for (int rt = 0; rt < kPfRT; ++rt) o[rt][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[rt][c].v, o[rt][d], 0, 0, 0);
        }
    }
  };

  // Two chunks are on their way from the cache while one is multiplied: chunk i+1 sits in
  // registers (asked for one trip earlier) and goes to the other LDS buffer after the products,
  // chunk i+2 is asked for before them.
  {
    Pieces pa, pb;
    request(seg_first, pa);
    request(seg_first + TRIP, pb);
    stage(0, pa, seg_first);
    __syncthreads();
    for (int t0 = seg_first; t0 <= block_last_pos; t0 += 2 * TRIP) {
      request(t0 + 2 * TRIP, pa);
      compute(t0, 0);
      stage(1, pb, t0 + TRIP);
      __syncthreads();
      if (t0 + TRIP > block_last_pos) break;
      request(t0 + 3 * TRIP, pb);
      compute(t0 + TRIP, 1);
      stage(0, pa, t0 + 2 * TRIP);
      __syncthreads();
    }
  }

  if constexpr (KH == 2) {
    // The waves of the second half hand what their rows have gathered (output, maximum, sum) to the
    // waves of the first half through LDS (every wave has passed the loop's last barrier: the staging
    // buffers are free), lane to lane: both halves hold a row's numbers in the same lanes.
    float* hand = reinterpret_cast<float*>(pf_lds);
    constexpr int ITEMS = DT * 4 + 2;   // per tile of a wave
    auto slot = [&](int rt, int item) { return hand + ((rt * ITEMS + item) * kPfWaves + wave) * kWave + lane; };
    if (half == 1 && wave_on) {
#pragma unroll
      for (int rt = 0; rt < kPfRT; ++rt) {
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
          for (int i = 0; i < 4; ++i) *slot(rt, d * 4 + i) = o[rt][d][i];
        *slot(rt, DT * 4) = m[rt];
        *slot(rt, DT * 4 + 1) = l[rt][0];
      }
    }
    __syncthreads();
    if (half == 1) return;
    if (wave_on) {
#pragma unroll
      for (int rt = 0; rt < kPfRT; ++rt) {
        const float m1 = *slot(rt, DT * 4), l1 = *slot(rt, DT * 4 + 1);
        const float m_all = fmaxf(m[rt], m1);
        // a half that has seen no key (maximum -FLT_MAX, sum 0) gets weight 0
        const float w0 = m[rt] > -0.5f * FLT_MAX ? __builtin_amdgcn_exp2f((m[rt] - m_all) * scale_log2) : 0.f;
        const float w1 = m1 > -0.5f * FLT_MAX ? __builtin_amdgcn_exp2f((m1 - m_all) * scale_log2) : 0.f;
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[rt][d][i] = w0 * o[rt][d][i] + w1 * *slot(rt, d * 4 + i);
        l[rt][0] = w0 * l[rt][0] + w1 * l1;
        m[rt] = m_all;
      }
    }
  }

  if (!wave_on) return;
#pragma unroll
  for (int rt = 0; rt < kPfRT; ++rt) {
    const int r = first + rt * 16 + n16;
    const float l_row = l[rt][0];
    if (r >= n_rows) continue;
    const float inv = l_row > 0.f ? 1.0f / l_row : 0.f;
    if (n_segs == 1) {
      uint16_t* orow = out + size_t(row0 + r) * out_stride + size_t(head) * HD + 4 * kq;
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        uint2 v;
        v.x = pack_bf16(o[rt][d][0] * inv, o[rt][d][1] * inv);
        v.y = pack_bf16(o[rt][d][2] * inv, o[rt][d][3] * inv);
        *reinterpret_cast<uint2*>(orow + d * 16) = v;
      }
    } else {   // this segment's share of the row: o / l, then m (in units of log2) and l
      float* dst = scratch + ((size_t(row0 + r) * nh + head) * max_segs + seg) * (HD + 4);
#pragma unroll
      for (int d = 0; d < DT; ++d)
        *reinterpret_cast<float4*>(dst + d * 16 + 4 * kq) =
            float4{o[rt][d][0] * inv, o[rt][d][1] * inv, o[rt][d][2] * inv, o[rt][d][3] * inv};
      if (kq == 0) { dst[HD] = m[rt] > -0.5f * FLT_MAX ? m[rt] * scale_log2 : -FLT_MAX; dst[HD + 1] = l_row; }
    }
  }
}

// Rows whose tile was cut into several segments: out = sum_s w_s o_s / sum_s w_s with
// w_s = l_s 2^(m_s - m), segments in order.  HD / 4 threads per row, four dims each.
template <int HD>
__global__ void __launch_bounds__(256)
    attention_prefill_merge_kernel(const float* __restrict__ scratch, uint16_t* __restrict__ out, int out_stride,
                                   const int* __restrict__ run_start, const int* __restrict__ seq_start, int nh,
                                   int seg_len, int max_segs, int tile_rows) {
  const int seq = blockIdx.y, head = blockIdx.z;
  const int row0 = run_start[seq], n_rows = run_start[seq + 1] - row0;
  constexpr int PER_ROW = HD / 4;
  const int r = blockIdx.x * (256 / PER_ROW) + threadIdx.x / PER_ROW, piece = threadIdx.x % PER_ROW;
  if (r >= n_rows) return;
  const int tile = r / tile_rows;
  const int tile_last_pos = seq_start[seq] + min((tile + 1) * tile_rows, n_rows) - 1;
  const int n_segs = tile_last_pos / seg_len + 1;
  if (n_segs == 1) return;   // stored directly
  const float* base = scratch + (size_t(row0 + r) * nh + head) * max_segs * (HD + 4);
  float m = -FLT_MAX;
  for (int s = 0; s < n_segs; ++s) m = fmaxf(m, base[s * (HD + 4) + HD]);
  float4 num = {0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  for (int s = 0; s < n_segs; ++s) {
    const float* p = base + s * (HD + 4);
    const float l = p[HD + 1];
    const float w = l > 0.f ? l * __builtin_amdgcn_exp2f(p[HD] - m) : 0.f;
    const float4 o = *reinterpret_cast<const float4*>(p + piece * 4);
    num.x = fmaf(w, o.x, num.x); num.y = fmaf(w, o.y, num.y); num.z = fmaf(w, o.z, num.z); num.w = fmaf(w, o.w, num.w);
    den += w;
  }
  const float inv = 1.0f / den;
  uint2 v;
  v.x = pack_bf16(num.x * inv, num.y * inv);
  v.y = pack_bf16(num.z * inv, num.w * inv);
  *reinterpret_cast<uint2*>(out + size_t(row0 + r) * out_stride + size_t(head) * HD + piece * 4) = v;
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_attention_prefill_supported(int nh, int nkv, int hd, int B) {
  return nkv > 0 && nh % nkv == 0 && (hd == 64 || hd == 128) && B >= 8 && (B & (B - 1)) == 0;
}

// How a launch is cut: query rows per workgroup and keys per segment.  Rows: 128, or 64 at head_dim 64
// when the launch is small (T rows that see about max_context - max_run / 2 keys each, counted in
// chunks of 128-row workgroups).  Keys per segment: 512 while that gives the chip fewer than kPfFill
// workgroups, longer (in multiples of 512) when tiles x heads x sequences already fill it, since
// every segment beyond the first costs a partial result per row and head in scratch.
struct PfPlan { int tile_rows, seg_len, halves; };
static PfPlan pf_plan(int T, int nh, int hd, int max_context, int max_run, int S) {
  PfPlan p{64 * kPfMaxRT, kPfSeg, 1};
  if (max_run <= 0 || S <= 0 || nh <= 0 || max_context <= 0) return p;
  if (T < max_run) T = max_run;
  const double seen = max_context - 0.5 * max_run > 64.0 ? max_context - 0.5 * max_run : 64.0;
  const double work = double(T) / 128.0 * (seen / kPfChunk) * nh;
  if (hd == 64 && work <= kPfSmallWork) p.tile_rows = 64;

  const long long base = static_cast<long long>((max_run + p.tile_rows - 1) / p.tile_rows) * nh * S;
  if (hd == 64 && p.tile_rows == 64 && base <= kPfFewGroups) p.halves = 2;
  const long long want = (kPfFill + base - 1) / base;
  long long len = (max_context + want - 1) / want;
  len = (len + kPfSeg - 1) / kPfSeg * kPfSeg;
  p.seg_len = static_cast<int>(len < kPfSeg ? kPfSeg : len > kPfSegMax ? kPfSegMax : len);
  return p;
}

// Keys per segment that a launch of these sizes cuts contexts into (T: rows in all).
int kvcm_attention_prefill_segment(int T, int nh, int hd, int max_context, int max_run, int S) {
  return pf_plan(T, nh, hd, max_context, max_run, S).seg_len;
}

// Query rows per workgroup of such a launch.
int kvcm_attention_prefill_tile_rows(int T, int nh, int hd, int max_context, int max_run, int S) {
  return pf_plan(T, nh, hd, max_context, max_run, S).tile_rows;
}

// Floats of scratch a launch needs: none while no row's context exceeds one segment.
long long kvcm_attention_prefill_scratch(int T, int nh, int hd, int max_context, int max_run, int S) {
  const int seg_len = pf_plan(T, nh, hd, max_context, max_run, S).seg_len;
  const long long segs = (max_context + seg_len - 1) / seg_len;
  return segs <= 1 ? 0 : static_cast<long long>(T) * nh * segs * (hd + 4);
}

// run_start [S+1]: first row of each sequence's run of consecutive positions (rows of a run are
// consecutive); seq_start [S]: position of a run's first row; tables [S][table_stride];
// max_run: the longest run (it sizes the launch); T: rows in all (run_start[S]); max_context: an
// upper bound of every row's context length (position + 1); scratch: see above; cos_sin: null when q is
// rotated already, else the step's table [T][hd / 2][2] (cos, sin) that q is rotated with as it is read.
int kvcm_attention_prefill(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                           const void* vcache, const int* tables, int table_stride, const int* run_start,
                           const int* seq_start, int S, int max_run, int T, int max_context, int nh, int nkv, int hd,
                           int B, float scale, float* scratch, long long scratch_floats, const float* cos_sin, hipStream_t s) {
  if (S == 0 || max_run == 0) return 0;
  KVCM_REQUIRE(kvcm_attention_prefill_supported(nh, nkv, hd, B),
               "attention_prefill: unsupported shape heads=%d kv_heads=%d head_dim=%d page=%d", nh, nkv, hd, B);
  KVCM_REQUIRE(S > 0 && max_run > 0 && S <= 65535 && nh <= 65535 && T >= max_run && max_context >= 1,
               "attention_prefill: bad sizes S=%d max_run=%d T=%d max_context=%d", S, max_run, T, max_context);
  KVCM_REQUIRE(scale > 0.f, "attention_prefill: the scale must be positive");
  KVCM_REQUIRE(q_stride >= nh * hd && out_stride >= nh * hd && q_stride % 8 == 0, "attention_prefill: bad row strides");
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(kcache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(vcache) % 16 == 0, "attention_prefill: operands must be 16-byte aligned");
  KVCM_REQUIRE(out_stride % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0, "attention_prefill: output must be 8-byte aligned");
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(cos_sin) % 16 == 0, "attention_prefill: the table of cos and sin must be 16-byte aligned");
  const PfPlan plan = pf_plan(T, nh, hd, max_context, max_run, S);
  const int seg_len = plan.seg_len;
  const int max_segs = (max_context + seg_len - 1) / seg_len;
  const long long need = kvcm_attention_prefill_scratch(T, nh, hd, max_context, max_run, S);
  KVCM_REQUIRE(need == 0 || (scratch && scratch_floats >= need && reinterpret_cast<uintptr_t>(scratch) % 16 == 0),
               "attention_prefill: scratch too small (%lld floats needed)", need);
  int b_shift = 0;
  while ((1 << b_shift) < B) ++b_shift;
  const long long units = static_cast<long long>((max_run + plan.tile_rows - 1) / plan.tile_rows) * max_segs * nh;
  KVCM_REQUIRE(units < (1ll << 31), "attention_prefill: too many workgroups");
  const dim3 grid(static_cast<unsigned>(units), S, 1);
  const uint16_t *qq = static_cast<const uint16_t*>(q), *kc = static_cast<const uint16_t*>(kcache),
                 *vc = static_cast<const uint16_t*>(vcache);
  const int merge_rows = 256 / (hd / 4);   // rows per workgroup of the merge
  const dim3 mgrid((max_run + merge_rows - 1) / merge_rows, S, nh);
  // LDS of a workgroup: two buffers of a trip's keys and values, and the page ids of one segment
#define KVCM_PF(HD, RT, KH)                                                                                                  \
  do {                                                                                                                       \
    const size_t lds = size_t(8) * kPfChunk * KH * HD + sizeof(int) * size_t(seg_len / B + 2);                              \
    static bool raised = false; /* a kernel may use more than 64 KiB of LDS once it has been told so */                    \
    if (lds > 65536 && !raised) {                                                                                            \
      KVCM_REQUIRE(hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<HD, RT, KH>),                 \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess,               \
                   "attention_prefill: the kernel may not use %zu bytes of LDS", lds);                                       \
      raised = true;                                                                                                         \
    }                                                                                                                        \
    attention_prefill_kernel<HD, RT, KH><<<grid, kPfGroupThreads * KH, lds, s>>>(                                            \
        qq, q_stride, static_cast<uint16_t*>(out), out_stride, kc, vc, tables, table_stride, run_start, seq_start, nh, nkv, \
        B, b_shift, scale, seg_len, max_segs, scratch, reinterpret_cast<const float2*>(cos_sin));                            \
  } while (0)
  if (hd == 64 && plan.tile_rows == 64 && plan.halves == 2) KVCM_PF(64, 1, 2);
  else if (hd == 64 && plan.tile_rows == 64) KVCM_PF(64, 1, 1);
  else if (hd == 64) KVCM_PF(64, 2, 1);
  else KVCM_PF(128, 2, 1);
#undef KVCM_PF
  if (max_segs > 1) {
    if (hd == 64)
      attention_prefill_merge_kernel<64><<<mgrid, 256, 0, s>>>(scratch, static_cast<uint16_t*>(out), out_stride, run_start,
                                                              seq_start, nh, seg_len, max_segs, plan.tile_rows);
    else
      attention_prefill_merge_kernel<128><<<mgrid, 256, 0, s>>>(scratch, static_cast<uint16_t*>(out), out_stride, run_start,
                                                               seq_start, nh, seg_len, max_segs, plan.tile_rows);
  }
  return launch_status("attention_prefill");
}

}  // extern "C"
