// C entry points of libkvcm_hip.so.  Every entry that launches returns 0 on success and a negative
// value on failure; kvcm_hip_last_error() then holds the reason (per calling thread).  Pointers are
// device pointers unless said otherwise; `*_dtype` arguments are KVCM_F32 or KVCM_BF16.  An entry
// checks on the host that sizes fit what its kernel assumes and launches nothing when they do not.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* kvcm_hip_last_error();

// Storage types of the `*_dtype` arguments.
enum { KVCM_F32 = 0, KVCM_BF16 = 1 };

// ---- decode-shaped products: out[M, N] = X[M, K] * W[N, K]^T, bfloat16 operands -------------
// How many slices of K a launch of this shape is cut into (0: the kernel does not take the shape).
int kvcm_gemm_skinny_splits(int M, int N, int K);

// S == 1 stores the result to `out`; S > 1 writes 32-bit partial sums [S][M][N] to `partials`,
// which the caller owns, and leaves `out` alone (kvcm_reduce_store adds them up).
int kvcm_gemm_skinny(const void* X, const void* W, float* partials, void* out, int out_dtype, int M, int N, int K,
                     int ldx, int ldw, int ldo, int S, hipStream_t stream);
int kvcm_reduce_store(const float* partials, void* out, int out_dtype, int M, int N, int ldo, int S, hipStream_t stream);
// Waves per workgroup of the shared-rows kernel for a bfloat16 product of this shape (0: another kernel takes it):
// chosen so that column tiles x splits x row blocks come to about one workgroup per CU.
int kvcm_gemm_skinny_waves(int M, int N, int K, int S, int swiglu);
// act = swiglu(rstd * (xg * [gate | up]^T)) for the rows xg and tile sums ss_in that a folded norm's producer left
// (kvcm_gemm8_residual_norm), by the shared-rows kernel; `preferred`: the widths at which it beats kvcm_gemm8.
int kvcm_gemm_skinny_swiglu_normed_preferred(int M, int I, int K);
int kvcm_gemm_skinny_swiglu_normed(const void* X, const void* W, const float* ss_in, int tiles_in, float eps, void* out,
                                   int M, int I, int K, int ldx, int ldw, int ldo, hipStream_t stream);

// The same product, whole (split where kvcm_gemm_skinny_splits says so, partial sums added up in
// split order, result in `out`), for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
// the reference, whose products go to cuBLAS with a workspace the library allocates.  The partial
// sums live in an array that is part of the library's device image instead of a buffer the caller
// brings; the call allocates nothing, on the host or on the device.
//
//   Limit: splits * M * N <= kvcm_gemm_skinny_noalloc_capacity() floats (2 Mi floats = 8 MiB,
//          held on every GPU the library runs on until the process ends); larger products are
//          refused with an error, nothing is launched.
//   Sharing: every call on a GPU uses that GPU's one array.  Two calls whose kernels may overlap
//          on one GPU (different streams, or different threads without ordering between their
//          streams) race on it; calls on one stream are ordered and safe.  Nothing in the array has
//          to start at zero: a call writes every partial sum it later reads.
//   The first call on a device looks the array's address up (no allocation either); do that
//          before a capture begins if the caller captures.
long long kvcm_gemm_skinny_noalloc_capacity();
int kvcm_gemm_skinny_noalloc(const void* X, const void* W, void* out, int out_dtype, int M, int N, int K, int ldx,
                             int ldw, int ldo, hipStream_t stream);

// ---- row-wise kernels (elementwise.hip) ------------------------------------------------------
int kvcm_embed(const int* ids, const void* table, int table_dtype, float* x, int T, int H, int V, hipStream_t s);
int kvcm_rmsnorm(float* x, const void* add, int add_dtype, const float* partials, int S, int T, const int* rows,
                 const void* w, int w_dtype, void* out, int out_dtype, int R, int H, float eps, int write_back,
                 hipStream_t s);
int kvcm_rope_cache(void* qkv, int dtype, int row_stride, const int* positions, const float* inv_freq, const int* slots,
                    void* kcache, void* vcache, int T, int nh, int nkv, int hd, int B, const float* partials, int S,
                    const float* cos_sin, int skip_q, hipStream_t s);
int kvcm_rope_table(const int* positions, const float* inv_freq, float* cos_sin, int T, int half, hipStream_t s);
int kvcm_swiglu(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t s);
int kvcm_add_residual(float* x, const void* y, int dtype, long long n, hipStream_t s);

// ---- products --------------------------------------------------------------------------------
int kvcm_gemm_skinny_swiglu_supported(int M, int I, int K);
int kvcm_gemm_skinny_swiglu(const void* X, const void* W, void* out, int out_dtype, int M, int I, int K, int ldx,
                            int ldw, int ldo, hipStream_t stream);
int kvcm_gemm_f32(const float* X, const float* W, float* Y, int M, int N, int K, int ldx, int ldw, int ldy, hipStream_t s);
int kvcm_gemm_bf16(const void* X, const void* W, void* Y, int out_dtype, int M, int N, int K, int ldx, int ldw, int ldy,
                   hipStream_t s);
// Products of at most 8 rows with the RMS norm around them folded in (gemm_rows8.hip).
int kvcm_gemm8_supported(int M, int N, int K);
int kvcm_gemm8(const void* X, int ldx, const void* W, int ldw, int M, int N, int K, const float* ss_in, int tiles_in,
               float eps, void* out, int out_dtype, int ldo, int swiglu, hipStream_t stream);
int kvcm_gemm8_residual_norm(const void* X, int ldx, const void* W, int ldw, int M, int N, int K, float* resid,
                             const void* g, int g_dtype, void* xg, float* ss_out, hipStream_t stream);
// The vendor library's product (hipBLASLt), bfloat16 operands and result, 32-bit accumulation, for
// the many-row products of prompt steps, where the reference calls cuBLAS (src/model/llama.cpp:45-52).
// `workspace` is device memory the caller owns (at least kvcm_gemm_library_workspace_bytes()).
long long kvcm_gemm_library_workspace_bytes();
int kvcm_gemm_library(const void* X, const void* W, void* out, int M, int N, int K, int ldx, int ldw, int ldo,
                      void* workspace, long long workspace_bytes, hipStream_t stream);
// Which algorithm of the library a shape runs: the heuristic's first choice until this has timed
// candidates on the shape's own operands (mode 1: the heuristic's choices, a few milliseconds; mode 2:
// every algorithm that supports the shape, at most max_seconds) and kept the fastest whose result
// agrees with the first choice's.  W: w_copies copies of the weights, w_copy_bytes apart, which timed
// calls go round (enough of them keep the weights out of the caches, as in a model of many layers).
// `check`: M * N bfloat16 + 8 bytes of device memory; `report` (host, may be null): microseconds of the
// first choice, of the kept one, candidates timed.  Synchronises the stream.
int kvcm_gemm_library_tuned(int M, int N, int K, int ldx, int ldw, int ldo);
int kvcm_gemm_library_tune(const void* X, const void* W, int w_copies, long long w_copy_bytes, void* out, int M, int N, int K,
                           int ldx, int ldw, int ldo, void* workspace, long long workspace_bytes, void* check, int mode,
                           double max_seconds, double* report, hipStream_t stream);

// ---- attention over the paged cache ----------------------------------------------------------
int kvcm_attention_generic(const void* q, int dtype, int q_stride, void* out, int out_stride, const void* kcache,
                           const void* vcache, const int* tables, int table_stride, const int* row_seq,
                           const int* ctx_lens, int T, int nh, int nkv, int hd, int B, float scale, int window,
                           hipStream_t s);
int kvcm_attention_decode(const void* q, int q_stride, void* out, int out_stride, const void* kcache, const void* vcache,
                          const int* tables, int table_stride, const int* row_seq, const int* ctx_lens, int T, int nh,
                          int nkv, int hd, int B, float scale, int max_context, float* scratch, long long scratch_floats,
                          hipStream_t s);
int kvcm_attention_decode_fused(const float* partials, int S, const void* qkv, int qkv_stride, const float* cos_sin,
                                const int* slots, void* kcache, void* vcache, const int* tables, int table_stride,
                                const int* row_seq, const int* ctx_lens, int T, int nh, int nkv, int hd, int B, float scale,
                                void* out, int out_stride, int max_context, float* scratch, long long scratch_floats,
                                hipStream_t s);
int kvcm_attention_prefill(const void* q, int q_stride, void* out, int out_stride, const void* kcache, const void* vcache,
                           const int* tables, int table_stride, const int* run_start, const int* seq_start, int S,
                           int max_run, int T, int max_context, int nh, int nkv, int hd, int B, float scale,
                           float* scratch, long long scratch_floats, const float* cos_sin, hipStream_t s);

// ---- sampling ---------------------------------------------------------------------------------
int kvcm_sample(const float* logits, int ld, const float* temperature, const uint64_t* seeds, const long long* request_ids,
                const int* token_index, int* out, int R, int V, hipStream_t s);

// ---- random weights (fill_normal.hip) ------------------------------------------------------------
// out[i] = mean + std * n(key, i), n standard normal by a counter-based rule that the host evaluates
// the same way; integer tables: a counter-based value mod `modulus`.
int kvcm_fill_normal(void* out, int dtype, long long n, uint64_t key, float mean, float std, hipStream_t s);
int kvcm_fill_index(int* out, long long n, uint64_t key, int modulus, hipStream_t s);

// ---- probes of the machine (probe.hip) -----------------------------------------------------------
int kvcm_probe_empty(int grid, int block, hipStream_t s);
int kvcm_probe_copy(const void* src, void* dst, long long bytes, int grid, hipStream_t s);      // moves 2 * bytes
int kvcm_probe_read(const void* src, long long bytes, void* sink, int grid, hipStream_t s);
// the same, every workgroup (of `waves` waves) reading a contiguous share with `inflight` 16-byte loads per lane on their way
int kvcm_probe_stream(const void* src, long long bytes, void* sink, int grid, int waves, int inflight, hipStream_t s);
int kvcm_probe_mfma(int iters, void* sink, int grid, hipStream_t s);   // grid * 4 waves * iters * 4 * 32768 flops
// What it costs workgroups of one launch to depend on one another (every wait inside is bounded: flags[0] counts
// workgroups that gave up, flags[1] wrong values): a barrier across G workgroups, `rounds` times; S sums per tile
// added by the tile's last workgroup to arrive, or by a second launch; a step of layers x phases as one launch of
// dependent phases, or as one launch per phase.
int kvcm_probe_barrier(float* data, unsigned* counter, unsigned* flags, int G, int rounds, int spin_cap, int fences, int awaited, hipStream_t s);
int kvcm_probe_sums(float* partials, unsigned* counters, float* out, int S, int tiles, int last_arriver, unsigned* flags, hipStream_t s);
int kvcm_probe_phases(const void* weights, const long long* phase_bytes, int phases, int layers, int persistent, int G,
                      unsigned* counters, float* act, unsigned* flags, void* sink, int spin_cap, hipStream_t s);

// ---- recorded steps ---------------------------------------------------------------------------
// A step program is the list of launches of one step, recorded once for a step shape and replayed
// with nothing but the step's metadata changed (the kernels read that from device memory).  The
// reference issues every launch of every step from its C++ step function
// (src/model/llama.cpp:54-141); here the parts that decide the launches are assembled per model,
// so the list is recorded while they run once and replayed natively afterwards.
//   `entry`  name of one of the launching entries above (the last argument of each is the stream);
//   `args`   the entry's arguments, one 64-bit slot each: pointers and integers as they are, a float
//            as its 32 bits in the low half; the stream's slot is ignored (a replay brings its own).
void* kvcm_program_new();
void kvcm_program_delete(void* program);
int kvcm_program_add(void* program, const char* entry, const uint64_t* args, int num_args);
int kvcm_program_size(void* program);
int kvcm_program_run(void* program, hipStream_t stream);


// ---- the engine's step loop (native_engine.hip) ---------------------------------------------------
// The reference's Engine (src/engine/engine.h:29-52: add, step, idle, take_finished) as an object a native
// caller holds.  It is made over a host core (scheduler, cache manager, batch builder: libkvcm_host.so,
// reached through the addresses of nine of its C functions: kvcm_sched_schedule_summary,
// kvcm_build_batch_from_plan_shaped, kvcm_sched_update_sampled, kvcm_last_error, kvcm_sched_add,
// kvcm_sched_idle, kvcm_sched_collect_finished, kvcm_finished_get, kvcm_finished_clear), the pinned and the
// device metadata buffers of the model's step function, the sampler's device and pinned id buffers, the
// engine's limits and a stream of its own.  A step runs here from schedule to update when its canonical
// shape has a recorded program (kvcm_program_*); the first step of a shape is recorded by whoever holds the
// model's parts (they decide the launches), and handed over with kvcm_engine_register.
void* kvcm_engine_new(void* core, const uint64_t* host_functions, int32_t* meta_host, int32_t* meta_dev, long long meta_ints,
                      int32_t* sampled_dev, int32_t* sampled_host, int max_sampled, int num_groups, int block_size,
                      int max_context, int max_tokens, int max_seqs, int max_logit_rows, int graph_rows, hipStream_t stream);
void kvcm_engine_delete(void* engine);
int kvcm_engine_add(void* engine, long long id, const int32_t* tokens, int n, int max_new_tokens, float temperature,
                    uint64_t sampler_seed, double arrival);
int kvcm_engine_idle(void* engine);
// 1: a step ran; 2: nothing was planned; 0: the planned step's shape has no program yet (record and register it).
int kvcm_engine_step(void* engine, double now, int64_t* info);
int kvcm_engine_take_finished(void* engine);
int kvcm_engine_finished_get(void* engine, int i, int64_t* info, double* times, int32_t* tokens, int cap);
void kvcm_engine_finished_clear(void* engine);
// The two halves of kvcm_engine_step, for callers that look at the plan first (out: 20 values, see
// native_engine.hip) or keep the scheduler's update to themselves (defer_update: teacher forcing).
int kvcm_engine_plan(void* engine, double now, int64_t* out);
int kvcm_engine_last_plan(void* engine, int64_t* out);      // the same report again, the scheduler not run
int kvcm_engine_run(void* engine, double now, int defer_update, int64_t* info);
int kvcm_engine_register(void* engine, void* program, int as_graph);
void kvcm_engine_stats(void* engine, int64_t* out);

#ifdef __cplusplus
}
#endif
