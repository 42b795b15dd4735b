// C entry points of libkvcm_hip.so that programs other than this package's Python layer call.
// Every entry returns 0 on success and a negative value on failure; kvcm_hip_last_error() then
// holds the reason (per calling thread).  Pointers are device pointers unless said otherwise.
#pragma once
#include <hip/hip_runtime.h>

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

#ifdef __cplusplus
}
#endif
