// The vendor library's matrix product for prompt steps: out[M, N] = X[M, K] * W[N, K]^T, bfloat16
// operands and result, 32-bit accumulation, through hipBLASLt.  The reference hands all its
// products to cuBLAS the same way (src/model/llama.cpp:45-52).  Called directly instead of through
// a tensor library so that the call is an ordinary launching entry of this library: a few
// microseconds of host time, and recordable into a step program.
//
// hipBLASLt is column-major: the row-major out[M, N] is the column-major [N, M] = W (as stored:
// column-major [K, N], transposed) times X (as stored: column-major [K, M]).  A plan (descriptors
// and an algorithm) is made once per shape and kept.  The algorithm is the first choice of the
// library's heuristic until kvcm_gemm_library_tune has timed candidates on the shape's own operands.
// Measured with the library that the tensor framework brings along (the one a process of this engine
// loads), at M = 2,048 and TinyLlama widths, weights from memory: the first choice 31.5 / 26.2 / 93.3 /
// 58.0 us for the four products of a layer, the fastest of the heuristic's 16 choices 30.2 / 24.4 / 87.7 /
// 56.6 us; timing all 246 algorithms that support such a shape there found nothing faster.
#include <hipblaslt/hipblaslt-ext.hpp>
#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"
#include "kvcm_hip.h"

namespace {

constexpr long long kWorkspaceBytes = 64ll << 20;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  int tuned = 0;                                        // the widest search this shape has had (0 none, 1 heuristic's choices, 2 all)
  std::vector<hipblasLtMatmulHeuristicResult_t> choices;   // what the heuristic offered, in its order
};

std::mutex g_lock;
hipblasLtHandle_t g_handle = nullptr;
std::map<std::tuple<int, int, int, int, int, int>, Plan> g_plans;

const char* status_name(hipblasStatus_t s) {
  switch (s) {
    case HIPBLAS_STATUS_SUCCESS: return "success";
    case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialized";
    case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
    case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
    case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
    case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
    default: return "error";
  }
}

#define KVCM_BLAS(call)                                                              \
  do {                                                                               \
    const hipblasStatus_t st_ = (call);                                              \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                                             \
      kvcm::set_error("gemm_library: %s: %s", #call, status_name(st_));              \
      return -2;                                                                     \
    }                                                                                \
  } while (0)

int make_plan(Plan& p, int M, int N, int K, int ldx, int ldw, int ldo) {
  KVCM_BLAS(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  KVCM_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
  KVCM_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
  KVCM_BLAS(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, ldw));   // W as stored, seen column-major
  KVCM_BLAS(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, ldx));   // X as stored, seen column-major
  KVCM_BLAS(hipblasLtMatrixLayoutCreate(&p.c, HIP_R_16BF, N, M, ldo));   // the result, seen column-major
  hipblasLtMatmulPreference_t pref = nullptr;
  KVCM_BLAS(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t cap = kWorkspaceBytes;
  hipblasStatus_t st = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap));
  hipblasLtMatmulHeuristicResult_t found[16];
  int n = 0;
  if (st == HIPBLAS_STATUS_SUCCESS)
    st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, 16, found, &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || n <= 0) {
    kvcm::set_error("gemm_library: the library has no algorithm for M=%d N=%d K=%d (%s)", M, N, K, status_name(st));
    return -2;
  }
  p.algo = found[0].algo;
  p.workspace = found[0].workspaceSize;
  p.choices.assign(found, found + n);
  return 0;
}

// The plan of a shape, made at its first use.  Call with g_lock held.
int plan_for(Plan*& plan, int M, int N, int K, int ldx, int ldw, int ldo) {
  if (g_handle == nullptr) KVCM_BLAS(hipblasLtCreate(&g_handle));
  const auto key = std::make_tuple(M, N, K, ldx, ldw, ldo);
  auto it = g_plans.find(key);
  if (it == g_plans.end()) {
    Plan p;
    if (int rc = make_plan(p, M, N, K, ldx, ldw, ldo)) return rc;
    it = g_plans.emplace(key, p).first;
  }
  plan = &it->second;   // entries of a std::map stay where they are
  return 0;
}

// result[0] = max |a - b|, result[1] = max |a| over two bfloat16 matrices of M rows (as unsigned bit
// patterns of non-negative floats, whose order is the floats' order); a NaN in either counts as a
// difference of infinity.
__global__ void __launch_bounds__(256)
    compare_kernel(const uint16_t* __restrict__ a, int lda, const uint16_t* __restrict__ b, int ldb, int M, int N, unsigned* result) {
  float diff = 0.f, top = 0.f;
  for (long long i = blockIdx.x * 256ll + threadIdx.x; i < static_cast<long long>(M) * N; i += gridDim.x * 256ll) {
    const size_t row = size_t(i / N), col = size_t(i % N);
    const float x = kvcm::bf16_bits_to_float(a[row * lda + col]), y = kvcm::bf16_bits_to_float(b[row * ldb + col]);
    const float d = fabsf(x - y);
    diff = fmaxf(diff, d == d ? d : __builtin_inff());
    top = fmaxf(top, fabsf(x));
  }
  atomicMax(result, __float_as_uint(diff));
  atomicMax(result + 1, __float_as_uint(top));
}

}  // namespace

extern "C" {

long long kvcm_gemm_library_workspace_bytes() { return kWorkspaceBytes; }

int kvcm_gemm_library(const void* X, const void* W, void* out, int M, int N, int K, int ldx, int ldw, int ldo,
                      void* workspace, long long workspace_bytes, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  KVCM_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_library: bad sizes M=%d N=%d K=%d", M, N, K);
  KVCM_REQUIRE(ldx >= K && ldw >= K && ldo >= N, "gemm_library: leading dimensions too small");
  KVCM_REQUIRE(X != nullptr && W != nullptr && out != nullptr, "gemm_library: null operand");
  // the plan's algorithm and workspace size are copied out under the lock: a tuning call on another
  // thread replaces them under the same lock (the descriptors of a plan never change once made)
  Plan* plan = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t algo_workspace = 0;
  {
    std::lock_guard<std::mutex> hold(g_lock);
    if (int rc = plan_for(plan, M, N, K, ldx, ldw, ldo)) return rc;
    algo = plan->algo;
    algo_workspace = plan->workspace;
  }
  KVCM_REQUIRE(static_cast<long long>(algo_workspace) <= workspace_bytes && (algo_workspace == 0 || workspace != nullptr),
               "gemm_library: the algorithm needs %zu bytes of workspace, %lld were given", algo_workspace, workspace_bytes);
  const float one = 1.0f, zero = 0.0f;
  KVCM_BLAS(hipblasLtMatmul(g_handle, plan->desc, &one, W, plan->a, X, plan->b, &zero, out, plan->c, out, plan->c,
                            &algo, workspace, algo_workspace, stream));
  return 0;
}

// How wide a search the shape's plan has had: 0 none (the heuristic's first choice), 1 the heuristic's
// choices were timed, 2 every algorithm of the library that supports the shape was.
int kvcm_gemm_library_tuned(int M, int N, int K, int ldx, int ldw, int ldo) {
  std::lock_guard<std::mutex> hold(g_lock);
  auto it = g_plans.find(std::make_tuple(M, N, K, ldx, ldw, ldo));
  return it == g_plans.end() ? 0 : it->second.tuned;
}

// Times candidate algorithms for this shape on these operands and keeps the fastest whose result
// agrees with the heuristic's first choice.  mode 1: the heuristic's choices (up to 16; a few
// milliseconds); mode 2: every algorithm of the library that supports the shape (seconds), at most
// `max_seconds` of search.  W: `w_copies` copies of the weight matrix, `w_copy_bytes` apart; timed calls
// go round them, so that with enough copies the weights come from memory as they do in a model of many
// layers and not from a cache.  `check`: M * N bfloat16 and 8 more bytes of device memory the caller owns.
// Synchronises the stream; not for use inside a capture.  `out` holds the product afterwards.
// report (host, may be null): [0] microseconds of the first choice, [1] of the kept one, [2] candidates timed.
int kvcm_gemm_library_tune(const void* X, const void* W, int w_copies, long long w_copy_bytes, void* out, int M, int N, int K,
                           int ldx, int ldw, int ldo, void* workspace, long long workspace_bytes, void* check, int mode,
                           double max_seconds, double* report, hipStream_t stream) {
  KVCM_REQUIRE(M > 0 && N > 0 && K > 0 && ldx >= K && ldw >= K && ldo >= N, "gemm_library_tune: bad sizes");
  KVCM_REQUIRE(X && W && out && check && (mode == 1 || mode == 2), "gemm_library_tune: null operand or unknown mode");
  KVCM_REQUIRE(w_copies >= 1 && (w_copies == 1 || w_copy_bytes >= static_cast<long long>(N - 1) * ldw * 2 + K * 2),
               "gemm_library_tune: copies of the weights overlap");
  std::lock_guard<std::mutex> hold(g_lock);
  Plan* plan = nullptr;
  if (int rc = plan_for(plan, M, N, K, ldx, ldw, ldo)) return rc;
  if (plan->tuned >= mode) return 0;
  const float one = 1.0f, zero = 0.0f;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  KVCM_REQUIRE(hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess, "gemm_library_tune: no events");
  long long turn = 1;
  // microseconds per call, or a negative value when the algorithm does not run
  auto time_of = [&](hipblasLtMatmulAlgo_t& algo, size_t need, int iters) -> float {
    if (static_cast<long long>(need) > workspace_bytes || (need > 0 && workspace == nullptr)) return -1.f;
    if (hipblasLtMatmul(g_handle, plan->desc, &one, W, plan->a, X, plan->b, &zero, out, plan->c, out, plan->c, &algo,
                        workspace, need, stream) != HIPBLAS_STATUS_SUCCESS) return -1.f;
    if (hipEventRecord(e0, stream) != hipSuccess) return -1.f;
    for (int i = 0; i < iters; ++i, ++turn)
      if (hipblasLtMatmul(g_handle, plan->desc, &one, static_cast<const char*>(W) + (turn % w_copies) * w_copy_bytes, plan->a, X,
                          plan->b, &zero, out, plan->c, out, plan->c, &algo, workspace, need, stream) != HIPBLAS_STATUS_SUCCESS)
        return -1.f;
    float ms = 0.f;
    if (hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
        hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.f;
    return ms * 1e3f / iters;
  };
  struct Timed { float us; hipblasLtMatmulAlgo_t algo; size_t need; };
  std::vector<Timed> timed;
  // the reference result and the first choice's time (after enough calls for the clock to have settled)
  hipblasLtMatmulAlgo_t first = plan->choices[0].algo;
  time_of(first, plan->choices[0].workspaceSize, 32);
  const float first_us = time_of(first, plan->choices[0].workspaceSize, 8);
  int rc = 0;
  unsigned* flags = reinterpret_cast<unsigned*>(static_cast<uint16_t*>(check) + size_t(M) * N);
  if (first_us < 0.f) { kvcm::set_error("gemm_library_tune: the heuristic's first choice does not run"); rc = -2; }
  if (rc == 0 && hipMemcpy2DAsync(check, size_t(N) * 2, out, size_t(ldo) * 2, size_t(N) * 2, M, hipMemcpyDeviceToDevice, stream) != hipSuccess) {
    kvcm::set_error("gemm_library_tune: copying the reference result failed"); rc = -2;
  }
  const auto began = std::chrono::steady_clock::now();
  auto out_of_time = [&] { return std::chrono::duration<double>(std::chrono::steady_clock::now() - began).count() > max_seconds; };
  if (rc == 0) {
    timed.push_back({first_us, first, plan->choices[0].workspaceSize});
    for (size_t i = 1; i < plan->choices.size(); ++i) {
      const float us = time_of(plan->choices[i].algo, plan->choices[i].workspaceSize, 8);
      if (us > 0.f) timed.push_back({us, plan->choices[i].algo, plan->choices[i].workspaceSize});
    }
    if (mode == 2) {
      std::vector<hipblasLtMatmulHeuristicResult_t> all;
      if (hipblaslt_ext::getAllAlgos(g_handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, HIP_R_16BF,
                                     HIP_R_16BF, HIP_R_16BF, HIP_R_16BF, HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
        for (auto& cand : all) {
          if (out_of_time()) break;
          size_t need = 0;
          if (hipblaslt_ext::matmulIsAlgoSupported(g_handle, plan->desc, &one, plan->a, plan->b, &zero, plan->c, plan->c,
                                                   cand.algo, need) != HIPBLAS_STATUS_SUCCESS) continue;
          const float us = time_of(cand.algo, need, 6);
          if (us > 0.f) timed.push_back({us, cand.algo, need});
        }
      }
    }
    // the fastest few again, longer, then the fastest of those whose result agrees with the first choice's
    std::sort(timed.begin(), timed.end(), [](const Timed& x, const Timed& y) { return x.us < y.us; });
    // (the first choice is always among them: rounds of the finalists alternate, so that a drift of the
    // clock does not favour who is timed first)
    std::stable_sort(timed.begin(), timed.end(), [](const Timed& x, const Timed& y) { return x.us < y.us; });
    const size_t finalists = std::min<size_t>(timed.size(), 8);
    {
      size_t at = 0;
      while (at < timed.size() && memcmp(&timed[at].algo, &first, sizeof(first)) != 0) ++at;
      if (at >= finalists && at < timed.size()) std::swap(timed[finalists - 1], timed[at]);
    }
    // (each finalist's time: the median of five rounds, which a single slow or fast round does not move)
    std::vector<std::vector<float>> rounds(finalists);
    for (int round = 0; round < 5; ++round)
      for (size_t i = 0; i < finalists; ++i) {
        const float us = time_of(timed[i].algo, timed[i].need, 16);
        rounds[i].push_back(us > 0.f ? us : 1e30f);
      }
    for (size_t i = 0; i < finalists; ++i) {
      std::sort(rounds[i].begin(), rounds[i].end());
      timed[i].us = rounds[i][2];
    }
    std::sort(timed.begin(), timed.begin() + finalists, [](const Timed& x, const Timed& y) { return x.us < y.us; });
    bool kept = false;
    for (size_t i = 0; i < finalists && !kept && timed[i].us < 1e29f; ++i) {
      unsigned host[2] = {0u, 0u};
      if (time_of(timed[i].algo, timed[i].need, 0) < 0.f) continue;   // its result into `out`
      if (hipMemsetAsync(flags, 0, 8, stream) != hipSuccess) break;
      compare_kernel<<<1024, 256, 0, stream>>>(static_cast<const uint16_t*>(out), ldo, static_cast<const uint16_t*>(check), N, M, N, flags);
      if (hipMemcpyAsync(host, flags, 8, hipMemcpyDeviceToHost, stream) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) break;
      float diff, top;
      memcpy(&diff, &host[0], 4); memcpy(&top, &host[1], 4);
      // two orders of a 32-bit sum differ by a rounding step of the bfloat16 result here and there
      if (diff <= top * (1.0f / 64.0f)) {
        plan->algo = timed[i].algo;
        plan->workspace = timed[i].need;
        kept = true;
        if (report) { report[0] = first_us; report[1] = timed[i].us; report[2] = double(timed.size()); }
      }
    }
    if (!kept) {   // nothing agreed (not even the first choice with itself): keep the first choice
      plan->algo = first;
      plan->workspace = plan->choices[0].workspaceSize;
      if (report) { report[0] = first_us; report[1] = first_us; report[2] = double(timed.size()); }
    }
    plan->tuned = mode;
    // leave the kept algorithm's product in `out`
    if (hipblasLtMatmul(g_handle, plan->desc, &one, W, plan->a, X, plan->b, &zero, out, plan->c, out, plan->c, &plan->algo,
                        workspace, plan->workspace, stream) != HIPBLAS_STATUS_SUCCESS) {
      kvcm::set_error("gemm_library_tune: the kept algorithm does not run"); rc = -2;
    }
  }
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  return rc;
}

}  // extern "C"
