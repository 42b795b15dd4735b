// The vendor library's matrix product for prompt steps: out[M, N] = X[M, K] * W[N, K]^T, bfloat16
// operands and result, 32-bit accumulation, through hipBLASLt.  The reference hands all its
// products to cuBLAS the same way (src/model/llama.cpp:45-52).  Called directly instead of through
// a tensor library so that the call is an ordinary launching entry of this library: a few
// microseconds of host time, and recordable into a step program.
//
// hipBLASLt is column-major: the row-major out[M, N] is the column-major [N, M] = W (as stored:
// column-major [K, N], transposed) times X (as stored: column-major [K, M]).  A plan (descriptors
// and the algorithm the library's heuristic picks) is made once per shape and kept.
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"
#include "kvcm_hip.h"

namespace {

constexpr long long kWorkspaceBytes = 64ll << 20;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
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
  hipblasLtMatmulHeuristicResult_t found[4];
  int n = 0;
  if (st == HIPBLAS_STATUS_SUCCESS)
    st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, 4, found, &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || n <= 0) {
    kvcm::set_error("gemm_library: the library has no algorithm for M=%d N=%d K=%d (%s)", M, N, K, status_name(st));
    return -2;
  }
  p.algo = found[0].algo;
  p.workspace = found[0].workspaceSize;
  return 0;
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
  const Plan* plan = nullptr;
  {
    std::lock_guard<std::mutex> hold(g_lock);
    if (g_handle == nullptr) KVCM_BLAS(hipblasLtCreate(&g_handle));
    const auto key = std::make_tuple(M, N, K, ldx, ldw, ldo);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
      Plan p;
      if (int rc = make_plan(p, M, N, K, ldx, ldw, ldo)) return rc;
      it = g_plans.emplace(key, p).first;
    }
    plan = &it->second;   // entries of a std::map stay where they are
  }
  KVCM_REQUIRE(static_cast<long long>(plan->workspace) <= workspace_bytes && (plan->workspace == 0 || workspace != nullptr),
               "gemm_library: the algorithm needs %zu bytes of workspace, %lld were given", plan->workspace, workspace_bytes);
  const float one = 1.0f, zero = 0.0f;
  KVCM_BLAS(hipblasLtMatmul(g_handle, plan->desc, &one, W, plan->a, X, plan->b, &zero, out, plan->c, out, plan->c,
                            &plan->algo, workspace, plan->workspace, stream));
  return 0;
}

}  // extern "C"
