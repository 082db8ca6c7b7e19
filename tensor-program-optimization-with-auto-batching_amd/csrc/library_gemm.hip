// Plain prefill-sized base linear through the vendor GEMM library (hipBLASLt):  y[T, N] (=|+=) x[T, K] . W[N, K]^T.
// No fusion is wanted here - it is a library GEMM on a row-major weight - so it is left to the library; the decode
// path (T <= 64) and everything fused stay on the kernels of this package.
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t ws = 0;
  int status = MLORA_OK;
};

using Key = std::tuple<int, int, int, int, int, int, int, size_t>;   // device, T, K, N, ldx, y_dtype, mode, workspace

std::mutex g_mu;
hipblasLtHandle_t g_handle[64] = {};
std::map<Key, Plan> g_plans;   // kept for the life of the process: a plan is a few descriptors and one algorithm choice

#define LT(call)                                                                                  \
  do {                                                                                            \
    hipblasStatus_t st_ = (call);                                                                 \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                                                          \
      p.status = mlora_set_error(MLORA_ERR_LAUNCH, "gemm_library: %s -> status %d", #call, (int)st_); \
      return p;                                                                                   \
    }                                                                                             \
  } while (0)

// Row-major y[T, N] = x[T, K] . W[N, K]^T is, column-major, D[N, T] = op_T(A[K, N]) . B[K, T] with A = W, B = x.
Plan make_plan(hipblasLtHandle_t h, int T, int K, int N, int ldx, int y_dtype, size_t ws_bytes) {
  Plan p;
  const hipDataType yt = y_dtype == MLORA_F32 ? HIP_R_32F : HIP_R_16F;
  LT(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
  LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
  LT(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16F, K, N, K));
  LT(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16F, K, T, ldx));
  LT(hipblasLtMatrixLayoutCreate(&p.c, yt, N, T, N));
  hipblasLtMatmulPreference_t pref = nullptr;
  LT(hipblasLtMatmulPreferenceCreate(&pref));
  LT(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws_bytes, sizeof(ws_bytes)));
  hipblasLtMatmulHeuristicResult_t res[1];
  int found = 0;
  const hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.a, p.b, p.c, p.c, pref, 1, res, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (hs != HIPBLAS_STATUS_SUCCESS || found < 1) {
    p.status = mlora_set_error(MLORA_ERR_UNSUPPORTED, "gemm_library: no algorithm for T=%d K=%d N=%d (status %d)", T, K, N, (int)hs);
    return p;
  }
  p.algo = res[0].algo;
  p.ws = res[0].workspaceSize;
  return p;
}

}  // namespace

extern "C" size_t mlora_gemm_library_workspace_bytes(void) { return (size_t)64 << 20; }

extern "C" int mlora_gemm_library(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W, int T, int K, int N,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  MLORA_CHECK(y && x && W, MLORA_ERR_INVALID, "gemm_library: null pointer");
  MLORA_CHECK(T >= 0 && K > 0 && N > 0 && ldx >= K, MLORA_ERR_INVALID, "gemm_library: bad shape T=%d K=%d N=%d ldx=%d", T, K, N, ldx);
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "gemm_library: bad y_dtype %d", y_dtype);
  MLORA_CHECK(mode == MLORA_STORE || (mode == MLORA_ACCUMULATE && y_dtype == MLORA_F32), MLORA_ERR_UNSUPPORTED,
              "gemm_library: accumulate needs an fp32 y");
  MLORA_CHECK(K % 8 == 0 && N % 8 == 0 && ldx % 8 == 0, MLORA_ERR_UNSUPPORTED, "gemm_library: need K, N, ldx %% 8 == 0");
  MLORA_CHECK(workspace || workspace_bytes == 0, MLORA_ERR_WORKSPACE, "gemm_library: workspace_bytes without a workspace");
  if (T == 0) return MLORA_OK;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return mlora_set_error(MLORA_ERR_LAUNCH, "gemm_library: no current device");
  Plan p;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_handle[dev] && hipblasLtCreate(&g_handle[dev]) != HIPBLAS_STATUS_SUCCESS)
      return mlora_set_error(MLORA_ERR_LAUNCH, "gemm_library: hipblasLtCreate failed");
    const Key key(dev, T, K, N, ldx, y_dtype, mode, workspace_bytes);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) it = g_plans.emplace(key, make_plan(g_handle[dev], T, K, N, ldx, y_dtype, workspace_bytes)).first;
    p = it->second;
  }
  if (p.status != MLORA_OK) return p.status;
  const float alpha = 1.f, beta = mode == MLORA_ACCUMULATE ? 1.f : 0.f;
  const hipblasStatus_t st = hipblasLtMatmul(g_handle[dev], p.desc, &alpha, W, p.a, x, p.b, &beta, y, p.c, y, p.c, &p.algo, workspace,
                                             workspace_bytes, (hipStream_t)stream);
  if (st != HIPBLAS_STATUS_SUCCESS) return mlora_set_error(MLORA_ERR_LAUNCH, "gemm_library: hipblasLtMatmul -> status %d", (int)st);
  return MLORA_OK;
}
