// Plain FP16 GEMM over already-dequantized weights through hipBLASLt: the
// second pass of the two-pass baseline the fused kernels are measured against.
// c[M,N] (row-major) = x[M,K] * w[N,K]^T, FP32 accumulation, FP16 output.
//
// The handle, its workspace and one plan per (M, N, K) -- descriptors plus the
// algorithm the heuristic picks -- are made once and kept, so a timed call is the
// matrix product alone, like a call of the fused entry points.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdio.h>

#include <map>
#include <mutex>
#include <tuple>

#include "../../include/w4_abi.h"

namespace {
thread_local char g_blas_msg[160] = "";
std::mutex g_mu;
hipblasLtHandle_t g_handle = nullptr;
void* g_ws = nullptr;
constexpr size_t WS_BYTES = 64u << 20;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
  hipblasLtMatmulAlgo_t algo;
};
std::map<std::tuple<int, int, int>, Plan> g_plans;

void destroy(Plan& p) {
  if (p.la) hipblasLtMatrixLayoutDestroy(p.la);
  if (p.lb) hipblasLtMatrixLayoutDestroy(p.lb);
  if (p.lc) hipblasLtMatrixLayoutDestroy(p.lc);
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  p = Plan{};
}

int fail(const char* what, int status) {
  snprintf(g_blas_msg, sizeof g_blas_msg, "%s: hipblas status %d", what, status);
  return W4_ERUNTIME;
}

// Handle and workspace: the handle is published only once both exist.
int ensure_handle() {
  if (g_handle) return W4_OK;
  void* ws = nullptr;
  if (hipMalloc(&ws, WS_BYTES) != hipSuccess) {
    snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: workspace allocation failed");
    return W4_ERUNTIME;
  }
  hipblasLtHandle_t h = nullptr;
  const hipblasStatus_t st = hipblasLtCreate(&h);
  if (st != HIPBLAS_STATUS_SUCCESS) {
    (void)hipFree(ws);
    return fail("hipblasLtCreate", (int)st);
  }
  g_ws = ws;
  g_handle = h;
  return W4_OK;
}

// Column-major view: C^T (N x M) = W (as K x N col-major, transposed) * X^T (K x M).
int make_plan(int M, int N, int K, Plan& p) {
#define BL(call)                                             \
  do {                                                       \
    const hipblasStatus_t st_ = (call);                      \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                     \
      if (pref) hipblasLtMatmulPreferenceDestroy(pref);      \
      destroy(p);                                            \
      return fail(#call, (int)st_);                          \
    }                                                        \
  } while (0)
  hipblasLtMatmulPreference_t pref = nullptr;
  BL(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  BL(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof ta));
  BL(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof tb));
  BL(hipblasLtMatrixLayoutCreate(&p.la, HIP_R_16F, K, N, K));  // W stored K x N col-major
  BL(hipblasLtMatrixLayoutCreate(&p.lb, HIP_R_16F, K, M, K));  // X stored K x M col-major
  BL(hipblasLtMatrixLayoutCreate(&p.lc, HIP_R_16F, N, M, N));  // C^T
  BL(hipblasLtMatmulPreferenceCreate(&pref));
  const size_t ws = WS_BYTES;
  BL(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws,
                                           sizeof ws));
  hipblasLtMatmulHeuristicResult_t heur[1];
  int found = 0;
  BL(hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.la, p.lb, p.lc, p.lc, pref, 1, heur,
                                     &found));
  hipblasLtMatmulPreferenceDestroy(pref);
  pref = nullptr;
  if (found < 1) {
    destroy(p);
    snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: no hipBLASLt algorithm");
    return W4_ERUNTIME;
  }
  p.algo = heur[0].algo;
#undef BL
  return W4_OK;
}
}  // namespace

extern "C" const char* w4_blas_last_error(void) { return g_blas_msg; }

extern "C" int w4_gemm_fp16_impl(const w4_half* w, const w4_half* x, w4_half* c, int M, int N,
                                 int K, w4_stream stream) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (int rc = ensure_handle()) return rc;
  const auto key = std::make_tuple(M, N, K);
  auto it = g_plans.find(key);
  if (it == g_plans.end()) {
    Plan p;
    if (int rc = make_plan(M, N, K, p)) return rc;
    it = g_plans.emplace(key, p).first;
  }
  const Plan& p = it->second;
  const float alpha = 1.0f, beta = 0.0f;
  const hipblasStatus_t st =
      hipblasLtMatmul(g_handle, p.desc, &alpha, w, p.la, x, p.lb, &beta, c, p.lc, c, p.lc, &p.algo,
                      g_ws, WS_BYTES, (hipStream_t)stream);
  if (st != HIPBLAS_STATUS_SUCCESS) return fail("hipblasLtMatmul", (int)st);
  return W4_OK;
}
