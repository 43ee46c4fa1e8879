// Plain FP16 GEMM over already-dequantized weights through hipBLASLt: the
// second pass of the two-pass baseline the fused kernels are measured against.
// c[M,N] (row-major) = x[M,K] * w[N,K]^T, FP32 accumulation, FP16 output.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdio.h>

#include <mutex>

#include "../../include/w4_abi.h"

namespace {
thread_local char g_blas_msg[160] = "";
std::mutex g_mu;
hipblasLtHandle_t g_handle = nullptr;
void* g_ws = nullptr;
constexpr size_t WS_BYTES = 64u << 20;
}  // namespace

extern "C" const char* w4_blas_last_error(void) { return g_blas_msg; }

// Column-major view: C^T (N x M) = W (as K x N col-major, transposed) * X^T (K x M).
extern "C" int w4_gemm_fp16_impl(const w4_half* w, const w4_half* x, w4_half* c, int M,
                                 int N, int K, w4_stream stream) {
  std::lock_guard<std::mutex> lk(g_mu);
#define BL(call)                                                              \
  do {                                                                        \
    hipblasStatus_t st_ = (call);                                             \
    if (st_ != HIPBLAS_STATUS_SUCCESS) {                                      \
      snprintf(g_blas_msg, sizeof g_blas_msg, "%s: hipblas status %d", #call, \
               (int)st_);                                                     \
      return W4_ERUNTIME;                                                     \
    }                                                                         \
  } while (0)
  if (!g_handle) {
    BL(hipblasLtCreate(&g_handle));
    if (hipMalloc(&g_ws, WS_BYTES) != hipSuccess) {
      snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: workspace allocation failed");
      return W4_ERUNTIME;
    }
  }
  hipblasLtMatmulDesc_t desc;
  hipblasLtMatrixLayout_t la, lb, lc;
  BL(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  BL(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof ta));
  BL(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof tb));
  BL(hipblasLtMatrixLayoutCreate(&la, HIP_R_16F, K, N, K));  // W stored K x N col-major
  BL(hipblasLtMatrixLayoutCreate(&lb, HIP_R_16F, K, M, K));  // X stored K x M col-major
  BL(hipblasLtMatrixLayoutCreate(&lc, HIP_R_16F, N, M, N));  // C^T
  hipblasLtMatmulPreference_t pref;
  BL(hipblasLtMatmulPreferenceCreate(&pref));
  size_t ws = WS_BYTES;
  BL(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES,
                                           &ws, sizeof ws));
  hipblasLtMatmulHeuristicResult_t heur[1];
  int found = 0;
  BL(hipblasLtMatmulAlgoGetHeuristic(g_handle, desc, la, lb, lc, lc, pref, 1, heur, &found));
  if (found < 1) {
    snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: no hipBLASLt algorithm");
    return W4_ERUNTIME;
  }
  const float alpha = 1.0f, beta = 0.0f;
  BL(hipblasLtMatmul(g_handle, desc, &alpha, w, la, x, lb, &beta, c, lc, c, lc,
                     &heur[0].algo, g_ws, WS_BYTES, (hipStream_t)stream));
  hipblasLtMatmulPreferenceDestroy(pref);
  hipblasLtMatrixLayoutDestroy(la);
  hipblasLtMatrixLayoutDestroy(lb);
  hipblasLtMatrixLayoutDestroy(lc);
  hipblasLtMatmulDescDestroy(desc);
#undef BL
  return W4_OK;
}
