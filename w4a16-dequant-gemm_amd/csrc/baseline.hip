// Plain FP16 GEMM over already-dequantized weights through hipBLASLt: the
// second pass of the two-pass baseline the fused kernels are measured against.
// c[M,N] (row-major) = x[M,K] * w[N,K]^T, FP32 accumulation, FP16 output.
//
// Per device: the handle, its workspace and one plan per (M, N, K) -- descriptors plus
// the algorithm the heuristic picks -- are made once and kept (at most MAX_PLANS of
// them; the least recently made goes first), so a timed call is the matrix product
// alone, like a call of the fused entry points.
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
constexpr size_t WS_BYTES = 64u << 20;
constexpr int MAX_DEVICES = 64;
constexpr size_t MAX_PLANS = 64;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
  hipblasLtMatmulAlgo_t algo;
};
struct PlanEntry {
  Plan plan;
  unsigned long long made = 0;  // creation order: the oldest is dropped when the map is full
};
struct DeviceState {
  hipblasLtHandle_t handle = nullptr;
  void* ws = nullptr;
  std::map<std::tuple<int, int, int>, PlanEntry> plans;
  unsigned long long clock = 0;
};
DeviceState g_dev[MAX_DEVICES];

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

// Handle and workspace of one device: the handle is published only once both exist.
int ensure_handle(DeviceState& d) {
  if (d.handle) return W4_OK;
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
  d.ws = ws;
  d.handle = h;
  return W4_OK;
}

// Column-major view: C^T (N x M) = W (as K x N col-major, transposed) * X^T (K x M).
int make_plan(hipblasLtHandle_t handle, int M, int N, int K, Plan& p) {
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
  BL(hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.la, p.lb, p.lc, p.lc, pref, 1, heur,
                                     &found));
  hipblasLtMatmulPreferenceDestroy(pref);
  pref = nullptr;
  if (found < 1) {
    destroy(p);
    snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: no hipBLASLt algorithm");
    return W4_ERUNTIME;
  }
  if (heur[0].workspaceSize > WS_BYTES) {  // the preference above caps it; never trust silently
    destroy(p);
    snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: algorithm wants %zu workspace bytes, have %zu",
             (size_t)heur[0].workspaceSize, WS_BYTES);
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
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    snprintf(g_blas_msg, sizeof g_blas_msg, "gemm_fp16: no current device");
    return W4_ERUNTIME;
  }
  std::lock_guard<std::mutex> lk(g_mu);
  DeviceState& d = g_dev[dev];
  if (int rc = ensure_handle(d)) return rc;
  const auto key = std::make_tuple(M, N, K);
  auto it = d.plans.find(key);
  if (it == d.plans.end()) {
    if (d.plans.size() >= MAX_PLANS) {
      auto oldest = d.plans.begin();
      for (auto j = d.plans.begin(); j != d.plans.end(); ++j)
        if (j->second.made < oldest->second.made) oldest = j;
      destroy(oldest->second.plan);
      d.plans.erase(oldest);
    }
    PlanEntry e;
    if (int rc = make_plan(d.handle, M, N, K, e.plan)) return rc;
    e.made = ++d.clock;
    it = d.plans.emplace(key, e).first;
  }
  const Plan& p = it->second.plan;
  const float alpha = 1.0f, beta = 0.0f;
  const hipblasStatus_t st =
      hipblasLtMatmul(d.handle, p.desc, &alpha, w, p.la, x, p.lb, &beta, c, p.lc, c, p.lc, &p.algo,
                      d.ws, WS_BYTES, (hipStream_t)stream);
  if (st != HIPBLAS_STATUS_SUCCESS) return fail("hipblasLtMatmul", (int)st);
  return W4_OK;
}
