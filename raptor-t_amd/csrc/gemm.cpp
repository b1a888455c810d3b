// Dense GEMM of the layer through hipBLASLt: row-major C[M,N] = A[M,K] . B[K,N], inputs and
// output in fp16 / bf16 / fp32, accumulation in fp32.
//
// Replaces kernels::MatMul (layers/kernels/mat_mul.cpp:9-96), which calls cublasGemmEx
// with the operands swapped to express a row-major product in a column-major library and
// accumulates in fp16; the same operand swap is used here, the accumulator is fp32, and a
// failure is reported to the caller instead of ending the process (mat_mul.cpp:60-70).
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "rt_common.h"

struct rt_gemm_ctx {
  hipblasLtHandle_t lt = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  int device = 0;
  std::mutex m;
  struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t ws = 0;
  };
  std::map<std::tuple<int64_t, int64_t, int64_t, int>, Plan> plans;
};

namespace {

#define LT_TRY(expr)                                                                     \
  do {                                                                                   \
    hipblasStatus_t s_ = (expr);                                                         \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return rt::fail(RT_EIO, "%s failed with hipblasStatus %d", #expr, int(s_)); \
  } while (0)

int make_plan(rt_gemm_ctx* ctx, int64_t m, int64_t n, int64_t k, int dtype, rt_gemm_ctx::Plan& p) {
  const hipDataType t = dtype == RT_F16 ? HIP_R_16F : (dtype == RT_BF16 ? HIP_R_16BF : HIP_R_32F);
  LT_TRY(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  hipblasOperation_t nop = HIPBLAS_OP_N;
  LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &nop, sizeof(nop)));
  LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &nop, sizeof(nop)));
  // column-major view: C^T[N,M] = B^T[N,K] . A^T[K,M]
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.la, t, n, k, n));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.lb, t, k, m, k));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.lc, t, n, m, n));
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
  LT_TRY(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ctx->workspace_bytes,
                                               sizeof(ctx->workspace_bytes)));
  hipblasLtMatmulHeuristicResult_t res[4];
  int found = 0;
  hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(ctx->lt, p.desc, p.la, p.lb, p.lc, p.lc, pref, 4, res, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (hs != HIPBLAS_STATUS_SUCCESS || found == 0)
    return rt::fail(RT_ENOSYS, "hipBLASLt has no algorithm for M=%lld N=%lld K=%lld dtype=%d (status %d)", (long long)m,
                    (long long)n, (long long)k, dtype, int(hs));
  p.algo = res[0].algo;
  p.ws = res[0].workspaceSize;
  return RT_OK;
}

void free_plan(rt_gemm_ctx::Plan& p) {
  if (p.la) hipblasLtMatrixLayoutDestroy(p.la);
  if (p.lb) hipblasLtMatrixLayoutDestroy(p.lb);
  if (p.lc) hipblasLtMatrixLayoutDestroy(p.lc);
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  p = rt_gemm_ctx::Plan();
}

}  // namespace

extern "C" {

int rt_gemm_create(rt_gemm_ctx** out) {
  RT_REQUIRE(out, RT_EINVAL, "NULL output");
  rt_gemm_ctx* ctx = new rt_gemm_ctx();
  if (hipGetDevice(&ctx->device) != hipSuccess) { delete ctx; return rt::fail(RT_EIO, "hipGetDevice failed: no usable GPU"); }
  hipblasStatus_t s = hipblasLtCreate(&ctx->lt);
  if (s != HIPBLAS_STATUS_SUCCESS) { delete ctx; return rt::fail(RT_EIO, "hipblasLtCreate failed with status %d", int(s)); }
  ctx->workspace_bytes = size_t(64) << 20;
  if (hipMalloc(&ctx->workspace, ctx->workspace_bytes) != hipSuccess) {
    hipblasLtDestroy(ctx->lt);
    delete ctx;
    return rt::fail(RT_ENOMEM, "could not allocate the 64 MiB GEMM workspace");
  }
  *out = ctx;
  return RT_OK;
}

int rt_gemm_destroy(rt_gemm_ctx* ctx) {
  if (!ctx) return RT_OK;
  for (auto& kv : ctx->plans) free_plan(kv.second);
  if (ctx->workspace) (void)hipFree(ctx->workspace);
  if (ctx->lt) hipblasLtDestroy(ctx->lt);
  delete ctx;
  return RT_OK;
}

int rt_gemm(rt_gemm_ctx* ctx, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int dtype,
            void* stream) {
  RT_REQUIRE(ctx && a && b && c, RT_EINVAL, "NULL argument");
  RT_REQUIRE(m >= 0 && n > 0 && k > 0, RT_EINVAL, "bad shape M=%lld N=%lld K=%lld", (long long)m, (long long)n, (long long)k);
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16 || dtype == RT_F32, RT_EINVAL, "unknown dtype %d", dtype);
  if (m == 0) return RT_OK;
  rt_gemm_ctx::Plan* plan;
  {
    std::lock_guard<std::mutex> lk(ctx->m);
    auto key = std::make_tuple(m, n, k, dtype);
    auto it = ctx->plans.find(key);
    if (it == ctx->plans.end()) {
      rt_gemm_ctx::Plan p;
      int rc = make_plan(ctx, m, n, k, dtype, p);
      if (rc) { free_plan(p); return rc; }
      it = ctx->plans.emplace(key, p).first;
    }
    plan = &it->second;
  }
  const float alpha = 1.0f, beta = 0.0f;
  LT_TRY(hipblasLtMatmul(ctx->lt, plan->desc, &alpha, b, plan->la, a, plan->lb, &beta, c, plan->lc, c, plan->lc,
                         &plan->algo, ctx->workspace, ctx->workspace_bytes, static_cast<hipStream_t>(stream)));
  return RT_OK;
}

}  // extern "C"
