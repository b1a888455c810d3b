// Dense GEMM of the layer through hipBLASLt: row-major C[M,N] = A[M,K] . B[K,N], inputs and
// output in fp16 / bf16 / fp32, accumulation in fp32.
//
// Replaces kernels::MatMul (layers/kernels/mat_mul.cpp:9-96), which calls cublasGemmEx
// with the operands swapped to express a row-major product in a column-major library and
// accumulates in fp16; the same operand swap is used here, the accumulator is fp32, and a
// failure is reported to the caller instead of ending the process (mat_mul.cpp:60-70).
//
// rt_gemm_bias_act runs the same product with the bias add, and optionally the tanh GELU, in
// the GEMM's epilogue: what BertIntermediate does with MatMul followed by add_bias_act_kernel
// (layers/bert_intermediate.cpp:22-30, layers/kernels/add_bias_act.cu:114-133) in one pass over
// the output.
//
// rt_gemm_bt takes B as Bt[N,K] (each output column's K weights contiguous), the b_trans = true
// case of kernels::MatMul: with both operands K-contiguous the library's kernels for these shapes
// run 8-20 % faster than with B[K,N], so a layer that owns its weights keeps them this way.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <map>
#include <vector>
#include <mutex>
#include <tuple>

#include "rt_common.h"

struct rt_gemm_ctx {
  hipblasLtHandle_t lt = nullptr;
  int tune_candidates = 64;         // heuristic results timed on a shape's first call (1 = take the first)
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
  // keyed by (M, N, K, dtype, mode); mode = epilogue | MODE_B_TRANS
  std::map<std::tuple<int64_t, int64_t, int64_t, int, int>, Plan> plans;
  // The fastest solutions (library indices, best first) of the first M seen of each (N, K, dtype,
  // mode).  A packed batch changes M with every batch and the best solution moves with it (the
  // number of output tiles against the number of CUs), so each further M times only these.
  std::map<std::tuple<int64_t, int64_t, int, int>, std::vector<int>> kind_best;
  int retune_candidates = 6;        // how many of kind_best a further M times (<= 1: take the first untimed)
};

namespace {

constexpr int MODE_B_TRANS = 16;   // B is handed over as Bt[N,K]

#define LT_TRY(expr)                                                                     \
  do {                                                                                   \
    hipblasStatus_t s_ = (expr);                                                         \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return rt::fail(RT_EIO, "%s failed with hipblasStatus %d", #expr, int(s_)); \
  } while (0)

// Times one candidate on the caller's operands (they are overwritten with the same product).
float time_algo(rt_gemm_ctx* ctx, const rt_gemm_ctx::Plan& p, const hipblasLtMatmulAlgo_t& algo, const void* a,
                const void* b, void* c, hipStream_t st, hipEvent_t e0, hipEvent_t e1) {
  const float alpha = 1.0f, beta = 0.0f;
  const int reps = 3;
  for (int r = 0; r <= reps; ++r) {               // the first run is a warm-up
    if (r == 1 && hipEventRecord(e0, st) != hipSuccess) return -1.f;
    if (hipblasLtMatmul(ctx->lt, p.desc, &alpha, b, p.la, a, p.lb, &beta, c, p.lc, c, p.lc, &algo, ctx->workspace,
                        ctx->workspace_bytes, st) != HIPBLAS_STATUS_SUCCESS)
      return -1.f;
  }
  float ms = -1.f;
  if (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
      hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
    return -1.f;
  return ms / reps;
}

// epilogue: RT_EPILOGUE_NONE, or bias / bias + GELU along the N columns of the row-major output
// (the rows of the column-major problem handed to the library, where it expects the bias).
int make_plan(rt_gemm_ctx* ctx, int64_t m, int64_t n, int64_t k, int dtype, int mode, const void* bias,
              rt_gemm_ctx::Plan& p, const void* a, const void* b, void* c, hipStream_t st) {
  const int epilogue = mode & ~MODE_B_TRANS;
  const bool b_trans = (mode & MODE_B_TRANS) != 0;
  const hipDataType t = dtype == RT_F16 ? HIP_R_16F : (dtype == RT_BF16 ? HIP_R_16BF : HIP_R_32F);
  LT_TRY(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  hipblasOperation_t nop = HIPBLAS_OP_N;
  const hipblasOperation_t first_op = b_trans ? HIPBLAS_OP_T : HIPBLAS_OP_N;
  LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &first_op, sizeof(first_op)));
  LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &nop, sizeof(nop)));
  if (epilogue != RT_EPILOGUE_NONE) {
    hipblasLtEpilogue_t ep = epilogue == RT_EPILOGUE_BIAS_GELU ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_BIAS;
    LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof(ep)));
    LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
    LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &t, sizeof(t)));
  }
  // column-major view: C^T[N,M] = B^T[N,K] . A^T[K,M]; a row-major Bt[N,K] is the column-major
  // K x N matrix whose transpose is the first operand
  if (b_trans)
    LT_TRY(hipblasLtMatrixLayoutCreate(&p.la, t, k, n, k));
  else
    LT_TRY(hipblasLtMatrixLayoutCreate(&p.la, t, n, k, n));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.lb, t, k, m, k));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.lc, t, n, m, n));
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  const bool can_time = hipStreamIsCapturing(st, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone;
  // A further M of a known kind: time the kind's best few (not the whole candidate list again).
  {
    auto known = ctx->kind_best.find(std::make_tuple(n, k, dtype, mode));
    if (known != ctx->kind_best.end() && !known->second.empty()) {
      const int want = ctx->retune_candidates < 1 ? 1 : ctx->retune_candidates;
      std::vector<int> index(known->second.begin(),
                             known->second.begin() + std::min<size_t>(known->second.size(), size_t(want)));
      std::vector<hipblasLtMatmulHeuristicResult_t> byindex;
      const float one = 1.0f, zero = 0.0f;
      if (hipblaslt_ext::getAlgosFromIndex(ctx->lt, index, byindex) == HIPBLAS_STATUS_SUCCESS) {
        std::vector<std::pair<hipblasLtMatmulAlgo_t, size_t>> ok;
        for (auto& r : byindex) {
          size_t ws = 0;
          if (hipblaslt_ext::matmulIsAlgoSupported(ctx->lt, p.desc, &one, p.la, p.lb, &zero, p.lc, p.lc, r.algo, ws) ==
                  HIPBLAS_STATUS_SUCCESS && ws <= ctx->workspace_bytes)
            ok.emplace_back(r.algo, ws);
        }
        if (!ok.empty()) {
          size_t best = 0;
          hipEvent_t e0 = nullptr, e1 = nullptr;
          if (ok.size() > 1 && can_time && hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
            float best_ms = -1.f;
            for (size_t i = 0; i < ok.size(); ++i) {
              const float ms = time_algo(ctx, p, ok[i].first, a, b, c, st, e0, e1);
              if (ms > 0.f && (best_ms < 0.f || ms < best_ms)) { best_ms = ms; best = i; }
            }
          }
          if (e0) (void)hipEventDestroy(e0);
          if (e1) (void)hipEventDestroy(e1);
          p.algo = ok[best].first;
          p.ws = ok[best].second;
          return RT_OK;
        }
      }
    }
  }
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
  LT_TRY(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ctx->workspace_bytes,
                                               sizeof(ctx->workspace_bytes)));
  constexpr int MAX_CAND = 64;
  std::vector<hipblasLtMatmulHeuristicResult_t> res(MAX_CAND);
  int found = 0;
  const int want = ctx->tune_candidates < 1 ? 1 : (ctx->tune_candidates > MAX_CAND ? MAX_CAND : ctx->tune_candidates);
  hipblasStatus_t hs =
      hipblasLtMatmulAlgoGetHeuristic(ctx->lt, p.desc, p.la, p.lb, p.lc, p.lc, pref, want, res.data(), &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (hs != HIPBLAS_STATUS_SUCCESS || found == 0)
    return rt::fail(RT_ENOSYS, "hipBLASLt has no algorithm for M=%lld N=%lld K=%lld dtype=%d (status %d)", (long long)m,
                    (long long)n, (long long)k, dtype, int(hs));
  res.resize(found);
  if (ctx->tune_candidates == RT_GEMM_TUNE_ALL) {
    // every solution the library has for these types, filtered to the ones that accept this problem
    std::vector<hipblasLtMatmulHeuristicResult_t> all;
    if (hipblaslt_ext::getAllAlgos(ctx->lt, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, first_op, HIPBLAS_OP_N, t, t, t, t,
                                   HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
      const float one = 1.0f, zero = 0.0f;
      for (auto& r : all) {
        size_t ws = 0;
        if (hipblaslt_ext::matmulIsAlgoSupported(ctx->lt, p.desc, &one, p.la, p.lb, &zero, p.lc, p.lc, r.algo, ws) !=
                HIPBLAS_STATUS_SUCCESS || ws > ctx->workspace_bytes)
          continue;
        r.workspaceSize = ws;
        r.state = HIPBLAS_STATUS_SUCCESS;
        res.push_back(r);
      }
      found = int(res.size());
    }
  }
  // The library's first suggestion is often not the fastest for these tall, K=768 shapes: time the
  // candidates once per kind on the caller's own operands (skipped while a graph is being captured),
  // then the best eight a second time (the ranking of near-equal candidates is noisy) and keep their order.
  std::vector<std::pair<float, int>> ranked;          // (milliseconds, position in res)
  if (found > 1 && can_time) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
      for (int i = 0; i < found; ++i) {
        if (res[i].state != HIPBLAS_STATUS_SUCCESS || res[i].workspaceSize > ctx->workspace_bytes) continue;
        const float ms = time_algo(ctx, p, res[i].algo, a, b, c, st, e0, e1);
        if (ms > 0.f) ranked.emplace_back(ms, i);
      }
      std::sort(ranked.begin(), ranked.end());
      if (ranked.size() > 8) ranked.resize(8);
      for (auto& r : ranked) {
        const float ms = time_algo(ctx, p, res[r.second].algo, a, b, c, st, e0, e1);
        if (ms > 0.f && ms < r.first) r.first = ms;
      }
      std::sort(ranked.begin(), ranked.end());
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  }
  const int best = ranked.empty() ? 0 : ranked[0].second;
  p.algo = res[best].algo;
  p.ws = res[best].workspaceSize;
  if (!ranked.empty()) {
    std::vector<int> order;
    for (auto& r : ranked) order.push_back(hipblaslt_ext::getIndexFromAlgo(res[r.second].algo));
    ctx->kind_best[std::make_tuple(n, k, dtype, mode)] = order;
  }
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

int rt_gemm_set_tuning(rt_gemm_ctx* ctx, int candidates) {
  RT_REQUIRE(ctx, RT_EINVAL, "NULL context");
  RT_REQUIRE((candidates >= 1 && candidates <= 64) || candidates == RT_GEMM_TUNE_ALL, RT_EINVAL,
             "candidates=%d must be in [1, 64] or RT_GEMM_TUNE_ALL", candidates);
  std::lock_guard<std::mutex> lk(ctx->m);
  ctx->tune_candidates = candidates;
  return RT_OK;
}

int rt_gemm_set_retuning(rt_gemm_ctx* ctx, int candidates) {
  RT_REQUIRE(ctx, RT_EINVAL, "NULL context");
  RT_REQUIRE(candidates >= 0 && candidates <= 8, RT_EINVAL, "candidates=%d must be in [0, 8]", candidates);
  std::lock_guard<std::mutex> lk(ctx->m);
  ctx->retune_candidates = candidates;
  return RT_OK;
}

}  // extern "C"

namespace {

int run_gemm(rt_gemm_ctx* ctx, const void* a, const void* b, const void* bias, void* c, int64_t m, int64_t n, int64_t k,
             int epilogue, bool b_trans, int dtype, void* stream) {
  RT_REQUIRE(ctx && a && b && c, RT_EINVAL, "NULL argument");
  RT_REQUIRE(m >= 0 && n > 0 && k > 0, RT_EINVAL, "bad shape M=%lld N=%lld K=%lld", (long long)m, (long long)n, (long long)k);
  RT_REQUIRE(dtype == RT_F16 || dtype == RT_BF16 || dtype == RT_F32, RT_EINVAL, "unknown dtype %d", dtype);
  if (m == 0) return RT_OK;
  const float alpha = 1.0f, beta = 0.0f;
  // the plan's descriptor carries the bias pointer: set and used under the lock
  std::lock_guard<std::mutex> lk(ctx->m);
  const int mode = epilogue | (b_trans ? MODE_B_TRANS : 0);
  auto key = std::make_tuple(m, n, k, dtype, mode);
  auto it = ctx->plans.find(key);
  if (it == ctx->plans.end()) {
    rt_gemm_ctx::Plan p;
    int rc = make_plan(ctx, m, n, k, dtype, mode, bias, p, a, b, c, static_cast<hipStream_t>(stream));
    if (rc) { free_plan(p); return rc; }
    it = ctx->plans.emplace(key, p).first;
  }
  rt_gemm_ctx::Plan* plan = &it->second;
  if (epilogue != RT_EPILOGUE_NONE)
    LT_TRY(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
  LT_TRY(hipblasLtMatmul(ctx->lt, plan->desc, &alpha, b, plan->la, a, plan->lb, &beta, c, plan->lc, c, plan->lc,
                         &plan->algo, ctx->workspace, ctx->workspace_bytes, static_cast<hipStream_t>(stream)));
  return RT_OK;
}

}  // namespace

extern "C" {

int rt_gemm(rt_gemm_ctx* ctx, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int dtype,
            void* stream) {
  return run_gemm(ctx, a, b, nullptr, c, m, n, k, RT_EPILOGUE_NONE, false, dtype, stream);
}

int rt_gemm_bias_act(rt_gemm_ctx* ctx, const void* a, const void* b, const void* bias, void* c, int64_t m, int64_t n,
                     int64_t k, int epilogue, int dtype, void* stream) {
  RT_REQUIRE(epilogue == RT_EPILOGUE_BIAS || epilogue == RT_EPILOGUE_BIAS_GELU, RT_EINVAL, "unknown epilogue %d", epilogue);
  RT_REQUIRE(bias, RT_EINVAL, "NULL bias");
  return run_gemm(ctx, a, b, bias, c, m, n, k, epilogue, false, dtype, stream);
}

int rt_gemm_bt(rt_gemm_ctx* ctx, const void* a, const void* bt, const void* bias, void* c, int64_t m, int64_t n,
               int64_t k, int epilogue, int dtype, void* stream) {
  RT_REQUIRE(epilogue == RT_EPILOGUE_NONE || epilogue == RT_EPILOGUE_BIAS || epilogue == RT_EPILOGUE_BIAS_GELU, RT_EINVAL,
             "unknown epilogue %d", epilogue);
  RT_REQUIRE(epilogue == RT_EPILOGUE_NONE || bias, RT_EINVAL, "NULL bias");
  return run_gemm(ctx, a, bt, epilogue == RT_EPILOGUE_NONE ? nullptr : bias, c, m, n, k, epilogue, true, dtype, stream);
}

}  // extern "C"
