// C[M, N] = X[M, K] * W[N, K]^T through hipBLASLt, for the many-row products of a
// prompt's portion (the reference hands its matrix products to the vendor's
// library too: infernum-cuda/src/inner/cuda/ops/matmul.rs:68-118, cublasGemmEx).
//
// Host code only.  What the library has to be asked once per shape (layouts, the
// choice of an algorithm) is kept per (M, N, K, dtype): a later call with the same
// shape costs one hipblasLtMatmul and no search.  Row-major X, W and C are the
// column-major operands of  C^T[N, M] = W^T-as-stored[K, N]^T * X-as-stored[K, M],
// that is A = W with a transposition, B = X without.
//
// bf16 operands and result with fp32 accumulation, or fp32 throughout (plain fp32
// arithmetic: HIPBLAS_COMPUTE_32F, no reduced-precision mode).
//
// The workspace belongs to the caller and must outlive the work put on the
// stream; calls on one stream share one workspace without harm.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdint.h>

#include <mutex>
#include <unordered_map>

namespace {

enum { IA_F32 = 0, IA_BF16 = 1 };
enum { IA_OK = 0, IA_ERR_BAD_ARG = 10001, IA_ERR_UNSUPPORTED = 10002, IA_ERR_LIBRARY = 10003 };

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

struct Key {
  int64_t m, n, k;
  int dtype;
  size_t workspace;
  bool operator==(const Key& o) const {
    return m == o.m && n == o.n && k == o.k && dtype == o.dtype && workspace == o.workspace;
  }
};
struct KeyHash {
  size_t operator()(const Key& x) const {
    uint64_t h = 1469598103934665603ull;
    for (uint64_t v : {(uint64_t)x.m, (uint64_t)x.n, (uint64_t)x.k, (uint64_t)x.dtype, (uint64_t)x.workspace}) {
      h ^= v;
      h *= 1099511628211ull;
    }
    return (size_t)h;
  }
};

std::mutex g_mu;
hipblasLtHandle_t g_handle = nullptr;
std::unordered_map<Key, Plan, KeyHash> g_plans;
int g_last_status = 0;          // the library's last status that was not a success
int g_in_flight = 0;            // calls between their lookup of a plan and the end of their hipblasLtMatmul
constexpr size_t kMaxPlans = 4096;

bool ok(hipblasStatus_t s) {
  if (s == HIPBLAS_STATUS_SUCCESS) return true;
  g_last_status = (int)s;
  return false;
}

void drop(Plan& p) {
  if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
  if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
  if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  p = Plan();
}

// Called with g_mu held.
int make_plan(const Key& key, Plan& p) {
  const hipDataType t = key.dtype == IA_BF16 ? HIP_R_16BF : HIP_R_32F;
  const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  hipblasLtMatmulPreference_t pref = nullptr;
  bool good = ok(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) &&
              ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta))) &&
              ok(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb))) &&
              ok(hipblasLtMatrixLayoutCreate(&p.a, t, key.k, key.n, key.k)) &&
              ok(hipblasLtMatrixLayoutCreate(&p.b, t, key.k, key.m, key.k)) &&
              ok(hipblasLtMatrixLayoutCreate(&p.c, t, key.n, key.m, key.n)) &&
              ok(hipblasLtMatmulPreferenceCreate(&pref));
  if (good) {
    const uint64_t ws = key.workspace;
    good = ok(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)));
  }
  int found = 0;
  hipblasLtMatmulHeuristicResult_t result;
  if (good)
    good = ok(hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, 1, &result, &found));
  if (pref) hipblasLtMatmulPreferenceDestroy(pref);
  if (!good) {
    drop(p);
    return IA_ERR_LIBRARY;
  }
  if (found < 1 || result.workspaceSize > key.workspace) {
    drop(p);
    return IA_ERR_UNSUPPORTED;
  }
  p.algo = result.algo;
  p.workspace = result.workspaceSize;
  return IA_OK;
}

}  // namespace

// X [M, K], W [N, K], C [M, N], contiguous, all bf16 (dtype 1) or all fp32 (dtype 0).  workspace: device
// memory of workspace_bytes (may be null with 0 bytes; the library then has fewer algorithms to choose from).
// Returns 0, 10001 for bad arguments, 10002 when the library has no algorithm for the shape, 10003 when a
// call into the library failed (ia_gemm_lt_last_status tells its status).
extern "C" int ia_gemm_lt(const void* X, const void* W, void* C, int M, int N, int K, int dtype, void* workspace,
                          size_t workspace_bytes, hipStream_t stream) {
  if (!X || !W || !C || M <= 0 || N <= 0 || K <= 0) return IA_ERR_BAD_ARG;
  if (dtype != IA_F32 && dtype != IA_BF16) return IA_ERR_BAD_ARG;
  if (!workspace) workspace_bytes = 0;
  Plan plan;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_handle && !ok(hipblasLtCreate(&g_handle))) {
      g_handle = nullptr;
      return IA_ERR_LIBRARY;
    }
    const Key key{M, N, K, dtype, workspace_bytes};
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
      // portions of prompts come in any length: the table is emptied when it has grown large, so that it stays
      // bounded; only while no call is between its lookup of a plan and the end of its hipblasLtMatmul
      if (g_plans.size() >= kMaxPlans && g_in_flight == 0) {
        for (auto& kv : g_plans) drop(kv.second);
        g_plans.clear();
      }
      Plan fresh;
      const int rc = make_plan(key, fresh);
      if (rc != IA_OK) return rc;
      it = g_plans.emplace(key, fresh).first;
    }
    plan = it->second;
    ++g_in_flight;          // the plan's descriptors stay alive until this call has used them
  }
  const float alpha = 1.0f, beta = 0.0f;
  const hipblasStatus_t s = hipblasLtMatmul(g_handle, plan.desc, &alpha, W, plan.a, X, plan.b, &beta, C, plan.c, C,
                                            plan.c, &plan.algo, workspace, workspace_bytes, stream);
  std::lock_guard<std::mutex> lock(g_mu);
  --g_in_flight;
  if (s != HIPBLAS_STATUS_SUCCESS) {
    g_last_status = (int)s;
    return IA_ERR_LIBRARY;
  }
  return IA_OK;
}

extern "C" int ia_gemm_lt_last_status() {
  std::lock_guard<std::mutex> lock(g_mu);
  return g_last_status;
}

// Number of shapes whose plan is kept.
extern "C" int ia_gemm_lt_plans() {
  std::lock_guard<std::mutex> lock(g_mu);
  return (int)g_plans.size();
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_gemm_lt)
