// The BLAS library's matrix product for many rows of activations, called directly:
// C[M, N] = A[M, K] * W[N, K]^T with bf16 operands, fp32 accumulation, bf16 or fp32 output, as
// the reference leaves its products to the library (serve/model.py:80-82,95,97,159).  A step that
// is launched kernel by kernel calls this a hundred times, so what a call costs on the host counts:
// the descriptors and the algorithm of a shape are looked up once and kept (a plan per device, M, N,
// K and output type), and a call is one hipblasLtMatmul with them.  Nothing is allocated here: the
// caller brings the workspace.  The library handle of a device and the plans live until the process
// ends.
//
// Row-major C = A W^T is, in the column-major terms of the library, C^T[N, M] = op_T(W) A^T with W
// seen as a K x N matrix of leading dimension K and A as a K x M matrix of leading dimension K.
#include "common.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  int failed = 0;            // the error of a shape that could not be planned (then nothing else is set)
};

constexpr int MAX_DEVICES = 64;
std::mutex mu;
hipblasLtHandle_t handles[MAX_DEVICES] = {};
std::map<std::tuple<int, int, int, int, int, size_t>, Plan> plans;   // (device, M, N, K, c_dtype, workspace) -> plan

#define LT_CHECK(call)                                   \
  do {                                                   \
    hipblasStatus_t st__ = (call);                       \
    if (st__ != HIPBLAS_STATUS_SUCCESS) return 1000 + (int)st__; \
  } while (0)

void destroy_plan(Plan* plan) {
  if (plan->desc) hipblasLtMatmulDescDestroy(plan->desc);
  if (plan->w) hipblasLtMatrixLayoutDestroy(plan->w);
  if (plan->a) hipblasLtMatrixLayoutDestroy(plan->a);
  if (plan->c) hipblasLtMatrixLayoutDestroy(plan->c);
  plan->desc = nullptr;
  plan->w = plan->a = plan->c = nullptr;
}

int fill_plan(hipblasLtHandle_t handle, int M, int N, int K, int c_dtype, size_t workspace_bytes, Plan* plan) {
  const hipDataType out = c_dtype == SA_F32 ? HIP_R_32F : HIP_R_16BF;
  LT_CHECK(hipblasLtMatmulDescCreate(&plan->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const int32_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
  LT_CHECK(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)));
  LT_CHECK(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)));
  LT_CHECK(hipblasLtMatrixLayoutCreate(&plan->w, HIP_R_16BF, K, N, K));
  LT_CHECK(hipblasLtMatrixLayoutCreate(&plan->a, HIP_R_16BF, K, M, K));
  LT_CHECK(hipblasLtMatrixLayoutCreate(&plan->c, out, N, M, N));
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_CHECK(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t ws = workspace_bytes;
  hipblasStatus_t st = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws,
                                                             sizeof(ws));
  hipblasLtMatmulHeuristicResult_t result;
  int found = 0;
  if (st == HIPBLAS_STATUS_SUCCESS)
    st = hipblasLtMatmulAlgoGetHeuristic(handle, plan->desc, plan->w, plan->a, plan->c, plan->c, pref, 1, &result,
                                         &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS) return 1000 + (int)st;
  if (found < 1 || result.state != HIPBLAS_STATUS_SUCCESS) return SA_ERR_UNSUPPORTED;
  plan->algo = result.algo;
  plan->workspace = result.workspaceSize;
  return 0;
}

// the plan of a shape, made at its first call (the lock is held).  A shape that cannot be planned
// keeps its error code (`failed`) and nothing else, so that it is neither planned again at every
// call nor leaves descriptors behind.
int make_plan(hipblasLtHandle_t handle, int M, int N, int K, int c_dtype, size_t workspace_bytes, Plan* plan) {
  const int rc = fill_plan(handle, M, N, K, c_dtype, workspace_bytes, plan);
  if (rc != 0) destroy_plan(plan);
  plan->failed = rc;
  return rc;
}

}  // namespace

// C = A W^T through hipBLASLt.  c_dtype SA_BF16 or SA_F32; `workspace` of `workspace_bytes` bytes is
// the library's scratch memory (calls that share it run in one stream).  Returns 0, an SA_ERR code,
// or 1000 + the library's status.
extern "C" int sa_blaslt_mm(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, void* workspace,
                            size_t workspace_bytes, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || !A || !W || !C || (c_dtype != SA_F32 && c_dtype != SA_BF16)) return SA_ERR_ARG;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return SA_ERR_ARG;
  hipblasLtHandle_t handle;
  const Plan* plan;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!handles[dev]) LT_CHECK(hipblasLtCreate(&handles[dev]));
    handle = handles[dev];
    const auto key = std::make_tuple(dev, M, N, K, c_dtype, workspace_bytes);
    auto it = plans.find(key);
    if (it == plans.end()) {
      Plan fresh;
      make_plan(handle, M, N, K, c_dtype, workspace_bytes, &fresh);
      it = plans.emplace(key, fresh).first;
    }
    plan = &it->second;                      // (entries of a std::map stay where they are)
    if (plan->failed != 0) return plan->failed;
  }
  if (plan->workspace > workspace_bytes) return SA_ERR_ARG;
  const float one = 1.f, zero = 0.f;
  LT_CHECK(hipblasLtMatmul(handle, plan->desc, &one, W, plan->w, A, plan->a, &zero, C, plan->c, C, plan->c,
                           &plan->algo, workspace, workspace_bytes, stream));
  return 0;
}
