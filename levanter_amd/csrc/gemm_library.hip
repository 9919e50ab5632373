// The vendor library's matrix product (hipBLASLt) behind the interface of lev_linear_mfma, for prompt-sized row counts:
//   y = act(a . w^T + bias) (+ residual),  a [M, K] bf16 (row stride lda), w [N, K] bf16, y [M, N] bf16 or f32.
// The reference leaves every matrix product to its compiler's library; here the library takes the large tiles
// (hundreds to thousands of rows), where its tuned kernels are ahead of gemm_tile_kernel on most shapes, and only
// with epilogues it has itself: bias, the tanh GELU ("gelu_new"), ReLU, and the residual as the C operand with beta = 1.
// Everything else (other activations, shapes it has no kernel for) returns LEV_LIBRARY_UNSUPPORTED and the caller
// runs the hand-written kernel. In the library's column-major terms the row-major problem is
//   D^T [N x M] = w_cm^T [N x K] . a_cm [K x M]  (+ C^T),  with w_cm = w seen as K x N (ld K), a_cm = a seen as K x M (ld lda),
// so that the bias, one value per row of D^T, is the per-output-column bias of the row-major result.
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

#define LEV_LIBRARY_UNSUPPORTED 1
#define LEV_LIB_MAX_DEVICES 64

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t lw = nullptr, la = nullptr, lc = nullptr, ld = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool ok = false;
};

// (device, M, N, K, lda, ldr, ldo, epilogue, output dtype, residual?)
typedef std::tuple<int, int, int, int, long, long, long, int, int, int> PlanKey;

std::mutex g_mutex;
hipblasLtHandle_t g_handle[LEV_LIB_MAX_DEVICES];
std::map<PlanKey, Plan> g_plans;

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

#define LIB_CHECK(call)                                                                                         \
  do {                                                                                                          \
    hipblasStatus_t s_ = (call);                                                                                \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return lev_fail("linear (library): %s: %s", #call, status_name(s_));       \
  } while (0)

int epilogue_of(int act, bool bias, uint32_t* out) {
  if (act == LEV_ACT_NONE) *out = bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT;
  else if (act == LEV_ACT_GELU_TANH) *out = bias ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_GELU;
  else if (act == LEV_ACT_RELU) *out = bias ? HIPBLASLT_EPILOGUE_RELU_BIAS : HIPBLASLT_EPILOGUE_RELU;
  else return LEV_LIBRARY_UNSUPPORTED;
  return 0;
}

int make_plan(hipblasLtHandle_t handle, Plan* p, int M, int N, int K, long lda, long ldr, long ldo, uint32_t epilogue, bool bias,
              bool residual, hipDataType out_type, size_t max_workspace) {
  LIB_CHECK(hipblasLtMatmulDescCreate(&p->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const int32_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
  LIB_CHECK(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)));
  LIB_CHECK(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)));
  LIB_CHECK(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)));
  if (bias) {
    const int32_t bias_type = HIP_R_32F;
    LIB_CHECK(hipblasLtMatmulDescSetAttribute(p->desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)));
  }
  LIB_CHECK(hipblasLtMatrixLayoutCreate(&p->lw, HIP_R_16BF, K, N, K));
  LIB_CHECK(hipblasLtMatrixLayoutCreate(&p->la, HIP_R_16BF, K, M, lda));
  LIB_CHECK(hipblasLtMatrixLayoutCreate(&p->lc, out_type, N, M, residual ? ldr : ldo));
  LIB_CHECK(hipblasLtMatrixLayoutCreate(&p->ld, out_type, N, M, ldo));
  hipblasLtMatmulPreference_t pref = nullptr;
  LIB_CHECK(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t ws = max_workspace;
  hipblasStatus_t s = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  hipblasLtMatmulHeuristicResult_t result[1];
  int found = 0;
  if (s == HIPBLAS_STATUS_SUCCESS)
    s = hipblasLtMatmulAlgoGetHeuristic(handle, p->desc, p->lw, p->la, p->lc, p->ld, pref, 1, result, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || found < 1) return LEV_LIBRARY_UNSUPPORTED;  // p->ok stays false: remembered, not asked again
  p->algo = result[0].algo;
  p->workspace = result[0].workspaceSize;
  p->ok = true;
  return 0;
}

}  // namespace

// Bytes of workspace the caller must bring (one size for every shape: the heuristic is asked for kernels within it).
extern "C" long lev_linear_library_workspace() { return 64L << 20; }

// Returns 0 (done), LEV_LIBRARY_UNSUPPORTED (nothing was launched: run the hand-written kernel) or -1 with a message.
extern "C" int lev_linear_library(const void* a, long lda, const void* w, const float* bias, const float* residual, long ldr,
                                  void* out, long ldo, void* workspace, long workspace_bytes, int M, int N, int K, int act,
                                  int out_dtype, hipStream_t stream) {
  LEV_REQUIRE(M > 0 && N > 0 && K > 0, "linear (library): bad sizes M=%d N=%d K=%d", M, N, K);
  LEV_REQUIRE(lda >= K && ldo >= N, "linear (library): row strides lda=%ld ldo=%ld are smaller than K=%d / N=%d", lda, ldo, K, N);
  LEV_REQUIRE(!residual || (ldr >= N && out_dtype == LEV_F32), "linear (library): a residual needs a float32 output and a row stride >= N");
  LEV_REQUIRE(out_dtype == LEV_F32 || out_dtype == LEV_BF16, "linear (library): unknown output dtype %d", out_dtype);
  uint32_t epilogue;
  if (epilogue_of(act, bias != nullptr, &epilogue)) return LEV_LIBRARY_UNSUPPORTED;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LEV_LIB_MAX_DEVICES) return lev_fail("linear (library): no current device");
  Plan plan;
  hipblasLtHandle_t handle;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_handle[dev]) LIB_CHECK(hipblasLtCreate(&g_handle[dev]));
    handle = g_handle[dev];
    const PlanKey key(dev, M, N, K, lda, residual ? ldr : 0, ldo, (int)epilogue, out_dtype, residual ? 1 : 0);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
      Plan p;
      const int rc = make_plan(handle, &p, M, N, K, lda, ldr, ldo, epilogue, bias != nullptr, residual != nullptr,
                               out_dtype == LEV_F32 ? HIP_R_32F : HIP_R_16BF, (size_t)workspace_bytes);
      if (rc < 0) return rc;
      it = g_plans.emplace(key, p).first;
    }
    plan = it->second;
  }
  if (!plan.ok) return LEV_LIBRARY_UNSUPPORTED;
  if (plan.workspace > (size_t)workspace_bytes || (plan.workspace > 0 && !workspace))
    return lev_fail("linear (library): the chosen kernel needs %zu bytes of workspace, %ld were brought", plan.workspace, workspace_bytes);
  if (bias) {  // the descriptor is shared by every call of this shape: the pointer is set under the lock, with the launch
    std::lock_guard<std::mutex> lock(g_mutex);
    const void* bp = bias;
    LIB_CHECK(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)));
    const float alpha = 1.0f, beta = residual ? 1.0f : 0.0f;
    LIB_CHECK(hipblasLtMatmul(handle, plan.desc, &alpha, w, plan.lw, a, plan.la, &beta, residual ? (const void*)residual : (const void*)out,
                              plan.lc, out, plan.ld, &plan.algo, workspace, plan.workspace, stream));
    return 0;
  }
  const float alpha = 1.0f, beta = residual ? 1.0f : 0.0f;
  LIB_CHECK(hipblasLtMatmul(handle, plan.desc, &alpha, w, plan.lw, a, plan.la, &beta, residual ? (const void*)residual : (const void*)out,
                            plan.lc, out, plan.ld, &plan.algo, workspace, plan.workspace, stream));
  return 0;
}
