// The vendor library's matrix product (hipBLASLt) behind the interface of lev_linear_mfma, for prompt-sized row counts:
//   y = act(a . w^T + bias) (+ residual),  a [M, K] bf16 (row stride lda), w [N, K] bf16, y [M, N] bf16 or f32.
// The reference leaves every matrix product to its compiler's library; here the library takes the large tiles
// (hundreds to thousands of rows), where its tuned kernels are ahead of gemm_tile_kernel on most shapes, and only
// with epilogues it has itself: bias, the tanh GELU ("gelu_new"), ReLU, and the residual as the C operand with beta = 1.
// Everything else (other activations, shapes it has no kernel for) returns LEV_LIBRARY_UNSUPPORTED and the caller
// runs the hand-written kernel. Which of the library's kernels runs a shape is not left to its heuristic alone: for
// 256 rows and more the heuristic's candidates are timed once (its first choice is up to twice slower than its best on row
// counts that are no multiple of the tile, 2,052 rows for instance); the other row counts up to the same multiple of 64 try
// only that kernel against the heuristic's first. In the library's column-major terms the row-major problem is
//   D^T [N x M] = w_cm^T [N x K] . a_cm [K x M]  (+ C^T),  with w_cm = w seen as K x N (ld K), a_cm = a seen as K x M (ld lda),
// so that the bias, one value per row of D^T, is the per-output-column bias of the row-major result.
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <chrono>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"

#define LEV_LIBRARY_UNSUPPORTED 1
#define LEV_LIB_MAX_DEVICES 64
#define LEV_LIB_CANDIDATES 16    // kernels asked of the heuristic for one shape
#define LEV_LIB_TUNE_MIN_ROWS 256  // below, a product is bound by reading its weight and a timing loop over one weight
                                   // (which then sits in the last-level cache) says nothing about the real step
#define LEV_LIB_TUNE_RUNS 4
#define LEV_LIB_ROW_BUCKET 64      // row counts up to the same multiple of this share one timing

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t lw = nullptr, la = nullptr, lc = nullptr, ld = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool ok = false;
  bool timed = false;  // the candidates have been timed on this shape and algo is the fastest of them
  std::vector<hipblasLtMatmulHeuristicResult_t> candidates;  // in the heuristic's order; algo starts as the first
};

// (device, M, N, K, lda, ldr, ldo, epilogue, output dtype, residual?)
typedef std::tuple<int, int, int, int, long, long, long, int, int, int> PlanKey;

std::mutex g_mutex;
hipblasLtHandle_t g_handle[LEV_LIB_MAX_DEVICES];
std::map<PlanKey, Plan> g_plans;
// What timing chose, by PlanKey with the row count replaced by its bucket (rows_bucket): the library's index of the kernel.
// Row counts of one bucket share it, so a serving run whose steps differ by a few rows times once, not once a row count.
std::map<PlanKey, int> g_timed_index;

int rows_bucket(int M) { return (M + LEV_LIB_ROW_BUCKET - 1) / LEV_LIB_ROW_BUCKET; }

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
  hipblasLtMatmulHeuristicResult_t result[LEV_LIB_CANDIDATES];
  int found = 0;
  if (s == HIPBLAS_STATUS_SUCCESS)
    s = hipblasLtMatmulAlgoGetHeuristic(handle, p->desc, p->lw, p->la, p->lc, p->ld, pref, LEV_LIB_CANDIDATES, result, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || found < 1) return LEV_LIBRARY_UNSUPPORTED;  // p->ok stays false: remembered, not asked again
  for (int i = 0; i < found; ++i)
    if (result[i].state == HIPBLAS_STATUS_SUCCESS && result[i].workspaceSize <= max_workspace) p->candidates.push_back(result[i]);
  if (p->candidates.empty()) return LEV_LIBRARY_UNSUPPORTED;
  p->algo = p->candidates[0].algo;
  p->workspace = p->candidates[0].workspaceSize;
  p->ok = true;
  return 0;
}

// 0: the heuristic's first kernel is taken; 1 (default): the candidates of a shape are timed at its first call outside a
// stream capture and the fastest is kept; 2: the timings are printed as well.
int tune_level() {
  static const int level = [] {
    const char* e = getenv("LEVANTER_AMD_GEMM_TUNE");
    return e ? atoi(e) : 1;
  }();
  return level;
}

// A buffer larger than the caches (32 MB of L2, 256 MB behind them), one per device, kept for the life of the process:
// sweeping it between two timed runs leaves nothing of the operands in a cache.
#define LEV_LIB_FLUSH_BYTES ((size_t)512 << 20)
void* flush_buffer() {
  static std::map<int, void*> buffers;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  auto it = buffers.find(dev);
  if (it != buffers.end()) return it->second;
  void* p = nullptr;
  if (hipMalloc(&p, LEV_LIB_FLUSH_BYTES) != hipSuccess) { (void)hipGetLastError(); p = nullptr; }
  buffers[dev] = p;
  return p;
}

// Times the given kernels on the call's own operands, writing to a buffer of its own (a product into the residual stream
// adds to its output, so the real output cannot take repeated runs), and gives the plan the fastest. The heuristic's order
// is a table look-up by size; on this chip its first kernel is often not the fastest one for the shape at hand.
// Allocates and synchronises: called only outside a stream capture. Returns the library's index of the kernel kept, or -1.
int time_candidates(hipblasLtHandle_t handle, Plan* p, const std::vector<hipblasLtMatmulHeuristicResult_t>& candidates, const void* a,
                    const void* w, const float* residual, void* workspace, int M, int N, long ldo, int out_dtype, hipStream_t stream) {
  p->timed = true;
  if (candidates.size() < 2) return -1;
  auto t_begin = std::chrono::steady_clock::now();
  const size_t bytes = (size_t)M * (size_t)ldo * (out_dtype == LEV_F32 ? 4 : 2);
  void* scratch = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipMalloc(&scratch, bytes) != hipSuccess) { (void)hipGetLastError(); return -1; }
  void* flush = flush_buffer();  // null if it could not be had: the runs are then timed on a warm weight
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    (void)hipGetLastError();
    if (e0) (void)hipEventDestroy(e0);
    (void)hipFree(scratch);
    return -1;
  }
  const float alpha = 1.0f, beta = residual ? 1.0f : 0.0f;
  const void* c = residual ? (const void*)residual : (const void*)scratch;
  float best = -1.0f;
  int best_i = 0;
  for (size_t i = 0; i < candidates.size(); ++i) {
    const hipblasLtMatmulHeuristicResult_t& cand = candidates[i];
    bool ok = true;
    float ms = -1.0f;
    // Every timed run behind a sweep over a buffer larger than the caches: in a model's step a product's weight has not
    // been touched since the step before, and the kernel that is fastest on a weight that waits in the last-level cache
    // (what a plain loop over one weight measures) is often not the fastest on one that comes from memory. The fastest
    // of the runs counts.
    for (int run = 0; run <= LEV_LIB_TUNE_RUNS && ok; ++run) {  // run 0 loads the kernel and is not timed
      if (run > 0) ok = (!flush || hipMemsetAsync(flush, run, LEV_LIB_FLUSH_BYTES, stream) == hipSuccess) &&
                        hipEventRecord(e0, stream) == hipSuccess;
      ok = ok && hipblasLtMatmul(handle, p->desc, &alpha, w, p->lw, a, p->la, &beta, c, p->lc, scratch, p->ld, &cand.algo, workspace,
                                 cand.workspaceSize, stream) == HIPBLAS_STATUS_SUCCESS;
      if (run > 0) {
        float t = 0.0f;
        ok = ok && hipEventRecord(e1, stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
             hipEventElapsedTime(&t, e0, e1) == hipSuccess;
        if (ok && (ms < 0.0f || t < ms)) ms = t;
      }
    }
    if (!ok || ms < 0.0f) { (void)hipGetLastError(); (void)hipStreamSynchronize(stream); continue; }
    if (tune_level() >= 2) {
      hipblasLtMatmulAlgo_t algo = cand.algo;
      fprintf(stderr, "linear (library) M=%d N=%d: candidate %zu (kernel %d) %.1f us\n", M, N, i, hipblaslt_ext::getIndexFromAlgo(algo),
              ms * 1000.0f);
    }
    if (best < 0.0f || ms < best) { best = ms; best_i = (int)i; }
  }
  if (best >= 0.0f) {
    p->algo = candidates[best_i].algo;
    p->workspace = candidates[best_i].workspaceSize;
    if (tune_level() >= 2)
      fprintf(stderr, "linear (library) M=%d N=%d: kept candidate %d after %.1f ms\n", M, N, best_i,
              std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t_begin).count());
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipStreamSynchronize(stream);
  (void)hipFree(scratch);
  return best >= 0.0f ? hipblaslt_ext::getIndexFromAlgo(p->algo) : -1;
}

// The kernel that timing chose for another row count of the plan's bucket, if the heuristic offers it for this row count
// too. (Asking the library for a kernel by its index instead makes it load its whole catalogue: a second at its first use.)
const hipblasLtMatmulHeuristicResult_t* candidate_of_index(const Plan* p, int index) {
  for (const hipblasLtMatmulHeuristicResult_t& cand : p->candidates) {
    hipblasLtMatmulAlgo_t algo = cand.algo;
    if (hipblaslt_ext::getIndexFromAlgo(algo) == index) return &cand;
  }
  return nullptr;
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
  // One lock for the look-up, the bias pointer (the descriptor is shared by every call of this shape) and the launch.
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_handle[dev]) LIB_CHECK(hipblasLtCreate(&g_handle[dev]));
  hipblasLtHandle_t handle = g_handle[dev];
  const PlanKey key(dev, M, N, K, lda, residual ? ldr : 0, ldo, (int)epilogue, out_dtype, residual ? 1 : 0);
  auto it = g_plans.find(key);
  if (it == g_plans.end()) {
    Plan p;
    const int rc = make_plan(handle, &p, M, N, K, lda, ldr, ldo, epilogue, bias != nullptr, residual != nullptr,
                             out_dtype == LEV_F32 ? HIP_R_32F : HIP_R_16BF, (size_t)workspace_bytes);
    if (rc < 0) return rc;
    it = g_plans.emplace(key, p).first;
  }
  Plan& plan = it->second;
  if (!plan.ok) return LEV_LIBRARY_UNSUPPORTED;
  if (bias) {
    const void* bp = bias;
    LIB_CHECK(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)));
  }
  if (!plan.timed && M >= LEV_LIB_TUNE_MIN_ROWS && tune_level() >= 1) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) { (void)hipGetLastError(); capturing = hipStreamCaptureStatusActive; }
    const bool may_time = capturing == hipStreamCaptureStatusNone;
    const PlanKey bucket(dev, rows_bucket(M), N, K, lda, residual ? ldr : 0, ldo, (int)epilogue, out_dtype, residual ? 1 : 0);
    auto known = g_timed_index.find(bucket);
    if (known == g_timed_index.end()) {
      if (may_time)
        g_timed_index[bucket] = time_candidates(handle, &plan, plan.candidates, a, w, residual, workspace, M, N, ldo, out_dtype, stream);
      else
        plan.timed = true;  // recorded into a graph with the heuristic's first kernel: eager calls of this shape keep it too,
                            // so that a replay and an eager run of the same product give the same bits
    } else {
      // Another row count of the bucket has been timed: its kernel against the heuristic's first for this row count (a
      // kernel that won at 264 rows can lose at 320, where its tiles divide the rows differently), not all sixteen again.
      plan.timed = true;  // whether the bucket's kernel is on offer or not: the plan is settled
      const hipblasLtMatmulHeuristicResult_t* theirs = known->second >= 0 ? candidate_of_index(&plan, known->second) : nullptr;
      if (tune_level() >= 2)
        fprintf(stderr, "linear (library) M=%d N=%d K=%d: kernel %d of its bucket is %s\n", M, N, K, known->second,
                theirs == &plan.candidates[0] ? "the heuristic's first" : (theirs ? "on offer" : "not on offer"));
      if (theirs && theirs != &plan.candidates[0]) {
        if (may_time) {
          std::vector<hipblasLtMatmulHeuristicResult_t> two = {*theirs, plan.candidates[0]};
          time_candidates(handle, &plan, two, a, w, residual, workspace, M, N, ldo, out_dtype, stream);
        } else {
          plan.algo = theirs->algo;
          plan.workspace = theirs->workspaceSize;
        }
      } else if (!theirs && may_time) {
        // the bucket's kernel is not offered for this row count: its own candidates then (the heuristic's first was up to
        // a third slower than their best at 304 and 320 rows of a 1600-wide layer, whose bucket was timed at 272)
        time_candidates(handle, &plan, plan.candidates, a, w, residual, workspace, M, N, ldo, out_dtype, stream);
      }
    }
  }
  if (plan.workspace > 0 && !workspace)
    return lev_fail("linear (library): the chosen kernel needs %zu bytes of workspace, none was brought", plan.workspace);
  const float alpha = 1.0f, beta = residual ? 1.0f : 0.0f;
  LIB_CHECK(hipblasLtMatmul(handle, plan.desc, &alpha, w, plan.lw, a, plan.la, &beta, residual ? (const void*)residual : (const void*)out,
                            plan.lc, out, plan.ld, &plan.algo, workspace, plan.workspace, stream));
  return 0;
}
