// Products of many rows: y = x . w^T in the vendor library (hipBLASLt), called directly.
// The reference hands the same products to its vendor library (yalis/external/model.py:449,
// 462-466, 717-722).  What this file adds to a plain library call: the descriptors and the
// chosen algorithm of every shape are kept, so that a call costs the host a few microseconds
// (through torch's matrix product it is about 19, four times a layer, which is what bounds a
// step of a prompt portion at the smaller shapes).  By default the algorithm is the library's
// first candidate, the same in every process, so that a step's bits do not depend on the run.
// On request (yk_gemm_library_tune) the candidates of a shape of up to 256 rows of x are timed
// once when the shape is first met and the fastest is kept: there the first is often not the best
// (128 rows at the 8B shapes, us, first / fastest: down-proj 58 / 39, o-proj 20 / 15, qkv 20 / 18),
// while from 512 rows on the first is as fast as any (and is what torch's product runs: the results
// are the same bits); the choice then depends on timing noise and may differ between two runs.
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"

namespace {

struct LtPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace_need = 0;  // scratch the chosen algorithm asks for
  int candidates = 0, chosen = 0;
};

struct LtDevice {
  hipblasLtHandle_t handle = nullptr;
  // (rows, columns, K, the three leading dimensions, float32 output)
  std::map<std::tuple<int, int, int, int, int, int, int>, LtPlan> plans;
};

// A process that meets ever new row counts (every portion length times every matrix of the model)
// would keep a plan for each: beyond this many the plans of a device are dropped and made again
// as their shapes come back (a plan is host memory only; making one takes some tens of microseconds).
constexpr size_t LT_MAX_PLANS = 4096;

void destroy_plan(LtPlan& plan) {
  if (plan.a) hipblasLtMatrixLayoutDestroy(plan.a);
  if (plan.b) hipblasLtMatrixLayoutDestroy(plan.b);
  if (plan.c) hipblasLtMatrixLayoutDestroy(plan.c);
  if (plan.desc) hipblasLtMatmulDescDestroy(plan.desc);
  plan = LtPlan();
}

std::mutex g_lt_mutex;
std::map<int, LtDevice> g_lt_devices;
int g_lt_tune = 0;
constexpr int LT_TUNE_MAX_ROWS = 256;

const char* lt_status(hipblasStatus_t s) {
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

#define LT_TRY(call, what)                                                                  \
  do {                                                                                      \
    hipblasStatus_t s_ = (call);                                                            \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return yk_fail(std::string(what) + ": " + lt_status(s_)); \
  } while (0)

}  // namespace

// 0 (the default): take the library's first candidate for every new shape; 1: for shapes of up to
// 256 rows of x, time its candidates once and keep the fastest.  Shapes already met keep what
// they have.
extern "C" int yk_gemm_library_tune(int on) {
  g_lt_tune = on != 0;
  return 0;
}

// y [M, N] (bfloat16, or float32 with y_dtype YK_F32) = x [M, K] . w [N, K]^T, bfloat16 operands,
// float32 accumulation.  `workspace` is the library's scratch (it may be null with 0 bytes).
// *info, when given, receives candidates * 256 + the index of the one in use.
// Under a graph capture nothing is timed: a shape first met there gets the first candidate.
extern "C" int yk_gemm_library(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int ldx,
                               int ldw, int ldy, void* workspace, size_t workspace_bytes, int* info,
                               hipStream_t stream) {
  YK_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_library: empty product");
  YK_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm_library: a leading dimension is shorter than its row");
  YK_REQUIRE(y_dtype == YK_BF16 || y_dtype == YK_F32, "gemm_library: the result is bfloat16 or float32");
  YK_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(y) % 16 == 0,
             "gemm_library: operands must be 16-byte aligned");
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return yk_fail("gemm_library: no current device");
  std::lock_guard<std::mutex> lock(g_lt_mutex);
  LtDevice& dev = g_lt_devices[device];
  if (!dev.handle) LT_TRY(hipblasLtCreate(&dev.handle), "gemm_library: hipblasLtCreate");
  const auto key = std::make_tuple(M, N, K, ldx, ldw, ldy, y_dtype);
  const float alpha = 1.f, beta = 0.f;
  auto it = dev.plans.find(key);
  if (it == dev.plans.end()) {
    // Row-major y = x . w^T is, in the library's column-major terms, Y (N x M) = W^T . X with
    // W stored K x N (leading dimension ldw) and X stored K x M (leading dimension ldx).
    LtPlan plan;
    struct Guard {  // a plan that fails half-made gives back what it holds
      LtPlan& plan;
      bool kept = false;
      ~Guard() {
        if (!kept) destroy_plan(plan);
      }
    } guard{plan};
    LT_TRY(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "gemm_library: descriptor");
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    LT_TRY(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "gemm_library: transa");
    LT_TRY(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "gemm_library: transb");
    LT_TRY(hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, N, ldw), "gemm_library: layout of w");
    LT_TRY(hipblasLtMatrixLayoutCreate(&plan.b, HIP_R_16BF, K, M, ldx), "gemm_library: layout of x");
    LT_TRY(hipblasLtMatrixLayoutCreate(&plan.c, y_dtype == YK_F32 ? HIP_R_32F : HIP_R_16BF, N, M, ldy), "gemm_library: layout of y");
    hipblasLtMatmulPreference_t pref = nullptr;
    LT_TRY(hipblasLtMatmulPreferenceCreate(&pref), "gemm_library: preference");
    LT_TRY(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes, sizeof(workspace_bytes)),
           "gemm_library: workspace preference");
    constexpr int WANT = 16;
    hipblasLtMatmulHeuristicResult_t found[WANT];
    int n_found = 0;
    hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(dev.handle, plan.desc, plan.a, plan.b, plan.c, plan.c, pref, WANT, found, &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (hs != HIPBLAS_STATUS_SUCCESS || n_found <= 0)
      return yk_fail("gemm_library: the vendor library has no kernel for " + std::to_string(M) + " x " + std::to_string(N) +
                     " x " + std::to_string(K));
    plan.candidates = n_found;
    plan.chosen = 0;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) capturing = hipStreamCaptureStatusNone;
    if (g_lt_tune && M <= LT_TUNE_MAX_ROWS && n_found > 1 && capturing == hipStreamCaptureStatusNone) {
      // every candidate writes the same y (beta is 0), so timing them does no harm
      hipEvent_t e0, e1;
      if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return yk_fail("gemm_library: no events");
      float best = 1e30f;
      for (int c = 0; c < n_found; ++c) {
        if (found[c].workspaceSize > workspace_bytes) continue;
        bool ok = true;
        float ms = 0.f;
        for (int rep = 0; rep < 4 && ok; ++rep) {  // the first run of a kernel is not counted
          if (rep == 1) ok = hipEventRecord(e0, stream) == hipSuccess;
          ok = ok && hipblasLtMatmul(dev.handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, y, plan.c, y, plan.c,
                               &found[c].algo, workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
        }
        if (hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) ok = false;
        if (ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess && ms < best) {
          best = ms;
          plan.chosen = c;
        }
      }
      (void)hipEventDestroy(e0);
      (void)hipEventDestroy(e1);
      (void)hipGetLastError();  // a candidate that failed to launch is simply not chosen
    }
    plan.algo = found[plan.chosen].algo;
    plan.workspace_need = found[plan.chosen].workspaceSize;
    if (dev.plans.size() >= LT_MAX_PLANS) {
      for (auto& kept : dev.plans) destroy_plan(kept.second);
      dev.plans.clear();
    }
    it = dev.plans.emplace(key, plan).first;
    guard.kept = true;
  }
  const LtPlan& plan = it->second;
  // (the plan was made with the workspace of the call that first met the shape)
  if (plan.workspace_need > workspace_bytes)
    return yk_fail("gemm_library: the algorithm kept for this shape needs " + std::to_string(plan.workspace_need) +
                   " bytes of workspace, this call brings " + std::to_string(workspace_bytes));
  if (info) *info = plan.candidates * 256 + plan.chosen;
  LT_TRY(hipblasLtMatmul(dev.handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, y, plan.c, y, plan.c, &plan.algo,
                         workspace, workspace_bytes, stream),
         "gemm_library: hipblasLtMatmul");
  return 0;
}
