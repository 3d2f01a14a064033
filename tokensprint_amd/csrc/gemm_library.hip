// Plain bfloat16 products with many rows, handed to the vendor library (hipBLASLt), as the
// reference hands every linear layer to its vendor library (engine/nn/base_layers.py:7-10).
// Called here directly rather than through the tensor framework: a plan (operation and
// layout descriptors, the algorithm the library's heuristic picks) is made once per
// (rows, columns, inner size, output type) and kept, so a call costs the launch and little
// else on the host; through the framework's matmul a call cost 18 us, more than most of
// these products run, and a prompt's step was bound by the host.
//
// C[M, N] = A[M, K] W[N, K]^T, all row-major.  To the library, which thinks in columns,
// that is C^T [N x M] = W^T-as-stored [K x N]^T * A-as-stored [K x M].
#include <hipblaslt/hipblaslt.h>

#include <mutex>
#include <unordered_map>

#include "common.h"

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

constexpr int kMaxDevices = 64;
hipblasLtHandle_t g_handle[kMaxDevices];
std::unordered_map<uint64_t, Plan> g_plans[kMaxDevices];
std::mutex g_mutex;

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

#define TS_BLAS(call)                                                          \
  do {                                                                         \
    hipblasStatus_t s_ = (call);                                               \
    if (s_ != HIPBLAS_STATUS_SUCCESS) TS_FAIL("gemm_library: %s: %s", #call, status_name(s_)); \
  } while (0)

int g_candidates = 1;      // algorithms of the heuristic's list that a plan is chosen from

// Seconds per call of one algorithm on the call's own operands (C is overwritten with the
// same product every time), or a negative number if the library refuses it.  Before every
// timed call `flush` is overwritten: a decode step reads each weight once, from HBM, and a
// weight left in the memory-side cache by the call before would favour other algorithms
// than the ones that are fastest then.
double time_algo(hipblasLtHandle_t handle, const Plan& p, const hipblasLtMatmulAlgo_t& algo,
                 const void* a, const void* w, void* c, void* workspace, size_t workspace_bytes,
                 void* flush, size_t flush_bytes, hipStream_t stream) {
  const float alpha = 1.f, beta = 0.f;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return -1.;
  if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return -1.; }
  double best = -1.;
  for (int i = 0; i < 4; ++i) {         // the first call is a warm-up (code, descriptors)
    bool ok = flush == nullptr || hipMemsetAsync(flush, i, flush_bytes, stream) == hipSuccess;
    ok = ok && hipEventRecord(e0, stream) == hipSuccess;
    ok = ok && hipblasLtMatmul(handle, p.desc, &alpha, w, p.w, a, p.a, &beta, c, p.c, c, p.c, &algo,
                               workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
    float ms = 0.f;
    ok = ok && hipEventRecord(e1, stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
         hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    if (!ok) { best = -1.; break; }
    if (i > 0 && (best < 0. || ms * 1e-3 < best)) best = ms * 1e-3;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return best;
}

// The plan of one (rows, columns, inner size, output type).  The heuristic's first choice
// is mostly right, but for a few rows against a large weight (decode steps of 9 to 64
// requests at the 8B and 32B shapes) it has been seen at a third of the rate of the list's
// best, and for 8,192 rows at N = 5,120 at three quarters.  So where the caller has asked
// for it (ts_gemm_library_candidates: the engine does during its warm-up, whose largest
// step and captured decode steps have the shapes the run is made of) the first entries of
// the list are run on the call's own operands and the fastest is kept, for weights from
// 2^20 elements.  Timing costs ten to a hundred milliseconds a plan, too much for a shape
// that a step meets once.  Under stream capture nothing can be timed and the first
// choice stands.
int make_plan(hipblasLtHandle_t handle, Plan& p, int M, int N, int K, int c_type,
              size_t workspace_bytes, const void* a, const void* w, void* c, void* workspace,
              hipStream_t stream) {
  const hipDataType out = c_type == TS_BF16 ? HIP_R_16BF : HIP_R_32F;
  TS_BLAS(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const hipblasOperation_t t = HIPBLAS_OP_T, n = HIPBLAS_OP_N;
  TS_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &t, sizeof(t)));
  TS_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &n, sizeof(n)));
  TS_BLAS(hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K));
  TS_BLAS(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, M, K));
  TS_BLAS(hipblasLtMatrixLayoutCreate(&p.c, out, N, M, N));
  hipblasLtMatmulPreference_t pref = nullptr;
  TS_BLAS(hipblasLtMatmulPreferenceCreate(&pref));
  TS_BLAS(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES,
                                                &workspace_bytes, sizeof(workspace_bytes)));
  constexpr int kMost = 16;
  hipblasLtMatmulHeuristicResult_t found[kMost];
  int count = 0;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  const bool tune = g_candidates > 1 && (int64_t)N * K >= (1 << 20) &&
                    hipStreamIsCapturing(stream, &capturing) == hipSuccess &&
                    capturing == hipStreamCaptureStatusNone;
  const int ask = tune ? (g_candidates < kMost ? g_candidates : kMost) : 1;
  const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.w, p.a, p.c, p.c,
                                                            pref, ask, found, &count);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || count < 1)
    TS_FAIL("gemm_library: the library has no algorithm for M=%d N=%d K=%d (%s)", M, N, K,
            status_name(s));
  int best = 0;
  if (tune && count > 1) {
    // larger than the memory-side cache; given back before this returns
    const size_t flush_bytes = (size_t)512 << 20;
    void* flush = nullptr;
    if (hipMalloc(&flush, flush_bytes) != hipSuccess) {
      (void)hipGetLastError();
      flush = nullptr;
    }
    // the first choice stands unless another is ahead by more than the timing's noise
    double best_seconds = -1.;
    for (int i = 0; i < count; ++i) {
      if (found[i].workspaceSize > workspace_bytes) continue;
      const double sec = time_algo(handle, p, found[i].algo, a, w, c, workspace, workspace_bytes,
                                   flush, flush_bytes, stream);
      if (sec <= 0.) continue;
      if (best_seconds < 0. || sec < 0.95 * best_seconds) { best_seconds = sec; best = i; }
    }
    if (flush != nullptr) {
      (void)hipStreamSynchronize(stream);
      (void)hipFree(flush);
    }
  }
  p.algo = found[best].algo;
  p.workspace = found[best].workspaceSize;
  return 0;
}

}  // namespace

// How many entries of the heuristic's list a plan for few rows is chosen from by timing
// them, from now on (1, the default: the first is taken untimed).  Plans already made keep
// their choice.
extern "C" void ts_gemm_library_candidates(int n) { g_candidates = n < 1 ? 1 : n; }

// `workspace`: device memory of `workspace_bytes` for the library's use during the call,
// the same for every call on a stream (calls on one stream run one after the other).
extern "C" int ts_gemm_library_bf16(const void* a, const void* w, void* c, int c_type, int M,
                                    int N, int K, void* workspace, size_t workspace_bytes,
                                    hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) TS_FAIL("gemm_library: K=%d", K);
  if (c_type != TS_BF16 && c_type != TS_F32) TS_FAIL("gemm_library: output type %d", c_type);
  if (((uintptr_t)a | (uintptr_t)w | (uintptr_t)c) & 15)
    TS_FAIL("gemm_library: operands must be 16-byte aligned");
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
    TS_FAIL("gemm_library: no current device below %d", kMaxDevices);
  Plan* plan;
  hipblasLtHandle_t handle;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_handle[device] == nullptr) TS_BLAS(hipblasLtCreate(&g_handle[device]));
    handle = g_handle[device];
    const uint64_t key = ((uint64_t)M << 42) ^ ((uint64_t)N << 21) ^ (uint64_t)K ^ ((uint64_t)c_type << 63);
    if ((uint64_t)M >= (1u << 21) || (uint64_t)N >= (1u << 21) || (uint64_t)K >= (1u << 21))
      TS_FAIL("gemm_library: a size beyond 2^21 (M=%d N=%d K=%d)", M, N, K);
    auto it = g_plans[device].find(key);
    if (it == g_plans[device].end()) {
      Plan p;
      if (make_plan(handle, p, M, N, K, c_type, workspace_bytes, a, w, c, workspace, stream)) return -1;
      it = g_plans[device].emplace(key, p).first;
    }
    plan = &it->second;     // entries of an unordered_map stay where they are
  }
  if (plan->workspace > workspace_bytes)
    TS_FAIL("gemm_library: the algorithm wants %zu bytes of workspace, %zu given", plan->workspace,
            workspace_bytes);
  const float alpha = 1.f, beta = 0.f;
  TS_BLAS(hipblasLtMatmul(handle, plan->desc, &alpha, w, plan->w, a, plan->a, &beta, c, plan->c, c,
                          plan->c, &plan->algo, workspace, workspace_bytes, stream));
  return 0;
}
