// Products of many rows by the vendor's library (hipBLASLt), called directly: Y (M, N) = X (M, K) . W (N, K)^T,
// bfloat16 in and out, float32 sums.  The reference hands its matrix products to the vendor's library as well
// (ext/amdgpu_ops.jl:453-465).
//
// What is kept per shape is a plan: the operation's and the operands' descriptors and the algorithm.  The first
// call of a shape asks the library for its candidate algorithms and, when tuning is asked for, runs each a few
// times on the operands at hand and keeps the fastest (a few milliseconds a shape; which one wins can differ from
// process to process, and with it the rounding of a bfloat16 result, so tuning is for measurements: without it the
// library's first choice runs, the same in every process); every later call is one
// hipblasLtMatmul with what the plan holds, a few microseconds of host time (torch.mm on the same library spends
// 20 to 30 us a call on the host, which is what steps of a few hundred tokens were bound by).
//
// Row-major operands are the library's column-major ones transposed: Y^T (N x M) = W (as K x N, transposed) . X^T
// (K x M).  Nothing here may be recorded into a graph (the library's kernels may clear their workspace with memset
// nodes, and tuning waits for events): a capturing stream is refused.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <algorithm>
#include <vector>
#include <map>
#include <mutex>
#include <tuple>

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  int candidates = 0;
  float best_us = 0.f;
};

typedef std::tuple<int, int, int, int, int, int, size_t, int> PlanKey;   // device, M, N, K, ldx, ldy, workspace bytes, tuned

std::mutex g_mutex;
std::map<PlanKey, Plan> g_plans;
std::map<int, hipblasLtHandle_t> g_handles;

// What the tuning runs overwrite between two measurements: more than the 256 MB of the memory-side cache.  One per
// device, allocated at the first tuning run and kept; without it (no memory) the measurements run on warm operands.
constexpr size_t FLUSH_BYTES = 384u << 20;
std::map<int, void*> g_flush;

void* flush_buffer() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  auto it = g_flush.find(dev);
  if (it != g_flush.end()) return it->second;
  void* p = nullptr;
  if (hipMalloc(&p, FLUSH_BYTES) != hipSuccess) {
    (void)hipGetLastError();
    p = nullptr;
  }
  g_flush[dev] = p;
  return p;
}

const char* status_name(hipblasStatus_t s) {
  switch (s) {
    case HIPBLAS_STATUS_SUCCESS: return "success";
    case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialized";
    case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
    case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
    case HIPBLAS_STATUS_ARCH_MISMATCH: return "architecture mismatch";
    case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
    case HIPBLAS_STATUS_INTERNAL_ERROR: return "internal error";
    case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
    default: return "error";
  }
}

#define LT_REQUIRE(call, what)                                                          \
  do {                                                                                  \
    hipblasStatus_t s_ = (call);                                                        \
    if (s_ != HIPBLAS_STATUS_SUCCESS) {                                                 \
      gs_set_error("library_gemm: %s: %s (%d)", what, status_name(s_), (int)s_);        \
      return -3;                                                                        \
    }                                                                                   \
  } while (0)

int run(hipblasLtHandle_t handle, const Plan& p, const void* X, const void* W, void* Y, void* ws, hipStream_t stream) {
  const float one = 1.f, zero = 0.f;
  LT_REQUIRE(hipblasLtMatmul(handle, p.desc, &one, W, p.a, X, p.b, &zero, Y, p.c, Y, p.c, &p.algo, ws, p.workspace, stream),
             "the product");
  return 0;
}

void destroy_plan(Plan& p) {
  if (p.desc) (void)hipblasLtMatmulDescDestroy(p.desc);
  if (p.a) (void)hipblasLtMatrixLayoutDestroy(p.a);
  if (p.b) (void)hipblasLtMatrixLayoutDestroy(p.b);
  if (p.c) (void)hipblasLtMatrixLayoutDestroy(p.c);
  p.desc = nullptr;
  p.a = p.b = p.c = nullptr;
}

// At most this many plans are kept.  A server sees a new row count in almost every step of mixed work; when the table is
// full the plans that were not tuned go (making one again costs some tens of microseconds), the tuned ones stay.
constexpr size_t MAX_PLANS = 512;

void make_room() {
  if (g_plans.size() < MAX_PLANS) return;
  for (auto it = g_plans.begin(); it != g_plans.end();) {
    if (std::get<7>(it->first) == 0) {
      destroy_plan(it->second);
      it = g_plans.erase(it);
    } else {
      ++it;
    }
  }
}

// Fills `p`; on failure whatever it has created so far is left in `p` for the caller to destroy.
int make_plan(hipblasLtHandle_t handle, Plan& p, const void* X, int ldx, const void* W, void* Y, int ldy, int M, int N, int K,
              void* ws, size_t ws_bytes, int tune, hipStream_t stream) {
  LT_REQUIRE(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "operation descriptor");
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  LT_REQUIRE(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "transpose of W");
  LT_REQUIRE(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "transpose of X");
  LT_REQUIRE(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, K), "layout of W");
  LT_REQUIRE(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, ldx), "layout of X");
  LT_REQUIRE(hipblasLtMatrixLayoutCreate(&p.c, HIP_R_16BF, N, M, ldy), "layout of Y");
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_REQUIRE(hipblasLtMatmulPreferenceCreate(&pref), "preference");
  const uint64_t max_ws = ws_bytes;
  {
    const hipblasStatus_t sp = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws,
                                                                     sizeof(max_ws));
    if (sp != HIPBLAS_STATUS_SUCCESS) (void)hipblasLtMatmulPreferenceDestroy(pref);
    LT_REQUIRE(sp, "workspace limit");
  }
  constexpr int WANT = 24;
  std::vector<hipblasLtMatmulHeuristicResult_t> found(WANT);
  int n = 0;
  hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.a, p.b, p.c, p.c, pref, tune ? WANT : 1, found.data(), &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || n <= 0) {
    gs_set_error("library_gemm: the library offers no algorithm for M=%d N=%d K=%d: %s", M, N, K, status_name(s));
    return -3;
  }
  found.resize(n);
  const float one = 1.f, zero = 0.f;
  int best = -1;
  float best_ms = 0.f;
  void* flush = tune && n > 1 ? flush_buffer() : nullptr;
  if (tune && n > 1) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
      if (e0) (void)hipEventDestroy(e0);
      gs_set_error("library_gemm: no events for the tuning run");
      return -2;
    }
    // Milliseconds of one product with candidate i, the mean of `runs` after one unmeasured; negative: it failed.
    // Before every run a buffer larger than the last-level cache is overwritten, so that the weight comes from
    // memory as it does in a model whose other weights have passed through the caches since its last use (measured
    // on operands that stay in the cache, the choice went to algorithms that are slower in the model).
    auto measure = [&](int i, int runs) -> float {
      if (found[i].state != HIPBLAS_STATUS_SUCCESS || found[i].workspaceSize > ws_bytes) return -1.f;
      float total = 0.f;
      for (int r = -1; r < runs; ++r) {
        if (flush) (void)hipMemsetAsync(flush, r & 1, FLUSH_BYTES, stream);
        (void)hipEventRecord(e0, stream);
        const bool ok = hipblasLtMatmul(handle, p.desc, &one, W, p.a, X, p.b, &zero, Y, p.c, Y, p.c, &found[i].algo, ws,
                                        found[i].workspaceSize, stream) == HIPBLAS_STATUS_SUCCESS;
        (void)hipEventRecord(e1, stream);
        float ms = 0.f;
        if (hipEventSynchronize(e1) != hipSuccess || !ok || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.f;
        if (r >= 0) total += ms;
      }
      return total / runs;
    };
    // a first look at every candidate, then the five fastest once more with more runs
    std::vector<std::pair<float, int>> order;
    for (int i = 0; i < n; ++i) {
      const float ms = measure(i, 3);
      if (ms >= 0.f) order.emplace_back(ms, i);
      ++p.candidates;
    }
    std::sort(order.begin(), order.end());
    // the library's own first choice stays unless another is faster by more than the measurements scatter
    float first_ms = -1.f;
    for (size_t j = 0; j < order.size() && j < 5; ++j) {
      const float ms = measure(order[j].second, 6);
      if (ms >= 0.f && order[j].second == 0) first_ms = ms;
      if (ms >= 0.f && (best < 0 || ms < best_ms)) {
        best = order[j].second;
        best_ms = ms;
      }
    }
    if (best > 0) {
      if (first_ms < 0.f) first_ms = measure(0, 6);
      if (first_ms >= 0.f && best_ms > 0.97f * first_ms) {
        best = 0;
        best_ms = first_ms;
      }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    p.best_us = best_ms * 1000.f;
  }
  if (best < 0) {
    for (int i = 0; i < n && best < 0; ++i)
      if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= ws_bytes) best = i;
    if (best < 0) {
      gs_set_error("library_gemm: every algorithm for M=%d N=%d K=%d wants more than %zu bytes of workspace", M, N, K, ws_bytes);
      return -3;
    }
  }
  p.algo = found[best].algo;
  p.workspace = found[best].workspaceSize;
  return 0;
}

}  // namespace

// Y (M, N) bfloat16, rows ldy apart = X (M, K) bfloat16, rows ldx apart . W (N, K)^T, W contiguous.  `workspace`:
// device memory the library's kernels may use, ws_bytes of it.  `tune`: 0 = the library's first choice; 1 = the first call
// of a shape measures the library's two dozen best guesses on these operands (Y is written several times, a few
// milliseconds) and keeps the fastest.  (Measuring every algorithm the library has for the problem, about a thousand,
// took a third of a second a shape and found nothing faster than the best of the two dozen.)
extern "C" int gs_library_gemm(const void* X, int ldx, const void* W, void* Y, int ldy, int M, int N, int K, void* workspace,
                               long ws_bytes, int tune, hipStream_t stream) {
  GS_REQUIRE(M > 0 && N > 0 && K > 0, "library_gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  GS_REQUIRE(X && W && Y && ldx >= K && ldy >= N, "library_gemm: operands missing or row strides %d, %d below K=%d, N=%d", ldx, ldy, K, N);
  GS_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)Y & 15) == 0 && ldx % 8 == 0 && ldy % 8 == 0 && K % 8 == 0,
             "library_gemm: operands must be 16-byte aligned, row strides and K multiples of 8");
  GS_REQUIRE(ws_bytes >= 0 && (ws_bytes == 0 || workspace), "library_gemm: a workspace size without a workspace");
  // While a stream records, a product whose plan exists is recorded like any launch; a plan is not made then (making
  // one asks the library and, when tuning, measures: neither belongs into a recording).
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  const bool recording = hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
  int dev = -1;
  GS_REQUIRE(hipGetDevice(&dev) == hipSuccess, "library_gemm: no current device");
  std::lock_guard<std::mutex> lock(g_mutex);
  hipblasLtHandle_t& handle = g_handles[dev];
  if (!handle) LT_REQUIRE(hipblasLtCreate(&handle), "the library's handle");
  const PlanKey key(dev, M, N, K, ldx, ldy, (size_t)ws_bytes, tune ? 1 : 0);
  auto it = g_plans.find(key);
  if (it == g_plans.end()) {
    GS_REQUIRE(!recording, "library_gemm: no plan yet for %d x %d x %d rows: run the product once before it is recorded into a graph", M, N, K);
    Plan p;
    if (int rc = make_plan(handle, p, X, ldx, W, Y, ldy, M, N, K, workspace, (size_t)ws_bytes, tune, stream)) {
      destroy_plan(p);
      return rc;
    }
    make_room();
    it = g_plans.emplace(key, p).first;
  }
  return run(handle, it->second, X, W, Y, workspace, stream);
}

// How many shapes have a plan, and for the shape given (if it has one) how many candidates were measured and the best
// one's microseconds: what a test or a log line can show.
extern "C" int gs_library_gemm_plans(int M, int N, int K, int* candidates, float* best_us) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (candidates) *candidates = 0;
  if (best_us) *best_us = 0.f;
  for (const auto& kv : g_plans)
    if (std::get<1>(kv.first) == M && std::get<2>(kv.first) == N && std::get<3>(kv.first) == K) {
      if (candidates) *candidates = kv.second.candidates;
      if (best_us) *best_us = kv.second.best_us;
    }
  return (int)g_plans.size();
}
