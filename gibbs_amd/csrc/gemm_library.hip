// The library's bfloat16 matrix product, called directly: C[n, o] = sum_k A[n, k] * W[o, k], float32
// accumulation, bfloat16 out.  hipBLASLt is what the prompt path's products run on (the reference's
// engine uses a library product for its prefill as well); called through PyTorch the same product costs
// the host about 20 us a call (dispatch, heuristics, descriptors), which is more than the device needs
// for a prompt portion of a few hundred rows: a step of 64 to 512 rows was bound by the host.  Here
// the descriptors and the algorithm are kept per shape, so a call is one hipblasLtMatmul.
//
// Which algorithm: the first of the library's heuristic, except for large steps (512 rows and more, a
// multiple of 256: whole prompts and prompt portions), where the heuristic's 24 best are timed once on
// the call's own activations and on copies of its weights that are taken in turn, so that the weights
// are read cold as in a model step, and the fastest is kept.  For the LFM2-1.2B shapes at 2,048 rows the
// heuristic's first choice is the fastest for the 16,384- and 6,144-wide products and 11 to 19 %
// slower than the best for the 2,048- and 3,072-wide ones (80 -> 68 us for w2).  Nothing is timed
// while the stream is being captured.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <stdlib.h>
#include <map>
#include <mutex>
#include <tuple>

namespace {
struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool timed = false;          // the algorithm was chosen by timing: such plans are kept
  unsigned long last_use = 0;

  void destroy() {
    if (desc) hipblasLtMatmulDescDestroy(desc);
    for (hipblasLtMatrixLayout_t l : {w, a, c})
      if (l) hipblasLtMatrixLayoutDestroy(l);
    desc = nullptr;
    w = a = c = nullptr;
  }
};
constexpr size_t WORKSPACE_BYTES = 64u << 20;   // what the heuristic may count on (stream-K kernels use some)
constexpr size_t FLUSH_BYTES = 320u << 20;      // copies of a weight matrix: more than L2 and the memory-side cache hold
constexpr int CANDIDATES = 24;
// Plans are kept per exact shape, and a scheduler that cuts prompts under a measured budget brings steps of
// any number of rows: beyond this many, the plan that was used longest ago goes (its descriptors are freed).
constexpr size_t MAX_PLANS = 192;
unsigned long use_clock = 0;
long timings_done = 0;
hipblasLtHandle_t handle = nullptr;
void* workspace = nullptr;
void* flush = nullptr;                          // allocated when the first shape is timed, kept
std::map<std::tuple<int, int, int, long, long, long>, Plan> plans;
std::mutex guard;

#define LT(call)                                                                               \
  do {                                                                                         \
    hipblasStatus_t st_ = (call);                                                              \
    if (st_ != HIPBLAS_STATUS_SUCCESS) return gibbs_fail("gemm_library: %s failed with status %d", #call, (int)st_); \
  } while (0)

// The fastest of the candidates on these operands; -1 if none could be timed.  The weights are copied
// several times into a large buffer and the candidates run over the copies in turn, so that each run
// reads its matrix cold, as in a model step (run on one matrix again and again, the candidates that
// win are those that like their weights in the memory-side cache).
int fastest(const Plan& p, const hipblasLtMatmulHeuristicResult_t* found, int n_found, const void* A, const void* W,
            void* C, size_t w_bytes, hipStream_t stream) {
  if (!flush && hipMalloc(&flush, FLUSH_BYTES) != hipSuccess) {
    flush = nullptr;
    (void)hipGetLastError();
    return -1;
  }
  const size_t stride = (w_bytes + 255) / 256 * 256;
  const int copies = (int)(FLUSH_BYTES / stride < 8 ? FLUSH_BYTES / stride : 8);
  if (copies < 2) return -1;
  for (int i = 0; i < copies; ++i)
    if (hipMemcpyAsync((char*)flush + i * stride, W, w_bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess) return -1;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1;
  const float one = 1.f, zero = 0.f;
  const int runs = 2 * copies;
  int best = -1;
  float best_ms = 0.f;
  for (int c = 0; c < n_found; ++c) {
    if (found[c].state != HIPBLAS_STATUS_SUCCESS || found[c].workspaceSize > WORKSPACE_BYTES) continue;
    auto run = [&](int i) {
      return hipblasLtMatmul(handle, p.desc, &one, (const char*)flush + (i % copies) * stride, p.w, A, p.a, &zero, C, p.c,
                             C, p.c, &found[c].algo, workspace, found[c].workspaceSize, stream);
    };
    if (run(0) != HIPBLAS_STATUS_SUCCESS) continue;           // (the first run also loads the kernel's code)
    bool ok = hipEventRecord(e0, stream) == hipSuccess;
    for (int i = 1; i <= runs && ok; ++i) ok = run(i) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipEventRecord(e1, stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
    float ms = 0.f;
    ok = ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    if (ok && (best < 0 || ms < best_ms)) {
      best = c;
      best_ms = ms;
    }
  }
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  (void)hipGetLastError();
  return best;
}

int make_plan(Plan& p, int N, int O, int I, long lda, long ldw, long ldc, const void* A, const void* W, void* C,
              hipStream_t stream) {
  // Column-major view: C' (O x N, ld ldc) = W'^T (W' is I x O, ld ldw) . A' (I x N, ld lda)
  LT(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const int32_t trans = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans)));
  LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)));
  LT(hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, I, O, ldw));
  LT(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, I, N, lda));
  LT(hipblasLtMatrixLayoutCreate(&p.c, HIP_R_16BF, O, N, ldc));
  hipblasLtMatmulPreference_t pref = nullptr;
  LT(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t room = WORKSPACE_BYTES;
  LT(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room)));
  static const bool timing = !(getenv("GIBBS_GEMM_TUNE") && atoi(getenv("GIBBS_GEMM_TUNE")) == 0);
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) capture = hipStreamCaptureStatusActive;
  const bool timed = timing && N >= 512 && N % 256 == 0 && capture == hipStreamCaptureStatusNone;
  hipblasLtMatmulHeuristicResult_t found[CANDIDATES];
  int n_found = 0;
  hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.w, p.a, p.c, p.c, pref, timed ? CANDIDATES : 1,
                                                       found, &n_found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || n_found < 1)
    return gibbs_fail("gemm_library: the library offers no algorithm for N=%d O=%d I=%d (status %d)", N, O, I, (int)st);
  int pick = 0;
  if (timed && n_found > 1) {
    const int best = fastest(p, found, n_found, A, W, C, (size_t)O * ldw * sizeof(bf16), stream);
    if (best >= 0) pick = best;
    p.timed = true;
    ++timings_done;
  }
  p.algo = found[pick].algo;
  p.workspace = found[pick].workspaceSize;
  if (p.workspace > WORKSPACE_BYTES) return gibbs_fail("gemm_library: the algorithm wants %zu bytes of workspace", p.workspace);
  return 0;
}
}  // namespace

// Creates the library's handle and the workspace; to be called once, outside any stream capture.
GIBBS_EXPORT int gibbs_gemm_library_init() {
  std::lock_guard<std::mutex> lock(guard);
  if (handle) return 0;
  LT(hipblasLtCreate(&handle));
  hipError_t e = hipMalloc(&workspace, WORKSPACE_BYTES);
  if (e != hipSuccess) {
    hipblasLtDestroy(handle);
    handle = nullptr;
    return gibbs_fail("gemm_library: workspace: %s", hipGetErrorString(e));
  }
  return 0;
}

// How many shapes have had their algorithm chosen by timing so far (a step during which this number
// grows took longer than its like will: whoever times steps leaves it out), and how many plans are kept.
GIBBS_EXPORT long gibbs_gemm_library_timings() { return timings_done; }
GIBBS_EXPORT long gibbs_gemm_library_plans() { return (long)plans.size(); }

// A: [N, I] bfloat16 (row stride lda), W: [O, I] bfloat16 (row stride ldw), C: [N, O] bfloat16 (row stride ldc).
GIBBS_EXPORT int gibbs_gemm_library(const void* A, const void* W, void* C, int N, int O, int I, long lda, long ldw,
                                    long ldc, hipStream_t stream) {
  GIBBS_REQUIRE(N > 0 && O > 0 && I > 0, "gemm_library: bad sizes N=%d O=%d I=%d", N, O, I);
  GIBBS_REQUIRE(lda >= I && ldw >= I && ldc >= O, "gemm_library: row strides shorter than rows");
  GIBBS_REQUIRE(handle != nullptr, "gemm_library: not initialised");
  Plan* plan;
  {
    std::lock_guard<std::mutex> lock(guard);
    const auto key = std::make_tuple(N, O, I, lda, ldw, ldc);
    auto it = plans.find(key);
    if (it == plans.end()) {
      if (plans.size() >= MAX_PLANS) {
        auto oldest = plans.end();
        for (auto j = plans.begin(); j != plans.end(); ++j)
          if (!j->second.timed && (oldest == plans.end() || j->second.last_use < oldest->second.last_use)) oldest = j;
        if (oldest != plans.end()) {
          oldest->second.destroy();
          plans.erase(oldest);
        }
      }
      Plan p;
      if (make_plan(p, N, O, I, lda, ldw, ldc, A, W, C, stream)) {
        p.destroy();
        return 1;
      }
      it = plans.emplace(key, p).first;
    }
    plan = &it->second;
    plan->last_use = ++use_clock;
  }
  const float one = 1.f, zero = 0.f;
  LT(hipblasLtMatmul(handle, plan->desc, &one, W, plan->w, A, plan->a, &zero, C, plan->c, C, plan->c, &plan->algo,
                     workspace, plan->workspace, stream));
  return 0;
}
