// The library's bfloat16 matrix product, called directly: C[n, o] = sum_k A[n, k] * W[o, k], float32
// accumulation, bfloat16 out.  hipBLASLt is what the prompt path's products run on (the reference's
// engine uses a library product for its prefill as well); called through PyTorch the same product costs
// the host about 20 us a call (dispatch, heuristics, descriptors), which is more than the device needs
// for a prompt portion of a few hundred rows: a step of 64 to 512 rows was bound by the host.  Here
// the descriptors and the algorithm that the library's heuristic picks are kept per shape, so a call is
// one hipblasLtMatmul.
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
};
constexpr size_t WORKSPACE_BYTES = 64u << 20;   // what the heuristic may count on (stream-K kernels use some)
hipblasLtHandle_t handle = nullptr;
void* workspace = nullptr;
std::map<std::tuple<int, int, int, long, long, long>, Plan> plans;
std::mutex guard;

#define LT(call)                                                                               \
  do {                                                                                         \
    hipblasStatus_t st_ = (call);                                                              \
    if (st_ != HIPBLAS_STATUS_SUCCESS) return gibbs_fail("gemm_library: %s failed with status %d", #call, (int)st_); \
  } while (0)

int make_plan(Plan& p, int N, int O, int I, long lda, long ldw, long ldc) {
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
  hipblasLtMatmulHeuristicResult_t found[1];
  int n_found = 0;
  hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.w, p.a, p.c, p.c, pref, 1, found, &n_found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || n_found < 1)
    return gibbs_fail("gemm_library: the library offers no algorithm for N=%d O=%d I=%d (status %d)", N, O, I, (int)st);
  p.algo = found[0].algo;
  p.workspace = found[0].workspaceSize;
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
      Plan p;
      if (make_plan(p, N, O, I, lda, ldw, ldc)) return 1;
      it = plans.emplace(key, p).first;
    }
    plan = &it->second;
  }
  const float one = 1.f, zero = 0.f;
  LT(hipblasLtMatmul(handle, plan->desc, &one, W, plan->w, A, plan->a, &zero, C, plan->c, C, plan->c, &plan->algo,
                     workspace, plan->workspace, stream));
  return 0;
}
