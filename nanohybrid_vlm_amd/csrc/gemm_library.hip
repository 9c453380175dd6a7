// y[M, N] = x[M, K] . w[N, K]^T in bfloat16 with float sums, by the vendor's matrix library (hipBLASLt), with the
// choice of its algorithm left to the caller: for a given shape the library names up to `want` algorithms it
// thinks suitable, best guess first, and the caller may run any of them. Its first guess is what a framework's
// matrix product gets; for products of few rows and a big weight, whose time is the time to stream the weight
// once, that guess is often far from the library's best (a 5120 x 17408 weight against 8 rows: 112 us by the
// first guess, 37 us by the fifth), so the engine times them on the model's own shapes and keeps the fastest.
// The reference's linears are library calls as well (nanovllm/layers/linear.py:88,192).
//
// A plan is the description of one shape with the list of its algorithms; plans live until the process ends
// (a model has a handful of shapes per batch size). Calls come from one host thread.
#include "nhv_common.h"
#include <hipblaslt/hipblaslt.h>
#include <vector>

namespace {

struct Plan {
  int M, N, K, out_dtype;
  hipblasLtMatmulDesc_t desc;
  hipblasLtMatrixLayout_t w, x, y;
  std::vector<hipblasLtMatmulHeuristicResult_t> algorithms;
};

hipblasLtHandle_t g_handle = nullptr;
std::vector<Plan> g_plans;

}  // namespace

#define NHV_BLAS(call)                                                                       \
  do {                                                                                       \
    hipblasStatus_t s_ = (call);                                                             \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return nhv_fail("%s failed with status %d", #call, (int)s_); \
  } while (0)

// Makes (or finds) the plan of a shape and writes its number to *plan and the number of its algorithms to *count.
// Only algorithms that need at most workspace_bytes of scratch memory are listed.
extern "C" int nhv_library_gemm_plan(int M, int N, int K, int out_dtype, int want, size_t workspace_bytes, int* plan,
                                     int* count) {
  NHV_REQUIRE(M > 0 && N > 0 && K > 0, "library product: empty shape %d x %d x %d", M, N, K);
  NHV_REQUIRE(out_dtype == NHV_BF16 || out_dtype == NHV_F32, "library product: result type %d", out_dtype);
  NHV_REQUIRE(want > 0 && want <= 256, "library product: %d algorithms asked for (1 to 256)", want);
  for (size_t i = 0; i < g_plans.size(); ++i) {
    const Plan& p = g_plans[i];
    if (p.M == M && p.N == N && p.K == K && p.out_dtype == out_dtype) {
      *plan = (int)i;
      *count = (int)p.algorithms.size();
      return 0;
    }
  }
  if (!g_handle) NHV_BLAS(hipblasLtCreate(&g_handle));
  Plan p;
  p.M = M, p.N = N, p.K = K, p.out_dtype = out_dtype;
  NHV_BLAS(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  // The library thinks in column-major matrices: w[N, K] in rows is a K x N matrix to it, taken transposed;
  // x[M, K] is K x M; and y[M, N] is N x M = w^T-as-stored . x-as-stored.
  const hipblasOperation_t transposed = HIPBLAS_OP_T, as_stored = HIPBLAS_OP_N;
  NHV_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)));
  NHV_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &as_stored, sizeof(as_stored)));
  NHV_BLAS(hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K));
  NHV_BLAS(hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, K, M, K));
  NHV_BLAS(hipblasLtMatrixLayoutCreate(&p.y, out_dtype == NHV_F32 ? HIP_R_32F : HIP_R_16BF, N, M, N));
  hipblasLtMatmulPreference_t preference;
  NHV_BLAS(hipblasLtMatmulPreferenceCreate(&preference));
  NHV_BLAS(hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                                 sizeof(workspace_bytes)));
  p.algorithms.resize(want);
  int found = 0;
  hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.w, p.x, p.y, p.y, preference, want,
                                                      p.algorithms.data(), &found);
  hipblasLtMatmulPreferenceDestroy(preference);
  if (s != HIPBLAS_STATUS_SUCCESS) return nhv_fail("library product %d x %d x %d: no algorithm (status %d)", M, N, K, (int)s);
  p.algorithms.resize(found);
  g_plans.push_back(p);
  *plan = (int)g_plans.size() - 1;
  *count = found;
  return 0;
}

// Runs algorithm number `algorithm` of a plan. The workspace must hold what the plan was made with.
extern "C" int nhv_library_gemm(int plan, int algorithm, const void* x, const void* w, void* y, void* workspace,
                                size_t workspace_bytes, hipStream_t stream) {
  NHV_REQUIRE(plan >= 0 && plan < (int)g_plans.size(), "library product: no plan %d", plan);
  Plan& p = g_plans[plan];
  NHV_REQUIRE(algorithm >= 0 && algorithm < (int)p.algorithms.size(), "library product: plan %d has %d algorithms, not %d",
              plan, (int)p.algorithms.size(), algorithm);
  NHV_REQUIRE(p.algorithms[algorithm].workspaceSize <= workspace_bytes, "library product: algorithm %d needs %zu bytes of "
              "workspace, %zu given", algorithm, p.algorithms[algorithm].workspaceSize, workspace_bytes);
  const float one = 1.f, zero = 0.f;
  NHV_BLAS(hipblasLtMatmul(g_handle, p.desc, &one, w, p.w, x, p.x, &zero, y, p.y, y, p.y, &p.algorithms[algorithm].algo,
                           workspace, workspace_bytes, stream));
  return 0;
}
