// The library's bf16 matrix product, called directly: out[M, N] = a[M, K] @ w[N, K]^T through
// hipBLASLt with the algorithm chosen by the caller among the library's own candidates.
//
// torch.mm asks the library for one candidate and takes it.  For the shapes of a decode step
// with tens of rows and of a 512-row portion of a prompt the first candidate is often not the
// fastest on this GPU, and a call through torch costs 18 us on the host.  Here the candidates of
// a shape are listed once (as_blas_plan), the caller times them in place and then names the one
// to run (as_blas_gemm); a call costs what hipblasLtMatmul costs.
//
// Row-major [M, K] x [N, K]^T is, column-major, D^T[N, M] = W (K x N, transposed) * A^T (K x M).
#include "common.h"

#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace {

constexpr int MAX_CANDIDATES = 16;

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  std::vector<hipblasLtMatmulHeuristicResult_t> candidates;
};

std::mutex g_mutex;
hipblasLtHandle_t g_handle = nullptr;
std::map<std::tuple<int, int, int, int, size_t>, Plan> g_plans;  // (M, N, K, out dtype, workspace bytes)

bool ok(hipblasStatus_t s) { return s == HIPBLAS_STATUS_SUCCESS; }

// The plan of a shape, made at its first use; nullptr if the library refuses.
Plan* plan_for(int M, int N, int K, int out_dtype, size_t workspace_bytes) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_handle && !ok(hipblasLtCreate(&g_handle))) return nullptr;
  const auto key = std::make_tuple(M, N, K, out_dtype, workspace_bytes);
  auto it = g_plans.find(key);
  if (it != g_plans.end()) return it->second.candidates.empty() ? nullptr : &it->second;
  Plan plan;
  const hipDataType out_type = out_dtype == DT_F32 ? HIP_R_32F : HIP_R_16BF;
  const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  bool good = ok(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) &&
              ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed))) &&
              ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain))) &&
              ok(hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, N, K)) &&
              ok(hipblasLtMatrixLayoutCreate(&plan.b, HIP_R_16BF, K, M, K)) &&
              ok(hipblasLtMatrixLayoutCreate(&plan.c, out_type, N, M, N));
  hipblasLtMatmulPreference_t pref = nullptr;
  good = good && ok(hipblasLtMatmulPreferenceCreate(&pref)) &&
         ok(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                                  sizeof(workspace_bytes)));
  if (good) {
    plan.candidates.resize(MAX_CANDIDATES);
    int found = 0;
    good = ok(hipblasLtMatmulAlgoGetHeuristic(g_handle, plan.desc, plan.a, plan.b, plan.c, plan.c, pref, MAX_CANDIDATES,
                                              plan.candidates.data(), &found));
    plan.candidates.resize(good ? found : 0);
  } else {
    plan.candidates.clear();
  }
  if (pref) hipblasLtMatmulPreferenceDestroy(pref);
  Plan& kept = g_plans[key] = plan;  // kept also when empty, so that the library is not asked again
  return kept.candidates.empty() ? nullptr : &kept;
}

}  // namespace

// The number of candidates the library offers for this shape (0: none, use another product).
extern "C" int as_blas_plan(int M, int N, int K, int out_dtype, size_t workspace_bytes) {
  if (M <= 0 || N <= 0 || K <= 0 || (out_dtype != DT_BF16 && out_dtype != DT_F32)) return 0;
  Plan* plan = plan_for(M, N, K, out_dtype, workspace_bytes);
  return plan ? (int)plan->candidates.size() : 0;
}

// The library's own number of a candidate's kernel (the same number names the same kernel for every
// shape, within one version of the library), -1 if there is none.
extern "C" int as_blas_candidate_index(int M, int N, int K, int out_dtype, size_t workspace_bytes, int candidate) {
  Plan* plan = plan_for(M, N, K, out_dtype, workspace_bytes);
  if (!plan || candidate < 0 || candidate >= (int)plan->candidates.size()) return -1;
  return hipblaslt_ext::getIndexFromAlgo(plan->candidates[candidate].algo);
}

// Makes the kernel with the library's number `index` (as_blas_candidate_index of another shape's
// candidate) a candidate of this shape: returns its place among the shape's candidates, adding it
// if the library says it can compute this shape within the workspace, or -1 if it cannot.
extern "C" int as_blas_adopt(int M, int N, int K, int out_dtype, size_t workspace_bytes, int index) {
  Plan* plan = plan_for(M, N, K, out_dtype, workspace_bytes);
  if (!plan || index < 0) return -1;
  std::lock_guard<std::mutex> lock(g_mutex);
  for (size_t i = 0; i < plan->candidates.size(); ++i)
    if (hipblaslt_ext::getIndexFromAlgo(plan->candidates[i].algo) == index) return (int)i;
  std::vector<int> wanted = {index};
  std::vector<hipblasLtMatmulHeuristicResult_t> found;
  if (!ok(hipblaslt_ext::getAlgosFromIndex(g_handle, wanted, found))) return -1;
  const float one = 1.f, zero = 0.f;
  for (auto& result : found) {
    size_t needs = 0;
    if (ok(hipblaslt_ext::matmulIsAlgoSupported(g_handle, plan->desc, &one, plan->a, plan->b, &zero, plan->c, plan->c,
                                                result.algo, needs)) &&
        needs <= workspace_bytes) {
      plan->candidates.push_back(result);
      return (int)plan->candidates.size() - 1;
    }
  }
  return -1;
}

// The library builds its table of kernels by number at the first look-up (a third of a second here);
// this makes that look-up, with the number of some candidate of some planned shape, so that a later
// as_blas_adopt in the middle of serving does not pay for it.  Returns 1 if a look-up was made.
extern "C" int as_blas_prepare_adoption() {
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto& kept : g_plans) {
    if (kept.second.candidates.empty()) continue;
    std::vector<int> wanted = {hipblaslt_ext::getIndexFromAlgo(kept.second.candidates[0].algo)};
    std::vector<hipblasLtMatmulHeuristicResult_t> found;
    return ok(hipblaslt_ext::getAlgosFromIndex(g_handle, wanted, found)) ? 1 : 0;
  }
  return 0;
}

// Runs candidate `candidate` of the shape's plan.  a [M, K], w [N, K] bf16; out [M, N] bf16 or fp32;
// workspace: device memory of at least workspace_bytes (the size the plan was made for).
extern "C" int as_blas_gemm(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K, int candidate,
                            void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (M <= 0) return AS_OK;
  if (N <= 0 || K <= 0 || !a || !w || !out || (workspace_bytes && !workspace)) return AS_BAD_SHAPE;
  if (out_dtype != DT_BF16 && out_dtype != DT_F32) return AS_BAD_DTYPE;
  Plan* plan = plan_for(M, N, K, out_dtype, workspace_bytes);
  if (!plan || candidate < 0 || candidate >= (int)plan->candidates.size()) return AS_BAD_SHAPE;
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t s = hipblasLtMatmul(g_handle, plan->desc, &one, w, plan->a, a, plan->b, &zero, out, plan->c, out,
                                            plan->c, &plan->candidates[candidate].algo, workspace, workspace_bytes, stream);
  return ok(s) ? AS_OK : AS_LAUNCH_FAILED;
}
