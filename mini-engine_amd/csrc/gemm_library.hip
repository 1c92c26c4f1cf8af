// Plain bfloat16 products through the GEMM library (hipBLASLt), called directly: C[M, N] = X[M, K] . W[N, K]^T
// with float32 accumulation, for the row counts where the library is ahead of the kernels of this
// folder (prompts). A call costs the host about 5 us (through torch's matmul: 18), which is what an
// eager step of a few hundred tokens is made of. The matmul descriptor, the layouts and the algorithm the
// library's heuristic picks are kept per (M, N, K, output type); the first product of a shape asks the
// heuristic (host work only), later ones only launch.
//
// Row-major operands are the library's column-major ones transposed: C^T[N, M] = W[N, K] . X^T[K, M],
// that is op(A) = W^T-of-column-major (transposed), op(B) = X as it lies.
#include "common.h"

#include <hipblaslt/hipblaslt.h>

#include <initializer_list>
#include <mutex>
#include <unordered_map>

namespace {

struct LibraryPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

constexpr size_t WORKSPACE_BYTES = 256u << 20;  // the most a product may ask for (the library's split-k kernels for
                                                // products of thousands of rows want tens of MB); allocated once
constexpr int MAX_CANDIDATES = 8;               // algorithms asked of the heuristic: the first whose workspace fits is taken
constexpr size_t MAX_PLANS = 2048;              // per output type; a serving loop's steps bring ever new row counts

std::mutex g_mutex;
hipblasLtHandle_t g_handle = nullptr;
void* g_workspace = nullptr;
std::unordered_map<uint64_t, LibraryPlan> g_plans[2];  // by output type

int make_plan(LibraryPlan& p, int M, int N, int K, int out_dtype) {
  const hipDataType out_type = out_dtype == ME_F32 ? HIP_R_32F : HIP_R_16BF;
  const hipblasOperation_t trans = HIPBLAS_OP_T, none = HIPBLAS_OP_N;
  if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans)) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &none, sizeof(none)) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, K, N, K) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, K, M, K) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.c, out_type, N, M, N) != HIPBLAS_STATUS_SUCCESS)
    return me_fail("me_gemm_bf16_library: the library refused the description of a %d x %d x %d product", M, N, K);
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS)
    return me_fail("me_gemm_bf16_library: no preference object");
  size_t most = WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &most, sizeof(most));
  hipblasLtMatmulHeuristicResult_t results[MAX_CANDIDATES];
  int found = 0;
  const hipblasStatus_t st =
      hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, MAX_CANDIDATES, results, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || found < 1)
    return me_fail("me_gemm_bf16_library: the library has no algorithm for a %d x %d x %d product (status %d)", M, N, K, (int)st);
  for (int i = 0; i < found; ++i)
    if (results[i].state == HIPBLAS_STATUS_SUCCESS && results[i].workspaceSize <= WORKSPACE_BYTES) {
      p.algo = results[i].algo;
      p.workspace = results[i].workspaceSize;
      return 0;
    }
  return me_fail("me_gemm_bf16_library: every algorithm for a %d x %d x %d product wants more than %zu bytes of workspace", M, N,
                 K, WORKSPACE_BYTES);
}

void destroy_plan(LibraryPlan& p) {
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  for (hipblasLtMatrixLayout_t l : {p.a, p.b, p.c})
    if (l) hipblasLtMatrixLayoutDestroy(l);
  p = LibraryPlan();
}

}  // namespace

// X [M, K] and W [N, K] bfloat16, C [M, N] bfloat16 or float32 (out_dtype), all contiguous. The first call
// creates the library's handle and a workspace of 256 MB that lives as long as the process; the first call
// for a shape must not come while a graph is being captured (it may load code), later ones may.
static int library_product(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype, bool accumulate,
                           hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return me_fail("me_gemm_bf16_library: K=%d", K);
  if (!X || !W || !C) return me_fail("me_gemm_bf16_library: null operand");
  if (out_dtype != ME_BF16 && out_dtype != ME_F32) return me_fail("me_gemm_bf16_library: unknown output type %d", out_dtype);
  if ((uint32_t)M >= (1u << 21) || (uint32_t)N >= (1u << 21) || (uint32_t)K >= (1u << 21))  // the plans' key packs 21 bits each
    return me_fail("me_gemm_bf16_library: sizes %d x %d x %d are beyond 2^21", M, N, K);
  LibraryPlan plan;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_handle) {
      if (hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) {
        g_handle = nullptr;
        return me_fail("me_gemm_bf16_library: the GEMM library could not be initialised");
      }
    }
    if (!g_workspace && hipMalloc(&g_workspace, WORKSPACE_BYTES) != hipSuccess) {
      g_workspace = nullptr;
      return me_fail("me_gemm_bf16_library: no memory for %zu bytes of workspace", WORKSPACE_BYTES);
    }
    auto& plans = g_plans[out_dtype == ME_F32 ? 1 : 0];
    const uint64_t key = ((uint64_t)(uint32_t)M << 42) ^ ((uint64_t)(uint32_t)N << 21) ^ (uint64_t)(uint32_t)K;
    auto it = plans.find(key);
    if (it == plans.end()) {
      if (plans.size() >= MAX_PLANS) {  // start over: the shapes in use come back within a few steps
        for (auto& kv : plans) destroy_plan(kv.second);
        plans.clear();
      }
      LibraryPlan fresh;
      if (make_plan(fresh, M, N, K, out_dtype)) {
        destroy_plan(fresh);
        return 1;
      }
      it = plans.emplace(key, fresh).first;
    }
    plan = it->second;
  }
  const float alpha = 1.f, beta = accumulate ? 1.f : 0.f;
  const hipblasStatus_t st = hipblasLtMatmul(g_handle, plan.desc, &alpha, W, plan.a, X, plan.b, &beta, C, plan.c, C, plan.c,
                                             &plan.algo, g_workspace, WORKSPACE_BYTES, stream);
  if (st != HIPBLAS_STATUS_SUCCESS) return me_fail("me_gemm_bf16_library: the product failed with status %d", (int)st);
  return 0;
}

extern "C" int me_gemm_bf16_library(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype,
                                    hipStream_t stream) {
  return library_product(X, W, C, M, N, K, out_dtype, false, stream);
}

// C[M, N] (float32) += X . W^T: the product added to what C holds, in the library's epilogue (a float32 sum per element).
extern "C" int me_gemm_bf16_library_add(const void* X, const void* W, float* C, int M, int N, int K, hipStream_t stream) {
  return library_product(X, W, C, M, N, K, ME_F32, true, stream);
}
