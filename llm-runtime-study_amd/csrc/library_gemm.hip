// The vendor library's matrix product for bfloat16 products of many rows, called here directly.
//
// out [M, N] = a [M, K] w[N, K]^T with float32 accumulation, out in bfloat16 or float32.  This is the
// one place where the product path uses a library (the reference leaves its products to
// torch.nn.Linear); everything the library needs (handle, workspace, the algorithm chosen for a shape)
// is made once and kept, so that a call inside a step, a recorded launch plan or a graph capture
// allocates nothing.
#include "common.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr size_t WORKSPACE_BYTES = 64u << 20;

struct Chosen {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t weights = nullptr, rows = nullptr, result = nullptr;
  hipblasLtMatmulAlgo_t algo;
};

hipblasLtHandle_t g_handle = nullptr;
void* g_workspace = nullptr;
std::mutex g_lock;
std::map<std::tuple<int, int, int, int, int, int>, Chosen> g_chosen;   // (m, n, k, lda, ldc, out is float32)

int prepare_locked() {
  if (!g_handle && hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) return lrs_fail("library_gemm: the matrix library could not be opened");
  if (!g_workspace && hipMalloc(&g_workspace, WORKSPACE_BYTES) != hipSuccess) {
    g_workspace = nullptr;
    return lrs_fail("library_gemm: could not allocate %zu bytes of workspace", WORKSPACE_BYTES);
  }
  return 0;
}

// In the library's column-major terms the result is C^T [N, M] = W (stored [K, N], transposed) times
// A^T (stored [K, M], as it is).
int choose(int m, int n, int k, int lda, int ldc, bool out_f32, Chosen& c) {
  const hipDataType out_type = out_f32 ? HIP_R_32F : HIP_R_16BF;
  if (hipblasLtMatmulDescCreate(&c.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return lrs_fail("library_gemm: no product description");
  const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  hipblasLtMatmulDescSetAttribute(c.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed));
  hipblasLtMatmulDescSetAttribute(c.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain));
  if (hipblasLtMatrixLayoutCreate(&c.weights, HIP_R_16BF, k, n, k) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&c.rows, HIP_R_16BF, k, m, lda) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&c.result, out_type, n, m, ldc) != HIPBLAS_STATUS_SUCCESS)
    return lrs_fail("library_gemm: no matrix layouts for m=%d n=%d k=%d", m, n, k);
  hipblasLtMatmulPreference_t preference = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&preference) != HIPBLAS_STATUS_SUCCESS) return lrs_fail("library_gemm: no preference object");
  const uint64_t workspace = WORKSPACE_BYTES;
  hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace, sizeof(workspace));
  hipblasLtMatmulHeuristicResult_t found[1];
  int count = 0;
  const hipblasStatus_t status = hipblasLtMatmulAlgoGetHeuristic(g_handle, c.desc, c.weights, c.rows, c.result, c.result, preference, 1, found, &count);
  hipblasLtMatmulPreferenceDestroy(preference);
  if (status != HIPBLAS_STATUS_SUCCESS || count < 1) return lrs_fail("library_gemm: the library offers no kernel for m=%d n=%d k=%d", m, n, k);
  c.algo = found[0].algo;
  return 0;
}

}  // namespace

// Opens the library and allocates its workspace now, so that no later call has to.  Safe to call again.
LRS_API int lrs_library_gemm_prepare() {
  std::lock_guard<std::mutex> hold(g_lock);
  return prepare_locked();
}

// out [M, N] (row stride ldc; bfloat16, or float32 if out_f32) = a [M, K] (row stride lda) times w [N, K]^T, bfloat16 inputs.
LRS_API int lrs_library_gemm(void* out, int out_f32, const void* a, const void* w, int m, int n, int k, int lda, int ldc, void* stream) {
  LRS_REQUIRE(m > 0 && n > 0 && k > 0 && lda >= k && ldc >= n, "library_gemm: bad sizes m=%d n=%d k=%d lda=%d ldc=%d", m, n, k, lda, ldc);
  LRS_REQUIRE(out && a && w, "library_gemm: out, a and w are required");
  Chosen* chosen = nullptr;
  {
    std::lock_guard<std::mutex> hold(g_lock);
    if (int rc = prepare_locked()) return rc;
    const auto key = std::make_tuple(m, n, k, lda, ldc, out_f32 ? 1 : 0);
    auto it = g_chosen.find(key);
    if (it == g_chosen.end()) {
      Chosen fresh;
      if (int rc = choose(m, n, k, lda, ldc, out_f32 != 0, fresh)) return rc;
      it = g_chosen.emplace(key, fresh).first;
    }
    chosen = &it->second;
  }
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t status = hipblasLtMatmul(g_handle, chosen->desc, &one, w, chosen->weights, a, chosen->rows, &zero, out, chosen->result,
                                                 out, chosen->result, &chosen->algo, g_workspace, WORKSPACE_BYTES, (hipStream_t)stream);
  if (status != HIPBLAS_STATUS_SUCCESS) return lrs_fail("library_gemm: the product failed with status %d (m=%d n=%d k=%d)", (int)status, m, n, k);
  return 0;
}
