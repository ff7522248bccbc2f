// hipBLASLt front end for the plain GEMMs of the lm_head path: one handle per device, the heuristic's first
// algorithm per problem shape, cached.
#include "lt_gemm.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace aa {
namespace lt {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
hipblasLtHandle_t g_handle[kMaxDevices] = {};

using Key = std::tuple<int, bool, bool, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, bool, bool>;
std::map<Key, hipblasLtMatmulAlgo_t> g_algos;

struct Problem {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  ~Problem() {
    if (a) hipblasLtMatrixLayoutDestroy(a);
    if (b) hipblasLtMatrixLayoutDestroy(b);
    if (d) hipblasLtMatrixLayoutDestroy(d);
    if (desc) hipblasLtMatmulDescDestroy(desc);
  }
};

}  // namespace

bool gemm(hipStream_t st, bool transA, bool transB, int64_t m, int64_t n, int64_t k, const void* A, int64_t lda,
          const void* B, int64_t ldb, void* D, int64_t ldd, bool out_f32, float beta, void* workspace,
          int64_t workspace_bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_handle[dev] && hipblasLtCreate(&g_handle[dev]) != HIPBLAS_STATUS_SUCCESS) return false;
  hipblasLtHandle_t handle = g_handle[dev];

  Problem p;
  const hipDataType out_type = out_f32 ? HIP_R_32F : HIP_R_16BF;
  if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return false;
  const hipblasOperation_t opa = transA ? HIPBLAS_OP_T : HIPBLAS_OP_N, opb = transB ? HIPBLAS_OP_T : HIPBLAS_OP_N;
  if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opa, sizeof(opa)) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opb, sizeof(opb)) != HIPBLAS_STATUS_SUCCESS)
    return false;
  if (hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, transA ? k : m, transA ? m : k, lda) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, transB ? n : k, transB ? k : n, ldb) != HIPBLAS_STATUS_SUCCESS ||
      hipblasLtMatrixLayoutCreate(&p.d, out_type, m, n, ldd) != HIPBLAS_STATUS_SUCCESS)
    return false;

  const Key key{dev, transA, transB, m, n, k, lda, ldb, ldd, out_f32, beta != 0.f};
  auto it = g_algos.find(key);
  if (it == g_algos.end()) {
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return false;
    const uint64_t max_ws = workspace ? (uint64_t)workspace_bytes : 0;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    hipblasLtMatmulHeuristicResult_t result[1];
    int found = 0;
    const hipblasStatus_t hs =
        hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.a, p.b, p.d, p.d, pref, 1, result, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (hs != HIPBLAS_STATUS_SUCCESS || found < 1) return false;
    it = g_algos.emplace(key, result[0].algo).first;
  }
  const float alpha = 1.f;
  return hipblasLtMatmul(handle, p.desc, &alpha, A, p.a, B, p.b, &beta, D, p.d, D, p.d, &it->second, workspace,
                         workspace ? (size_t)workspace_bytes : 0, st) == HIPBLAS_STATUS_SUCCESS;
}

}  // namespace lt
}  // namespace aa
