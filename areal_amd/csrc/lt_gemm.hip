// hipBLASLt front end for the plain GEMMs of the lm_head path: one handle per device, one algorithm per problem
// shape, cached.  The library's heuristic ranks its kernels without running them, and its first choice is up to
// 30 % slower than its second for some row counts (e.g. m = 4096, k = 151936: n = 11520 runs at 1 258 TFLOP/s with
// the first and 1 560 with the second, n = 12288 the other way round).  So the first time a shape is seen with
// beta == 0 (the output is overwritten, a trial run does no harm) the leading candidates are timed on the caller's
// stream with the caller's operands and the fastest is kept.  That blocks the host for a few GEMM durations, once
// per shape; AREAL_AMD_GEMM_TUNE=0 turns it off, and a capturing stream is never timed.  AREAL_AMD_GEMM_TUNE_LOG=1
// prints the timings.  Which candidate wins depends on the operands too (the matrix cores clock down on data with
// many bit flips), which is one more reason to time with the caller's own data.
#include "lt_gemm.h"

#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <cstdlib>
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

constexpr int kCandidates = 4;

bool tuning_enabled() {
  static const bool on = [] {
    const char* v = std::getenv("AREAL_AMD_GEMM_TUNE");
    return !(v && v[0] == '0');
  }();
  return on;
}

bool stream_is_capturing(hipStream_t st) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(st, &status) != hipSuccess || status != hipStreamCaptureStatusNone;
}

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
    hipblasLtMatmulHeuristicResult_t result[kCandidates];
    int found = 0;
    const bool tune = beta == 0.f && tuning_enabled() && !stream_is_capturing(st);
    const hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.a, p.b, p.d, p.d, pref,
                                                               tune ? kCandidates : 1, result, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (hs != HIPBLAS_STATUS_SUCCESS || found < 1) return false;
    int best = 0;
    if (tune && found > 1) {
      hipEvent_t e0 = nullptr, e1 = nullptr;
      if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
        const float one = 1.f, zero = 0.f;
        float best_ms = -1.f;
        for (int c = 0; c < found; ++c) {
          auto run = [&] {
            return hipblasLtMatmul(handle, p.desc, &one, A, p.a, B, p.b, &zero, D, p.d, D, p.d, &result[c].algo, workspace,
                                   workspace ? (size_t)workspace_bytes : 0, st) == HIPBLAS_STATUS_SUCCESS;
          };
          float ms = 0.f;
          if (!run() || hipEventRecord(e0, st) != hipSuccess || !run() || hipEventRecord(e1, st) != hipSuccess ||
              hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
            continue;
          if (std::getenv("AREAL_AMD_GEMM_TUNE_LOG"))
            fprintf(stderr, "[areal_amd] gemm m=%lld n=%lld k=%lld f32=%d: candidate %d %.3f ms\n", (long long)m,
                    (long long)n, (long long)k, (int)out_f32, c, ms);
          if (best_ms < 0.f || ms < best_ms) {
            best_ms = ms;
            best = c;
          }
        }
      }
      if (e0) hipEventDestroy(e0);
      if (e1) hipEventDestroy(e1);
    }
    it = g_algos.emplace(key, result[best].algo).first;
  }
  const float alpha = 1.f;
  return hipblasLtMatmul(handle, p.desc, &alpha, A, p.a, B, p.b, &beta, D, p.d, D, p.d, &it->second, workspace,
                         workspace ? (size_t)workspace_bytes : 0, st) == HIPBLAS_STATUS_SUCCESS;
}

}  // namespace lt
}  // namespace aa
