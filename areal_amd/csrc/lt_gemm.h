// Plain bf16 GEMMs through hipBLASLt (the library's tuned kernels for matrices that need no fused epilogue).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aa {
namespace lt {

constexpr int64_t kWorkspaceBytes = 128ll << 20;  // scratch handed to the library (stream-K partial tiles)

// Column-major D[m, n] = op(A) op(B) + beta * D with bf16 A, B, fp32 accumulation, D bf16 or fp32 (ldd rows apart).
// op(X) = X^T when transX.  A is stored [m, k] (or [k, m] when transA) with leading dimension lda, B likewise.
// A row-major matrix X[r, c] with row stride ld is the column-major matrix X^T[c, r] with leading dimension ld.
// Enqueues on `st`; returns false if the library refuses the problem (nothing enqueued).
bool gemm(hipStream_t st, bool transA, bool transB, int64_t m, int64_t n, int64_t k, const void* A, int64_t lda,
          const void* B, int64_t ldb, void* D, int64_t ldd, bool out_f32, float beta, void* workspace,
          int64_t workspace_bytes);

}  // namespace lt
}  // namespace aa
