// Declarations shared between the translation units of libclblas_amd.so.
// Nothing here is part of the exported C ABI.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace cba {

// Complex element, laid out as the reference's FloatComplex / DoubleComplex (cl_float2 /
// cl_double2, src/clBLAS-complex.h:25-26: real part first).
template <typename R> struct Cx { R re, im; };

// Debug-only override of the GEMM tile choice: index into the per-type tile table taken
// from the environment variable CLBLAS_AMD_GEMM_TILE, or -1.
int forced_gemm_tile();

// Debug-only integer knob from the environment (tile walk order experiments), or `dflt`.
int debug_env_int(const char *name, int dflt);

// Library-owned device scratch for `stream` on the current device, at least `bytes` long.
// Grown on demand; earlier, smaller buffers stay alive until clblasTeardown so that work
// already enqueued on them remains valid.  Returns nullptr if the allocation fails.
void *workspace_get(hipStream_t stream, size_t bytes);
void workspace_release_all();

// Raises a kernel's dynamic LDS limit (needed above 64 KiB); cached per function.
hipError_t ensure_dynamic_lds(const void *fn, size_t bytes);

// Column-major GEMM launchers.  Arguments are already validated and folded to column
// major; pointers already include their element offsets.
hipError_t sgemm_colmajor(bool transA, bool transB, int M, int N, int K, float alpha, const float *A, int64_t lda,
                          const float *B, int64_t ldb, float beta, float *C, int64_t ldc, hipStream_t stream);
hipError_t dgemm_colmajor(bool transA, bool transB, int M, int N, int K, double alpha, const double *A,
                          int64_t lda, const double *B, int64_t ldb, double beta, double *C, int64_t ldc,
                          hipStream_t stream);

// Complex variants: conjA / conjB conjugate the elements of op(A) / op(B) (clblasConjTrans).
hipError_t cgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<float> alpha,
                          const Cx<float> *A, int64_t lda, const Cx<float> *B, int64_t ldb, Cx<float> beta,
                          Cx<float> *C, int64_t ldc, hipStream_t stream);
hipError_t zgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<double> alpha,
                          const Cx<double> *A, int64_t lda, const Cx<double> *B, int64_t ldb, Cx<double> beta,
                          Cx<double> *C, int64_t ldc, hipStream_t stream);

// Column-major TRSM drivers (same conventions).
hipError_t strsm_colmajor(bool right, bool lower, bool trans, bool unit, int M, int N, float alpha, const float *A,
                          int64_t lda, float *B, int64_t ldb, hipStream_t stream);
hipError_t dtrsm_colmajor(bool right, bool lower, bool trans, bool unit, int M, int N, double alpha,
                          const double *A, int64_t lda, double *B, int64_t ldb, hipStream_t stream);

}  // namespace cba
