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
// `kind` separates buffers that are alive at the same time (0: split-K partial sums,
// 1: the operand copy of an in-place routine).
void *workspace_get(hipStream_t stream, size_t bytes, int kind = 0);
void workspace_release_all();

// Raises a kernel's dynamic LDS limit (needed above 64 KiB); cached per function.
hipError_t ensure_dynamic_lds(const void *fn, size_t bytes);

// Triangular structure of a GEMM-shaped call (SYRK, TRMM).
//   tri_c: only the lower (1) / upper (2) triangle of C is computed and stored.
//   tri_a / tri_b: op(A)(m,k) / op(B)(k,n) is triangular: entries with k > x (1) or k < x (2),
//   x = m resp. n, count as zero whatever memory holds; unit_* = 1: the diagonal counts as
//   one, 2: as zero (strict triangle), 3: as its real part (diagonal of a Hermitian matrix).
//   herm_c (with tri_c, complex types): C is Hermitian, its diagonal is stored with zero
//   imaginary parts.
struct GemmTri {
    int tri_c = 0, tri_a = 0, tri_b = 0, unit_a = 0, unit_b = 0, herm_c = 0;
    bool any() const { return tri_c || tri_a || tri_b; }
};

// Column-major GEMM launchers.  Arguments are already validated and folded to column
// major; pointers already include their element offsets.
hipError_t sgemm_colmajor(bool transA, bool transB, int M, int N, int K, float alpha, const float *A, int64_t lda,
                          const float *B, int64_t ldb, float beta, float *C, int64_t ldc, hipStream_t stream,
                          const GemmTri *tri = nullptr);
hipError_t dgemm_colmajor(bool transA, bool transB, int M, int N, int K, double alpha, const double *A,
                          int64_t lda, const double *B, int64_t ldb, double beta, double *C, int64_t ldc,
                          hipStream_t stream, const GemmTri *tri = nullptr);

// Complex variants: conjA / conjB conjugate the elements of op(A) / op(B) (clblasConjTrans).
hipError_t cgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<float> alpha,
                          const Cx<float> *A, int64_t lda, const Cx<float> *B, int64_t ldb, Cx<float> beta,
                          Cx<float> *C, int64_t ldc, hipStream_t stream, const GemmTri *tri = nullptr);
hipError_t zgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<double> alpha,
                          const Cx<double> *A, int64_t lda, const Cx<double> *B, int64_t ldb, Cx<double> beta,
                          Cx<double> *C, int64_t ldc, hipStream_t stream, const GemmTri *tri = nullptr);

// The four launchers above behind one name (conjA / conjB are ignored by the real types).
template <typename T>
hipError_t launch_gemm(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, T alpha, const T *A,
                       int64_t lda, const T *B, int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream,
                       const GemmTri *tri = nullptr);

// Column-major SYRK / TRMM / SYMM drivers built on the GEMM launchers (level3.hip).
//   syrk: C <- alpha op(A) op(A)^T + beta C on the `lower` / upper triangle of C (N x N).
//   trmm: B <- alpha op(A) B (left) or alpha B op(A) (right), A triangular, in place.
//   symm: C <- alpha A B + beta C (left) or alpha B A + beta C (right), A symmetric with only
//         its `lower` / upper triangle stored.
template <typename T>
hipError_t syrk_colmajor(bool lower, bool trans, int N, int K, T alpha, const T *A, int64_t lda, T beta, T *C,
                         int64_t ldc, hipStream_t stream);
template <typename T>
hipError_t trmm_colmajor(bool right, bool lower, bool trans, bool conj, bool unit, int M, int N, T alpha, const T *A,
                         int64_t lda, T *B, int64_t ldb, hipStream_t stream);
template <typename T>
hipError_t symm_colmajor(bool right, bool lower, int M, int N, T alpha, const T *A, int64_t lda, const T *B,
                         int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream);
// syr2k: C <- alpha (op(A) op(B)^T + op(B) op(A)^T) + beta C on one triangle of C.
template <typename T>
hipError_t syr2k_colmajor(bool lower, bool trans, int N, int K, T alpha, const T *A, int64_t lda, const T *B,
                          int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream);
// herk: C <- alpha op(A) op(A)^H + beta C; her2k: C <- alpha op(A) op(B)^H + conj(alpha) op(B) op(A)^H
// + beta C; op = identity or conjugate transpose (`ctrans`), real beta (and alpha for herk), C Hermitian.
template <typename R>
hipError_t herk_colmajor(bool lower, bool ctrans, int N, int K, R alpha, const Cx<R> *A, int64_t lda, R beta,
                         Cx<R> *C, int64_t ldc, hipStream_t stream);
template <typename R>
hipError_t her2k_colmajor(bool lower, bool ctrans, int N, int K, Cx<R> alpha, const Cx<R> *A, int64_t lda,
                          const Cx<R> *B, int64_t ldb, R beta, Cx<R> *C, int64_t ldc, hipStream_t stream);
// hemm: as symm with A Hermitian (complex types).
template <typename T>
hipError_t hemm_colmajor(bool right, bool lower, int M, int N, T alpha, const T *A, int64_t lda, const T *B,
                         int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream);


// Column-major TRSM driver (trsm.hip), all four types: solves op(A) X = alpha B (left) or
// X op(A) = alpha B (right) in place; `conj` conjugates op(A) (complex, clblasConjTrans).
template <typename T>
hipError_t trsm_colmajor(bool right, bool lower, bool trans, bool conj, bool unit, int M, int N, T alpha, const T *A,
                         int64_t lda, T *B, int64_t ldb, hipStream_t stream);

}  // namespace cba
