// Builds the reference's own CPU statement of GEMM / TRSM -- the "naive BLAS" its kernel
// test tool checks against -- straight from the reference tree, for use as a second
// opinion on oracle.c.  TEST INFRASTRUCTURE ONLY.
//
// The reference file is included by path from where it lies
// (REF_ROOT/src/library/tools/ktest/naive/naive_blas.cpp); no reference text is copied into
// this repository.  That file has no includes of its own, so the headers it relies on
// (all present in this image) are pulled in first.
#include <CL/cl.h>

#include <cmath>
#include <cstddef>
#include <cstdlib>
#include <string>
using std::isnan;

#include REF_NAIVE_BLAS_CPP

// Scalar of type T (a real, or a complex made of two R) read from its address.
template <typename T, typename R> static T ref_scalar(const void *p) {
    T z;
    *(R *)&z = ((const R *)p)[0];
    if (sizeof(T) == 2 * sizeof(R)) ((R *)&z)[1] = ((const R *)p)[1];
    return z;
}

extern "C" {

void ref_naive_sgemm(int order, int transA, int transB, size_t M, size_t N, size_t K, float alpha, const float *A,
                     size_t lda, const float *B, size_t ldb, float beta, float *C, size_t ldc) {
    NaiveBlas::gemm<float>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasTranspose)transA,
                           (NaiveBlas::clblasTranspose)transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

void ref_naive_dgemm(int order, int transA, int transB, size_t M, size_t N, size_t K, double alpha,
                     const double *A, size_t lda, const double *B, size_t ldb, double beta, double *C,
                     size_t ldc) {
    NaiveBlas::gemm<double>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasTranspose)transA,
                            (NaiveBlas::clblasTranspose)transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

// Complex: alpha / beta are passed by address (re, im); matrices are interleaved pairs with
// the layout of FloatComplex / DoubleComplex.
void ref_naive_cgemm(int order, int transA, int transB, size_t M, size_t N, size_t K, const float *alpha,
                     const void *A, size_t lda, const void *B, size_t ldb, const float *beta, void *C, size_t ldc) {
    NaiveBlas::FloatComplex al, be;
    al.s[0] = alpha[0]; al.s[1] = alpha[1];
    be.s[0] = beta[0]; be.s[1] = beta[1];
    NaiveBlas::gemm<NaiveBlas::FloatComplex>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasTranspose)transA,
                                  (NaiveBlas::clblasTranspose)transB, M, N, K, al, (const NaiveBlas::FloatComplex *)A, lda,
                                  (const NaiveBlas::FloatComplex *)B, ldb, be, (NaiveBlas::FloatComplex *)C, ldc);
}

void ref_naive_zgemm(int order, int transA, int transB, size_t M, size_t N, size_t K, const double *alpha,
                     const void *A, size_t lda, const void *B, size_t ldb, const double *beta, void *C,
                     size_t ldc) {
    NaiveBlas::DoubleComplex al, be;
    al.s[0] = alpha[0]; al.s[1] = alpha[1];
    be.s[0] = beta[0]; be.s[1] = beta[1];
    NaiveBlas::gemm<NaiveBlas::DoubleComplex>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasTranspose)transA,
                                   (NaiveBlas::clblasTranspose)transB, M, N, K, al, (const NaiveBlas::DoubleComplex *)A, lda,
                                   (const NaiveBlas::DoubleComplex *)B, ldb, be, (NaiveBlas::DoubleComplex *)C, ldc);
}

void ref_naive_strsm(int order, int side, int uplo, int transA, int diag, size_t M, size_t N, float alpha,
                     const float *A, size_t lda, float *B, size_t ldb) {
    NaiveBlas::trsm<float>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasSide)side, (NaiveBlas::clblasUplo)uplo,
                           (NaiveBlas::clblasTranspose)transA, (NaiveBlas::clblasDiag)diag, M, N, alpha, A, lda, B,
                           ldb);
}

void ref_naive_dtrsm(int order, int side, int uplo, int transA, int diag, size_t M, size_t N, double alpha,
                     const double *A, size_t lda, double *B, size_t ldb) {
    NaiveBlas::trsm<double>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasSide)side,
                            (NaiveBlas::clblasUplo)uplo, (NaiveBlas::clblasTranspose)transA,
                            (NaiveBlas::clblasDiag)diag, M, N, alpha, A, lda, B, ldb);
}

// SYRK and TRMM of the reference's naive BLAS; scalars by address, T selected by `type`
// (0 float, 1 double, 2 FloatComplex, 3 DoubleComplex).
#define REF_DISPATCH(CALL)                                                            \
    switch (type) {                                                                   \
    case 0: { typedef float T; typedef float R; CALL; break; }                        \
    case 1: { typedef double T; typedef double R; CALL; break; }                      \
    case 2: { typedef NaiveBlas::FloatComplex T; typedef float R; CALL; break; }      \
    default: { typedef NaiveBlas::DoubleComplex T; typedef double R; CALL; break; }   \
    }

void ref_naive_syrk(int type, int order, int uplo, int trans, size_t N, size_t K, const void *alpha, const void *A,
                    size_t lda, const void *beta, void *C, size_t ldc) {
    REF_DISPATCH((NaiveBlas::syrk<T>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasUplo)uplo,
                                     (NaiveBlas::clblasTranspose)trans, N, K, ref_scalar<T, R>(alpha), (const T *)A,
                                     lda, ref_scalar<T, R>(beta), (T *)C, ldc)))
}

void ref_naive_syr2k(int type, int order, int uplo, int trans, size_t N, size_t K, const void *alpha, const void *A,
                     size_t lda, const void *B, size_t ldb, const void *beta, void *C, size_t ldc) {
    REF_DISPATCH((NaiveBlas::syr2k<T>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasUplo)uplo,
                                      (NaiveBlas::clblasTranspose)trans, N, K, ref_scalar<T, R>(alpha), (const T *)A,
                                      lda, (const T *)B, ldb, ref_scalar<T, R>(beta), (T *)C, ldc)))
}

void ref_naive_trmm(int type, int order, int side, int uplo, int trans, int diag, size_t M, size_t N,
                    const void *alpha, const void *A, size_t lda, void *B, size_t ldb) {
    REF_DISPATCH((NaiveBlas::trmm<T>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasSide)side,
                                     (NaiveBlas::clblasUplo)uplo, (NaiveBlas::clblasTranspose)trans,
                                     (NaiveBlas::clblasDiag)diag, M, N, ref_scalar<T, R>(alpha), (const T *)A, lda,
                                     (T *)B, ldb)))
}

void ref_naive_trsm(int type, int order, int side, int uplo, int trans, int diag, size_t M, size_t N,
                    const void *alpha, const void *A, size_t lda, void *B, size_t ldb) {
    REF_DISPATCH((NaiveBlas::trsm<T>((NaiveBlas::clblasOrder)order, (NaiveBlas::clblasSide)side,
                                     (NaiveBlas::clblasUplo)uplo, (NaiveBlas::clblasTranspose)trans,
                                     (NaiveBlas::clblasDiag)diag, M, N, ref_scalar<T, R>(alpha), (const T *)A, lda,
                                     (T *)B, ldb)))
}

}  // extern "C"
