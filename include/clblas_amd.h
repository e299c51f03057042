/*
 * clblas_amd.h -- C ABI of the MI355X (gfx950) BLAS-3 core that stands in for the
 * xGEMM / xTRSM path of clBLAS.
 *
 * The entry points keep clBLAS's names, argument order and status codes.  The only
 * differences to the reference prototypes are the ones a HIP back end forces:
 *   - `cl_mem` matrices become device pointers (`const float *`, `double *`, ...);
 *     element offsets (offA/offB/offC) are kept and are added to those pointers,
 *   - the five trailing queue/event arguments
 *       (numCommandQueues, commandQueues, numEventsInWaitList, eventWaitList, events)
 *     collapse into one `hipStream_t stream`; stream order supplies both the wait and
 *     the completion semantics.
 * Every call returns after enqueueing its work on `stream`.
 *
 * The library is plain C ABI: no C++ or torch types cross it.
 */
#ifndef CLBLAS_AMD_H_
#define CLBLAS_AMD_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same opaque stream type as <hip/hip_runtime_api.h>; repeating the typedef is legal. */
typedef struct ihipStream_t *hipStream_t;

/* In C++ the enumerations get a fixed underlying type (int, what a C compiler gives them on this
 * ABI anyway), so that a value outside the enumerators - which a C caller can pass and which the
 * entry points answer with clblasInvalidValue - is a valid value to read in the C++ implementation
 * as well. */
#ifdef __cplusplus
#define CLBLAS_AMD_ENUM_BASE : int
#else
#define CLBLAS_AMD_ENUM_BASE
#endif

/* Enumerations: numeric values identical to reference src/clBLAS.h:78-113. */
typedef enum clblasOrder_ CLBLAS_AMD_ENUM_BASE {
    clblasRowMajor = 0,
    clblasColumnMajor = 1
} clblasOrder;

typedef enum clblasTranspose_ CLBLAS_AMD_ENUM_BASE {
    clblasNoTrans = 0,
    clblasTrans = 1,
    clblasConjTrans = 2 /* same as clblasTrans for real types (xgemm.cc:330-335) */
} clblasTranspose;

typedef enum clblasUplo_ CLBLAS_AMD_ENUM_BASE {
    clblasUpper = 0,
    clblasLower = 1
} clblasUplo;

typedef enum clblasDiag_ CLBLAS_AMD_ENUM_BASE {
    clblasUnit = 0,
    clblasNonUnit = 1
} clblasDiag;

typedef enum clblasSide_ CLBLAS_AMD_ENUM_BASE {
    clblasLeft = 0,
    clblasRight = 1
} clblasSide;

/* Status codes: numeric values identical to reference src/clBLAS.h:123-155
 * (the OpenCL aliases keep the OpenCL numbers they had there). */
typedef enum clblasStatus_ CLBLAS_AMD_ENUM_BASE {
    clblasSuccess = 0,
    clblasInvalidValue = -30,         /* CL_INVALID_VALUE: bad enum argument */
    clblasInvalidCommandQueue = -36,  /* CL_INVALID_COMMAND_QUEUE */
    clblasInvalidContext = -34,
    clblasInvalidMemObject = -38,
    clblasInvalidDevice = -33,
    clblasInvalidEventWaitList = -57,
    clblasOutOfResources = -5,        /* a HIP launch or allocation failed */
    clblasOutOfHostMemory = -6,
    clblasInvalidOperation = -59,
    clblasCompilerNotAvailable = -3,
    clblasBuildProgramFailure = -11,
    clblasNotImplemented = -1024,
    clblasNotInitialized = -1023,
    clblasInvalidMatA = -1022,
    clblasInvalidMatB = -1021,
    clblasInvalidMatC = -1020,
    clblasInvalidVecX = -1019,
    clblasInvalidVecY = -1018,
    clblasInvalidDim = -1017,
    clblasInvalidLeadDimA = -1016,
    clblasInvalidLeadDimB = -1015,
    clblasInvalidLeadDimC = -1014,
    clblasInvalidIncX = -1013,
    clblasInvalidIncY = -1012,
    clblasInsufficientMemMatA = -1011,
    clblasInsufficientMemMatB = -1010,
    clblasInsufficientMemMatC = -1009,
    clblasInsufficientMemVecX = -1008,
    clblasInsufficientMemVecY = -1007
} clblasStatus;

/* Complex scalars and matrix elements: real part in s[0], imaginary part in s[1].
 * Same size, alignment, element order and by-value calling convention as the reference's
 * FloatComplex / DoubleComplex (src/clBLAS-complex.h:25-26: cl_float2 / cl_double2). */
typedef struct FloatComplex_ { float s[2]; } __attribute__((aligned(8))) FloatComplex;
typedef struct DoubleComplex_ { double s[2]; } __attribute__((aligned(16))) DoubleComplex;

/* Replaces clblasGetVersion (src/clBLAS.h:176-177, src/library/blas/init.c:33-41).
 * Reports this library's own version. Always clblasSuccess. */
clblasStatus clblasGetVersion(unsigned int *major, unsigned int *minor, unsigned int *patch);

/* Replaces clblasSetup (src/clBLAS.h:196-197, src/library/blas/init.c:43-223).
 * Checks that a gfx950 device is current and its code object loads.  No routine of this library
 * requires it: where the reference's S/C/Z TRSM return clblasNotInitialized without it
 * (src/library/blas/functor/functor_xtrsm.cc:57-59), these run (as the reference's GEMM and
 * DTRSM paths do, which never ask).  clblasNotInitialized is never returned. */
clblasStatus clblasSetup(void);

/* Replaces clblasTeardown (src/clBLAS.h:208-209, src/library/blas/init.c:232-263).
 * Waits for every device that holds library-owned scratch buffers (hipDeviceSynchronize) and
 * frees them; buffers of a device that cannot be waited for (one of its streams is being
 * captured) are kept. */
void clblasTeardown(void);

/* Replaces clblasSgemm (src/clBLAS.h:7382-7405, src/library/blas/xgemm.cc:667-723).
 *   C <- alpha * op(A) * op(B) + beta * C, fp32.  beta == 0 means C is not read.
 * Validation order and codes follow xgemm.cc:685-706 and generic/common.c:585-688:
 *   null A/B/C -> clblasInvalidMat{A,B,C}; if K != 0 sizes of A then B; sizes of C.
 * K == 0 computes C <- beta*C (the reference kernel loop is undefined there). */
clblasStatus clblasSgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB,
                         size_t M, size_t N, size_t K, float alpha,
                         const float *A, size_t offA, size_t lda,
                         const float *B, size_t offB, size_t ldb, float beta,
                         float *C, size_t offC, size_t ldc, hipStream_t stream);

/* clblasSgemm for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, validation, kernels and results (bit for bit) as clblasSgemm, but
 * the partial sums of a K split or of a sliced last round of tiles go to a fixed array of
 * CLBLAS_AMD_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process
 * ends, instead of to a per-stream buffer allocated on first use: the call allocates nothing.
 * A call that would need more scratch than that (small C with very deep K: K ranges x N x M
 * rounded up to 64, x 4 bytes) returns clblasOutOfResources and enqueues nothing; calls that
 * need no scratch (the large ones) have no size limit.  All calls on one GPU share the array:
 * calls in order on one stream are safe, calls that overlap in time on one GPU race.
 * The array's device address is looked up once per GPU, by clblasSetup or by the first call on
 * that GPU; that first call must not be made on a stream that is being captured (it returns
 * clblasInvalidOperation then): call clblasSetup, or make one call outside a capture, first. */
#define CLBLAS_AMD_NOALLOC_SCRATCH_BYTES (32u << 20)
clblasStatus clblasSgemmNoAlloc(clblasOrder order, clblasTranspose transA, clblasTranspose transB,
                                size_t M, size_t N, size_t K, float alpha,
                                const float *A, size_t offA, size_t lda,
                                const float *B, size_t offB, size_t ldb, float beta,
                                float *C, size_t offC, size_t ldc, hipStream_t stream);

/* Replaces clblasDgemm (src/clBLAS.h:7463-7486, src/library/blas/xgemm.cc:728-783). */
clblasStatus clblasDgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB,
                         size_t M, size_t N, size_t K, double alpha,
                         const double *A, size_t offA, size_t lda,
                         const double *B, size_t offB, size_t ldb, double beta,
                         double *C, size_t offC, size_t ldc, hipStream_t stream);

/* Replaces clblasCgemm (src/clBLAS.h:7538-7561, src/library/blas/xgemm.cc:788-845).
 *   C <- alpha * op(A) * op(B) + beta * C, complex fp32; clblasConjTrans is the conjugate
 * transpose.  beta == 0+0i means C is not read.  Arithmetic follows the complex TYPE_MAD /
 * TYPE_MAD_WRITE of AutoGemm/KernelOpenCL.py:106-165.  Validation as clblasSgemm.
 * Matrices need only 4-byte alignment. */
clblasStatus clblasCgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB,
                         size_t M, size_t N, size_t K, FloatComplex alpha,
                         const FloatComplex *A, size_t offA, size_t lda,
                         const FloatComplex *B, size_t offB, size_t ldb, FloatComplex beta,
                         FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream);

/* Replaces clblasZgemm (src/clBLAS.h:7622-7645, src/library/blas/xgemm.cc:850-905).
 * Matrices need only 8-byte alignment. */
clblasStatus clblasZgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB,
                         size_t M, size_t N, size_t K, DoubleComplex alpha,
                         const DoubleComplex *A, size_t offA, size_t lda,
                         const DoubleComplex *B, size_t offB, size_t ldb, DoubleComplex beta,
                         DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream);

/* Replaces clblasStrsm (src/clBLAS.h:7988-8008, src/library/blas/xtrsm.cc:1600-1661).
 *   side == Left : solve op(A) * X = alpha * B,  A is M x M
 *   side == Right: solve X * op(A) = alpha * B,  A is N x N
 * X overwrites B (M x N).  Only the `uplo` triangle of A is read and, with
 * diag == Unit, not its diagonal.  Validation follows doTrsm
 * (src/library/blas/functor/functor_xtrsm.cc:57-75): null A/B -> clblasInvalidMat{A,B},
 * then A (msize x msize), then B (M x N). */
clblasStatus clblasStrsm(clblasOrder order, clblasSide side, clblasUplo uplo,
                         clblasTranspose transA, clblasDiag diag, size_t M, size_t N,
                         float alpha, const float *A, size_t offA, size_t lda,
                         float *B, size_t offB, size_t ldb, hipStream_t stream);

/* Replaces clblasDtrsm (src/clBLAS.h:8063-8083, src/library/blas/xtrsm.cc:1663-1785). */
clblasStatus clblasDtrsm(clblasOrder order, clblasSide side, clblasUplo uplo,
                         clblasTranspose transA, clblasDiag diag, size_t M, size_t N,
                         double alpha, const double *A, size_t offA, size_t lda,
                         double *B, size_t offB, size_t ldb, hipStream_t stream);

/* Replaces clblasCtrsm (src/clBLAS.h:8132-8152, src/library/blas/xtrsm.cc:1789-1850).
 * transA == clblasConjTrans solves with the conjugate transpose of A. */
clblasStatus clblasCtrsm(clblasOrder order, clblasSide side, clblasUplo uplo,
                         clblasTranspose transA, clblasDiag diag, size_t M, size_t N,
                         FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                         FloatComplex *B, size_t offB, size_t ldb, hipStream_t stream);

/* Replaces clblasZtrsm (src/clBLAS.h:8202-8222, src/library/blas/xtrsm.cc:1852-1914). */
clblasStatus clblasZtrsm(clblasOrder order, clblasSide side, clblasUplo uplo,
                         clblasTranspose transA, clblasDiag diag, size_t M, size_t N,
                         DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                         DoubleComplex *B, size_t offB, size_t ldb, hipStream_t stream);

/* ---- GEMM-shaped neighbours on the same MFMA core: SYRK, TRMM, SYMM, SYR2K (all four types), HERK, HER2K, HEMM ---- */

/* Replace clblas{S,D,C,Z}syrk (src/clBLAS.h:8278-8503, src/library/blas/xsyrk.c:27-233).
 *   C <- alpha * op(A) * op(A)^T + beta * C, C is N x N and only its `uplo` triangle is read
 * or written; op(A) is N x K (transA == NoTrans: A is N x K, else K x N).  Validation follows
 * doSyrk (xsyrk.c:56-72): null A/C -> clblasInvalidMat{A,C}; clblasConjTrans with a complex
 * type -> clblasInvalidValue; sizes of A, then C (K == 0 -> clblasInvalidDim). */
clblasStatus clblasSsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         float alpha, const float *A, size_t offA, size_t lda, float beta,
                         float *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8278-8297 */
clblasStatus clblasDsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         double alpha, const double *A, size_t offA, size_t lda, double beta,
                         double *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8350-8369 */
clblasStatus clblasCsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda, FloatComplex beta,
                         FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8416-8435 */
clblasStatus clblasZsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda, DoubleComplex beta,
                         DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8484-8503 */

/* Replace clblas{S,D,C,Z}trmm (src/clBLAS.h:7696-7928, src/library/blas/xtrmm.c:27-245).
 *   side == Left : B <- alpha * op(A) * B,  A is M x M
 *   side == Right: B <- alpha * B * op(A),  A is N x N
 * A triangular; only its `uplo` triangle is read and, with diag == Unit, not its diagonal.
 * Validation as clblas?trsm (xtrmm.c:47-64).  Uses a library-owned M x N device workspace. */
clblasStatus clblasStrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA,
                         clblasDiag diag, size_t M, size_t N, float alpha,
                         const float *A, size_t offA, size_t lda,
                         float *B, size_t offB, size_t ldb, hipStream_t stream); /* src/clBLAS.h:7696-7716 */
clblasStatus clblasDtrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA,
                         clblasDiag diag, size_t M, size_t N, double alpha,
                         const double *A, size_t offA, size_t lda,
                         double *B, size_t offB, size_t ldb, hipStream_t stream); /* src/clBLAS.h:7771-7791 */
clblasStatus clblasCtrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA,
                         clblasDiag diag, size_t M, size_t N, FloatComplex alpha,
                         const FloatComplex *A, size_t offA, size_t lda,
                         FloatComplex *B, size_t offB, size_t ldb, hipStream_t stream); /* src/clBLAS.h:7838-7858 */
clblasStatus clblasZtrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA,
                         clblasDiag diag, size_t M, size_t N, DoubleComplex alpha,
                         const DoubleComplex *A, size_t offA, size_t lda,
                         DoubleComplex *B, size_t offB, size_t ldb, hipStream_t stream); /* src/clBLAS.h:7908-7928 */

/* Replace clblas{S,D,C,Z}symm (src/clBLAS.h:8897-9145, src/library/blas/xsymm.c:33-429).
 *   side == Left : C <- alpha * A * B + beta * C,  A is M x M
 *   side == Right: C <- alpha * B * A + beta * C,  A is N x N
 * A symmetric (not Hermitian), only its `uplo` triangle is read; B and C are M x N.
 * Validation follows doSymm (xsymm.c:50-71): null A/B/C, sizes of A, B, C in that order. */
clblasStatus clblasSsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N,
                         float alpha, const float *A, size_t offA, size_t lda,
                         const float *B, size_t offB, size_t ldb, float beta,
                         float *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8897-8919 */
clblasStatus clblasDsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N,
                         double alpha, const double *A, size_t offA, size_t lda,
                         const double *B, size_t offB, size_t ldb, double beta,
                         double *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8978-9000 */
clblasStatus clblasCsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N,
                         FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                         const FloatComplex *B, size_t offB, size_t ldb, FloatComplex beta,
                         FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9051-9073 */
clblasStatus clblasZsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N,
                         DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                         const DoubleComplex *B, size_t offB, size_t ldb, DoubleComplex beta,
                         DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9123-9145 */

/* Replace clblas{S,D,C,Z}syr2k (src/clBLAS.h:8568-8819, src/library/blas/xsyr2k.c:27-251).
 *   C <- alpha * (op(A) * op(B)^T + op(B) * op(A)^T) + beta * C on the `uplo` triangle of the
 * N x N matrix C; op(A), op(B) are N x K.  Validation follows doSyr2k (xsyr2k.c:58-76): null
 * A/B/C, clblasConjTrans with a complex type -> clblasInvalidValue, sizes of A, B, then C. */
clblasStatus clblasSsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          float alpha, const float *A, size_t offA, size_t lda,
                          const float *B, size_t offB, size_t ldb, float beta,
                          float *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8568-8589 */
clblasStatus clblasDsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          double alpha, const double *A, size_t offA, size_t lda,
                          const double *B, size_t offB, size_t ldb, double beta,
                          double *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8648-8669 */
clblasStatus clblasCsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                          const FloatComplex *B, size_t offB, size_t ldb, FloatComplex beta,
                          FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8722-8743 */
clblasStatus clblasZsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                          const DoubleComplex *B, size_t offB, size_t ldb, DoubleComplex beta,
                          DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:8798-8819 */

/* Replace clblas{C,Z}herk (src/clBLAS.h:9389-9476, src/library/blas/xherk.c:132-210).
 *   C <- alpha * op(A) * op(A)^H + beta * C, alpha and beta real, C Hermitian N x N: only its
 * `uplo` triangle is read or written, imaginary parts of its diagonal are ignored on input and
 * stored as zero.  transA is NoTrans or ConjTrans; Trans is rejected with clblasInvalidValue, xherk.c:69-71. */
clblasStatus clblasCherk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         float alpha, const FloatComplex *A, size_t offA, size_t lda, float beta,
                         FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9389-9407 */
clblasStatus clblasZherk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         double alpha, const DoubleComplex *A, size_t offA, size_t lda, double beta,
                         DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9458-9476 */

/* Replace clblas{C,Z}her2k (src/clBLAS.h:9545-9644, src/library/blas/xher2k.c:155-245).
 *   C <- alpha * op(A) * op(B)^H + conj(alpha) * op(B) * op(A)^H + beta * C, beta real, C
 * Hermitian as for herk.  Validation follows doHer2k (xher2k.c:73-97). */
clblasStatus clblasCher2k(clblasOrder order, clblasUplo uplo, clblasTranspose trans, size_t N, size_t K,
                          FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                          const FloatComplex *B, size_t offB, size_t ldb, float beta,
                          FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9545-9566 */
clblasStatus clblasZher2k(clblasOrder order, clblasUplo uplo, clblasTranspose trans, size_t N, size_t K,
                          DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                          const DoubleComplex *B, size_t offB, size_t ldb, double beta,
                          DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9623-9644 */

/* Replace clblas{C,Z}hemm (src/clBLAS.h:9224-9326, src/library/blas/xhemm.c:36-112).
 *   side == Left : C <- alpha * A * B + beta * C,  A Hermitian M x M
 *   side == Right: C <- alpha * B * A + beta * C,  A Hermitian N x N
 * Only the `uplo` triangle of A is read; imaginary parts of its diagonal are ignored.
 * Validation and row-major folding are SYMM's (xhemm.c:69-73 -> doSymm, xsymm.c:50-124). */
clblasStatus clblasChemm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N,
                         FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                         const FloatComplex *B, size_t offB, size_t ldb, FloatComplex beta,
                         FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9224-9245 */
clblasStatus clblasZhemm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N,
                         DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                         const DoubleComplex *B, size_t offB, size_t ldb, DoubleComplex beta,
                         DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream); /* src/clBLAS.h:9305-9326 */

/* ---- Workspace and diagnostics.  These four have no counterpart in the reference: clBLAS allocates
 * and frees its temporaries inside every call (src/library/blas/xtrsm.cc:1186-1207, 1499-1500) and
 * logs nothing; this library keeps scratch buffers per (device, stream) and lets the caller
 * manage them. ---- */

/* Waits for `stream` (hipStreamSynchronize) and frees the scratch buffers kept for it on the current
 * device.  Call it before destroying the stream.  clblasInvalidOperation, and nothing freed, if the
 * stream is being captured.  Without it a process still holds a bounded amount: at most 32 streams per
 * device keep buffers, the least recently used one is evicted (after a device synchronisation; none if
 * that fails) when another appears - never one that a running call has been handed buffers of, nor
 * one whose buffers were handed out while the stream was being captured.
 * A HIP graph captured from calls of this library holds raw pointers into its stream's buffers: do not
 * call this for that stream, nor clblasTeardown, while such a graph can still be launched. */
clblasStatus clblasAmdReleaseStream(hipStream_t stream);

/* Makes sure the scratch buffers of `stream` on the current device are at least this large
 * (bytes; 0 leaves a buffer alone):
 *   gemm_bytes  GEMM-shaped calls (every routine of this library ends in them) that cut K into
 *               ranges (ranges x M x N elements, M rounded up to 64, at most 512 ranges) or slice
 *               their last round of tiles (at most 256 tiles of 256 x 128 elements);
 *   trmm_bytes  TRMM's copy of B (M x N elements, M rounded up to 64), and the full N x N product
 *               (N rounded up to 64, times N elements) of a rank-k update - SYRK, SYR2K, HERK,
 *               HER2K - of a small C with a deep K (N <= 704 and K >= 4096), which also takes
 *               gemm_bytes for its K ranges;
 *   trsm_bytes  TRSM's packed diagonal blocks (real types: 135 168 elements per 512 rows of the
 *               triangle or part thereof; complex types: 104 448 real elements per 256 rows).
 * A later call on the stream whose needs fit allocates nothing, so it can be the first thing recorded
 * into a HIP graph.  A call that would have to allocate while its stream is being captured returns
 * clblasInvalidOperation, enqueues nothing - routines made of several launches find out before the
 * first one - and leaves the capture valid. */
clblasStatus clblasAmdReserveWorkspace(hipStream_t stream, size_t gemm_bytes, size_t trmm_bytes, size_t trsm_bytes);

/* Number of streams that hold scratch buffers, and the bytes of their buffers (current ones plus
 * outgrown ones that are parked until the stream is released). */
void clblasAmdWorkspaceStats(size_t *streams, size_t *bytes);

/* The tile choice of clblasSgemm (type 's') / clblasDgemm ('d') / clblasCgemm ('c') / clblasZgemm ('z') for a plain M x N x K product, as a
 * function that launches nothing: the chosen tile (index into the type's tile table), its number of K
 * ranges and tail slices, the cost the choice model puts on every tile in one K range (negative: tile not
 * offered) and the tiles' dimensions (bm, bn, bk per tile, 3 ints each; `costs` and `dims` hold max_tiles
 * entries).  Returns the number of tiles in the table, -1 for bad arguments.  (The answer is for the product
 * as given, in one piece: the launcher may in addition make a strip of up to 64 rows or columns beyond a
 * multiple of 128 as a product of its own where this same model prices the two pieces lower.)
 * clblasAmdTileModelParam reads (set == 0) or sets one parameter of one tile's model - which: 0 the
 * efficiency credited to the tile, 1 the factor for a workgroup alone on its CU, 2 the fixed time per
 * workgroup as a depth, 3 the price of a sliced tail in rounds, 4 the credit of the deep-panel form, 5 the
 * factor on the efficiency in a launch that cuts K into ranges, 6 the factor on the efficiency where the
 * operands are streamed from HBM - returning 0, or -1 for no such tile or parameter.  Both exist for clblas_amd/fit_tile_model.py, which
 * refits the parameters to measured times; setting parameters while another thread is inside a GEMM call
 * is not supported.  No counterpart in the reference (its selection table is generated at build time,
 * src/library/blas/AutoGemm/KernelSelection.py). */
int clblasAmdTileModelQuery(char type, size_t M, size_t N, size_t K, int *tile, int *splits, int *tail_slices,
                            double *costs, int *dims, int max_tiles);
int clblasAmdTileModelParam(char type, int tile, int which, double *value, int set);

/* The TRSM kernel that solves a diagonal block by substitution synchronises its wavefronts through
 * flags in LDS; a wait for a flag gives up after a bounded number of polls (so that a mistake in the
 * library would end in a wrong result, not in a hung GPU).  This reads, for the current GPU, how many
 * waits have ever given up since the library was loaded - zero unless the library is broken or the
 * debugging variable CLBLAS_AMD_TRSM_POLL_LIMIT makes the bound tiny - and, with reset != 0, sets the
 * count back to zero.  It waits for the device (a blocking copy).  No counterpart in the reference. */
clblasStatus clblasAmdTrsmPollTimeouts(unsigned int *count, int reset);

/* Describes the last GEMM kernel the calling thread launched (kernel family, tile, transposes,
 * sizes, grid, K ranges), as text; returns the number of kernel launches the thread has issued
 * through this library.  With CLBLAS_AMD_LOG=1 in the environment every launch also prints
 * such a line on stderr. */
size_t clblasAmdLastDispatch(char *text, size_t size);

/* The library reads its debugging environment variables (CLBLAS_AMD_*) once, at first use.
 * This reads them again.  Debugging only: not to be called while another thread is inside a
 * library call. */
void clblasAmdReloadDebugEnv(void);

#ifdef __cplusplus
}
#endif

#endif /* CLBLAS_AMD_H_ */
