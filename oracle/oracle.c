/*
 * oracle.c -- CPU restatement of the clBLAS xGEMM / xTRSM hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links or calls this file; it is
 * used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py as the
 * checker / the timed CPU reference.
 *
 * Every function names the reference lines (relative to the clBLAS source tree) it follows.
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   oracle_{s,d}gemm        - README.md:77-156 and src/samples/example_sgemm.c:31-73 fixed
 *                             inputs with hand-computed expected outputs; integer-exact inputs
 *                             (src/tests/include/blas-random.h:60-93) against exact integer
 *                             products; closed forms (identity, rank-1, alpha=0, NaN in C with
 *                             beta=0); transposition and row/column-major identities; the
 *                             reference's own naive gemm compiled from
 *                             src/library/tools/ktest/naive/naive_blas.cpp (oracle/_ref).
 *   oracle_{s,d}gemm_exact  - same integer-exact inputs (must reproduce them exactly).
 *   oracle_{c,z}gemm(_exact)- Gaussian-integer inputs against exact integer products for every
 *                             order / transpose / conjugate combination; closed forms (i*i,
 *                             identity, Hermitian products have real diagonals, alpha / beta
 *                             rotations by i); conjugation identities; the reference's own
 *                             naive complex gemm (oracle/_ref).
 *   oracle_{s,d}trsm_naive  - TRSM_extratest closed form (src/tests/correctness/corr-trsm.cpp:
 *                             240-452, X_r = r+1); src/samples/example_strsm.c:30-63 fixed
 *                             input; oracle/_ref naive trsm; residual identities.
 *   oracle_{c,z}trsm_naive  - src/samples/example_ctrsm.c fixed input solved exactly; oracle/_ref
 *                             naive trsm<FloatComplex/DoubleComplex>; residual against a complex
 *                             product computed with numpy; real-embedding identity (a complex
 *                             system with zero imaginary parts equals the real routine).
 *   oracle_{s,d}trsm_blocked- the same, plus agreement with the naive solver within the
 *                             reference's own per-element bound (trsm-delta.h:44-240 style),
 *                             NaN-poisoned unused triangle, zero-diagonal -> 1 behaviour.
 *   oracle_{s,d,c,z}{syrk,trmm,symm} (level3.inc)
 *                           - exact-integer inputs against exact integer products for every
 *                             order / side / triangle / transpose / diagonal combination with
 *                             the unused triangle NaN-poisoned; the reference's own naive syrk
 *                             and trmm (oracle/_ref); SYMM, which has no naive statement in the
 *                             reference, against oracle GEMM on the explicitly symmetrised
 *                             matrix; TRMM followed by TRSM returns the input.
 *   oracle_{s,d,c,z}syr2k, oracle_{c,z}{herk,her2k,hemm} (level3.inc)
 *                           - src/samples/example_{ssyr2k.c,cherk.cpp,cher2k.c,chemm.cpp} fixed
 *                             inputs against exact expected values (complex diagonals with
 *                             non-zero imaginary parts included); exact-integer inputs against
 *                             products evaluated with numpy for every order / side / triangle /
 *                             transpose combination, unused triangle NaN-poisoned; the
 *                             reference's own naive syr2k (oracle/_ref); HEMM against oracle
 *                             GEMM on the explicitly formed Hermitian matrix; HER2K with B == A
 *                             against HERK.  (The reference has no naive herk / her2k / hemm.)
 *   oracle_trsm_ref_inputs, oracle_trsm_hp (trsm_reftest.inc)
 *                           - see the header of that file (tests/test_oracle_trsm_reftest.py).
 *   oracle_check_*          - expectations of src/tests/functional/func-error.cpp:58-104 and
 *                             the branch table of generic/common.c:585-688.
 *   Bit-for-bit output of the OpenCL kernels (implementation-defined `mad` contraction,
 *   AutoGemm/KernelOpenCL.py:100) is NOT pinned: no OpenCL device exists to run them.
 *   Parity is judged with the K*eps bound, as the task states.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* enum values of src/clBLAS.h:78-155 */
enum { ROW_MAJOR = 0, COL_MAJOR = 1 };
enum { NO_TRANS = 0, TRANS = 1, CONJ_TRANS = 2 };
enum { UPPER = 0, LOWER = 1 };
enum { UNIT = 0, NON_UNIT = 1 };
enum { LEFT = 0, RIGHT = 1 };
enum {
    ST_SUCCESS = 0,
    ST_INVALID_VALUE = -30,
    ST_NOT_IMPLEMENTED = -1024,
    ST_INVALID_MAT_A = -1022,
    ST_INVALID_MAT_B = -1021,
    ST_INVALID_MAT_C = -1020,
    ST_INVALID_DIM = -1017,
    ST_INVALID_LD_A = -1016,
    ST_INVALID_LD_B = -1015,
    ST_INVALID_LD_C = -1014,
    ST_INSUFF_A = -1011,
    ST_INSUFF_B = -1010,
    ST_INSUFF_C = -1009
};

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------ */
/* Argument checks                                                                       */
/* ------------------------------------------------------------------------------------ */

/* checkMatrixSizes, src/library/blas/generic/common.c:585-688.  which: 0=A 1=B 2=C.
 * mem_elems: size of the buffer in elements, or 0 for "unknown / large enough". */
static int check_matrix_sizes(int order, int trans, size_t M, size_t N, size_t off, size_t ld, size_t mem_elems,
                              int which) {
    size_t matr;
    int tra;
    if (M == 0 || N == 0) return ST_INVALID_DIM; /* :601-603 */
    tra = (order == ROW_MAJOR && trans != NO_TRANS) || (order == COL_MAJOR && trans == NO_TRANS); /* :606-607 */
    if (tra) {
        if (ld < M) return ST_INVALID_LD_A + which; /* :610-624 */
        matr = (N - 1) * ld + M;                    /* :625 */
    } else {
        if (ld < N) return ST_INVALID_LD_A + which; /* :628-641 */
        matr = (M - 1) * ld + N;                    /* :642 */
    }
    if (mem_elems != 0 && off + matr > mem_elems) return ST_INSUFF_A + which; /* :670-684 */
    return ST_SUCCESS;
}

/* clblasSgemm / clblasDgemm front-end checks, src/library/blas/xgemm.cc:685-706.
 * haveX: nonzero if the X object is valid (checkMemObjects, generic/common.c:837-900). */
int oracle_check_gemm(int order, int transA, int transB, size_t M, size_t N, size_t K, int haveA, size_t offA,
                      size_t lda, size_t memA, int haveB, size_t offB, size_t ldb, size_t memB, int haveC,
                      size_t offC, size_t ldc, size_t memC) {
    int st;
    if (!haveA) return ST_INVALID_MAT_A;
    if (!haveB) return ST_INVALID_MAT_B;
    if (!haveC) return ST_INVALID_MAT_C;
    if (K != 0) {
        if ((st = check_matrix_sizes(order, transA, M, K, offA, lda, memA, 0))) return st;
        if ((st = check_matrix_sizes(order, transB, K, N, offB, ldb, memB, 1))) return st;
    }
    return check_matrix_sizes(order, NO_TRANS, M, N, offC, ldc, memC, 2);
}

/* doTrsm checks, src/library/blas/functor/functor_xtrsm.cc:57-75. */
int oracle_check_trsm(int order, int side, int transA, size_t M, size_t N, int haveA, size_t offA, size_t lda,
                      size_t memA, int haveB, size_t offB, size_t ldb, size_t memB) {
    int st;
    size_t msize = side == LEFT ? M : N;
    if (!haveA) return ST_INVALID_MAT_A;
    if (!haveB) return ST_INVALID_MAT_B;
    if ((st = check_matrix_sizes(order, transA, msize, msize, offA, lda, memA, 0))) return st;
    return check_matrix_sizes(order, NO_TRANS, M, N, offB, ldb, memB, 1);
}

/* ------------------------------------------------------------------------------------ */
/* GEMM                                                                                  */
/* ------------------------------------------------------------------------------------ */

/* Column-major kernel arithmetic, src/library/blas/AutoGemm/KernelOpenCL.py:
 *   :311-422  one accumulator per C element, k strictly ascending, TYPE_MAD = mad(a,b,acc)
 *             (restated as a fused multiply-add)
 *   :100-104  epilogue  C = alpha*acc + beta*C  (beta != 0)   or   C = alpha*acc (beta == 0,
 *             C never read)
 * Element addressing: :68-81.  The loops are arranged so that rows of C vectorise; every
 * element still sees k = 0,1,2,... in order. */
#define GEMM_COLMAJOR(NAME, T, FMA)                                                                         \
    static void NAME(int tA, int tB, size_t M, size_t N, size_t K, T alpha, const T *A, size_t lda,         \
                     const T *B, size_t ldb, T beta, T *C, size_t ldc) {                                    \
        const size_t MBLK = 64;                                                                              \
        ptrdiff_t nb;                                                                                        \
        const ptrdiff_t n_mblk = (ptrdiff_t)((M + MBLK - 1) / MBLK);                                         \
        _Pragma("omp parallel for schedule(dynamic, 1)")                                                     \
        for (nb = 0; nb < n_mblk; ++nb) {                                                                    \
            const size_t m0 = (size_t)nb * MBLK;                                                             \
            const size_t mlen = (M - m0) < MBLK ? (M - m0) : MBLK;                                           \
            T acc[64];                                                                                       \
            T apan[64];                                                                                      \
            size_t n, k, i;                                                                                  \
            for (n = 0; n < N; ++n) {                                                                        \
                for (i = 0; i < mlen; ++i) acc[i] = (T)0;                                                    \
                for (k = 0; k < K; ++k) {                                                                    \
                    const T b = tB ? B[n + k * ldb] : B[k + n * ldb];                                        \
                    if (tA) {                                                                                \
                        for (i = 0; i < mlen; ++i) apan[i] = A[k + (m0 + i) * lda];                          \
                    } else {                                                                                 \
                        const T *ap = A + m0 + k * lda;                                                      \
                        for (i = 0; i < mlen; ++i) apan[i] = ap[i];                                          \
                    }                                                                                        \
                    _Pragma("omp simd")                                                                      \
                    for (i = 0; i < mlen; ++i) acc[i] = FMA(apan[i], b, acc[i]);                             \
                }                                                                                            \
                {                                                                                            \
                    T *cp = C + m0 + n * ldc;                                                                \
                    if (beta == (T)0) {                                                                      \
                        for (i = 0; i < mlen; ++i) cp[i] = alpha * acc[i];                                   \
                    } else {                                                                                 \
                        for (i = 0; i < mlen; ++i) cp[i] = alpha * acc[i] + beta * cp[i];                    \
                    }                                                                                        \
                }                                                                                            \
            }                                                                                                \
        }                                                                                                    \
    }

GEMM_COLMAJOR(sgemm_colmajor, float, fmaf)
GEMM_COLMAJOR(dgemm_colmajor, double, fma)

/* Front end: checks (xgemm.cc:685-706), ConjTrans -> Trans for real types (xgemm.cc:330-335),
 * row-major folded to column-major by swapping the operands (xgemm.cc:40-61). */
#define GEMM_FRONT(NAME, T, CORE)                                                                            \
    int NAME(int order, int transA, int transB, size_t M, size_t N, size_t K, T alpha, const T *A,          \
             size_t offA, size_t lda, const T *B, size_t offB, size_t ldb, T beta, T *C, size_t offC,       \
             size_t ldc) {                                                                                   \
        int st = oracle_check_gemm(order, transA, transB, M, N, K, A != NULL, offA, lda, 0, B != NULL, offB, \
                                   ldb, 0, C != NULL, offC, ldc, 0);                                         \
        int tA, tB;                                                                                          \
        if (st) return st;                                                                                   \
        tA = transA != NO_TRANS;                                                                             \
        tB = transB != NO_TRANS;                                                                             \
        if (order == ROW_MAJOR)                                                                              \
            CORE(tB, tA, N, M, K, alpha, B + offB, ldb, A + offA, lda, beta, C + offC, ldc);                 \
        else                                                                                                 \
            CORE(tA, tB, M, N, K, alpha, A + offA, lda, B + offB, ldb, beta, C + offC, ldc);                 \
        return ST_SUCCESS;                                                                                   \
    }

GEMM_FRONT(oracle_sgemm, float, sgemm_colmajor)
GEMM_FRONT(oracle_dgemm, double, dgemm_colmajor)

/* High-precision evaluation of selected elements of a column-major GEMM, plus the magnitude
 * term of the parity bound   |C - C_ref| <= c * K * eps * (|alpha| |A||B| + |beta| |C|).
 * Products and sums are carried in a wider type (double for fp32 data, long double for fp64
 * data).  rows/cols list `count` element positions; exact[i] and mag[i] are written.
 * Not a restatement of reference code: this is the yardstick both the reference result and
 * ours are measured against. */
#define GEMM_EXACT(NAME, T, W, ABSW)                                                                         \
    void NAME(int tA, int tB, size_t K, T alpha, const T *A, size_t lda, const T *B, size_t ldb, T beta,    \
              const T *C, size_t ldc, size_t count, const int64_t *rows, const int64_t *cols, double *exact, \
              double *mag) {                                                                                 \
        ptrdiff_t i;                                                                                         \
        _Pragma("omp parallel for schedule(static)")                                                         \
        for (i = 0; i < (ptrdiff_t)count; ++i) {                                                             \
            const size_t m = (size_t)rows[i], n = (size_t)cols[i];                                           \
            W s = 0, sa = 0;                                                                                 \
            size_t k;                                                                                        \
            for (k = 0; k < K; ++k) {                                                                        \
                const W a = tA ? A[k + m * lda] : A[m + k * lda];                                            \
                const W b = tB ? B[n + k * ldb] : B[k + n * ldb];                                            \
                s += a * b;                                                                                  \
                sa += ABSW(a * b);                                                                           \
            }                                                                                                \
            {                                                                                                \
                W r = (W)alpha * s, g = ABSW((W)alpha) * sa;                                                 \
                if (!(beta == (T)0)) {                                                                       \
                    r += (W)beta * (W)C[m + n * ldc];                                                        \
                    g += ABSW((W)beta * (W)C[m + n * ldc]);                                                  \
                }                                                                                            \
                exact[i] = (double)r;                                                                        \
                mag[i] = (double)g;                                                                          \
            }                                                                                                \
        }                                                                                                    \
    }

GEMM_EXACT(oracle_sgemm_exact, float, double, fabs)
GEMM_EXACT(oracle_dgemm_exact, double, long double, fabsl)

/* Complex GEMM (clblasCgemm / clblasZgemm, src/library/blas/xgemm.cc:788-905).  Elements are
 * interleaved (re, im) pairs, as cl_float2 / cl_double2 (src/clBLAS-complex.h:25-26).
 * Column-major kernel arithmetic, src/library/blas/AutoGemm/KernelOpenCL.py:
 *   :106-141  TYPE_MAD, four mads per k in this order (x' = imaginary part negated when the
 *             operand is conjugated; the four macro variants differ only in where the minus
 *             signs sit, which is exact):
 *                 s0 = mad( a0,  b0, s0);  s0 = mad(-a1', b1', s0);
 *                 s1 = mad( a0, b1', s1);  s1 = mad( a1', b0,  s1);
 *   :142-165  TYPE_MAD_WRITE: reg = alpha*reg as  r0 = reg0*al0; r0 = mad(-al1, reg1, r0);
 *             r1 = reg1*al0; r1 = mad(al1, reg0, r1);  then (beta != 0 only)
 *             r0 = mad(be0, c0, r0); r0 = mad(-be1, c1, r0); r1 = mad(be1, c0, r1);
 *             r1 = mad(be0, c1, r1).
 * beta == 0+0i never reads C (isZero<FloatComplex>, xgemm.cc:94-101). */
#define CGEMM_COLMAJOR(NAME, R, FMA)                                                                         \
    static void NAME(int tA, int cA, int tB, int cB, size_t M, size_t N, size_t K, const R *alpha,          \
                     const R *A, size_t lda, const R *B, size_t ldb, const R *beta, R *C, size_t ldc) {     \
        const size_t MBLK = 64;                                                                              \
        ptrdiff_t nb;                                                                                        \
        const ptrdiff_t n_mblk = (ptrdiff_t)((M + MBLK - 1) / MBLK);                                         \
        const int beta_zero = beta[0] == (R)0 && beta[1] == (R)0;                                            \
        _Pragma("omp parallel for schedule(dynamic, 1)")                                                     \
        for (nb = 0; nb < n_mblk; ++nb) {                                                                    \
            const size_t m0 = (size_t)nb * MBLK;                                                             \
            const size_t mlen = (M - m0) < MBLK ? (M - m0) : MBLK;                                           \
            R s0[64], s1[64], a0[64], a1[64];                                                                \
            size_t n, k, i;                                                                                  \
            for (n = 0; n < N; ++n) {                                                                        \
                for (i = 0; i < mlen; ++i) s0[i] = s1[i] = (R)0;                                             \
                for (k = 0; k < K; ++k) {                                                                    \
                    const R *bp = tB ? B + 2 * (n + k * ldb) : B + 2 * (k + n * ldb);                        \
                    const R b0 = bp[0], b1 = cB ? -bp[1] : bp[1];                                            \
                    for (i = 0; i < mlen; ++i) {                                                             \
                        const R *ap = tA ? A + 2 * (k + (m0 + i) * lda) : A + 2 * (m0 + i + k * lda);        \
                        a0[i] = ap[0];                                                                       \
                        a1[i] = cA ? -ap[1] : ap[1];                                                         \
                    }                                                                                        \
                    _Pragma("omp simd")                                                                      \
                    for (i = 0; i < mlen; ++i) {                                                             \
                        s0[i] = FMA(a0[i], b0, s0[i]);                                                       \
                        s0[i] = FMA(-a1[i], b1, s0[i]);                                                      \
                        s1[i] = FMA(a0[i], b1, s1[i]);                                                       \
                        s1[i] = FMA(a1[i], b0, s1[i]);                                                       \
                    }                                                                                        \
                }                                                                                            \
                for (i = 0; i < mlen; ++i) {                                                                 \
                    R *cp = C + 2 * (m0 + i + n * ldc);                                                      \
                    R r0 = s0[i] * alpha[0], r1;                                                             \
                    r0 = FMA(-alpha[1], s1[i], r0);                                                          \
                    r1 = s1[i] * alpha[0];                                                                   \
                    r1 = FMA(alpha[1], s0[i], r1);                                                           \
                    if (!beta_zero) {                                                                        \
                        const R c0 = cp[0], c1 = cp[1];                                                      \
                        r0 = FMA(beta[0], c0, r0);                                                           \
                        r0 = FMA(-beta[1], c1, r0);                                                          \
                        r1 = FMA(beta[1], c0, r1);                                                           \
                        r1 = FMA(beta[0], c1, r1);                                                           \
                    }                                                                                        \
                    cp[0] = r0;                                                                              \
                    cp[1] = r1;                                                                              \
                }                                                                                            \
            }                                                                                                \
        }                                                                                                    \
    }

CGEMM_COLMAJOR(cgemm_colmajor, float, fmaf)
CGEMM_COLMAJOR(zgemm_colmajor, double, fma)

/* Front end: checks as for the real types (xgemm.cc:807-829), ConjTrans kept
 * (correctTranspose is the identity for complex types, xgemm.cc:334-335), row-major folded
 * by swapping the operands together with their transpose flags (xgemm.cc:40-61).
 * alpha / beta point at (re, im); A, B, C at interleaved elements; offsets and leading
 * dimensions count complex elements. */
#define CGEMM_FRONT(NAME, R, CORE)                                                                           \
    int NAME(int order, int transA, int transB, size_t M, size_t N, size_t K, const R *alpha, const R *A,   \
             size_t offA, size_t lda, const R *B, size_t offB, size_t ldb, const R *beta, R *C, size_t offC, \
             size_t ldc) {                                                                                   \
        int st = oracle_check_gemm(order, transA, transB, M, N, K, A != NULL, offA, lda, 0, B != NULL, offB, \
                                   ldb, 0, C != NULL, offC, ldc, 0);                                         \
        int tA, tB, cA, cB;                                                                                  \
        if (st) return st;                                                                                   \
        tA = transA != NO_TRANS;                                                                             \
        tB = transB != NO_TRANS;                                                                             \
        cA = transA == CONJ_TRANS;                                                                           \
        cB = transB == CONJ_TRANS;                                                                           \
        if (order == ROW_MAJOR)                                                                              \
            CORE(tB, cB, tA, cA, N, M, K, alpha, B + 2 * offB, ldb, A + 2 * offA, lda, beta, C + 2 * offC,   \
                 ldc);                                                                                       \
        else                                                                                                 \
            CORE(tA, cA, tB, cB, M, N, K, alpha, A + 2 * offA, lda, B + 2 * offB, ldb, beta, C + 2 * offC,   \
                 ldc);                                                                                       \
        return ST_SUCCESS;                                                                                   \
    }

CGEMM_FRONT(oracle_cgemm, float, cgemm_colmajor)
CGEMM_FRONT(oracle_zgemm, double, zgemm_colmajor)

/* Complex counterpart of the high-precision yardstick above.  exact[2i], exact[2i+1]: real
 * and imaginary part; mag[i] bounds the magnitude of everything summed into either part:
 *   (|al0|+|al1|) * sum_k (|a0|+|a1|)(|b0|+|b1|) + (|be0|+|be1|)(|c0|+|c1|). */
#define CGEMM_EXACT(NAME, R, W, ABSW)                                                                        \
    void NAME(int tA, int cA, int tB, int cB, size_t K, const R *alpha, const R *A, size_t lda, const R *B, \
              size_t ldb, const R *beta, const R *C, size_t ldc, size_t count, const int64_t *rows,          \
              const int64_t *cols, double *exact, double *mag) {                                             \
        ptrdiff_t i;                                                                                         \
        const int beta_zero = beta[0] == (R)0 && beta[1] == (R)0;                                            \
        _Pragma("omp parallel for schedule(static)")                                                         \
        for (i = 0; i < (ptrdiff_t)count; ++i) {                                                             \
            const size_t m = (size_t)rows[i], n = (size_t)cols[i];                                           \
            W s0 = 0, s1 = 0, sa = 0, r0, r1, g;                                                             \
            size_t k;                                                                                        \
            for (k = 0; k < K; ++k) {                                                                        \
                const R *ap = tA ? A + 2 * (k + m * lda) : A + 2 * (m + k * lda);                            \
                const R *bp = tB ? B + 2 * (n + k * ldb) : B + 2 * (k + n * ldb);                            \
                const W a0 = ap[0], a1 = cA ? -(W)ap[1] : (W)ap[1];                                          \
                const W b0 = bp[0], b1 = cB ? -(W)bp[1] : (W)bp[1];                                          \
                s0 += a0 * b0 - a1 * b1;                                                                     \
                s1 += a0 * b1 + a1 * b0;                                                                     \
                sa += (ABSW(a0) + ABSW(a1)) * (ABSW(b0) + ABSW(b1));                                         \
            }                                                                                                \
            r0 = (W)alpha[0] * s0 - (W)alpha[1] * s1;                                                        \
            r1 = (W)alpha[0] * s1 + (W)alpha[1] * s0;                                                        \
            g = (ABSW((W)alpha[0]) + ABSW((W)alpha[1])) * sa;                                                \
            if (!beta_zero) {                                                                                \
                const W c0 = C[2 * (m + n * ldc)], c1 = C[2 * (m + n * ldc) + 1];                            \
                r0 += (W)beta[0] * c0 - (W)beta[1] * c1;                                                     \
                r1 += (W)beta[0] * c1 + (W)beta[1] * c0;                                                     \
                g += (ABSW((W)beta[0]) + ABSW((W)beta[1])) * (ABSW(c0) + ABSW(c1));                          \
            }                                                                                                \
            exact[2 * i] = (double)r0;                                                                       \
            exact[2 * i + 1] = (double)r1;                                                                   \
            mag[i] = (double)g;                                                                              \
        }                                                                                                    \
    }

CGEMM_EXACT(oracle_cgemm_exact, float, double, fabs)
CGEMM_EXACT(oracle_zgemm_exact, double, long double, fabsl)

/* ------------------------------------------------------------------------------------ */
/* SYRK / TRMM / SYMM (the GEMM-shaped neighbours), all four types: level3.inc            */
/* ------------------------------------------------------------------------------------ */
#define P s
#define R float
#define NC 1
#include "level3.inc"
#undef P
#undef R
#undef NC
#define P d
#define R double
#define NC 1
#include "level3.inc"
#undef P
#undef R
#undef NC
#define P c
#define R float
#define NC 2
#include "level3.inc"
#undef P
#undef R
#undef NC
#define P z
#define R double
#define NC 2
#include "level3.inc"
#undef P
#undef R
#undef NC

/* ------------------------------------------------------------------------------------ */
/* TRSM                                                                                  */
/* ------------------------------------------------------------------------------------ */

/* Row-by-row substitution followed by a scaling with alpha: the reference's own CPU
 * statement of TRSM, src/library/tools/ktest/naive/naive_blas.cpp:632-684.
 * MatrixAccessor semantics (naive_blas.cpp:480-528): element (r,c) of op(A). */
#define ACC_A(T, r, c) (a_rowstride * (r) + a_colstride * (c))
#define TRSM_NAIVE(NAME, T)                                                                                  \
    int NAME(int order, int side, int uplo, int transA, int diag, size_t M, size_t N, T alpha, const T *A,  \
             size_t offA, size_t lda, T *B, size_t offB, size_t ldb) {                                       \
        int st = oracle_check_trsm(order, side, transA, M, N, A != NULL, offA, lda, 0, B != NULL, offB, ldb, \
                                   0);                                                                       \
        size_t rowsA, colsB, i, j, k, a_rowstride, a_colstride, b_rowstride, b_colstride;                    \
        int rev, tra;                                                                                        \
        if (st) return st;                                                                                   \
        A += offA;                                                                                           \
        B += offB;                                                                                           \
        rowsA = side == LEFT ? M : N;                                                                        \
        colsB = side == LEFT ? N : M;                                                                        \
        /* element (r,c) of op(A) and of B (viewed as rowsA x colsB) */                                      \
        tra = transA != NO_TRANS;                                                                            \
        rev = (uplo == UPPER) ^ tra;              /* :650 */                                                 \
        if (side == RIGHT) {                      /* :651-655: solve the transposed system */                \
            tra = !tra;                                                                                      \
            rev = !rev;                                                                                      \
        }                                                                                                    \
        if ((order == COL_MAJOR) != tra) { a_rowstride = 1; a_colstride = lda; }                             \
        else { a_rowstride = lda; a_colstride = 1; }                                                         \
        if ((order == COL_MAJOR) != (side == RIGHT)) { b_rowstride = 1; b_colstride = ldb; }                 \
        else { b_rowstride = ldb; b_colstride = 1; }                                                         \
        for (i = 0; i < rowsA; ++i) {                                                                        \
            const size_t row = rev ? rowsA - i - 1 : i;                                                      \
            for (j = 0; j < colsB; ++j) {                                                                    \
                const size_t boundK = rev ? rowsA - row - 1 : row;                                           \
                T tmp = (T)0;                                                                                \
                for (k = 0; k <= boundK; ++k) {                                                              \
                    const size_t col = rev ? rowsA - k - 1 : k;                                              \
                    if (col == row) {                                                                        \
                        const T a = diag == UNIT ? (T)1 : A[ACC_A(T, row, col)];                             \
                        tmp = (B[b_rowstride * row + b_colstride * j] - tmp) / a;                            \
                    } else {                                                                                 \
                        tmp = tmp + A[ACC_A(T, row, col)] * B[b_rowstride * col + b_colstride * j];          \
                    }                                                                                        \
                }                                                                                            \
                B[b_rowstride * row + b_colstride * j] = tmp;                                                \
            }                                                                                                \
        }                                                                                                    \
        for (i = 0; i < rowsA; ++i)                                                                          \
            for (j = 0; j < colsB; ++j)                                                                      \
                B[b_rowstride * i + b_colstride * j] = B[b_rowstride * i + b_colstride * j] * alpha;         \
        return ST_SUCCESS;                                                                                   \
    }

TRSM_NAIVE(oracle_strsm_naive, float)
TRSM_NAIVE(oracle_dtrsm_naive, double)

/* The same statement for complex elements (interleaved re, im; alpha by address): the template
 * above instantiated with FloatComplex / DoubleComplex, whose product and quotient are
 * naive_blas.cpp:300-390 ((a*b).re = ar*br - ai*bi, (a*b).im = ar*bi + br*ai;
 * a/b = (ar*br + ai*bi, br*ai - ar*bi) / (br^2 + bi^2)).  transA == ConjTrans conjugates every
 * element read from A (MatrixAccessor conj_, naive_blas.cpp:494, 466-472).  Right-hand sides
 * are independent of each other, so the loop over them is outermost here (and parallel); the
 * arithmetic on each is in the reference's order. */
#define CTRSM_NAIVE(NAME, R)                                                                                   \
    int NAME(int order, int side, int uplo, int transA, int diag, size_t M, size_t N, const R *alpha,          \
             const R *A, size_t offA, size_t lda, R *B, size_t offB, size_t ldb) {                             \
        int st = oracle_check_trsm(order, side, transA, M, N, A != NULL, offA, lda, 0, B != NULL, offB, ldb,   \
                                   0);                                                                         \
        size_t rowsA, colsB, a_rowstride, a_colstride, b_rowstride, b_colstride;                               \
        ptrdiff_t jj;                                                                                          \
        int rev, tra;                                                                                          \
        const R csign = transA == CONJ_TRANS ? (R)-1 : (R)1;                                                   \
        if (st) return st;                                                                                     \
        A += 2 * offA;                                                                                         \
        B += 2 * offB;                                                                                         \
        rowsA = side == LEFT ? M : N;                                                                          \
        colsB = side == LEFT ? N : M;                                                                          \
        tra = transA != NO_TRANS;                                                                              \
        rev = (uplo == UPPER) ^ tra;                                                                           \
        if (side == RIGHT) {                                                                                   \
            tra = !tra;                                                                                        \
            rev = !rev;                                                                                        \
        }                                                                                                      \
        if ((order == COL_MAJOR) != tra) { a_rowstride = 1; a_colstride = lda; }                               \
        else { a_rowstride = lda; a_colstride = 1; }                                                           \
        if ((order == COL_MAJOR) != (side == RIGHT)) { b_rowstride = 1; b_colstride = ldb; }                   \
        else { b_rowstride = ldb; b_colstride = 1; }                                                           \
        _Pragma("omp parallel for schedule(static)")                                                           \
        for (jj = 0; jj < (ptrdiff_t)colsB; ++jj) {                                                            \
            const size_t j = (size_t)jj;                                                                       \
            size_t i, k;                                                                                       \
            for (i = 0; i < rowsA; ++i) {                                                                      \
                const size_t row = rev ? rowsA - i - 1 : i;                                                    \
                const size_t boundK = rev ? rowsA - row - 1 : row;                                             \
                R *bx = B + 2 * (b_rowstride * row + b_colstride * j);                                         \
                R tr = 0, ti = 0;                                                                              \
                for (k = 0; k <= boundK; ++k) {                                                                \
                    const size_t col = rev ? rowsA - k - 1 : k;                                                \
                    const R *ap = A + 2 * (a_rowstride * row + a_colstride * col);                             \
                    if (col == row) {                                                                          \
                        const R ar = diag == UNIT ? (R)1 : ap[0], ai = diag == UNIT ? (R)0 : csign * ap[1];    \
                        const R nr = bx[0] - tr, ni = bx[1] - ti, div = ar * ar + ai * ai;                     \
                        tr = (nr * ar + ni * ai) / div;                                                        \
                        ti = (ar * ni - nr * ai) / div;                                                        \
                    } else {                                                                                   \
                        const R ar = ap[0], ai = csign * ap[1];                                                \
                        const R *bp = B + 2 * (b_rowstride * col + b_colstride * j);                           \
                        const R pr = ar * bp[0] - ai * bp[1], pi = ar * bp[1] + bp[0] * ai;                    \
                        tr = tr + pr;                                                                          \
                        ti = ti + pi;                                                                          \
                    }                                                                                          \
                }                                                                                              \
                bx[0] = tr;                                                                                    \
                bx[1] = ti;                                                                                    \
            }                                                                                                  \
            for (i = 0; i < rowsA; ++i) {                                                                      \
                R *bx = B + 2 * (b_rowstride * i + b_colstride * j);                                           \
                const R xr = bx[0], xi = bx[1];                                                                \
                bx[0] = xr * alpha[0] - xi * alpha[1];                                                         \
                bx[1] = xr * alpha[1] + alpha[0] * xi;                                                         \
            }                                                                                                  \
        }                                                                                                      \
        return ST_SUCCESS;                                                                                     \
    }

CTRSM_NAIVE(oracle_ctrsm_naive, float)
CTRSM_NAIVE(oracle_ztrsm_naive, double)

/* The reference's device algorithm for DTRSM: gpu_dtrsm128, src/library/blas/xtrsm.cc:1136-1507.
 *   1. InvA <- explicit inverses of the NB x NB (NB = 128) diagonal blocks of A
 *      (diag_dtrtri128, xtrsm.cc:790-1134): every 16x16 diagonal block is inverted
 *      column by column (trtri/diag_dtrtri_lower_128_16.cpp:85-165,
 *      trtri/diag_dtrtri_upper_128_16.cpp), unit diagonal forced to 1, a zero diagonal
 *      entry replaced by 1 (:87-96), rows/columns past the matrix read as zero (:67-74);
 *      then blocks are doubled 16->32->64->128 with
 *        lower: inv21 = -inv22 * (A21 * inv11)   (triple_dgemm_update_128_*_PART{1,2}_L.cpp)
 *        upper: inv12 = -inv11 * (A12 * inv22)   (triple_dgemm_update_128_*_R.cpp)
 *   2. block sweep X_i = op(InvA_ii) * B_i, B_rest = -op(A_rest,i) X_i + (alpha|1) B_rest with
 *      the public DGEMM, writing X to a zeroed M x N temporary that is copied back at the
 *      end (xtrsm.cc:1186-1192, 1229-1497).
 * The same algorithm is used here for fp32 (the reference routes STRSM through its legacy
 * solver instead, gens/trsm.c:1213-1456; its bit pattern is not restated). */
#define REAL float
#define FN(name) name##_s
#define ORACLE_TRSM_BLOCKED oracle_strsm_blocked
#define GEMM_CORE sgemm_colmajor
#include "trsm_blocked.inc"
#undef REAL
#undef FN
#undef ORACLE_TRSM_BLOCKED
#undef GEMM_CORE

#define REAL double
#define FN(name) name##_d
#define ORACLE_TRSM_BLOCKED oracle_dtrsm_blocked
#define GEMM_CORE dgemm_colmajor
#include "trsm_blocked.inc"
#undef REAL
#undef FN
#undef ORACLE_TRSM_BLOCKED
#undef GEMM_CORE

/* ------------------------------------------------------------------------------------ */
/* Seeded input generators (portable: splitmix64, identical on every host)               */
/* ------------------------------------------------------------------------------------ */

static inline uint64_t mix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ULL;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}
/* counter-based: value i of stream `seed` */
static inline uint64_t rnd_u64(uint64_t seed, uint64_t i) { return mix64(mix64(seed) + i * 0x9e3779b97f4a7c15ULL); }
static inline double rnd_unit(uint64_t seed, uint64_t i) { /* [0,1) with 53 bits */
    return (double)(rnd_u64(seed, i) >> 11) * (1.0 / 9007199254740992.0);
}

/* uniform [-1,1) */
void oracle_fill_uniform_f32(float *x, size_t n, uint64_t seed) {
    ptrdiff_t i;
    _Pragma("omp parallel for schedule(static)")
    for (i = 0; i < (ptrdiff_t)n; ++i) {
        /* 24 random bits so that the value is exactly representable in fp32 */
        x[i] = (float)((double)(rnd_u64(seed, (uint64_t)i) >> 40) * (1.0 / 8388608.0) - 1.0);
    }
}
void oracle_fill_uniform_f64(double *x, size_t n, uint64_t seed) {
    ptrdiff_t i;
    _Pragma("omp parallel for schedule(static)")
    for (i = 0; i < (ptrdiff_t)n; ++i) x[i] = 2.0 * rnd_unit(seed, (uint64_t)i) - 1.0;
}
/* normal(0,1), Box-Muller on two counter-based uniforms */
void oracle_fill_normal_f64(double *x, size_t n, uint64_t seed) {
    ptrdiff_t i;
    _Pragma("omp parallel for schedule(static)")
    for (i = 0; i < (ptrdiff_t)n; ++i) {
        double u1 = 1.0 - rnd_unit(seed, 2 * (uint64_t)i); /* (0,1] */
        double u2 = rnd_unit(seed, 2 * (uint64_t)i + 1);
        x[i] = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
    }
}
void oracle_fill_normal_f32(float *x, size_t n, uint64_t seed) {
    ptrdiff_t i;
    _Pragma("omp parallel for schedule(static)")
    for (i = 0; i < (ptrdiff_t)n; ++i) {
        double u1 = 1.0 - rnd_unit(seed, 2 * (uint64_t)i);
        double u2 = rnd_unit(seed, 2 * (uint64_t)i + 1);
        x[i] = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2));
    }
}
/* signed integers in (-limit, limit): the reference tests' exact-arithmetic inputs,
 * random<T>(limit) = +-(rand() % limit), src/tests/include/blas-math.h:232-246 */
void oracle_fill_int_f32(float *x, size_t n, uint64_t seed, uint32_t limit) {
    size_t i;
    for (i = 0; i < n; ++i) {
        uint64_t r = rnd_u64(seed, i);
        float v = (float)((r >> 8) % limit);
        x[i] = (r & 1) ? -v : v;
    }
}
void oracle_fill_int_f64(double *x, size_t n, uint64_t seed, uint32_t limit) {
    size_t i;
    for (i = 0; i < n; ++i) {
        uint64_t r = rnd_u64(seed, i);
        double v = (double)((r >> 8) % limit);
        x[i] = (r & 1) ? -v : v;
    }
}

/* Well-conditioned triangular matrix of order n, column-major with leading dimension ld:
 * strict triangle uniform[-1,1)/n, diagonal uniform[1,2); the other triangle (and, if
 * poison_diag, the diagonal) is NaN so that any illegal read shows in the result, as in the
 * reference tests (src/tests/include/blas-random.h:258-263, 311-317). */
#define FILL_TRI(NAME, T)                                                                                    \
    void NAME(T *a, size_t n, size_t ld, int lower, int poison_diag, uint64_t seed) {                        \
        ptrdiff_t c;                                                                                         \
        _Pragma("omp parallel for schedule(static)")                                                         \
        for (c = 0; c < (ptrdiff_t)n; ++c) {                                                                 \
            size_t r;                                                                                        \
            for (r = 0; r < n; ++r) {                                                                        \
                uint64_t idx = (uint64_t)r + (uint64_t)c * n;                                                \
                T v;                                                                                         \
                if (r == (size_t)c) v = poison_diag ? (T)NAN : (T)(1.0 + rnd_unit(seed, idx));               \
                else if ((lower && r > (size_t)c) || (!lower && r < (size_t)c))                              \
                    v = (T)((2.0 * rnd_unit(seed, idx) - 1.0) / (double)n);                                  \
                else v = (T)NAN;                                                                             \
                a[r + (size_t)c * ld] = v;                                                                   \
            }                                                                                                \
        }                                                                                                    \
    }
FILL_TRI(oracle_fill_tri_f32, float)
FILL_TRI(oracle_fill_tri_f64, double)

/* ------------------------------------------------------------------------------------ */
/* The reference TRSM test's input family and a long double solver to judge against       */
/* ------------------------------------------------------------------------------------ */
#include "trsm_reftest.inc"
