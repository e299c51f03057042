// SYRK, SYR2K, HERK, HER2K, TRMM, SYMM and HEMM as GEMM-shaped calls on the MFMA GEMM core.
//
// The reference runs these through its generated solver kernels (src/library/blas/xsyrk.c,
// xtrmm.c, xsymm.c; xsymm.c:150-330 already composes SYMM from GEMM passes).  Here each is
// one or two launches of the GEMM kernel's triangular variant:
//   SYRK  one launch; only the tiles that touch the stored triangle of C exist, tiles on
//         the diagonal store element-wise.
//   TRMM  B is copied to a workspace W, then B <- alpha op(A) W (or alpha W op(A)) with the
//         triangular operand masked in LDS and the panels in its zero half skipped.
//   SYMM  A = T + S^T with T the stored triangle and S its strict part:
//         C <- alpha T B + beta C, then C <- alpha S^T B + C (two half-depth launches, no
//         workspace).
//   SYR2K two SYRK-shaped launches (A B^T, then B A^T accumulated).
//   HERK / HER2K  the same with the second operand conjugate-transposed; the diagonal of C is
//         stored with zero imaginary parts (the reference does this in its GEMM epilogue,
//         src/library/blas/gens/clTemplates/gemm.cl:1034-1056; xherk.c:88-110, xher2k.c:96-149).
//   HEMM  as SYMM with a conjugated mirror pass; the stored diagonal counts with its real
//         part only (xhemm.c:36-112 -> doSymm).
#include "gemm_kernel.hpp"
#include "internal.h"

namespace cba {

template <> hipError_t launch_gemm<float>(bool tA, bool tB, bool, bool, int M, int N, int K, float alpha,
                                          const float *A, int64_t lda, const float *B, int64_t ldb, float beta,
                                          float *C, int64_t ldc, hipStream_t s, const GemmTri *tri) {
    return sgemm_colmajor(tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s, tri);
}
template <> hipError_t launch_gemm<double>(bool tA, bool tB, bool, bool, int M, int N, int K, double alpha,
                                           const double *A, int64_t lda, const double *B, int64_t ldb, double beta,
                                           double *C, int64_t ldc, hipStream_t s, const GemmTri *tri) {
    return dgemm_colmajor(tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s, tri);
}
template <> hipError_t launch_gemm<Cx<float>>(bool tA, bool tB, bool cA, bool cB, int M, int N, int K,
                                              Cx<float> alpha, const Cx<float> *A, int64_t lda, const Cx<float> *B,
                                              int64_t ldb, Cx<float> beta, Cx<float> *C, int64_t ldc, hipStream_t s,
                                              const GemmTri *tri) {
    return cgemm_colmajor(tA, tB, cA, cB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s, tri);
}
template <> hipError_t launch_gemm<Cx<double>>(bool tA, bool tB, bool cA, bool cB, int M, int N, int K,
                                               Cx<double> alpha, const Cx<double> *A, int64_t lda,
                                               const Cx<double> *B, int64_t ldb, Cx<double> beta, Cx<double> *C,
                                               int64_t ldc, hipStream_t s, const GemmTri *tri) {
    return zgemm_colmajor(tA, tB, cA, cB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s, tri);
}

// dst(m, n) = src(m, n) for an M x N column-major matrix; block b covers rows
// [256 * (b % m_blocks), +256) of column b / m_blocks.
template <typename T>
__global__ void __launch_bounds__(256)
copy_matrix_kernel(int M, int N, int m_blocks, const T *src, int64_t lds_, T *dst, int64_t ldd) {
    const int m = (blockIdx.x % m_blocks) * 256 + threadIdx.x;
    const int n = blockIdx.x / m_blocks;
    if (m < M && n < N) dst[(int64_t)n * ldd + m] = src[(int64_t)n * lds_ + m];
}

// C(m, n) <- alpha W(m, n) + beta C(m, n) on the lower / upper triangle of the N x N matrix C; beta == 0
// does not read C; herm: the diagonal of C is read without and stored with a zero imaginary part.
// Block b covers rows [256 * (b % m_blocks), +256) of column b / m_blocks.
template <typename T>
__global__ void __launch_bounds__(256)
triangle_axpy_kernel(int N, int m_blocks, bool lower, bool herm, T alpha, const T *W, int64_t ldw, T beta, T *C,
                     int64_t ldc) {
    const int m = (blockIdx.x % m_blocks) * 256 + threadIdx.x;
    const int n = blockIdx.x / m_blocks;
    if (m >= N || n >= N || (lower ? m < n : m > n)) return;
    T *c = C + (int64_t)n * ldc + m;
    T r = el_scale(alpha, W[(int64_t)n * ldw + m]);
    const bool diag = herm && m == n;
    if (!el_is_zero(beta)) r = el_axpy(beta, diag ? el_real_only(*c) : *c, r);
    if (diag) r = el_real_only(r);
    *c = r;
}

// A rank-k update of a small C with a deep K.  The kernels that store one triangle of C do not cut K
// into ranges, so a handful of tiles would walk through all of K on a handful of CUs (DSYRK 64 x 2^21:
// one workgroup, 0.4 s).  Such a product runs as a plain GEMM - both triangles, twice the flops, but
// with a K split over every CU - into a library-owned N x N buffer, and a small pass folds the wanted
// triangle into C.  Used while the full square has at most 128 tiles of 64 x 64 (N <= 704) and K >= 4096.
static inline bool rank_k_is_deep(int N, int K) {
    const int64_t n64 = (N + 63) / 64;
    return n64 * n64 <= 128 && K >= 4096;
}
template <typename T>
static hipError_t rank_k_deep(bool lower, bool herm, bool tA, bool tB, bool cA, bool cB, int N, int K, T alpha,
                              const T *A, int64_t lda, const T *B, int64_t ldb, T beta, T *C, int64_t ldc,
                              hipStream_t stream) {
    const int64_t ldw = ((int64_t)N + 63) / 64 * 64;
    void *wv = nullptr;
    hipError_t err = workspace_get(stream, (size_t)ldw * N * sizeof(T), 1, &wv);
    if (err != hipSuccess) return err;
    T *W = (T *)wv;
    err = launch_gemm<T>(tA, tB, cA, cB, N, N, K, el_one<T>(), A, lda, B, ldb, T(), W, ldw, stream);
    if (err != hipSuccess) return err;
    const int mb = (N + 255) / 256;
    dispatch_record().launches++;
    return launch_kernel(triangle_axpy_kernel<T>, dim3((unsigned)(mb * N)), dim3(256), 0, stream, N, mb, lower, herm,
                         alpha, (const T *)W, ldw, beta, C, ldc);
}

template <typename T>
hipError_t syrk_colmajor(bool lower, bool trans, int N, int K, T alpha, const T *A, int64_t lda, T beta, T *C,
                         int64_t ldc, hipStream_t stream) {
    if (rank_k_is_deep(N, K))
        return rank_k_deep<T>(lower, false, trans, !trans, false, false, N, K, alpha, A, lda, A, lda, beta, C, ldc, stream);
    GemmTri tri;
    tri.tri_c = lower ? 1 : 2;
    // op(A) op(A)^T: the second operand is the same matrix with the opposite transpose flag.
    return launch_gemm<T>(trans, !trans, false, false, N, N, K, alpha, A, lda, A, lda, beta, C, ldc, stream, &tri);
}

template <typename T>
hipError_t trmm_colmajor(bool right, bool lower, bool trans, bool conj, bool unit, int M, int N, T alpha, const T *A,
                         int64_t lda, T *B, int64_t ldb, hipStream_t stream) {
    const int64_t ldw = ((int64_t)M + 63) / 64 * 64;
    void *wv = nullptr;
    hipError_t err = workspace_get(stream, (size_t)ldw * N * sizeof(T), 1, &wv);
    if (err != hipSuccess) return err;
    T *W = (T *)wv;
    const int mb = (M + 255) / 256;
    if ((int64_t)mb * N > 0x7fffffffLL) return hipErrorInvalidValue;
    dispatch_record().launches++;
    err = launch_kernel(copy_matrix_kernel<T>, dim3((unsigned)((int64_t)mb * N)), dim3(256), 0, stream, M, N, mb,
                        (const T *)B, ldb, W, ldw);
    if (err != hipSuccess) return err;
    GemmTri tri;
    const bool op_lower = lower != trans;  // op(A) is lower triangular
    if (!right) {
        // op(A)(m,k): lower keeps k <= m
        tri.tri_a = op_lower ? 1 : 2;
        tri.unit_a = unit ? 1 : 0;
        return launch_gemm<T>(trans, false, conj, false, M, N, M, alpha, A, lda, W, ldw, T(), B, ldb, stream, &tri);
    }
    // op(A)(k,n): lower keeps k >= n
    tri.tri_b = op_lower ? 2 : 1;
    tri.unit_b = unit ? 1 : 0;
    return launch_gemm<T>(false, trans, false, conj, M, N, N, alpha, W, ldw, A, lda, T(), B, ldb, stream, &tri);
}

template <typename T>
hipError_t symm_colmajor(bool right, bool lower, int M, int N, T alpha, const T *A, int64_t lda, const T *B,
                         int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream) {
    GemmTri stored, mirrored;
    hipError_t err;
    if (!right) {
        // stored triangle as it lies: lower keeps k <= m; its strict part read transposed
        // fills the other side: op(A)(m,k) = A(k,m), stored for k > m (lower) / k < m (upper).
        stored.tri_a = lower ? 1 : 2;
        mirrored.tri_a = lower ? 2 : 1;
        mirrored.unit_a = 2;
        err = launch_gemm<T>(false, false, false, false, M, N, M, alpha, A, lda, B, ldb, beta, C, ldc, stream, &stored);
        if (err != hipSuccess) return err;
        return launch_gemm<T>(true, false, false, false, M, N, M, alpha, A, lda, B, ldb, el_one<T>(), C, ldc, stream,
                              &mirrored);
    }
    // A is the second operand, op(A)(k,n): lower keeps k >= n.
    stored.tri_b = lower ? 2 : 1;
    mirrored.tri_b = lower ? 1 : 2;
    mirrored.unit_b = 2;
    err = launch_gemm<T>(false, false, false, false, M, N, N, alpha, B, ldb, A, lda, beta, C, ldc, stream, &stored);
    if (err != hipSuccess) return err;
    return launch_gemm<T>(false, true, false, false, M, N, N, alpha, B, ldb, A, lda, el_one<T>(), C, ldc, stream,
                          &mirrored);
}

template <typename T>
hipError_t syr2k_colmajor(bool lower, bool trans, int N, int K, T alpha, const T *A, int64_t lda, const T *B,
                          int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream) {
    if (rank_k_is_deep(N, K)) {
        hipError_t e = rank_k_deep<T>(lower, false, trans, !trans, false, false, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream);
        if (e != hipSuccess) return e;
        return rank_k_deep<T>(lower, false, trans, !trans, false, false, N, K, alpha, B, ldb, A, lda, el_one<T>(), C, ldc, stream);
    }
    GemmTri tri;
    tri.tri_c = lower ? 1 : 2;
    // C <- alpha op(A) op(B)^T + beta C, then C <- alpha op(B) op(A)^T + C
    hipError_t err =
        launch_gemm<T>(trans, !trans, false, false, N, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, &tri);
    if (err != hipSuccess) return err;
    return launch_gemm<T>(trans, !trans, false, false, N, N, K, alpha, B, ldb, A, lda, el_one<T>(), C, ldc, stream,
                          &tri);
}

template <typename R>
hipError_t herk_colmajor(bool lower, bool ctrans, int N, int K, R alpha, const Cx<R> *A, int64_t lda, R beta,
                         Cx<R> *C, int64_t ldc, hipStream_t stream) {
    typedef Cx<R> T;
    if (rank_k_is_deep(N, K))
        return rank_k_deep<T>(lower, true, ctrans, !ctrans, ctrans, !ctrans, N, K, T{alpha, (R)0}, A, lda, A, lda,
                              T{beta, (R)0}, C, ldc, stream);
    GemmTri tri;
    tri.tri_c = lower ? 1 : 2;
    tri.herm_c = 1;
    // A A^H (second operand conjugate-transposed) or A^H A (first operand)
    return launch_gemm<T>(ctrans, !ctrans, ctrans, !ctrans, N, N, K, T{alpha, (R)0}, A, lda, A, lda, T{beta, (R)0}, C,
                          ldc, stream, &tri);
}

template <typename R>
hipError_t her2k_colmajor(bool lower, bool ctrans, int N, int K, Cx<R> alpha, const Cx<R> *A, int64_t lda,
                          const Cx<R> *B, int64_t ldb, R beta, Cx<R> *C, int64_t ldc, hipStream_t stream) {
    typedef Cx<R> T;
    if (rank_k_is_deep(N, K)) {
        hipError_t e = rank_k_deep<T>(lower, true, ctrans, !ctrans, ctrans, !ctrans, N, K, alpha, A, lda, B, ldb,
                                      T{beta, (R)0}, C, ldc, stream);
        if (e != hipSuccess) return e;
        return rank_k_deep<T>(lower, true, ctrans, !ctrans, ctrans, !ctrans, N, K, T{alpha.re, -alpha.im}, B, ldb, A, lda,
                              el_one<T>(), C, ldc, stream);
    }
    GemmTri tri;
    tri.tri_c = lower ? 1 : 2;
    tri.herm_c = 1;
    // C <- alpha op(A) op(B)^H + beta C, then C <- conj(alpha) op(B) op(A)^H + C
    // (the two passes of xher2k.c:117-149)
    hipError_t err = launch_gemm<T>(ctrans, !ctrans, ctrans, !ctrans, N, N, K, alpha, A, lda, B, ldb, T{beta, (R)0}, C,
                                    ldc, stream, &tri);
    if (err != hipSuccess) return err;
    return launch_gemm<T>(ctrans, !ctrans, ctrans, !ctrans, N, N, K, T{alpha.re, -alpha.im}, B, ldb, A, lda,
                          el_one<T>(), C, ldc, stream, &tri);
}

template <typename T>
hipError_t hemm_colmajor(bool right, bool lower, int M, int N, T alpha, const T *A, int64_t lda, const T *B,
                         int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream) {
    // As SYMM, with A = T + S^H: the mirrored pass conjugates, and the diagonal of the stored
    // triangle counts with its real part only.
    GemmTri stored, mirrored;
    hipError_t err;
    if (!right) {
        stored.tri_a = lower ? 1 : 2;
        stored.unit_a = 3;
        mirrored.tri_a = lower ? 2 : 1;
        mirrored.unit_a = 2;
        err = launch_gemm<T>(false, false, false, false, M, N, M, alpha, A, lda, B, ldb, beta, C, ldc, stream, &stored);
        if (err != hipSuccess) return err;
        return launch_gemm<T>(true, false, true, false, M, N, M, alpha, A, lda, B, ldb, el_one<T>(), C, ldc, stream,
                              &mirrored);
    }
    stored.tri_b = lower ? 2 : 1;
    stored.unit_b = 3;
    mirrored.tri_b = lower ? 1 : 2;
    mirrored.unit_b = 2;
    err = launch_gemm<T>(false, false, false, false, M, N, N, alpha, B, ldb, A, lda, beta, C, ldc, stream, &stored);
    if (err != hipSuccess) return err;
    return launch_gemm<T>(false, true, false, true, M, N, N, alpha, B, ldb, A, lda, el_one<T>(), C, ldc, stream,
                          &mirrored);
}

#define CBA_INSTANTIATE(T)                                                                                         \
    template hipError_t syrk_colmajor<T>(bool, bool, int, int, T, const T *, int64_t, T, T *, int64_t, hipStream_t); \
    template hipError_t trmm_colmajor<T>(bool, bool, bool, bool, bool, int, int, T, const T *, int64_t, T *, int64_t, \
                                         hipStream_t);                                                             \
    template hipError_t symm_colmajor<T>(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *,   \
                                         int64_t, hipStream_t);                                                    \
    template hipError_t syr2k_colmajor<T>(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *,  \
                                          int64_t, hipStream_t);
CBA_INSTANTIATE(float)
CBA_INSTANTIATE(double)
CBA_INSTANTIATE(Cx<float>)
CBA_INSTANTIATE(Cx<double>)
#undef CBA_INSTANTIATE
#define CBA_INSTANTIATE_HERM(R)                                                                                     \
    template hipError_t herk_colmajor<R>(bool, bool, int, int, R, const Cx<R> *, int64_t, R, Cx<R> *, int64_t,       \
                                         hipStream_t);                                                              \
    template hipError_t her2k_colmajor<R>(bool, bool, int, int, Cx<R>, const Cx<R> *, int64_t, const Cx<R> *,       \
                                          int64_t, R, Cx<R> *, int64_t, hipStream_t);                               \
    template hipError_t hemm_colmajor<Cx<R>>(bool, bool, int, int, Cx<R>, const Cx<R> *, int64_t, const Cx<R> *,    \
                                             int64_t, Cx<R>, Cx<R> *, int64_t, hipStream_t);
CBA_INSTANTIATE_HERM(float)
CBA_INSTANTIATE_HERM(double)
#undef CBA_INSTANTIATE_HERM

}  // namespace cba
