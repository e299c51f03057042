// Blocked triangular solve for gfx950: substitution on the diagonal blocks, MFMA GEMM for
// everything off the diagonal.
//
// Stands where the reference has gpu_dtrsm128 (src/library/blas/xtrsm.cc:1136-1507) and,
// for STRSM, the legacy block solver (src/library/blas/gens/trsm.c:1213-1456).  The
// reference inverts every 128x128 diagonal block (trtri kernels) and then alternates
// "X_i = inv(A_ii) B_i" with a trailing DGEMM update, using an M x N temporary.  Here the
// diagonal blocks are solved directly by substitution (one wavefront lane per right-hand
// side, the block's triangle broadcast from LDS), the sweep is recursive so that almost all
// flops land in large-K GEMM updates, and B is solved in place without a temporary.
// The block sweep directions are those of xtrsm.cc:1226-1477; alpha is applied exactly once
// to every element of B (xtrsm.cc:1236-1240).
//
// A zero on a non-unit diagonal gives Inf/NaN (1/0), as in the textbook algorithm; the
// reference's inversion kernel substitutes 1 instead (trtri/diag_dtrtri_lower_128_16.cpp:93-96).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "internal.h"

namespace cba {

// Solves one diagonal block against every right-hand side it touches.
//
// The block is the nb x nb (nb <= NBL) triangle at A(i0,i0).  "Equation order" p = 0..nb-1
// walks the block forward (index p) or backward (index nb-1-p) so that equation p only
// involves unknowns q < p.  coef(p,q) is the factor of unknown q in equation p:
//   left :  op(A)(ip, iq)        right:  op(A)(iq, ip)
// so with teff = trans XOR right it is A[ip + iq*lda] (teff false) or A[iq + ip*lda].
// Right-hand side j (a column of B for side=left, a row of B for side=right) has its
// element r at B[(i0+r)*sr + j*sj].
template <typename T, int NBL, bool RIGHT, bool FORWARD>
__global__ void __launch_bounds__(64)
trsm_diag_kernel(const T *__restrict__ Ablk, int64_t lda, bool teff, bool unit, int nb, T alpha,
                 T *__restrict__ Bblk, int64_t ldb, int nrhs) {
    __shared__ __attribute__((aligned(16))) T E[NBL * NBL];
    __shared__ T Dinv[NBL];
    constexpr int TP = NBL + 2;  // pitch of the transposed right-hand-side staging (left side)
    __shared__ __attribute__((aligned(16))) T stage[RIGHT ? 1 : 64 * TP];

    const int lane = threadIdx.x;
    // ---- triangle into LDS in equation order; only the referenced triangle is read ----
    for (int e = lane; e < NBL * NBL; e += 64) {
        // Make the index that is contiguous in memory vary fastest across lanes.
        int p, q;
        if (teff != !FORWARD) { q = e % NBL; p = e / NBL; } else { p = e % NBL; q = e / NBL; }
        T val = (T)0;
        if (q < p && p < nb) {
            int ip = FORWARD ? p : nb - 1 - p, iq = FORWARD ? q : nb - 1 - q;
            val = teff ? Ablk[iq + (int64_t)ip * lda] : Ablk[ip + (int64_t)iq * lda];
        }
        E[p * NBL + q] = val;
    }
    if (lane < NBL) {
        T d = (T)1;
        if (!unit && lane < nb) {
            int ip = FORWARD ? lane : nb - 1 - lane;
            d = (T)1 / Ablk[ip + (int64_t)ip * lda];
        }
        Dinv[lane] = d;
    }

    const int64_t j0 = (int64_t)blockIdx.x * 64;
    const int64_t j = j0 + lane;
    T x[NBL];

    if (RIGHT) {
        // element r of rhs j: Bblk[j + r*ldb]; lanes run along j: coalesced.
#pragma unroll
        for (int p = 0; p < NBL; ++p) {
            int r = FORWARD ? p : nb - 1 - p;
            x[p] = (p < nb && j < nrhs) ? Bblk[j + (int64_t)r * ldb] : (T)0;
        }
        __syncthreads();
    } else {
        // element r of rhs j: Bblk[r + j*ldb]; contiguous along r, so go through LDS:
        // lanes read runs along r, then each lane picks up its own column.
        for (int e = lane; e < 64 * NBL; e += 64) {
            int r = e % NBL, c = e / NBL;
            T v = (T)0;
            if (r < nb && j0 + c < nrhs) v = Bblk[r + (j0 + c) * ldb];
            stage[c * TP + r] = v;
        }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < NBL; ++p) {
            // p >= nb are padding equations (x = 0); clamp the index, the value is unused.
            int r = FORWARD ? p : (nb - 1 - p < 0 ? 0 : nb - 1 - p);
            x[p] = (p < nb) ? stage[lane * TP + r] : (T)0;
        }
    }

    // ---- substitution, all in registers; E and Dinv are wave-uniform LDS broadcasts ----
#pragma unroll
    for (int p = 0; p < NBL; ++p) {
        T acc = alpha * x[p];
#pragma unroll
        for (int q = 0; q < p; ++q) acc = fma(-E[p * NBL + q], x[q], acc);
        x[p] = acc * Dinv[p];
    }

    if (RIGHT) {
#pragma unroll
        for (int p = 0; p < NBL; ++p) {
            int r = FORWARD ? p : nb - 1 - p;
            if (p < nb && j < nrhs) Bblk[j + (int64_t)r * ldb] = x[p];
        }
    } else {
        __syncthreads();
#pragma unroll
        for (int p = 0; p < NBL; ++p) {
            int r = FORWARD ? p : (nb - 1 - p < 0 ? 0 : nb - 1 - p);
            if (p < nb) stage[lane * TP + r] = x[p];
        }
        __syncthreads();
        for (int e = lane; e < 64 * NBL; e += 64) {
            int r = e % NBL, c = e / NBL;
            if (r < nb && j0 + c < nrhs) Bblk[r + (j0 + c) * ldb] = stage[c * TP + r];
        }
    }
}

template <typename T> struct GemmOf;
template <> struct GemmOf<float> {
    static hipError_t run(bool tA, bool tB, int M, int N, int K, float alpha, const float *A, int64_t lda,
                          const float *B, int64_t ldb, float beta, float *C, int64_t ldc, hipStream_t s) {
        return sgemm_colmajor(tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s);
    }
};
template <> struct GemmOf<double> {
    static hipError_t run(bool tA, bool tB, int M, int N, int K, double alpha, const double *A, int64_t lda,
                          const double *B, int64_t ldb, double beta, double *C, int64_t ldc, hipStream_t s) {
        return dgemm_colmajor(tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s);
    }
};

template <typename T, int NBL> struct TrsmDriver {
    bool right, trans, unit, forward, teff;
    int M, N;
    const T *A;
    int64_t lda;
    T *B;
    int64_t ldb;
    hipStream_t stream;

    hipError_t leaf(int i0, int nb, T alpha) {
        const T *Ablk = A + i0 + (int64_t)i0 * lda;
        const int nrhs = right ? M : N;
        T *Bblk = right ? B + (int64_t)i0 * ldb : B + i0;
        dim3 grid((unsigned)((nrhs + 63) / 64)), block(64);
        if (right) {
            if (forward)
                hipLaunchKernelGGL((trsm_diag_kernel<T, NBL, true, true>), grid, block, 0, stream, Ablk, lda, teff,
                                   unit, nb, alpha, Bblk, ldb, nrhs);
            else
                hipLaunchKernelGGL((trsm_diag_kernel<T, NBL, true, false>), grid, block, 0, stream, Ablk, lda, teff,
                                   unit, nb, alpha, Bblk, ldb, nrhs);
        } else {
            if (forward)
                hipLaunchKernelGGL((trsm_diag_kernel<T, NBL, false, true>), grid, block, 0, stream, Ablk, lda, teff,
                                   unit, nb, alpha, Bblk, ldb, nrhs);
            else
                hipLaunchKernelGGL((trsm_diag_kernel<T, NBL, false, false>), grid, block, 0, stream, Ablk, lda,
                                   teff, unit, nb, alpha, Bblk, ldb, nrhs);
        }
        return hipGetLastError();
    }

    // Off-diagonal update of the block range `dst` (length nd, start d0) with the solved
    // range `src` (length ns, start s0):   B_dst <- beta * B_dst - coupling * X_src.
    hipError_t update(int d0, int nd, int s0, int ns, T beta) {
        if (!right) {
            // rows: B[d0.., :] -= op(A)[d0.., s0..] * B[s0.., :]
            const T *Ablk = trans ? A + s0 + (int64_t)d0 * lda : A + d0 + (int64_t)s0 * lda;
            return GemmOf<T>::run(trans, false, nd, N, ns, (T)-1, Ablk, lda, B + s0, ldb, beta, B + d0, ldb, stream);
        }
        // columns: B[:, d0..] -= B[:, s0..] * op(A)[s0.., d0..]
        const T *Ablk = trans ? A + d0 + (int64_t)s0 * lda : A + s0 + (int64_t)d0 * lda;
        return GemmOf<T>::run(false, trans, M, nd, ns, (T)-1, B + (int64_t)s0 * ldb, ldb, Ablk, lda, beta,
                              B + (int64_t)d0 * ldb, ldb, stream);
    }

    // Solves the diagonal range [i0, i0+n); every element of B in the range is scaled by
    // alpha exactly once (in the first leaf that touches it or as beta of its first update).
    hipError_t solve(int i0, int n, T alpha) {
        if (n <= NBL) return leaf(i0, n, alpha);
        // Split at a multiple of NBL near the middle.
        const int blocks = (n + NBL - 1) / NBL;
        const int n_lo = ((blocks + 1) / 2) * NBL;  // length of the low-index part
        const int n_hi = n - n_lo;
        hipError_t e;
        if (forward) {
            if ((e = solve(i0, n_lo, alpha)) != hipSuccess) return e;
            if ((e = update(i0 + n_lo, n_hi, i0, n_lo, alpha)) != hipSuccess) return e;
            return solve(i0 + n_lo, n_hi, (T)1);
        }
        if ((e = solve(i0 + n_lo, n_hi, alpha)) != hipSuccess) return e;
        if ((e = update(i0, n_lo, i0 + n_lo, n_hi, alpha)) != hipSuccess) return e;
        return solve(i0, n_lo, (T)1);
    }
};

template <typename T>
static hipError_t trsm_colmajor(bool right, bool lower, bool trans, bool unit, int M, int N, T alpha, const T *A,
                                int64_t lda, T *B, int64_t ldb, hipStream_t stream) {
    TrsmDriver<T, 32> d;
    d.right = right; d.trans = trans; d.unit = unit;
    // Left: equations run forward when op(A) is lower triangular; right: when it is upper.
    d.forward = right ? (lower == trans) : (lower != trans);
    d.teff = trans != right;
    d.M = M; d.N = N; d.A = A; d.lda = lda; d.B = B; d.ldb = ldb; d.stream = stream;
    return d.solve(0, right ? N : M, alpha);
}

hipError_t strsm_colmajor(bool right, bool lower, bool trans, bool unit, int M, int N, float alpha, const float *A,
                          int64_t lda, float *B, int64_t ldb, hipStream_t stream) {
    return trsm_colmajor<float>(right, lower, trans, unit, M, N, alpha, A, lda, B, ldb, stream);
}

hipError_t dtrsm_colmajor(bool right, bool lower, bool trans, bool unit, int M, int N, double alpha,
                          const double *A, int64_t lda, double *B, int64_t ldb, hipStream_t stream) {
    return trsm_colmajor<double>(right, lower, trans, unit, M, N, alpha, A, lda, B, ldb, stream);
}

}  // namespace cba
