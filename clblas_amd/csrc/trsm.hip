// Blocked triangular solve for gfx950: substitution on the diagonal blocks, MFMA GEMM for
// everything off the diagonal.
//
// Stands where the reference has gpu_dtrsm128 (src/library/blas/xtrsm.cc:1136-1507) and,
// for STRSM, the legacy block solver (src/library/blas/gens/trsm.c:1213-1456).  The
// reference inverts every 128x128 diagonal block (trtri kernels) and then alternates
// "X_i = inv(A_ii) B_i" with a trailing DGEMM update, using an M x N temporary.  Here the
// diagonal blocks (128 x 128) are solved directly by substitution inside one kernel (eight
// wavefronts, one lane per right-hand side, the block's triangle broadcast from LDS), the
// sweep is recursive so that almost all flops land in large-K GEMM updates, and B is solved
// in place without a temporary.
// The block sweep directions are those of xtrsm.cc:1226-1477; alpha is applied exactly once
// to every element of B (xtrsm.cc:1236-1240).
//
// A zero on a non-unit diagonal gives Inf/NaN (1/0), as in the textbook algorithm; the
// reference's inversion kernel substitutes 1 instead (trtri/diag_dtrtri_lower_128_16.cpp:93-96).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "internal.h"

namespace cba {

// Solves one diagonal block (up to 128 x 128) against 64 right-hand sides per workgroup.
//
// The block is the nb x nb (nb <= NB) triangle at A(i0,i0).  "Equation order" P = 0..nb-1
// walks the block forward (index P) or backward (index nb-1-P) so that equation P only
// involves unknowns Q < P.  coef(P,Q) is the factor of unknown Q in equation P:
//   left :  op(A)(iP, iQ)        right:  op(A)(iQ, iP)
// so with teff = trans XOR right it is A[iP + iQ*lda] (teff false) or A[iQ + iP*lda].
// Right-hand side j is a column of B for side=left (element r at B[r + j*ldb]) and a row
// of B for side=right (element r at B[j + r*ldb]).
//
// Work split: 8 wavefronts, wavefront w owns equations [16w, 16w+16) and keeps them in
// registers, one lane per right-hand side.  Step s: wavefront s finishes its 16 unknowns
// by substitution (each new unknown is folded into the remaining equations at once, so
// the FMAs of one step are independent) and publishes them through LDS; after the
// barrier every later wavefront subtracts the 16 x 16 coupling block times those unknowns.
// The triangle sits in LDS as 36 blocks of 16 x 16, read as wave-uniform broadcasts one
// column ahead of the FMAs that use them.
// Only the referenced triangle of A is read (never the other one, nor a unit diagonal).
// For side=left a right-hand side is a column of B, so giving each lane "its" column
// directly would make every load touch 64 different columns; the panel is instead moved
// between HBM and registers through an LDS staging area with lanes running along the
// contiguous direction (the area reuses the triangle's LDS before and after the solve).
template <typename T> struct TrsmLeaf {
    static constexpr int NB = 128, IB = 16, NBLK = NB / IB, CW = 64, THREADS = 64 * NBLK;
    static constexpr int EP = IB + 16 / (int)sizeof(T);   // column pitch of an E block: columns stay 16-byte aligned
    static constexpr int N_EBLK = NBLK * (NBLK + 1) / 2;  // blocks (bi,bj), bi >= bj, at bi*(bi+1)/2 + bj
    static constexpr int E_ELEMS = N_EBLK * IB * EP;
    static constexpr int X_ELEMS = 2 * IB * CW;
    static constexpr int SP = NB + 2;                     // pitch of the right-hand-side staging area
    static constexpr int S_ELEMS = CW * SP;               // shares LDS with E (used before and after it)
    static_assert(S_ELEMS <= E_ELEMS + X_ELEMS, "staging area must fit in the E/X region");
    static constexpr size_t SMEM = (size_t)(E_ELEMS + X_ELEMS + NB) * sizeof(T);
};

// IB values of one E-block column (16-byte LDS reads; the address is wave-uniform).
template <typename T, int IB> static __device__ __forceinline__ void load_e_column(const T *src, T (&dst)[IB]) {
    constexpr int V = 16 / (int)sizeof(T);
    typedef T VT __attribute__((ext_vector_type(V)));
#pragma unroll
    for (int p = 0; p < IB; p += V) {
        VT v = *reinterpret_cast<const VT *>(src + p);
#pragma unroll
        for (int e = 0; e < V; ++e) dst[p + e] = v[e];
    }
}

template <typename T, bool RIGHT, bool FORWARD>
__global__ void __launch_bounds__(TrsmLeaf<T>::THREADS)
trsm_diag_kernel(const T *__restrict__ Ablk, int64_t lda, bool teff, bool unit, int nb, T alpha,
                 T *__restrict__ Bblk, int64_t ldb, int nrhs) {
    typedef TrsmLeaf<T> L;
    constexpr int IB = L::IB, CW = L::CW, EP = L::EP, NT = L::THREADS;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *E = reinterpret_cast<T *>(smem_raw);
    T *X = E + L::E_ELEMS;
    T *Dinv = X + L::X_ELEMS;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    const int64_t j0 = (int64_t)blockIdx.x * CW;
    const int64_t j = j0 + lane;
    const bool col_ok = j < nrhs;
    T y[IB];

    // ---- triangle: issue its loads first so that they overlap the right-hand-side traffic.
    //      Element e of the (block, q, p) enumeration; only the referenced triangle is read. ----
    constexpr int E_ITERS = L::N_EBLK * IB * IB / NT;
    static_assert(L::N_EBLK * IB * IB % NT == 0, "triangle fill must divide over the workgroup");
    auto e_coords = [&](int u, int &blk, int &p, int &q) {
        const int e = tid + u * NT;
        blk = e / (IB * IB);
        const int w = e % (IB * IB);
        // Let the index that is contiguous in memory vary fastest across lanes.
        if (teff) { q = w % IB; p = w / IB; } else { p = w % IB; q = w / IB; }
    };
    auto e_slot = [&](int u) {
        int blk, p, q;
        e_coords(u, blk, p, q);
        return blk * (IB * EP) + q * EP + p;
    };
    T eval[E_ITERS];
#pragma unroll
    for (int u = 0; u < E_ITERS; ++u) {
        int blk, p, q;
        e_coords(u, blk, p, q);
        int bi = 0;
        while ((bi + 1) * (bi + 2) / 2 <= blk) ++bi;
        const int bj = blk - bi * (bi + 1) / 2;
        const int P = bi * IB + p, Q = bj * IB + q;
        eval[u] = (T)0;
        if (Q < P && P < nb) {
            const int ip = FORWARD ? P : nb - 1 - P, iq = FORWARD ? Q : nb - 1 - Q;
            eval[u] = teff ? Ablk[iq + (int64_t)ip * lda] : Ablk[ip + (int64_t)iq * lda];
        }
    }
    T dval = (T)1;
    if (tid < L::NB && !unit && tid < nb) {
        const int ip = FORWARD ? tid : nb - 1 - tid;
        dval = Ablk[ip + (int64_t)ip * lda];
    }

    // ---- this wavefront's 16 equations of right-hand side j into registers ----
    if (RIGHT) {
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            const int P = wave * IB + p;
            const int r = FORWARD ? P : nb - 1 - P;
            T v = (T)0;
            if (P < nb && col_ok) v = Bblk[j + (int64_t)r * ldb];
            y[p] = alpha * v;
        }
    } else {
        T *S = E;  // staging area, overwritten by the triangle afterwards
        // All loads are issued before the first LDS write so that their latencies overlap.
        constexpr int NLD = CW * (L::NB / 2) / NT;
        T v0[NLD], v1[NLD];
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int e = tid + u * NT;
            const int c = e / (L::NB / 2), r = (e % (L::NB / 2)) * 2;
            v0[u] = (T)0;
            v1[u] = (T)0;
            if (j0 + c < nrhs) {
                const T *src = Bblk + r + (j0 + c) * ldb;
                if (r < nb) v0[u] = src[0];
                if (r + 1 < nb) v1[u] = src[1];
            }
        }
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int e = tid + u * NT;
            const int c = e / (L::NB / 2), r = (e % (L::NB / 2)) * 2;
            S[c * L::SP + r] = v0[u];
            S[c * L::SP + r + 1] = v1[u];
        }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            const int P = wave * IB + p;
            const int r = FORWARD ? P : (nb - 1 - P < 0 ? 0 : nb - 1 - P);
            y[p] = (P < nb) ? alpha * S[lane * L::SP + r] : (T)0;
        }
        __syncthreads();
    }

    // ---- triangle into LDS (its loads were issued first, see above) ----
#pragma unroll
    for (int u = 0; u < E_ITERS; ++u) E[e_slot(u)] = eval[u];
    if (tid < L::NB) Dinv[tid] = (T)1 / dval;
    __syncthreads();

#pragma unroll 1
    for (int s = 0; s < L::NBLK; ++s) {
        T *Xs = X + (s & 1) * (IB * CW);
        if (wave == s) {
            const T *Ed = E + (s * (s + 1) / 2 + s) * (IB * EP);
            T dinv[IB];
            load_e_column<T, IB>(Dinv + s * IB, dinv);
            T ea[IB], eb[IB];
            load_e_column<T, IB>(Ed, ea);
#pragma unroll
            for (int q = 0; q < IB; q += 2) {
                load_e_column<T, IB>(Ed + (q + 1) * EP, eb);
                __builtin_amdgcn_sched_barrier(0);
                {
                    const T x = y[q] * dinv[q];
                    y[q] = x;
                    Xs[q * CW + lane] = x;
#pragma unroll
                    for (int p = q + 1; p < IB; ++p) y[p] = fma(-ea[p], x, y[p]);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (q + 2 < IB) load_e_column<T, IB>(Ed + (q + 2) * EP, ea);
                __builtin_amdgcn_sched_barrier(0);
                {
                    const T x = y[q + 1] * dinv[q + 1];
                    y[q + 1] = x;
                    Xs[(q + 1) * CW + lane] = x;
#pragma unroll
                    for (int p = q + 2; p < IB; ++p) y[p] = fma(-eb[p], x, y[p]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
        if (wave > s && wave * IB < nb) {
            const T *Eo = E + (wave * (wave + 1) / 2 + s) * (IB * EP);
            T xs[IB];
#pragma unroll
            for (int q = 0; q < IB; ++q) xs[q] = Xs[q * CW + lane];
            T ea[IB], eb[IB];
            load_e_column<T, IB>(Eo, ea);
#pragma unroll
            for (int q = 0; q < IB; q += 2) {
                load_e_column<T, IB>(Eo + (q + 1) * EP, eb);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int p = 0; p < IB; ++p) y[p] = fma(-ea[p], xs[q], y[p]);
                __builtin_amdgcn_sched_barrier(0);
                if (q + 2 < IB) load_e_column<T, IB>(Eo + (q + 2) * EP, ea);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int p = 0; p < IB; ++p) y[p] = fma(-eb[p], xs[q + 1], y[p]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    if (RIGHT) {
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            const int P = wave * IB + p;
            const int r = FORWARD ? P : nb - 1 - P;
            if (P < nb && col_ok) Bblk[j + (int64_t)r * ldb] = y[p];
        }
    } else {
        T *S = E;
        __syncthreads();  // every wavefront is done with the triangle
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            const int P = wave * IB + p;
            const int r = FORWARD ? P : (nb - 1 - P < 0 ? 0 : nb - 1 - P);
            if (P < nb) S[lane * L::SP + r] = y[p];
        }
        __syncthreads();
        constexpr int NLD = CW * (L::NB / 2) / NT;
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int e = tid + u * NT;
            const int c = e / (L::NB / 2), r = (e % (L::NB / 2)) * 2;
            if (j0 + c < nrhs) {
                T *dst = Bblk + r + (j0 + c) * ldb;
                if (r < nb) dst[0] = S[c * L::SP + r];
                if (r + 1 < nb) dst[1] = S[c * L::SP + r + 1];
            }
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

template <typename T> struct TrsmDriver {
    static constexpr int NBL = TrsmLeaf<T>::NB;
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
        typedef TrsmLeaf<T> L;
        void (*fn)(const T *, int64_t, bool, bool, int, T, T *, int64_t, int);
        if (right) fn = forward ? trsm_diag_kernel<T, true, true> : trsm_diag_kernel<T, true, false>;
        else fn = forward ? trsm_diag_kernel<T, false, true> : trsm_diag_kernel<T, false, false>;
        if (L::SMEM > 64 * 1024) {
            hipError_t e = ensure_dynamic_lds((const void *)fn, L::SMEM);
            if (e != hipSuccess) return e;
        }
        dim3 grid((unsigned)((nrhs + L::CW - 1) / L::CW)), block(L::THREADS);
        hipLaunchKernelGGL(fn, grid, block, L::SMEM, stream, Ablk, lda, teff, unit, nb, alpha, Bblk, ldb, nrhs);
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
    TrsmDriver<T> d;
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
