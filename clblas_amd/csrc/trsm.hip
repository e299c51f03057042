// Blocked triangular solve for gfx950: substitution on the diagonal blocks, MFMA GEMM for
// everything off the diagonal.
//
// Stands where the reference has gpu_dtrsm128 (src/library/blas/xtrsm.cc:1136-1507) and,
// for STRSM, the legacy block solver (src/library/blas/gens/trsm.c:1213-1456).  The
// reference inverts every 128x128 diagonal block (trtri kernels) and then alternates
// "X_i = inv(A_ii) B_i" with a trailing DGEMM update, using an M x N temporary.  Here the
// diagonal blocks (256 x 256) are solved inside one kernel by block substitution over their
// 16 x 16 sub-blocks on the MFMA units (only the 16 x 16 diagonal sub-triangles are inverted,
// by substitution, in a packing pass), the sweep is recursive so that almost all flops land
// in large-K GEMM updates, and B is solved in place without a temporary.
// The block sweep directions are those of xtrsm.cc:1226-1477; alpha is applied exactly once
// to every element of B (xtrsm.cc:1236-1240).
//
// Complex types (clblasCtrsm / clblasZtrsm, xtrsm.cc:1789-1914) run through the same driver and
// kernels: the packing pass conjugates for clblasConjTrans and splits every sub-block into real
// planes, the leaf does four real MFMAs per complex product, the updates are CGEMM / ZGEMM.
//
// A zero on a non-unit diagonal gives Inf/NaN (1/0); the reference's inversion kernel
// substitutes 1 instead (trtri/diag_dtrtri_lower_128_16.cpp:93-96).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.hpp"
#include "internal.h"

namespace cba {

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef double f64x4_t __attribute__((ext_vector_type(4)));

// 16 x 16 x 4 MFMA: D[i][j] += sum_k A[i][k] B[k][j]; lane l supplies A[l%16][l/16] and
// B[l/16][l%16] and holds D[krow(l/16, v)][l%16] in accumulator element v (layouts checked
// on the device).
template <typename T> struct Mma16;
template <> struct Mma16<double> {
    typedef f64x4_t Acc;
    static __device__ __forceinline__ Acc run(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __host__ __device__ __forceinline__ int krow(int g, int v) { return g + 4 * v; }
};
template <> struct Mma16<float> {
    typedef f32x4_t Acc;
    static __device__ __forceinline__ Acc run(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    static __host__ __device__ __forceinline__ int krow(int g, int v) { return 4 * g + v; }
};

// Diagonal blocks (up to 256 x 256) are solved in 16 x 16 sub-blocks on the MFMA units.
//
// "Equation order" P = 0..nb-1 walks a diagonal block forward (index P) or backward (index
// nb-1-P) so that equation P only involves unknowns Q <= P.  coef(P,Q) is the factor of
// unknown Q in equation P:   left: op(A)(iP, iQ)   right: op(A)(iQ, iP),
// so with teff = trans XOR right it is A[iP + iQ*lda] (teff false) or A[iQ + iP*lda].
// In that order every diagonal block is lower triangular, L = (L_ws), 16 x 16 sub-blocks of
// 16 x 16, and the solve is the block substitution
//     X_s = inv(L_ss) Y_s ;   Y_w -= L_ws X_s  (w > s)        s = 0..15.
// A packing pass (trsm_pack_kernel, once per call, all diagonal blocks at once) reads the
// referenced triangle of A - never the other one, nor a unit diagonal - inverts the sixteen
// small triangles L_ss by substitution and writes, per diagonal block, the 136 sub-blocks
// inv(L_ss) and -L_ws in the order the MFMA "A" operand wants them: entry [lane][c] is
// element (p = lane%16, q = krow(lane/16, c)), so a lane fetches its four values of a
// sub-block with one or two 16-byte loads and nothing is broadcast.  Row w's sub-blocks
// (w,0..w) are consecutive, so each wavefront streams its own row straight from memory
// (L2), two steps ahead of their use.
// (The reference inverts whole 128 x 128 blocks, trtri/*.cpp; inverting only the 16 x 16
// ones keeps the result much closer to plain substitution.)
//
// Leaf kernel: one workgroup = one diagonal block x CW = 16 or 32 right-hand sides, 16
// wavefronts; wavefront w owns equations [16w, 16w+16) as CW/16 accumulator blocks of 16 x 16
// (lane l: right-hand side l%16 of each block, equations krow(l/16, v)).  Accumulator layout and
// MFMA "B" operand layout coincide, so Y_s feeds the MFMAs as it is and X_s goes to the
// other wavefronts through LDS in the same per-lane order.  Step s: wavefronts w > s subtract
// L_ws X_s (4 MFMAs per block); wavefront s+1 then computes X_(s+1) (4 per block) and publishes it
// while the others are still updating; one barrier per step.
// For side=left a right-hand side is a column of B; the panel moves between HBM and the
// accumulator layout through an LDS staging area so that global accesses run along columns.
template <typename T, bool RIGHT = false> struct TrsmLeaf {
    typedef typename Elem<T>::Real R;
    static constexpr bool CPLX = Elem<T>::CPLX;
    static constexpr int NB = 256, IB = 16, NBLK = NB / IB, THREADS = 64 * NBLK;
    // Right-hand sides per workgroup.  16: two workgroups fit a CU and cover each other's
    // serial solves (DTRSM left 2048: 0.36 -> 0.31 ms, 4096: 1.36 -> 1.28 ms, 8192 x 512: 1.52 ->
    // 1.34 ms).  Side = right with real elements keeps 32: its right-hand sides are rows of B,
    // and 16 of them are too short a run of memory (8192: 0.5 - 1.5 % slower with 16).
    static constexpr int CW = (RIGHT && !CPLX) ? 32 : 16, NBK = CW / 16;
    static constexpr int N_EBLK = NBLK * (NBLK + 1) / 2;  // sub-blocks (bi,bj), bi >= bj, at bi*(bi+1)/2 + bj
    // Packed sub-block: PLANES x 64 lanes x 4 reals.  Real: the values.  Complex: real parts,
    // imaginary parts, negated imaginary parts (so that no sign has to be flipped in the solve).
    static constexpr int PLANES = CPLX ? 3 : 1;
    static constexpr int SUB_REALS = PLANES * IB * IB;
    static constexpr int PACK_REALS = N_EBLK * SUB_REALS;  // per diagonal block
    static constexpr int NP = CPLX ? 2 : 1;                // accumulators per block (re, im)
    static constexpr int X_REALS = 2 * NP * NBK * 64 * 4;  // two buffers of X_s in per-lane order
    static constexpr int SP = NB + 2;                      // pitch of the right-hand-side staging area
    static constexpr int S_ELEMS = CW * SP;
    static constexpr size_t SMEM = (size_t)X_REALS * sizeof(R) + (size_t)S_ELEMS * sizeof(T);
};

// Element helpers for the packing pass (real and complex).
static __device__ __forceinline__ float tr_conj_if(float x, bool) { return x; }
static __device__ __forceinline__ double tr_conj_if(double x, bool) { return x; }
template <typename R> static __device__ __forceinline__ Cx<R> tr_conj_if(Cx<R> x, bool c) { return Cx<R>{x.re, c ? -x.im : x.im}; }
static __device__ __forceinline__ float tr_mul(float a, float b) { return a * b; }
static __device__ __forceinline__ double tr_mul(double a, double b) { return a * b; }
template <typename R> static __device__ __forceinline__ Cx<R> tr_mul(Cx<R> a, Cx<R> b) {
    return Cx<R>{a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
static __device__ __forceinline__ float tr_sub(float a, float b) { return a - b; }
static __device__ __forceinline__ double tr_sub(double a, double b) { return a - b; }
template <typename R> static __device__ __forceinline__ Cx<R> tr_sub(Cx<R> a, Cx<R> b) { return Cx<R>{a.re - b.re, a.im - b.im}; }
static __device__ __forceinline__ float tr_div(float a, float b) { return a / b; }
static __device__ __forceinline__ double tr_div(double a, double b) { return a / b; }
template <typename R> static __device__ __forceinline__ Cx<R> tr_div(Cx<R> a, Cx<R> b) {
    const R d = b.re * b.re + b.im * b.im;
    return Cx<R>{(a.re * b.re + a.im * b.im) / d, (a.im * b.re - a.re * b.im) / d};
}
// Writes value v (to be used as it is) into the planes of a packed sub-block at index w.
static __device__ __forceinline__ void tr_put(float *sub, int w, float v) { sub[w] = v; }
static __device__ __forceinline__ void tr_put(double *sub, int w, double v) { sub[w] = v; }
template <typename R> static __device__ __forceinline__ void tr_put(R *sub, int w, Cx<R> v) {
    sub[w] = v.re;
    sub[256 + w] = v.im;
    sub[512 + w] = -v.im;
}

// Packs all diagonal blocks of the n x n triangle (see above).  Workgroup (bi, b) of 256
// threads packs sub-block row bi of diagonal block b (rows/columns [256 b, 256 b + nb)).
// `conj` conjugates the coefficients (complex, clblasConjTrans).
template <typename T, bool FORWARD>
__global__ void __launch_bounds__(256)
trsm_pack_kernel(const T *__restrict__ A, int64_t lda, int n, bool teff, bool conj, bool unit,
                 typename Elem<T>::Real *__restrict__ pack) {
    typedef TrsmLeaf<T> L;
    typedef typename Elem<T>::Real R;
    typedef Mma16<R> M;
    constexpr int IB = L::IB;
    __shared__ T Ld[IB][IB + 1];  // the diagonal sub-triangle, then its inverse
    const int tid = threadIdx.x;
    const int bi = blockIdx.x;
    const int i0 = blockIdx.y * L::NB;
    const int nb = n - i0 < L::NB ? n - i0 : L::NB;
    const T *Ablk = A + i0 + (int64_t)i0 * lda;
    R *out = pack + (int64_t)blockIdx.y * L::PACK_REALS + (int64_t)(bi * (bi + 1) / 2) * L::SUB_REALS;
    auto coef = [&](int P, int Q) -> T {  // Q <= P < nb
        const int ip = FORWARD ? P : nb - 1 - P, iq = FORWARD ? Q : nb - 1 - Q;
        return tr_conj_if(teff ? Ablk[iq + (int64_t)ip * lda] : Ablk[ip + (int64_t)iq * lda], conj);
    };
    // off-diagonal sub-blocks (bi, 0..bi-1), negated; rows past nb are zero
    for (int e = tid; e < bi * IB * IB; e += 256) {
        const int bj = e / (IB * IB), w = e % (IB * IB);
        const int lane = w / 4, c = w % 4;
        const int P = bi * IB + lane % 16, Q = bj * IB + M::krow(lane / 16, c);
        // Q < P always holds here; Q < nb follows from P < nb
        tr_put(out + bj * L::SUB_REALS, w, (P < nb) ? tr_sub(T(), coef(P, Q)) : T());
    }
    // diagonal sub-triangle into LDS (identity where the block is short)
    {
        const int p = tid / IB, q = tid % IB;
        const int P = bi * IB + p, Q = bi * IB + q;
        T v = T();
        if (p == q) {
            v = el_one<T>();
            if (!unit && P < nb) v = coef(P, P);
        } else if (q < p && P < nb) {
            v = coef(P, Q);
        }
        Ld[p][q] = v;
    }
    __syncthreads();
    // invert: thread zc < 16 solves L z = e_zc by substitution
    T z[IB];
    const int zc = tid;
    if (tid < IB) {
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            T acc = (p == zc) ? el_one<T>() : T();
#pragma unroll
            for (int q = 0; q < IB; ++q)
                if (q < p) acc = tr_sub(acc, tr_mul(Ld[p][q], z[q]));
            z[p] = (p < zc) ? T() : tr_div(acc, Ld[p][p]);
        }
    }
    __syncthreads();
    if (tid < IB) {
#pragma unroll
        for (int p = 0; p < IB; ++p) Ld[p][zc] = z[p];
    }
    __syncthreads();
    {
        const int lane = tid / 4, c = tid % 4;
        tr_put(out + bi * L::SUB_REALS, tid, Ld[lane % 16][M::krow(lane / 16, c)]);
    }
}

template <typename T, bool RIGHT, bool FORWARD>
__global__ void __launch_bounds__(TrsmLeaf<T>::THREADS)
trsm_diag_kernel(const typename Elem<T>::Real *__restrict__ packed, int nb, T alpha, T *__restrict__ Bblk,
                 int64_t ldb, int nrhs) {
    typedef TrsmLeaf<T, RIGHT> L;
    typedef typename Elem<T>::Real R;
    typedef Mma16<R> M;
    typedef typename M::Acc Acc;
    constexpr bool CPLX = L::CPLX;
    constexpr int IB = L::IB, CW = L::CW, NBK = L::NBK, NT = L::THREADS, NBLK = L::NBLK, NP = L::NP;
    constexpr int PLANES = L::PLANES;
    constexpr int V = 16 / (int)sizeof(R);  // reals per 16 bytes
    typedef R VT __attribute__((ext_vector_type(V)));
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    R *X = reinterpret_cast<R *>(smem_raw);
    T *S = reinterpret_cast<T *>(X + L::X_REALS);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, jj = lane & 15;
    const int64_t j0 = (int64_t)blockIdx.x * CW;
    const int nsteps = (nb + IB - 1) / IB;  // sub-block rows that exist

    // A lane's values of sub-block (wave, s): MFMA "A" operand, plane pl, chunk c = element c.
    const R *erow = packed + (int64_t)(wave * (wave + 1) / 2) * L::SUB_REALS + lane * 4;
    auto load_e = [&](int s, R (&a)[PLANES][4]) {
#pragma unroll
        for (int pl = 0; pl < PLANES; ++pl) {
            const R *src = erow + s * L::SUB_REALS + pl * (IB * IB);
#pragma unroll
            for (int c = 0; c < 4; c += V) {
                VT t = *reinterpret_cast<const VT *>(src + c);
#pragma unroll
                for (int e = 0; e < V && c + e < 4; ++e) a[pl][c + e] = t[e];
            }
        }
    };
    constexpr int RING = CPLX ? 2 : 3;  // sub-blocks in flight: this step's and the next one or two
    R ea[RING][PLANES][4];
#pragma unroll
    for (int s = 0; s < RING - 1; ++s)
        if (s <= wave && wave < nsteps) load_e(s, ea[s]);

    // ---- right-hand sides into the accumulator layout: y[.][k][v] = alpha * b(equation krow(g,v)
    //      of this wavefront, right-hand side j0 + 16k + jj); complex: [0] real, [1] imaginary ----
    Acc y[NP][NBK];
    auto put_y = [&](int k, int v, T b) {
        const T ab = el_scale(alpha, b);
        if constexpr (CPLX) { y[0][k][v] = ab.re; y[1][k][v] = ab.im; } else { y[0][k][v] = ab; }
    };
    auto get_y = [&](int k, int v) -> T {
        if constexpr (CPLX) return T{y[0][k][v], y[1][k][v]};
        else return y[0][k][v];
    };
    auto mem_row = [&](int P) { return FORWARD ? P : nb - 1 - P; };
    if (RIGHT) {
#pragma unroll
        for (int k = 0; k < NBK; ++k) {
            const int64_t j = j0 + 16 * k + jj;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int P = wave * IB + M::krow(g, v);
                T b = T();
                if (P < nb && j < nrhs) b = Bblk[j + (int64_t)mem_row(P) * ldb];
                put_y(k, v, b);
            }
        }
    } else {
        constexpr int NLD = CW * (L::NB / 2) / NT;
        // (kept as real components: arrays of complex structs end up in scratch memory)
        constexpr int NC = CPLX ? 2 : 1;
        R v0[NLD][NC], v1[NLD][NC];
        auto split = [&](T t, R (&out)[NC]) {
            if constexpr (CPLX) { out[0] = t.re; out[1] = t.im; } else { out[0] = t; }
        };
        auto join = [&](const R (&in)[NC]) -> T {
            if constexpr (CPLX) return T{in[0], in[1]};
            else return in[0];
        };
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int e = tid + u * NT;
            const int c = e / (L::NB / 2), r = (e % (L::NB / 2)) * 2;
#pragma unroll
            for (int q = 0; q < NC; ++q) v0[u][q] = v1[u][q] = (R)0;
            if (j0 + c < nrhs) {
                const T *src = Bblk + r + (j0 + c) * ldb;
                if (r < nb) split(src[0], v0[u]);
                if (r + 1 < nb) split(src[1], v1[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int e = tid + u * NT;
            const int c = e / (L::NB / 2), r = (e % (L::NB / 2)) * 2;
            S[c * L::SP + r] = join(v0[u]);
            S[c * L::SP + r + 1] = join(v1[u]);
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < NBK; ++k)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int P = wave * IB + M::krow(g, v);
                put_y(k, v, (P < nb) ? S[(16 * k + jj) * L::SP + mem_row(P)] : T());
            }
    }

    // out (+)= E * in for one sub-block E (this lane's packed values e) and the blocks `in` in
    // MFMA "B" operand order.  Complex: Re += er*inr + (-ei)*ini, Im += er*ini + ei*inr.
    auto block_mma = [&](const R (&e)[PLANES][4], const Acc (&in)[NP][NBK], Acc (&out)[NP][NBK]) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int k = 0; k < NBK; ++k) {
                if constexpr (CPLX) {
                    out[0][k] = M::run(e[0][c], in[0][k][c], out[0][k]);
                    out[1][k] = M::run(e[0][c], in[1][k][c], out[1][k]);
                    out[0][k] = M::run(e[2][c], in[1][k][c], out[0][k]);
                    out[1][k] = M::run(e[1][c], in[0][k][c], out[1][k]);
                } else {
                    out[0][k] = M::run(e[0][c], in[0][k][c], out[0][k]);
                }
            }
    };
    // X_s = inv(L_ss) Y_s by the wavefront that owns row s; published in buffer s & 1.
    auto solve_row = [&](int s) {
        Acc x[NP][NBK];
#pragma unroll
        for (int pp = 0; pp < NP; ++pp)
#pragma unroll
            for (int k = 0; k < NBK; ++k) x[pp][k] = Acc{0, 0, 0, 0};
        block_mma(ea[s % RING], y, x);
        R *Xs = X + (s & 1) * (NP * NBK * 64 * 4);
#pragma unroll
        for (int pp = 0; pp < NP; ++pp)
#pragma unroll
            for (int k = 0; k < NBK; ++k) {
                y[pp][k] = x[pp][k];
                *reinterpret_cast<Acc *>(Xs + ((pp * NBK + k) * 64 + lane) * 4) = x[pp][k];
            }
    };
    if (wave == 0) solve_row(0);
    __syncthreads();
    // Step s: every row w > s subtracts L_ws X_s; the owner of row s+1 then solves it at once,
    // while the other wavefronts are still updating, so each step costs one barrier and the
    // solves stay off the critical path of everyone else.
#pragma unroll
    for (int s = 0; s < NBLK; ++s) {
        if (s < nsteps) {  // uniform over the workgroup
            const R *Xs = X + (s & 1) * (NP * NBK * 64 * 4);
            // Sub-block (wave, s+RING-1) goes into the ring slot that step s-1 used.  With a ring
            // of two it is the one solve_row(s+1) needs below, so it is requested first; with
            // three it is requested behind this step's MFMAs.
            const bool fetch = s + RING - 1 <= wave && wave < nsteps;
            if (RING == 2 && fetch) load_e(s + RING - 1, ea[(s + RING - 1) % RING]);
            if (wave > s && wave < nsteps) {
                Acc xb[NP][NBK];
#pragma unroll
                for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                    for (int k = 0; k < NBK; ++k)
                        xb[pp][k] = *reinterpret_cast<const Acc *>(Xs + ((pp * NBK + k) * 64 + lane) * 4);
                block_mma(ea[s % RING], xb, y);
                __builtin_amdgcn_sched_barrier(0);
                if (wave == s + 1) solve_row(s + 1);
            }
            if (RING > 2 && fetch) load_e(s + RING - 1, ea[(s + RING - 1) % RING]);
            __syncthreads();
        }
    }

    if (RIGHT) {
#pragma unroll
        for (int k = 0; k < NBK; ++k) {
            const int64_t j = j0 + 16 * k + jj;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int P = wave * IB + M::krow(g, v);
                if (P < nb && j < nrhs) Bblk[j + (int64_t)mem_row(P) * ldb] = get_y(k, v);
            }
        }
    } else {
        // The staging area was last read before the first barrier of the solve.
#pragma unroll
        for (int k = 0; k < NBK; ++k)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int P = wave * IB + M::krow(g, v);
                if (P < nb) S[(16 * k + jj) * L::SP + mem_row(P)] = get_y(k, v);
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

template <typename T> struct TrsmDriver {
    typedef typename Elem<T>::Real R;
    static constexpr int NBL = TrsmLeaf<T>::NB;
    bool right, trans, conj, unit, forward, teff;
    int M, N;
    const T *A;
    int64_t lda;
    T *B;
    int64_t ldb;
    hipStream_t stream;
    const R *pack;  // packed diagonal blocks, TrsmLeaf<T>::PACK_REALS each

    static T minus_one() { return el_scale_host(-1); }
    static T el_scale_host(int v) {
        if constexpr (Elem<T>::CPLX) return T{(R)v, (R)0};
        else return (T)v;
    }

    // Packs every diagonal block of the triangle (one launch per call).
    hipError_t prepare() {
        typedef TrsmLeaf<T> L;
        const int n = right ? N : M;
        const int nblk = (n + NBL - 1) / NBL;
        void *wv = nullptr;
        hipError_t we = workspace_get(stream, (size_t)nblk * L::PACK_REALS * sizeof(R), 2, &wv);
        if (we != hipSuccess) return we;
        R *w = (R *)wv;
        pack = w;
        dispatch_record().launches++;
        if (forward)
            return launch_kernel(trsm_pack_kernel<T, true>, dim3(L::NBLK, nblk), dim3(256), 0, stream, A, lda, n, teff,
                                 conj, unit, w);
        return launch_kernel(trsm_pack_kernel<T, false>, dim3(L::NBLK, nblk), dim3(256), 0, stream, A, lda, n, teff,
                             conj, unit, w);
    }

    template <bool RIGHT> hipError_t leaf_side(int i0, int nb, T alpha) {
        typedef TrsmLeaf<T, RIGHT> L;
        const int nrhs = RIGHT ? M : N;
        T *Bblk = RIGHT ? B + (int64_t)i0 * ldb : B + i0;
        const R *packed = pack + (int64_t)(i0 / NBL) * L::PACK_REALS;
        void (*fn)(const R *, int, T, T *, int64_t, int) =
            forward ? trsm_diag_kernel<T, RIGHT, true> : trsm_diag_kernel<T, RIGHT, false>;
        if (L::SMEM > 64 * 1024) {
            hipError_t e = ensure_dynamic_lds((const void *)fn, L::SMEM);
            if (e != hipSuccess) return e;
        }
        dim3 grid((unsigned)((nrhs + L::CW - 1) / L::CW)), block(L::THREADS);
        dispatch_record().launches++;
        return launch_kernel(fn, grid, block, L::SMEM, stream, packed, nb, alpha, Bblk, ldb, nrhs);
    }
    hipError_t leaf(int i0, int nb, T alpha) { return right ? leaf_side<true>(i0, nb, alpha) : leaf_side<false>(i0, nb, alpha); }

    // Off-diagonal update of the block range `dst` (length nd, start d0) with the solved
    // range `src` (length ns, start s0):   B_dst <- beta * B_dst - coupling * X_src.
    hipError_t update(int d0, int nd, int s0, int ns, T beta) {
        if (!right) {
            // rows: B[d0.., :] -= op(A)[d0.., s0..] * B[s0.., :]
            const T *Ablk = trans ? A + s0 + (int64_t)d0 * lda : A + d0 + (int64_t)s0 * lda;
            return launch_gemm<T>(trans, false, conj, false, nd, N, ns, minus_one(), Ablk, lda, B + s0, ldb, beta, B + d0,
                                  ldb, stream);
        }
        // columns: B[:, d0..] -= B[:, s0..] * op(A)[s0.., d0..]
        const T *Ablk = trans ? A + d0 + (int64_t)s0 * lda : A + s0 + (int64_t)d0 * lda;
        return launch_gemm<T>(false, trans, false, conj, M, nd, ns, minus_one(), B + (int64_t)s0 * ldb, ldb, Ablk, lda, beta,
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
            return solve(i0 + n_lo, n_hi, el_scale_host(1));
        }
        if ((e = solve(i0 + n_lo, n_hi, alpha)) != hipSuccess) return e;
        if ((e = update(i0, n_lo, i0 + n_lo, n_hi, alpha)) != hipSuccess) return e;
        return solve(i0, n_lo, el_scale_host(1));
    }
};

template <typename T>
hipError_t trsm_colmajor(bool right, bool lower, bool trans, bool conj, bool unit, int M, int N, T alpha, const T *A,
                         int64_t lda, T *B, int64_t ldb, hipStream_t stream) {
    TrsmDriver<T> d;
    d.right = right; d.trans = trans; d.conj = conj && Elem<T>::CPLX; d.unit = unit;
    // Left: equations run forward when op(A) is lower triangular; right: when it is upper.
    d.forward = right ? (lower == trans) : (lower != trans);
    d.teff = trans != right;
    d.M = M; d.N = N; d.A = A; d.lda = lda; d.B = B; d.ldb = ldb; d.stream = stream;
    hipError_t e = d.prepare();
    if (e != hipSuccess) return e;
    return d.solve(0, right ? N : M, alpha);
}

template hipError_t trsm_colmajor<float>(bool, bool, bool, bool, bool, int, int, float, const float *, int64_t, float *,
                                         int64_t, hipStream_t);
template hipError_t trsm_colmajor<double>(bool, bool, bool, bool, bool, int, int, double, const double *, int64_t,
                                          double *, int64_t, hipStream_t);
template hipError_t trsm_colmajor<Cx<float>>(bool, bool, bool, bool, bool, int, int, Cx<float>, const Cx<float> *,
                                             int64_t, Cx<float> *, int64_t, hipStream_t);
template hipError_t trsm_colmajor<Cx<double>>(bool, bool, bool, bool, bool, int, int, Cx<double>, const Cx<double> *,
                                              int64_t, Cx<double> *, int64_t, hipStream_t);

}  // namespace cba
