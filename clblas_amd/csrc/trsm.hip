// Blocked triangular solve for gfx950: substitution on the diagonal blocks, MFMA GEMM for
// everything off the diagonal.
//
// Stands where the reference has gpu_dtrsm128 (src/library/blas/xtrsm.cc:1136-1507) and,
// for STRSM, the legacy block solver (src/library/blas/gens/trsm.c:1213-1456).  The
// reference inverts every 128x128 diagonal block (trtri kernels) and then alternates
// "X_i = inv(A_ii) B_i" with a trailing DGEMM update, using an M x N temporary.  Here the
// diagonal blocks (512 x 512, 256 x 256 for complex types) are solved inside one kernel by block substitution over their
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
// B[l/16][l%16] and holds D[hw(l/16, v)][l%16] in accumulator element v, hw(g, v) = 4g + v for FP32
// and g + 4v for FP64 (layouts checked
// on the device).
template <typename T> struct Mma16;
template <> struct Mma16<double> {
    typedef f64x4_t Acc;
    static __device__ __forceinline__ Acc run(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    // Which equation of a sub-block a row of the MFMA stands for is free, as long as the coefficients
    // are packed to match: row i stands for equation arow(i) = 4 (i % 4) + i / 4, so that the four
    // rows g + 4v that a lane holds are the neighbouring equations krow(g, v) = 4g + v (one run of
    // memory per lane, as for FP32, instead of four).
    static __host__ __device__ __forceinline__ int krow(int g, int v) { return 4 * g + v; }
    static __host__ __device__ __forceinline__ int arow(int i) { return 4 * (i % 4) + i / 4; }
};
template <> struct Mma16<float> {
    typedef f32x4_t Acc;
    static __device__ __forceinline__ Acc run(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    static __host__ __device__ __forceinline__ int krow(int g, int v) { return 4 * g + v; }
    static __host__ __device__ __forceinline__ int arow(int i) { return i; }
};

// Diagonal blocks (up to 512 x 512; complex types 256 x 256) are solved in 16 x 16 sub-blocks on the MFMA units.
//
// "Equation order" P = 0..nb-1 walks a diagonal block forward (index P) or backward (index
// nb-1-P) so that equation P only involves unknowns Q <= P.  coef(P,Q) is the factor of
// unknown Q in equation P:   left: op(A)(iP, iQ)   right: op(A)(iQ, iP),
// so with teff = trans XOR right it is A[iP + iQ*lda] (teff false) or A[iQ + iP*lda].
// In that order every diagonal block is lower triangular, L = (L_ws), NBLK x NBLK sub-blocks of
// 16 x 16 (NBLK = 32 for real types, 16 for complex ones), and the solve is the block substitution
//     X_s = inv(L_ss) Y_s ;   Y_w -= L_ws X_s  (w > s)        s = 0..NBLK-1.
// A packing pass (trsm_pack_kernel, once per call, all diagonal blocks at once) reads the
// referenced triangle of A - never the other one, nor a unit diagonal - inverts the
// small triangles L_ss by substitution and writes, per diagonal block, the NBLK (NBLK+1)/2 sub-blocks
// inv(L_ss) and -L_ws in the order the MFMA "A" operand wants them: value c of lane `lane` is
// element (p = arow(lane%16), q = krow(lane/16, c)), filed at packed_at(lane, c), so a lane fetches its
// four values of a sub-block with one or two 16-byte loads and nothing is broadcast.  Row w's sub-blocks
// (w,0..w) are consecutive, so each wavefront streams its own row straight from memory
// (L2), one to three sub-blocks ahead of their use.
// (The reference inverts whole 128 x 128 blocks, trtri/*.cpp; inverting only the 16 x 16
// ones keeps the result much closer to plain substitution.)
//
// Leaf kernel: one workgroup = one diagonal block x CW = 16 or 32 right-hand sides, 16
// wavefronts; wavefront w owns sub-block rows w (and w+16), each as CW/16 accumulator blocks of
// 16 x 16 (lane l: right-hand side l%16 of each block, equations krow(l/16, v)).  Accumulator layout
// and MFMA "B" operand layout coincide, so Y_s feeds the MFMAs as it is and X_s goes to the
// other wavefronts through LDS in the same per-lane order.  A row subtracts L_ws X_s (4 MFMAs per
// block) for every s below it as the X_s appear, then computes X_w (4 per block) and publishes
// it; the wavefronts are synchronised by one flag per X_s in LDS, not by barriers.
// Every wavefront moves its own rows between memory and the accumulator layout directly (side = left:
// a right-hand side is a column of B, and the loads of a row block touch one cache line per column;
// side = right: a row of B); a row is written back as soon as it is solved.
template <typename T, bool RIGHT = false, bool WIDE = false> struct TrsmLeaf {
    typedef typename Elem<T>::Real R;
    static constexpr bool CPLX = Elem<T>::CPLX;
    // Row blocks per wavefront.  Real types: two, i.e. a leaf of 512 equations.  The updates of
    // the second row block fill the MFMA pipes while the serial chain of the first 256 equations
    // runs, and the 256-row GEMM update between two leaves of 256 (a launch of its own, short of
    // work: 17 us against 14 us for a leaf at 2048 right-hand sides) is gone.  Complex types keep
    // one row block (their packed sub-blocks are three times the size; LDS and registers).
    static constexpr int WAVES = 16, RW = CPLX ? 1 : 2;
    static constexpr int IB = 16, NB = WAVES * IB * RW, NBLK = NB / IB, THREADS = 64 * WAVES;
    static constexpr int CW = WIDE ? 32 : 16, NBK = CW / 16;
    static constexpr int N_EBLK = NBLK * (NBLK + 1) / 2;  // sub-blocks (bi,bj), bi >= bj, at bi*(bi+1)/2 + bj
    // Packed sub-block: PLANES x 64 lanes x 4 reals.  Real: the values.  Complex: real parts,
    // imaginary parts, negated imaginary parts (so that no sign has to be flipped in the solve).
    static constexpr int PLANES = CPLX ? 3 : 1;
    static constexpr int SUB_REALS = PLANES * IB * IB;
    static constexpr int PACK_REALS = N_EBLK * SUB_REALS;  // per diagonal block
    static constexpr int NP = CPLX ? 2 : 1;                // accumulators per block (re, im)
    static constexpr int XS_REALS = NP * NBK * 64 * 4;     // one X_s in per-lane order
    static constexpr int X_REALS = NBLK * XS_REALS;        // every X_s keeps a slot of its own
    // LDS: the X slots, then one "published" flag per step.
    static constexpr size_t FLAGS_AT = ((size_t)X_REALS * sizeof(R) + 15) / 16 * 16;
    static constexpr size_t SMEM = FLAGS_AT + NBLK * sizeof(int);
    static constexpr int PACK_CHUNK = 8;                   // sub-blocks per workgroup of the packing pass
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
// Place of value c (0..3) of lane `lane` in a plane of a packed sub-block: the plane is a row of 16-byte
// pieces, piece k of all 64 lanes together, so that one load instruction of a wavefront reads 1 KB in one
// run (whole cache lines; FP32: a lane's four values are one piece anyway).
template <typename R> static __host__ __device__ __forceinline__ int packed_at(int lane, int c) {
    constexpr int V = 16 / (int)sizeof(R);
    return (c / V) * (64 * V) + lane * V + c % V;
}
// Writes value v (to be used as it is) into the planes of a packed sub-block, value w % 4 of lane w / 4.
static __device__ __forceinline__ void tr_put(float *sub, int w, float v) { sub[packed_at<float>(w / 4, w % 4)] = v; }
static __device__ __forceinline__ void tr_put(double *sub, int w, double v) { sub[packed_at<double>(w / 4, w % 4)] = v; }
template <typename R> static __device__ __forceinline__ void tr_put(R *sub, int w, Cx<R> v) {
    const int at = packed_at<R>(w / 4, w % 4);
    sub[at] = v.re;
    sub[256 + at] = v.im;
    sub[512 + at] = -v.im;
}

// Packs all diagonal blocks of the n x n triangle (see above).  Workgroup (bi, chunk, b) of 256
// threads packs up to PACK_CHUNK sub-blocks of sub-block row bi of diagonal block b (rows/columns
// [NB b, NB b + nb)).
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
    constexpr int CHUNKS = L::NBLK / L::PACK_CHUNK;
    const int tid = threadIdx.x;
    const int bi = blockIdx.x / CHUNKS, chunk = blockIdx.x % CHUNKS;
    if (chunk > bi / L::PACK_CHUNK) return;  // nothing of row bi lies in this chunk
    const int i0 = blockIdx.y * L::NB;
    const int nb = n - i0 < L::NB ? n - i0 : L::NB;
    const T *Ablk = A + i0 + (int64_t)i0 * lda;
    R *out = pack + (int64_t)blockIdx.y * L::PACK_REALS + (int64_t)(bi * (bi + 1) / 2) * L::SUB_REALS;
    auto coef = [&](int P, int Q) -> T {  // Q <= P < nb
        const int ip = FORWARD ? P : nb - 1 - P, iq = FORWARD ? Q : nb - 1 - Q;
        return tr_conj_if(teff ? Ablk[iq + (int64_t)ip * lda] : Ablk[ip + (int64_t)iq * lda], conj);
    };
    // off-diagonal sub-blocks (bi, bj) of this chunk, bj < bi, negated; rows past nb are zero
    const int bj_lo = chunk * L::PACK_CHUNK;
    const int bj_hi = bj_lo + L::PACK_CHUNK < bi ? bj_lo + L::PACK_CHUNK : bi;
    for (int e = bj_lo * IB * IB + tid; e < bj_hi * IB * IB; e += 256) {
        const int bj = e / (IB * IB), w = e % (IB * IB);
        const int lane = w / 4, c = w % 4;
        const int P = bi * IB + M::arow(lane % 16), Q = bj * IB + M::krow(lane / 16, c);
        // Q < P always holds here; Q < nb follows from P < nb
        tr_put(out + bj * L::SUB_REALS, w, (P < nb) ? tr_sub(T(), coef(P, Q)) : T());
    }
    if (chunk != bi / L::PACK_CHUNK) return;  // the chunk that holds column bi also inverts (bi, bi)
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
    // invert: thread zc < 16 solves L z = e_zc by substitution.  The sixteen reciprocals of the diagonal
    // are taken first, all at once: one division's latency instead of sixteen in a row.
    __shared__ T Rd[IB];
    if (tid < IB) Rd[tid] = tr_div(el_one<T>(), Ld[tid][tid]);
    __syncthreads();
    T z[IB];
    const int zc = tid;
    if (tid < IB) {
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            T acc = (p == zc) ? el_one<T>() : T();
#pragma unroll
            for (int q = 0; q < IB; ++q)
                if (q < p) acc = tr_sub(acc, tr_mul(Ld[p][q], z[q]));
            z[p] = (p < zc) ? T() : tr_mul(acc, Rd[p]);
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
        tr_put(out + bi * L::SUB_REALS, tid, Ld[M::arow(lane % 16)][M::krow(lane / 16, c)]);
    }
}

template <int N> struct IntC { static constexpr int value = N; };

// Number of flag waits of trsm_diag_kernel that gave up at their poll limit since the library was
// loaded (per GPU).  A wait that gives up lets its wavefront go on with whatever the slot holds - a
// wrong result instead of a hang - so this counter staying at zero is what says that no result
// was ever produced that way.  Only touched on that path; read by clblasAmdTrsmPollTimeouts.
__device__ unsigned int trsm_poll_timeouts = 0;

template <typename T, bool RIGHT, bool FORWARD, bool WIDE>
__global__ void __launch_bounds__(TrsmLeaf<T>::THREADS)
trsm_diag_kernel(const typename Elem<T>::Real *__restrict__ packed, int nb, T alpha, T *__restrict__ Bblk,
                 int64_t ldb, int nrhs, int poll_limit) {
    typedef TrsmLeaf<T, RIGHT, WIDE> L;
    typedef typename Elem<T>::Real R;
    typedef Mma16<R> M;
    typedef typename M::Acc Acc;
    constexpr bool CPLX = L::CPLX;
    constexpr int IB = L::IB, CW = L::CW, NBK = L::NBK, NBLK = L::NBLK, NP = L::NP;
    constexpr int PLANES = L::PLANES, RW = L::RW, WAVES = L::WAVES;
    constexpr int V = 16 / (int)sizeof(R);  // reals per 16 bytes
    constexpr int CH = 4 / V;               // 16-byte pieces of an accumulator block
    typedef R VT __attribute__((ext_vector_type(V)));
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    R *X = reinterpret_cast<R *>(smem_raw);
    int *published = reinterpret_cast<int *>(smem_raw + L::FLAGS_AT);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, jj = lane & 15;
    const int64_t j0 = (int64_t)blockIdx.x * CW;
    const int nsteps = (nb + IB - 1) / IB;  // sub-block rows that exist
    if (tid < NBLK) published[tid] = 0;
    __syncthreads();  // the only barrier: from here on every wavefront runs at its own pace

    // This wavefront owns the sub-block rows wave + WAVES*h, h < RW.
    // A lane's values of sub-block (row, s): MFMA "A" operand, plane pl, chunk c = element c.
    const R *erow[RW];
#pragma unroll
    for (int h = 0; h < RW; ++h) {
        const int row = wave + WAVES * h;
        erow[h] = packed + (int64_t)(row * (row + 1) / 2) * L::SUB_REALS + lane * V;
    }
    auto load_e = [&](int h, int s, R (&a)[PLANES][4]) {
#pragma unroll
        for (int pl = 0; pl < PLANES; ++pl) {
            const R *src = erow[h] + s * L::SUB_REALS + pl * (IB * IB);
#pragma unroll
            for (int c = 0; c < 4; c += V) {
                VT t = *reinterpret_cast<const VT *>(src + (c / V) * (64 * V));
#pragma unroll
                for (int e = 0; e < V && c + e < 4; ++e) a[pl][c + e] = t[e];
            }
        }
    };
    // A wavefront finishes its first row block before it starts on its second, so one ring of
    // sub-blocks in flight serves both, one after the other.
    constexpr int RING = CPLX ? 2 : 4;  // sub-blocks in flight: the current one and the next one to three
    R ea[RING][PLANES][4];
    // Every wavefront requests the same number of sub-blocks at the same places of the program, needed
    // or not (a row's own diagonal sub-block again once it is past it): with requests under
    // conditions the compiler can only wait for ALL outstanding loads before each use, which puts a
    // full memory latency into every step.
    auto prefetch = [&](int h, int s) {
        const int row = wave + WAVES * h;
        load_e(h, s < row ? s : row, ea[s % RING]);
    };
    // Real types keep each row's own diagonal sub-block (its inverse) in registers of its own, requested
    // first of all, so that a solve never waits for memory; the complex kernels have no registers
    // to spare for that and take it from the ring.
    constexpr bool DIAG_REGS = !CPLX && !(WIDE && sizeof(R) == 8);  // (FP64 with 32 right-hand sides: no registers to spare either)
    R ed[DIAG_REGS ? RW : 1][PLANES][4];
    if constexpr (DIAG_REGS) {
#pragma unroll
        for (int h = 0; h < RW; ++h) load_e(h, wave + WAVES * h, ed[h]);
    }
#pragma unroll
    for (int s = 0; s < RING - 1; ++s) prefetch(0, s);
    constexpr int LOADS_PER_SUB = PLANES * (4 / V);  // load instructions per sub-block and lane
    // Waits until at most n of this wavefront's global loads are outstanding (they return in order).
    auto wait_loads = [&](int n) {
        switch (n) {  // (n is known at compile time where this is used)
            case 0: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(0)); break;
            case 1: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(1)); break;
            case 2: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(2)); break;
            case 3: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(3)); break;
            case 4: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(4)); break;
            case 5: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(5)); break;
            case 6: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(6)); break;
            default: __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(0)); break;
        }
    };

    // ---- right-hand sides into the accumulator layout: y[h][.][k][v] = alpha * b(equation
    //      krow(g,v) of row block h of this wavefront, right-hand side j0 + 16k + jj); complex: [0]
    //      real, [1] imaginary ----
    Acc y[RW][NP][NBK];
    auto put_y = [&](int h, int k, int v, T b) {
        const T ab = el_scale(alpha, b);
        if constexpr (CPLX) { y[h][0][k][v] = ab.re; y[h][1][k][v] = ab.im; } else { y[h][0][k][v] = ab; }
    };
    auto get_y = [&](int h, int k, int v) -> T {
        if constexpr (CPLX) return T{y[h][0][k][v], y[h][1][k][v]};
        else return y[h][0][k][v];
    };
    auto mem_row = [&](int P) { return FORWARD ? P : nb - 1 - P; };
    // Element (equation P, right-hand side j) of the panel: rows of B for side = left, columns for right.
    auto at = [&](int P, int64_t j) -> int64_t {
        return RIGHT ? j + (int64_t)mem_row(P) * ldb : (int64_t)mem_row(P) + j * ldb;
    };
    // Every wavefront fetches its own rows straight into the accumulator layout (side = left: the four
    // loads of a row block touch the same 16 cache lines, one per right-hand side) and writes each row
    // back as soon as it is solved: no staging through LDS, no barrier, and both ends of the kernel
    // overlap with the solve.
    // Side = left: a lane's four equations krow(g, 0..3) = 4g .. 4g+3 are neighbours in memory.
    constexpr bool ROWS4 = !RIGHT;
    constexpr int RPE = CPLX ? 2 : 1;  // reals per element
    typedef R rx4u_t __attribute__((ext_vector_type(4 * RPE), aligned(sizeof(R))));
    auto elem_of = [&](const rx4u_t &t, int v) -> T {
        if constexpr (CPLX) return T{t[2 * v], t[2 * v + 1]};
        else return t[v];
    };
    auto set_elem = [&](rx4u_t &t, int v, T x) {
        if constexpr (CPLX) { t[2 * v] = x.re; t[2 * v + 1] = x.im; } else { t[v] = x; }
    };
#pragma unroll
    for (int h = 0; h < RW; ++h)
#pragma unroll
        for (int k = 0; k < NBK; ++k) {
            const int64_t j = j0 + 16 * k + jj;
            const int P0 = (wave + WAVES * h) * IB + M::krow(g, 0);
            if (ROWS4 && P0 + 3 < nb && j < nrhs) {
                if constexpr (ROWS4) {
                    const rx4u_t t = *reinterpret_cast<const rx4u_t *>(Bblk + (FORWARD ? at(P0, j) : at(P0 + 3, j)));
#pragma unroll
                    for (int v = 0; v < 4; ++v) put_y(h, k, v, elem_of(t, FORWARD ? v : 3 - v));
                }
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int P = (wave + WAVES * h) * IB + M::krow(g, v);
                    // (every lane loads, from a harmless address if it has no element: loads under
                    // conditions are waited for one by one)
                    const bool have = P < nb && j < nrhs;
                    const T b = Bblk[have ? at(P, j) : 0];
                    put_y(h, k, v, have ? b : T());
                }
            }
        }
    auto store_row = [&](int h) {
#pragma unroll
        for (int k = 0; k < NBK; ++k) {
            const int64_t j = j0 + 16 * k + jj;
            const int P0 = (wave + WAVES * h) * IB + M::krow(g, 0);
            if (ROWS4 && P0 + 3 < nb && j < nrhs) {
                if constexpr (ROWS4) {
                    rx4u_t t;
#pragma unroll
                    for (int v = 0; v < 4; ++v) set_elem(t, FORWARD ? v : 3 - v, get_y(h, k, v));
                    *reinterpret_cast<rx4u_t *>(Bblk + (FORWARD ? at(P0, j) : at(P0 + 3, j))) = t;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int P = (wave + WAVES * h) * IB + M::krow(g, v);
                    if (P < nb && j < nrhs) Bblk[at(P, j)] = get_y(h, k, v);
                }
            }
        }
    };

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
    // A block of X in LDS: 16-byte pieces, each piece of all 64 lanes together, so that the lanes of a
    // 16-byte access are 16 bytes apart (no bank conflicts for FP64 either).
    auto x_put = [&](R *Xs, int pp, int k, const Acc &a) {
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            VT t;
#pragma unroll
            for (int e = 0; e < V; ++e) t[e] = a[ch * V + e];
            *reinterpret_cast<VT *>(Xs + (((pp * NBK + k) * CH + ch) * 64 + lane) * V) = t;
        }
    };
    auto x_get = [&](const R *Xs, int pp, int k) -> Acc {
        Acc a;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            const VT t = *reinterpret_cast<const VT *>(Xs + (((pp * NBK + k) * CH + ch) * 64 + lane) * V);
#pragma unroll
            for (int e = 0; e < V; ++e) a[ch * V + e] = t[e];
        }
        return a;
    };
    // There are no barriers between the steps.  Every X_s has an LDS slot of its own and a flag that
    // its owner sets once the slot is written; a wavefront that needs X_s polls the flag.  LDS
    // operations of one wavefront are carried out in order, so a wavefront that reads the flag as
    // set reads the complete X_s after it.  A wavefront takes its row blocks one after the other:
    // row w needs X_0 .. X_(w-1) as they appear, is solved and published; then row w+16 is brought up
    // to date with everything published so far and follows the chain until its own turn.  The chain
    // "update row s+1 with X_s, solve, publish X_(s+1)" thus competes for the MFMA pipes only with
    // rows that are about to be needed and with wavefronts catching up, not with 31 - s updates
    // per step that a barrier would all put in front of the next solve.
    // Every flag a wavefront waits for belongs to a lower row, so the waits end; the poll count is
    // bounded all the same, so that a mistake would show as a wrong result and not as a hang.
    auto publish = [&](int s) {
        asm volatile("" ::: "memory");  // (compiler only) the X_s stores stay in front of the flag store
        if (lane == 0) __hip_atomic_store(published + s, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    auto wait_for = [&](int s, bool urgent) {
        int polls = 0;
        for (; polls < poll_limit; ++polls) {
            // (an atomic load: a plain one may be hoisted out of the loop, a volatile one is compiled as
            // a flat access, which also waits for every outstanding global load)
            if (__builtin_amdgcn_readfirstlane(
                    __hip_atomic_load(published + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) != 0)
                break;
            if (!urgent) __builtin_amdgcn_s_sleep(1);
        }
        if (polls >= poll_limit && lane == 0) atomicAdd(&trsm_poll_timeouts, 1u);
        asm volatile("" ::: "memory");  // (compiler only) the X_s loads stay behind the flag load
    };
    // Row block h of this wavefront: updates with X_0 .. X_(row-1), then X_row = inv(L_row,row) Y.
    // The loop runs over groups of RING steps so that the register ring is indexed by constants;
    // every step of a group requests a sub-block, needed or not (see above), and only steps up to
    // the row's own do any work.
    auto run_row = [&](auto hcst) __attribute__((always_inline)) {
        constexpr int h = decltype(hcst)::value;
        const int row = wave + WAVES * h;
        if (row >= nsteps) return;
        if constexpr (h > 0) {
#pragma unroll
            for (int s = 0; s < RING - 1; ++s) prefetch(h, s);
        }
        // Steps are taken two at a time wherever the row is not about to be solved: both X read together,
        // the two products on separate accumulators so that their MFMAs alternate.  One step at a time
        // costs a wavefront the latencies of a step (flag, X, four dependent MFMAs, the way round the
        // loop) every time, a wavefront that falls behind the chain makes the chain wait when its row's
        // turn comes, and the last rows of a leaf are finished by such wavefronts alone.  The X are
        // published in order, so the flag of the later one covers both; a second row block starts
        // behind the chain (X_0 .. X_(row - WAVES) were published before this wavefront published its
        // previous row) and needs no flags there.  The last PAIR_GAP steps before the solve go one by
        // one: they are not to wait for a second X.
        // (Which steps are paired depends on the row only, so the order of summation is fixed.)
        constexpr int PAIR_GAP = 3;
        constexpr bool PAIRS = RING >= 4 && !(WIDE && sizeof(R) == 8);
        Acc y2[NP][NBK];
#pragma unroll
        for (int pp = 0; pp < NP; ++pp)
#pragma unroll
            for (int k = 0; k < NBK; ++k) y2[pp][k] = Acc{0, 0, 0, 0};
        bool next_done = false;
        constexpr bool SOLVE_AT_ONCE = DIAG_REGS && !WIDE;
        bool solved = false;
#pragma nounroll
        for (int s0 = 0; s0 <= row; s0 += RING) {
#pragma unroll
            for (int j = 0; j < RING; ++j) {
                const int s = s0 + j;
                {  // sub-block (row, s+RING-1) into the slot that step s-1 used
                    const int nxt = s + RING - 1;
                    load_e(h, nxt < row ? nxt : row, ea[(j + RING - 1) % RING]);
                }
                if (PAIRS && next_done) {  // this step went with the one before
                    next_done = false;
                } else if (PAIRS && j % 2 == 0 && s + 1 <= row - PAIR_GAP) {
                    if constexpr (PAIRS) {
                        // (the X are published in order: the flag of the later one covers both)
                        if (s + 1 > row - WAVES) wait_for(s + 1, false);
                        wait_loads((RING - 2) * LOADS_PER_SUB);
                        Acc xa[NP][NBK], xb[NP][NBK];
                        const R *Xa = X + s * L::XS_REALS, *Xb = Xa + L::XS_REALS;
#pragma unroll
                        for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                            for (int k = 0; k < NBK; ++k) {
                                xa[pp][k] = x_get(Xa, pp, k);
                                xb[pp][k] = x_get(Xb, pp, k);
                            }
#pragma unroll
                        for (int c = 0; c < 4; ++c)
#pragma unroll
                            for (int k = 0; k < NBK; ++k) {
                                y[h][0][k] = M::run(ea[j][0][c], xa[0][k][c], y[h][0][k]);
                                y2[0][k] = M::run(ea[(j + 1) % RING][0][c], xb[0][k][c], y2[0][k]);
                            }
                        __builtin_amdgcn_sched_barrier(0);
                        next_done = true;
                    }
                } else if (s < row) {
                    const bool solves_next = s + 1 == row;
                    if (solves_next) __builtin_amdgcn_s_setprio(2);
                    wait_for(s, solves_next);
                    // Said explicitly: left to itself the compiler, which cannot know which of the
                    // conditional uses were executed, waits for all outstanding loads.
                    wait_loads((RING - 1) * LOADS_PER_SUB);
                    Acc xb[NP][NBK];
                    const R *Xs = X + s * L::XS_REALS;
#pragma unroll
                    for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                        for (int k = 0; k < NBK; ++k) xb[pp][k] = x_get(Xs, pp, k);
                    block_mma(ea[j], xb, y[h]);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (SOLVE_AT_ONCE) {
                        // The row's last update is followed by its solve without going round the loop
                        // (a request for coefficients, tests, a taken branch: 300 cycles on the chain).
                        if (solves_next) {
                            if constexpr (PAIRS) y[h][0][0] += y2[0][0];
                            Acc x = Acc{0, 0, 0, 0};
#pragma unroll
                            for (int c = 0; c < 4; ++c) x = M::run(ed[h][0][c], y[h][0][0][c], x);
                            y[h][0][0] = x;
                            x_put(X + row * L::XS_REALS, 0, 0, x);
                            publish(row);
                            __builtin_amdgcn_s_setprio(0);
                            store_row(h);
                            solved = true;
                        }
                    }
                } else if (s == row && !(SOLVE_AT_ONCE && solved)) {  // every update is in: solve and publish
                    if constexpr (PAIRS) {
#pragma unroll
                        for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                            for (int k = 0; k < NBK; ++k) y[h][pp][k] += y2[pp][k];
                    }
                    Acc x[NP][NBK];
#pragma unroll
                    for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                        for (int k = 0; k < NBK; ++k) x[pp][k] = Acc{0, 0, 0, 0};
                    if constexpr (DIAG_REGS) {
                        block_mma(ed[h], y[h], x);
                    } else {
                        wait_loads((RING - 1) * LOADS_PER_SUB);
                        block_mma(ea[j], y[h], x);
                    }
                    R *Xs = X + s * L::XS_REALS;
#pragma unroll
                    for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                        for (int k = 0; k < NBK; ++k) {
                            y[h][pp][k] = x[pp][k];
                            x_put(Xs, pp, k, x[pp][k]);
                        }
                    publish(s);
                    __builtin_amdgcn_s_setprio(0);
                    store_row(h);
                }
            }
        }
    };
    if constexpr (DIAG_REGS) {
        if (wave == 0) wait_loads((RING - 1) * LOADS_PER_SUB);  // its diagonal sub-block is needed at once
    }
    run_row(IntC<0>{});
    if constexpr (RW > 1) run_row(IntC<1>{});
    static_assert(RW <= 2, "one run_row call per row block");
}

// ---------------------------------------------------------------------------------------------
// Real types: diagonal blocks of 512 x 512 solved with explicitly inverted 64 x 64 triangles.
//
// The reference inverts its diagonal blocks by doubling - 16 x 16 triangles by substitution, then
// inv21 = -inv22 (A21 inv11) for 32, 64 and 128 (trtri/diag_dtrtri_lower_128_16.cpp:60-160,
// trtri/triple_dgemm_update_128_16_PART1_L.cpp:44-160, ..._32_PART1_L.cpp, ..._64_PART1_L.cpp) - and
// multiplies by the inverses.  The same here up to 64 x 64 ("super-blocks" of four sub-block rows):
// the packing pass files, for sub-block row r = 4S + i, the sub-blocks -L(r, q) for q < 4S and the
// sub-blocks Inv_S(i, j), j <= i, of the inverted triangle at q = 4S + j - one uniform row of
// MFMA "A" operands - and the solve of a diagonal block is eight steps
//     X_S = Inv_S Y_S ;   Y_r += (-L(r, 4S..4S+3)) X_S   for every sub-block row r beyond S.
// Substitution over 16-row sub-blocks needs 32 dependent steps whose latencies (flag, X out of LDS, four
// dependent MFMAs, X into LDS) do not overlap with the bulk of the MFMA work; with the inverses the
// serial part of a step is one product per owner and everything else is work for all sixteen
// wavefronts between two barriers.
//
// Workgroup: one diagonal block x 16 NBK right-hand sides, 16 wavefronts, wavefront w owning sub-block
// rows w and w + 16 (accumulators, as above); super-block S is owned by four consecutive
// wavefronts, one per SIMD.  Step S:
//   A  the four owners: X_r = sum_{j<=i} Inv_S(i, j) Y_(4S+j), the Y of the other owners out of LDS
//      (written at the end of the step before); X_r to LDS and to memory.           barrier
//   B  every wavefront, each row beyond S it owns: four products with the X of S; then the row's
//      coefficients of the next step are requested; owners of S + 1 file their Y.      barrier
// The schedule is fixed, so results are reproducible bit for bit.
template <typename R> struct TrsmBlock {
    static constexpr int IB = 16, WAVES = 8, RW = 4, NB = WAVES * IB * RW, NBLK = NB / IB;
    static constexpr int SBR = 4, SB = SBR * IB, NS = NB / SB;  // sub-block rows per super-block, its order, super-blocks
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int SUB_REALS = IB * IB;
    static constexpr int N_EBLK = NBLK * (NBLK + 1) / 2;
    static constexpr int PACK_REALS = N_EBLK * SUB_REALS;
    static constexpr int PACK_CHUNK = 8;                        // sub-blocks per copying workgroup of the packing pass
    static constexpr int COPY_GROUPS = NBLK * (NBLK / PACK_CHUNK);
    typedef double Work;                                        // the inversion runs in FP64 for both types
    static constexpr size_t PACK_SMEM = (size_t)(2 * SB * SB + SB) * sizeof(Work);
};

// Packing pass of the above.  blockIdx.y: diagonal block.  blockIdx.x < COPY_GROUPS: workgroup
// (bi, chunk) negates and files up to PACK_CHUNK sub-blocks (bi, bj), bj < 4 (bi / 4), of sub-block row bi;
// blockIdx.x >= COPY_GROUPS: super-block S = blockIdx.x - COPY_GROUPS is inverted and its ten sub-blocks filed.
// Only the referenced triangle is read, and no diagonal when `unit`; rows past the end of a short
// block count as rows of the identity.
template <typename T, bool FORWARD>
__global__ void __launch_bounds__(256)
trsm_pack_inv_kernel(const T *__restrict__ A, int64_t lda, int n, bool teff, bool unit, T *__restrict__ pack) {
    typedef TrsmBlock<T> L;
    typedef Mma16<T> M;
    typedef typename L::Work W;
    constexpr int IB = L::IB, SB = L::SB;
    extern __shared__ __attribute__((aligned(16))) unsigned char pack_smem[];
    const int tid = threadIdx.x;
    const int i0 = blockIdx.y * L::NB;
    const int nb = n - i0 < L::NB ? n - i0 : L::NB;
    const T *Ablk = A + i0 + (int64_t)i0 * lda;
    T *out_blk = pack + (int64_t)blockIdx.y * L::PACK_REALS;
    auto coef = [&](int P, int Q) -> T {  // Q <= P < nb
        const int ip = FORWARD ? P : nb - 1 - P, iq = FORWARD ? Q : nb - 1 - Q;
        return teff ? Ablk[iq + (int64_t)ip * lda] : Ablk[ip + (int64_t)iq * lda];
    };
    if ((int)blockIdx.x < L::COPY_GROUPS) {
        constexpr int CHUNKS = L::NBLK / L::PACK_CHUNK;
        const int bi = blockIdx.x / CHUNKS, chunk = blockIdx.x % CHUNKS;
        if (bi * IB >= nb) return;
        const int below = (bi / L::SBR) * L::SBR;  // sub-block columns left of the row's super-block
        const int bj_lo = chunk * L::PACK_CHUNK;
        const int bj_hi = bj_lo + L::PACK_CHUNK < below ? bj_lo + L::PACK_CHUNK : below;
        T *out = out_blk + (int64_t)(bi * (bi + 1) / 2) * L::SUB_REALS;
        for (int e = bj_lo * IB * IB + tid; e < bj_hi * IB * IB; e += 256) {
            const int bj = e / (IB * IB), w = e % (IB * IB);
            const int lane = w / 4, c = w % 4;
            const int P = bi * IB + M::arow(lane % 16), Q = bj * IB + M::krow(lane / 16, c);
            out[bj * L::SUB_REALS + packed_at<T>(lane, c)] = (P < nb) ? -coef(P, Q) : (T)0;
        }
        return;
    }
    const int sb = blockIdx.x - L::COPY_GROUPS;
    const int P0 = sb * SB;
    if (P0 >= nb) return;
    W(*Ls)[SB] = reinterpret_cast<W(*)[SB]>(pack_smem);                       // the triangle, later A21 inv11
    W(*Iv)[SB] = reinterpret_cast<W(*)[SB]>(pack_smem + sizeof(W) * SB * SB);  // its inverse
    W *Rd = reinterpret_cast<W *>(pack_smem + 2 * sizeof(W) * SB * SB);        // reciprocals of the diagonal
    for (int e = tid; e < SB * SB; e += 256) {
        const int p = e / SB, q = e % SB;
        const int P = P0 + p, Q = P0 + q;
        W v = 0;
        if (p == q) v = (unit || P >= nb) ? (W)1 : (W)coef(P, P);
        else if (q < p && P < nb) v = (W)coef(P, Q);
        Ls[p][q] = v;
        Iv[p][q] = 0;
    }
    __syncthreads();
    if (tid < SB) Rd[tid] = (W)1 / Ls[tid][tid];
    __syncthreads();
    // the four 16 x 16 triangles on the diagonal, by substitution: thread (d, zc) solves L_dd z = e_zc
    if (tid < SB) {
        const int d = tid / IB, zc = tid % IB, o = d * IB;
        W z[IB];
#pragma unroll
        for (int p = 0; p < IB; ++p) {
            W acc = (p == zc) ? (W)1 : (W)0;
#pragma unroll
            for (int q = 0; q < IB; ++q)
                if (q < p) acc -= Ls[o + p][o + q] * z[q];
            z[p] = (p < zc) ? (W)0 : acc * Rd[o + p];
        }
#pragma unroll
        for (int p = 0; p < IB; ++p) Iv[o + p][o + zc] = z[p];
    }
    __syncthreads();
    // doubling: with inv11 (h x h at offset c0) and inv22 (h x h at c0 + h) known,
    //   T = A21 inv11 (into the place of A21), then inv21 = -inv22 T.
    // (The sums run over all h terms - the triangular factors hold their zeros - so that the loops
    // have fixed lengths and their LDS reads are issued back to back.)
    auto level = [&](auto hc) {
        constexpr int h = decltype(hc)::value;
        constexpr int PER = h / 8;  // all the A21 of one level: SB / (2h) pairs of h x h elements, h / 8 per thread
        W t[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int o = tid + 256 * u;
            const int pr = o / (h * h), i = (o % (h * h)) / h, j = o % h;
            const int c0 = pr * 2 * h, r0 = c0 + h;
            W acc = 0;
#pragma unroll
            for (int k = 0; k < h; ++k) acc += Ls[r0 + i][c0 + k] * Iv[c0 + k][c0 + j];
            t[u] = acc;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int o = tid + 256 * u;
            const int pr = o / (h * h), i = (o % (h * h)) / h, j = o % h;
            Ls[pr * 2 * h + h + i][pr * 2 * h + j] = t[u];
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int o = tid + 256 * u;
            const int pr = o / (h * h), i = (o % (h * h)) / h, j = o % h;
            const int c0 = pr * 2 * h, r0 = c0 + h;
            W acc = 0;
#pragma unroll
            for (int k = 0; k < h; ++k) acc += Iv[r0 + i][r0 + k] * Ls[r0 + k][c0 + j];
            t[u] = -acc;
        }
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int o = tid + 256 * u;
            const int pr = o / (h * h), i = (o % (h * h)) / h, j = o % h;
            Iv[pr * 2 * h + h + i][pr * 2 * h + j] = t[u];
        }
        __syncthreads();
    };
    level(IntC<16>{});
    level(IntC<32>{});
    static_assert(SB == 64, "two doubling levels");
    // the ten sub-blocks (4 sb + i, 4 sb + j), j <= i, in MFMA operand order
    for (int o = tid; o < 10 * IB * IB; o += 256) {
        const int blk = o / (IB * IB), w = o % (IB * IB);
        const int i = blk < 1 ? 0 : blk < 3 ? 1 : blk < 6 ? 2 : 3, j = blk - i * (i + 1) / 2;
        const int lane = w / 4, c = w % 4;
        const int r = sb * L::SBR + i, q = sb * L::SBR + j;
        out_blk[(int64_t)(r * (r + 1) / 2 + q) * L::SUB_REALS + packed_at<T>(lane, c)] =
            (T)Iv[i * IB + M::arow(lane % 16)][j * IB + M::krow(lane / 16, c)];
    }
}

template <typename T, bool RIGHT, bool FORWARD, int NBK>
__global__ void __launch_bounds__(TrsmBlock<T>::THREADS)
trsm_block_kernel(const T *__restrict__ packed, int nb, T alpha, T *__restrict__ Bblk, int64_t ldb, int nrhs) {
    typedef TrsmBlock<T> L;
    typedef T R;
    typedef Mma16<R> M;
    typedef typename M::Acc Acc;
    constexpr int IB = L::IB, WAVES = L::WAVES, RW = L::RW, SBR = L::SBR, NS = L::NS, CW = 16 * NBK;
    static_assert(WAVES == 2 * SBR && RW * WAVES * IB == L::NB, "two sets of SBR owners, RW rows each");
    constexpr int V = 16 / (int)sizeof(R);  // reals per 16 bytes
    constexpr int CH = 4 / V;               // 16-byte pieces of an accumulator block
    typedef R VT __attribute__((ext_vector_type(V)));
    // LDS: X of the last two steps (step S in half S % 2) and the Y that the owners of the coming step
    // exchange; one accumulator block per (sub-block row of the super-block, block of 16 right-hand
    // sides), in per-lane order.
    __shared__ __attribute__((aligned(16))) R Xb[2][SBR * NBK * 256];
    __shared__ __attribute__((aligned(16))) R Yb[SBR * NBK * 256];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int own_i = wave % SBR;  // the wavefront owns row own_i of the super-blocks SET, SET + 2, ... (SET = wave / SBR)
    const int g = lane >> 4, jj = lane & 15;
    const int64_t j0 = (int64_t)blockIdx.x * CW;
    const int nsteps = (nb + IB - 1) / IB;        // sub-block rows that exist
    const int nsuper = (nb + L::SB - 1) / L::SB;  // super-blocks that exist

    // The two sets of owners run different programs (their turns alternate), each in straight-line code:
    // the body is instantiated per set and a wavefront enters the one of its set.  Both instances execute
    // the same number of barriers.
    auto body = [&](auto setc) __attribute__((always_inline)) {
        constexpr int SET = decltype(setc)::value;
        // Row h of this wavefront: sub-block row (2h + set) SBR + own_i.  Its packed sub-blocks are consecutive.
        auto row_of = [&](int h) __attribute__((always_inline)) { return (2 * h + SET) * SBR + own_i; };
        // (Addresses are kept as a wavefront-uniform pointer plus a 32-bit lane offset, so that they live in
        // scalar registers.)
        const uint32_t lane_off = (uint32_t)lane * V;
        // Sub-blocks first .. first + 3 of row h (clamped to the row's own sub-blocks) into four register blocks.
        auto fetch4 = [&](int h, int first, R (&dst)[SBR][4]) __attribute__((always_inline)) {
            const int row = row_of(h);
            const R *rowp = packed + (int64_t)(row * (row + 1) / 2) * L::SUB_REALS;
    #pragma unroll
            for (int q = 0; q < SBR; ++q) {
                int sidx = first + q;
                sidx = sidx < 0 ? 0 : (sidx < row ? sidx : row);
                const R *src = rowp + sidx * L::SUB_REALS;
    #pragma unroll
                for (int c = 0; c < 4; c += V) {
                    const VT t = *reinterpret_cast<const VT *>(src + (c / V) * (64 * V) + lane_off);
    #pragma unroll
                    for (int x = 0; x < V; ++x) dst[q][c + x] = t[x];
                }
            }
        };
        // Coefficients in flight: for the wavefront's next turn as an owner the sub-blocks of its near update
        // (ecn) and of the inverse (eca); for its far updates one step's sub-blocks of the rows 1 .. 3 (row 0 of a
        // wavefront lies in super-block 0 or 1 and takes no far update).
        // (TWO_CRIT false: one set of registers for both - the inverse is then requested into the near update's
        // registers as soon as that update's MFMAs are issued, and the solve waits for it.)
        constexpr bool TWO_CRIT = true;
        R ecn[SBR][4], eca_own[TWO_CRIT ? SBR : 1][4], ef[RW - 1][SBR][4];
        R(&eca)[SBR][4] = *reinterpret_cast<R(*)[SBR][4]>(TWO_CRIT ? &eca_own[0] : &ecn[0]);
        // ---- right-hand sides into the accumulator layout (as in trsm_diag_kernel) ----
        Acc y[RW][NBK];
        auto mem_row = [&](int P) __attribute__((always_inline)) { return FORWARD ? P : nb - 1 - P; };
        auto at = [&](int P, int64_t j) __attribute__((always_inline)) -> int64_t {
            return RIGHT ? j + (int64_t)mem_row(P) * ldb : (int64_t)mem_row(P) + j * ldb;
        };
        constexpr bool ROWS4 = !RIGHT;
        typedef R rx4u_t __attribute__((ext_vector_type(4), aligned(sizeof(R))));
        // Requests in the order of need: the right-hand sides of row 0 (every wavefront's first turn as an owner),
        // that turn's coefficients, the other rows, the first far update's coefficients.
        auto load_rhs = [&](int h) __attribute__((always_inline)) {
    #pragma unroll
            for (int k = 0; k < NBK; ++k) {
                const int64_t j = j0 + 16 * k + jj;
                const int P0 = row_of(h) * IB + M::krow(g, 0);
                if (ROWS4 && P0 + 3 < nb && j < nrhs) {
                    if constexpr (ROWS4) {
                        const rx4u_t t = *reinterpret_cast<const rx4u_t *>(Bblk + (FORWARD ? at(P0, j) : at(P0 + 3, j)));
    #pragma unroll
                        for (int v = 0; v < 4; ++v) y[h][k][v] = alpha * t[FORWARD ? v : 3 - v];
                    }
                } else {
    #pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int P = P0 + v;
                        const bool have = P < nb && j < nrhs;
                        const T b = Bblk[have ? at(P, j) : 0];
                        y[h][k][v] = have ? alpha * b : (T)0;
                    }
                }
            }
        };
        load_rhs(0);
        // first turn: super-block `set`, row 0
        if constexpr (TWO_CRIT) {
            fetch4(0, (SET - 1) * SBR, ecn);
            fetch4(0, SET * SBR, eca);
        } else {
            fetch4(0, 0, ecn);  // set 0: its inverse; set 1: its near update with X_0
        }
    #pragma unroll
        for (int h = 1; h < RW; ++h) load_rhs(h);
    #pragma unroll
        for (int h = 1; h < RW; ++h) fetch4(h, 0, ef[h - 1]);
        auto store_row = [&](int h) __attribute__((always_inline)) {
    #pragma unroll
            for (int k = 0; k < NBK; ++k) {
                const int64_t j = j0 + 16 * k + jj;
                const int P0 = row_of(h) * IB + M::krow(g, 0);
                if (ROWS4 && P0 + 3 < nb && j < nrhs) {
                    if constexpr (ROWS4) {
                        rx4u_t t;
    #pragma unroll
                        for (int v = 0; v < 4; ++v) t[FORWARD ? v : 3 - v] = y[h][k][v];
                        *reinterpret_cast<rx4u_t *>(Bblk + (FORWARD ? at(P0, j) : at(P0 + 3, j))) = t;
                    }
                } else {
    #pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int P = P0 + v;
                        if (P < nb && j < nrhs) Bblk[at(P, j)] = y[h][k][v];
                    }
                }
            }
        };
        // An accumulator block in LDS: 16-byte pieces, each piece of all 64 lanes together.
        auto blk_put = [&](R *buf, int i, int k, const Acc &a) __attribute__((always_inline)) {
    #pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                VT t;
    #pragma unroll
                for (int x = 0; x < V; ++x) t[x] = a[ch * V + x];
                *reinterpret_cast<VT *>(buf + (((i * NBK + k) * CH + ch) * 64 + lane) * V) = t;
            }
        };
        auto blk_get = [&](const R *buf, int i, int k) __attribute__((always_inline)) -> Acc {
            Acc a;
    #pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                const VT t = *reinterpret_cast<const VT *>(buf + (((i * NBK + k) * CH + ch) * 64 + lane) * V);
    #pragma unroll
                for (int x = 0; x < V; ++x) a[ch * V + x] = t[x];
            }
            return a;
        };
        // out += E in for one sub-block E (this lane's values) and NBK blocks in MFMA "B" operand order
        auto block_mma = [&](const R (&ev)[4], const Acc (&in)[NBK], Acc (&out)[NBK]) {
    #pragma unroll
            for (int c = 0; c < 4; ++c)
    #pragma unroll
                for (int k = 0; k < NBK; ++k) out[k] = M::run(ev[c], in[k][c], out[k]);
        };
        // Far update with the X of step s (in half s % 2 of Xb): rows HMIN .. RW-1 of this wavefront take
        // y += (-L(row, 4s .. 4s+3)) X_s, the rows in the inner loop so that consecutive MFMAs are independent;
        // then each row's sub-blocks of step s + 1 are requested.
        auto far = [&](auto sc, auto hminc) __attribute__((always_inline)) {
            constexpr int s = decltype(sc)::value, HMIN = decltype(hminc)::value;
            if constexpr (HMIN < RW && s >= 0) {
                const R *X = Xb[s % 2];
    #pragma unroll
                for (int q = 0; q < SBR; ++q) {
                    Acc in[NBK];
    #pragma unroll
                    for (int k = 0; k < NBK; ++k) in[k] = blk_get(X, q, k);
    #pragma unroll
                    for (int c = 0; c < 4; ++c)
    #pragma unroll
                        for (int h = HMIN; h < RW; ++h) {
                            if (row_of(h) < nsteps) {
    #pragma unroll
                                for (int k = 0; k < NBK; ++k) y[h][k] = M::run(ef[h - 1][q][c], in[k][c], y[h][k]);
                            }
                        }
                }
                // (The requests for the next step's sub-blocks stay behind this step's MFMAs: hoisted above
                // them they would need a second set of registers.)
    #pragma unroll
                for (int h = HMIN; h < RW; ++h)
    #pragma unroll
                    for (int k = 0; k < NBK; ++k) asm volatile("" : "+v"(y[h][k]) : : "memory");
    #pragma unroll
                for (int h = HMIN; h < RW; ++h) fetch4(h, (s + 1) * SBR, ef[h - 1]);
            }
        };

        if constexpr (SET == 0) {  // owners of super-block 0 file their Y
    #pragma unroll
            for (int k = 0; k < NBK; ++k) blk_put(Yb, own_i, k, y[0][k]);
        }
        __syncthreads();
        // Step S, two halves with a barrier after each:
        //   first   owners of S (set S % 2, their row S / 2):  A  X = sum_{j <= i} Inv(i, j) Y_j, filed and stored
        //           the other set:                              far update with X_(S-1) on all its unsolved rows
        //   second  owners of S:                                far update with X_(S-1) on the rows beyond S + 1
        //           the other set (owners of S + 1):            N  near update of its row of S + 1 with X_S; Y filed
        // Every row thus takes the X of an earlier super-block of its own set's one half-step after it appears
        // and the X of the other set's three half-steps after, always in the same order.
        auto step = [&](auto Sc) __attribute__((always_inline)) {
            constexpr int S = decltype(Sc)::value;
            constexpr int HO = S / 2;        // the owners' row
            constexpr int HN = (S + 1) / 2;  // the row of S + 1 in the other set
            constexpr bool mine = SET == S % 2;
            if constexpr (mine) {
                if (row_of(HO) < nsteps) {
                    Acc x[NBK];
    #pragma unroll
                    for (int k = 0; k < NBK; ++k) x[k] = Acc{0, 0, 0, 0};
    #pragma unroll
                    for (int q = 0; q < SBR; ++q) {
                        if (q < own_i) {
                            Acc in[NBK];
    #pragma unroll
                            for (int k = 0; k < NBK; ++k) in[k] = blk_get(Yb, q, k);
                            block_mma(eca[q], in, x);
                        } else if (q == own_i) {
                            block_mma(eca[q], y[HO], x);
                        }
                    }
    #pragma unroll
                    for (int k = 0; k < NBK; ++k) {
                        y[HO][k] = x[k];
                        blk_put(Xb[S % 2], own_i, k, x[k]);
                    }
                    // X to memory now, while this wavefront has nothing to do until the barrier.  (All rows stored
                    // at the end of the kernel instead: 28.8 -> 30.7 us per FP64 leaf.)
                    store_row(HO);
                }
                // the coefficients of the next turn as an owner: super-block S + 2, row HO + 1
                if constexpr (HO + 1 < RW) {
    #pragma unroll
                    for (int k = 0; k < NBK; ++k) asm volatile("" : "+v"(y[HO][k]) : : "memory");
                    fetch4(HO + 1, (S + 1) * SBR, ecn);
                    if constexpr (TWO_CRIT) fetch4(HO + 1, (S + 2) * SBR, eca);
                }
            } else {
                far(IntC<S - 1>{}, IntC<(S + 1) / 2>{});
            }
            __syncthreads();
            if constexpr (mine) {
                far(IntC<S - 1>{}, IntC<S / 2 + 1>{});
            } else if constexpr (HN < RW && S + 1 < NS) {
                if (row_of(HN) < nsteps) {
    #pragma unroll
                    for (int q = 0; q < SBR; ++q) {
                        Acc in[NBK];
    #pragma unroll
                        for (int k = 0; k < NBK; ++k) in[k] = blk_get(Xb[S % 2], q, k);
                        block_mma(ecn[q], in, y[HN]);
                    }
                    if constexpr (!TWO_CRIT) {
    #pragma unroll
                        for (int k = 0; k < NBK; ++k) asm volatile("" : "+v"(y[HN][k]) : : "memory");
                        fetch4(HN, (S + 1) * SBR, ecn);
                    }
    #pragma unroll
                    for (int k = 0; k < NBK; ++k) blk_put(Yb, own_i, k, y[HN][k]);
                }
            }
            __syncthreads();
        };
        if (0 < nsuper) step(IntC<0>{});
        if (1 < nsuper) step(IntC<1>{});
        if (2 < nsuper) step(IntC<2>{});
        if (3 < nsuper) step(IntC<3>{});
        if (4 < nsuper) step(IntC<4>{});
        if (5 < nsuper) step(IntC<5>{});
        if (6 < nsuper) step(IntC<6>{});
        if (7 < nsuper) step(IntC<7>{});
    };
    if (wave / SBR == 0) body(IntC<0>{}); else body(IntC<1>{});
    static_assert(NS == 8, "one step call per super-block");
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
    bool inv_leaf;  // real types: the block solve with inverted 64 x 64 triangles (else substitution over 16-row sub-blocks)

    static T minus_one() { return el_scale_host(-1); }
    static T el_scale_host(int v) {
        if constexpr (Elem<T>::CPLX) return T{(R)v, (R)0};
        else return (T)v;
    }

    // Packs every diagonal block of the triangle (one launch per call).
    hipError_t prepare() {
        const int n = right ? N : M;
        const int nblk = (n + NBL - 1) / NBL;
        void *wv = nullptr;
        if constexpr (!Elem<T>::CPLX) {
            if (!inv_leaf) return prepare_substitution(n, nblk);
            typedef TrsmBlock<T> L;
            hipError_t we = workspace_get(stream, (size_t)nblk * L::PACK_REALS * sizeof(R), 2, &wv);
            if (we != hipSuccess) return we;
            pack = (const R *)wv;
            void (*fn)(const T *, int64_t, int, bool, bool, T *) =
                forward ? trsm_pack_inv_kernel<T, true> : trsm_pack_inv_kernel<T, false>;
            hipError_t e = ensure_dynamic_lds((const void *)fn, L::PACK_SMEM);
            if (e != hipSuccess) return e;
            dispatch_record().launches++;
            return launch_kernel(fn, dim3(L::COPY_GROUPS + L::NS, nblk), dim3(256), L::PACK_SMEM, stream, A, lda, n, teff, unit,
                                 (T *)wv);
        } else {
            return prepare_substitution(n, nblk);
        }
    }
    hipError_t prepare_substitution(int n, int nblk) {
        typedef TrsmLeaf<T> L;
        void *wv = nullptr;
        hipError_t we = workspace_get(stream, (size_t)nblk * L::PACK_REALS * sizeof(R), 2, &wv);
        if (we != hipSuccess) return we;
        R *w = (R *)wv;
        pack = w;
        dispatch_record().launches++;
        if (forward)
            return launch_kernel(trsm_pack_kernel<T, true>, dim3(L::NBLK * (L::NBLK / L::PACK_CHUNK), nblk), dim3(256), 0, stream, A, lda, n, teff,
                                 conj, unit, w);
        return launch_kernel(trsm_pack_kernel<T, false>, dim3(L::NBLK * (L::NBLK / L::PACK_CHUNK), nblk), dim3(256), 0, stream, A, lda, n, teff,
                             conj, unit, w);
    }

    // Real types: the block solve with inverted 64 x 64 triangles, NBK blocks of 16 right-hand sides per workgroup.
    template <bool RIGHT, int NBK> hipError_t block_side(int i0, int nb, T alpha) {
        if constexpr (!Elem<T>::CPLX) {
            typedef TrsmBlock<T> L;
            const int nrhs = RIGHT ? M : N;
            T *Bblk = RIGHT ? B + (int64_t)i0 * ldb : B + i0;
            const T *packed = pack + (int64_t)(i0 / NBL) * L::PACK_REALS;
            void (*fn)(const T *, int, T, T *, int64_t, int) =
                forward ? trsm_block_kernel<T, RIGHT, true, NBK> : trsm_block_kernel<T, RIGHT, false, NBK>;
            dim3 grid((unsigned)((nrhs + 16 * NBK - 1) / (16 * NBK))), block(L::THREADS);
            dispatch_record().launches++;
            return launch_kernel(fn, grid, block, 0, stream, packed, nb, alpha, Bblk, ldb, nrhs);
        } else {
            return hipErrorNotSupported;
        }
    }

    template <bool RIGHT, bool WIDE> hipError_t leaf_side(int i0, int nb, T alpha) {
        typedef TrsmLeaf<T, RIGHT, WIDE> L;
        const int nrhs = RIGHT ? M : N;
        T *Bblk = RIGHT ? B + (int64_t)i0 * ldb : B + i0;
        const R *packed = pack + (int64_t)(i0 / NBL) * L::PACK_REALS;
        void (*fn)(const R *, int, T, T *, int64_t, int, int) =
            forward ? trsm_diag_kernel<T, RIGHT, true, WIDE> : trsm_diag_kernel<T, RIGHT, false, WIDE>;
        if (L::SMEM > 64 * 1024) {
            hipError_t e = ensure_dynamic_lds((const void *)fn, L::SMEM);
            if (e != hipSuccess) return e;
        }
        dim3 grid((unsigned)((nrhs + L::CW - 1) / L::CW)), block(L::THREADS);
        dispatch_record().launches++;
        // (2^22 polls: far beyond any wait of a leaf that works, short enough that a mistake ends in seconds)
        const int poll_limit = knobs().trsm_poll_limit > 0 ? knobs().trsm_poll_limit : (1 << 22);
        return launch_kernel(fn, grid, block, L::SMEM, stream, packed, nb, alpha, Bblk, ldb, nrhs, poll_limit);
    }
    // Right-hand sides per workgroup.  Real types: 16, or 32 (each sub-block of coefficients is then
    // used twice) where that makes the launch shorter, or for FP32 with side = right, whose right-hand sides
    // are rows of B: 16 floats are too short a run of memory.  A leaf kernel has a CU to itself and lasts
    // about as long whatever the number of workgroups in its round, so a launch costs rounds x time per
    // round: FP64 30 us with 16 and 52 us with 32 right-hand sides per workgroup, FP32 21 and 34.  One round
    // of 32 beats two of 16 (4097 .. 8192 right-hand sides), two rounds of 32 lose against three of 16
    // (8193 .. 12288: DTRSM 9216 64.0 -> 66.6 TFLOP/s), and so on.
    static bool wide_leaf_pays(int nrhs) {
        const int64_t rounds16 = ((int64_t)(nrhs + 15) / 16 + 255) / 256, rounds32 = ((int64_t)(nrhs + 31) / 32 + 255) / 256;
        const double wide_over_narrow = sizeof(R) == 8 ? 52.0 / 30.0 : 34.0 / 21.0;
        return (double)rounds32 * wide_over_narrow < (double)rounds16;
    }
    hipError_t leaf(int i0, int nb, T alpha) {
        const int nrhs = right ? M : N;
        if constexpr (!Elem<T>::CPLX) {
            if (!inv_leaf) {
                bool wide = wide_leaf_pays(nrhs) || (right && sizeof(R) == 4);
                if (knobs().trsm_wide >= 0) wide = knobs().trsm_wide != 0;
                if (wide) return right ? leaf_side<true, true>(i0, nb, alpha) : leaf_side<false, true>(i0, nb, alpha);
                return right ? leaf_side<true, false>(i0, nb, alpha) : leaf_side<false, false>(i0, nb, alpha);
            }
            const bool two = sizeof(R) == 4 && (nrhs > 256 * 16 || right);
            if constexpr (sizeof(R) == 4) {
                if (two) return right ? block_side<true, 2>(i0, nb, alpha) : block_side<false, 2>(i0, nb, alpha);
            }
            return right ? block_side<true, 1>(i0, nb, alpha) : block_side<false, 1>(i0, nb, alpha);
        } else {
            return right ? leaf_side<true, false>(i0, nb, alpha) : leaf_side<false, false>(i0, nb, alpha);
        }
    }

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
    d.inv_leaf = !Elem<T>::CPLX && knobs().trsm_leaf != 0;
    hipError_t e = d.prepare();
    if (e != hipSuccess) return e;
    return d.solve(0, right ? N : M, alpha);
}

hipError_t trsm_poll_timeouts_read(unsigned int *count, bool reset) {
    unsigned int v = 0;
    hipError_t e = hipMemcpyFromSymbol(&v, HIP_SYMBOL(trsm_poll_timeouts), sizeof v);
    if (e != hipSuccess) return e;
    if (count) *count = v;
    if (reset && v != 0) {
        const unsigned int zero = 0;
        e = hipMemcpyToSymbol(HIP_SYMBOL(trsm_poll_timeouts), &zero, sizeof zero);
    }
    return e;
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
