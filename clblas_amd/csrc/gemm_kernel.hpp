// MFMA GEMM kernel for gfx950 (CDNA4): FP32, FP64 and their complex counterparts, all
// transpose / conjugate combinations; the TRI variants also serve SYRK, SYR2K, HERK, HER2K,
// TRMM, SYMM and HEMM.
//
// Computes (column-major, after the host has folded row-major calls)
//     C(m,n) <- alpha * sum_k opA(m,k) * opB(k,n) + beta * C(m,n)
// which is the contract of the reference's AutoGemm kernels
// (src/library/blas/AutoGemm/KernelOpenCL.py:311-452): one accumulator per C element,
// alpha/beta applied once in the epilogue, beta == 0 never reads C.
//
// Structure of one workgroup (BM x BN macro tile of C, waves arranged WAVES_M x WAVES_N):
//   * Panels of depth BK travel HBM -> LDS without passing through registers wherever the
//     LDS image is a plain copy of memory: `buffer_load_dwordx4 ... lds` writes each wave's
//     64 x 16 bytes to consecutive LDS addresses.  That covers operands contiguous along the
//     tile edge (As[k][m], Bs[k][n]) and k-contiguous panels, kept as As[m][k] / Bs[n][k]
//     with their 16-byte slots XOR-swizzled by the row so that fragment reads stay
//     bank-conflict free.  Each lane of such a load names its own source address, so the rows
//     of As[m][k] are stored block by block (all rows of MFMA block 0, then block 1, ...)
//     while a lane still owns VM consecutive rows of C for its 16-byte stores.
//   * Two LDS stages; the loads of panel p+1 are issued during panel p,
//     one at a time behind the MFMAs of its first steps (in front of them they cost several
//     per cent), and one barrier per panel publishes the next stage.  All but the last few
//     panels run straight-line code, two panels per loop trip.  Buffer descriptors are
//     re-based every panel and sized to the exact footprint of the operand, so the hardware
//     range check turns every access past the end of the matrix into a zero (also on the
//     LDS path): no extra launch and no per-element branch is needed for M/N remainders or
//     for the K remainder of tile-edge-contiguous operands; the K remainder of a
//     k-contiguous panel is real memory (the next column) and is cleared in LDS before use.
//   * Each wave owns a WM x WN sub-tile as TM x TN MFMA blocks
//     (v_mfma_f32_32x32x2_f32 / v_mfma_f64_16x16x4_f64).  The MFMA "B" operand carries the
//     A matrix and the "A" operand carries the B matrix, so that the lane index of the
//     result runs along m, the contiguous direction of C.  The m coordinates are
//     interleaved between blocks so that one 16-byte LDS read feeds VM blocks and one
//     16-byte global store writes VM consecutive rows of C.
//   * Complex types (interleaved re/im, src/library/blas/AutoGemm/KernelOpenCL.py:106-165)
//     run on the same real MFMAs with the same lane <-> k mapping: a lane reads whole
//     (re, im) elements and every block of C keeps two accumulators,
//         Re += ar*br,  Re += ai*(-bi),  Im += ar*bi,  Im += ai*br
//     - four MFMAs per block and step, all of their flops useful, the only extra work one
//     sign flip per B element.  Conjugation moves that flip to br and/or negates Im at the end.
//   * Kernels instantiated with TRI = true additionally honour triangular structure (only a
//     triangle of C exists; an operand is triangular: its zero half is skipped and the
//     diagonal band is masked in LDS) and the sliced tail (the tiles of a partly filled last
//     round are cut into K ranges); see GemmParams.  The plain instantiations carry none of it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "internal.h"

namespace cba {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elem { typedef T Real; static constexpr bool CPLX = false; };
template <typename R> struct Elem<Cx<R>> { typedef R Real; static constexpr bool CPLX = true; };

// Element arithmetic shared by the kernels.  The complex forms follow the operation order
// of the reference's TYPE_MAD / TYPE_MAD_WRITE macros (KernelOpenCL.py:106-165).
template <typename T> __host__ __device__ __forceinline__ T el_one() { return (T)1; }
template <> __host__ __device__ __forceinline__ Cx<float> el_one<Cx<float>>() { return Cx<float>{1.f, 0.f}; }
template <> __host__ __device__ __forceinline__ Cx<double> el_one<Cx<double>>() { return Cx<double>{1.0, 0.0}; }
__host__ __device__ __forceinline__ bool el_is_zero(float x) { return x == 0.f; }
__host__ __device__ __forceinline__ bool el_is_zero(double x) { return x == 0.0; }
template <typename R> __host__ __device__ __forceinline__ bool el_is_zero(Cx<R> x) { return x.re == (R)0 && x.im == (R)0; }
__device__ __forceinline__ float el_add(float a, float b) { return a + b; }
__device__ __forceinline__ double el_add(double a, double b) { return a + b; }
template <typename R> __device__ __forceinline__ Cx<R> el_add(Cx<R> a, Cx<R> b) { return Cx<R>{a.re + b.re, a.im + b.im}; }
// alpha * x
__device__ __forceinline__ float el_scale(float alpha, float x) { return alpha * x; }
__device__ __forceinline__ double el_scale(double alpha, double x) { return alpha * x; }
template <typename R> __device__ __forceinline__ Cx<R> el_scale(Cx<R> alpha, Cx<R> x) {
    R re = x.re * alpha.re;
    re = fma(-alpha.im, x.im, re);
    R im = x.im * alpha.re;
    im = fma(alpha.im, x.re, im);
    return Cx<R>{re, im};
}
// x with its imaginary part dropped (x itself for real types)
__device__ __forceinline__ float el_real_only(float x) { return x; }
__device__ __forceinline__ double el_real_only(double x) { return x; }
template <typename R> __device__ __forceinline__ Cx<R> el_real_only(Cx<R> x) { return Cx<R>{x.re, (R)0}; }
// r + beta * c
__device__ __forceinline__ float el_axpy(float beta, float c, float r) { return r + beta * c; }
__device__ __forceinline__ double el_axpy(double beta, double c, double r) { return r + beta * c; }
template <typename R> __device__ __forceinline__ Cx<R> el_axpy(Cx<R> beta, Cx<R> c, Cx<R> r) {
    R re = fma(beta.re, c.re, r.re);
    re = fma(-beta.im, c.im, re);
    R im = fma(beta.im, c.re, r.im);
    im = fma(beta.re, c.im, im);
    return Cx<R>{re, im};
}
// s + op(a) * op(b), op = conjugate where flagged (flags are ignored for real types)
__device__ __forceinline__ float el_mad(float a, bool, float b, bool, float s) { return fmaf(a, b, s); }
__device__ __forceinline__ double el_mad(double a, bool, double b, bool, double s) { return fma(a, b, s); }
template <typename R> __device__ __forceinline__ Cx<R> el_mad(Cx<R> a, bool ca, Cx<R> b, bool cb, Cx<R> s) {
    const R ai = ca ? -a.im : a.im, bi = cb ? -b.im : b.im;
    R re = fma(a.re, b.re, s.re);
    re = fma(-ai, bi, re);
    R im = fma(a.re, bi, s.im);
    im = fma(ai, b.re, im);
    return Cx<R>{re, im};
}

// Vector of N elements of T: `type` with natural alignment (LDS), `utype` with only element
// alignment (global C may be misaligned by offC / ldc); get/set address element e.
template <typename T, int N> struct Vec;
template <> struct Vec<float, 1> {
    typedef float type; typedef float utype;
    template <typename V> static __device__ __forceinline__ float get(const V &v, int) { return v; }
    template <typename V> static __device__ __forceinline__ void set(V &v, int, float x) { v = x; }
};
template <> struct Vec<double, 1> {
    typedef double type; typedef double utype;
    template <typename V> static __device__ __forceinline__ double get(const V &v, int) { return v; }
    template <typename V> static __device__ __forceinline__ void set(V &v, int, double x) { v = x; }
};
#define CBA_REAL_VEC(T, N, BASE, ALIGN)                                                          \
    template <> struct Vec<T, N> {                                                               \
        typedef BASE type;                                                                       \
        typedef T utype __attribute__((ext_vector_type(N), aligned(ALIGN)));                     \
        template <typename V> static __device__ __forceinline__ T get(const V &v, int e) { return v[e]; }   \
        template <typename V> static __device__ __forceinline__ void set(V &v, int e, T x) { v[e] = x; }    \
    };
CBA_REAL_VEC(float, 2, f32x2, 4)
CBA_REAL_VEC(float, 4, f32x4, 4)
CBA_REAL_VEC(double, 2, f64x2, 8)
#undef CBA_REAL_VEC
#define CBA_CPLX_VEC(R, N, BASE, ALIGN)                                                          \
    template <> struct Vec<Cx<R>, N> {                                                           \
        typedef BASE type;                                                                       \
        typedef R utype __attribute__((ext_vector_type(2 * N), aligned(ALIGN)));                 \
        template <typename V> static __device__ __forceinline__ Cx<R> get(const V &v, int e) {   \
            return Cx<R>{v[2 * e], v[2 * e + 1]};                                                \
        }                                                                                        \
        template <typename V> static __device__ __forceinline__ void set(V &v, int e, Cx<R> x) { \
            v[2 * e] = x.re;                                                                     \
            v[2 * e + 1] = x.im;                                                                 \
        }                                                                                        \
    };
CBA_CPLX_VEC(float, 1, f32x2, 4)
CBA_CPLX_VEC(float, 2, f32x4, 4)
CBA_CPLX_VEC(double, 1, f64x2, 8)
#undef CBA_CPLX_VEC

template <typename T> struct Mma;

template <> struct Mma<float> {
    static constexpr int MB = 32;    // block edge
    static constexpr int KS = 2;     // k per instruction
    static constexpr int NACC = 16;  // accumulator elements per lane
    typedef f32x16 Acc;
    static __device__ __forceinline__ Acc run(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // Row of the 32x32 result held in accumulator element v of lane `lane`.
    static __device__ __forceinline__ int row(int v, int lane) {
        return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
    }
};

template <> struct Mma<double> {
    static constexpr int MB = 16;
    static constexpr int KS = 4;
    static constexpr int NACC = 4;
    typedef f64x4 Acc;
    static __device__ __forceinline__ Acc run(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int v, int lane) {
        return (lane >> 4) + 4 * v;
    }
};

// FP32 on the 16x16x4 instruction (the operand and result layout of the FP64 one, but for the rows of a
// result column: four consecutive ones per lane): for wave tiles of 16 rows or columns, i.e. workgroups of
// four wavefronts on tiles below 64x64.
struct MmaF32Small {
    static constexpr int MB = 16;
    static constexpr int KS = 4;
    static constexpr int NACC = 4;
    typedef f32x4 Acc;
    static __device__ __forceinline__ Acc run(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int v, int lane) {
        return 4 * (lane >> 4) + v;
    }
};

// The instruction for a wave tile of WM x WN elements of real type R.
template <typename R, int WM, int WN> struct MmaFor { typedef Mma<R> type; };
template <int WM, int WN> struct MmaFor<float, WM, WN> {
    typedef typename std::conditional<WM % 32 == 0 && WN % 32 == 0, Mma<float>, MmaF32Small>::type type;
};

template <typename T> struct GemmParams {
    const T *A;
    const T *B;
    T *C;
    int64_t lda, ldb, ldc;
    int64_t a_bytes, b_bytes;  // exact footprint of op-A / op-B storage, from A / B
    int M, N, K;
    int conj_a, conj_b;  // complex types: conjugate op-A / op-B elements
    T alpha, beta;
    int tiles_m, tiles_n;
    int group_m;      // tile rows walked together (L2 locality)
    int xcd_remap;    // 1: give each XCD a contiguous chunk of the tile list
    int stagger;      // 1: every other workgroup of the first round starts late (see the kernel)
    int k_per_split;  // multiple of BK; >= K when the K loop is not split
    T *ws;            // split-K partial sums: ws[split * ws_slice + n * ws_ld + m]
    int64_t ws_ld, ws_slice;
    // Triangular structure (kernels built with TRI only; all zero otherwise).
    //   tri_c: store only the lower (1: m >= n) or upper (2: m <= n) triangle of C; tiles
    //          wholly outside it are not enumerated at all (grid = number of active tiles).
    //   tri_a / tri_b: op(A)(m,k) / op(B)(k,n) is triangular: elements with k > x (1) or
    //          k < x (2), x = m resp. n, count as zero whatever memory holds; unit_* = 1: the
    //          diagonal k == x counts as one, 2: as zero, 3: as its real part.  Panels outside
    //          the triangle are skipped.
    //   herm_c (with tri_c, complex types): the diagonal of C is read and stored with a zero
    //          imaginary part.
    //   rev_m / rev_n: walk the tile rows / columns from the far end (longest tiles first).
    int tri_c, tri_a, tri_b, unit_a, unit_b, rev_m, rev_n, herm_c;
    // Sliced tail (TRI kernels only): the last tiles of the list - those of the final, partly
    // filled round of 256 CUs - are each cut into `tail_slices` K ranges of `tail_kps`, so that
    // the round lasts 1/tail_slices as long.  Workgroup ids from `tail_first` on are slices
    // (tile tail_first + u / tail_slices, slice u % tail_slices); slice u stores its partial
    // tile to ws + u * BM * BN (tile-local, pitch BM) and tail_reduce_kernel finishes C.
    int tail_first, tail_slices, tail_kps;
};

// Tile row / column of entry `tile` of the tile list (bm x bn tiles).  Full grid: groups of
// `group_m` tile rows, column by column inside a group, so that concurrently running
// workgroups of one XCD share A and B panels in that XCD's L2.  With tri_c only the tiles that
// touch the stored triangle exist: row r holds the columns [0, last] (lower) or
// [first, tiles_n) (upper); they are walked the same way and the walk is replayed here until
// `tile` is reached.
template <typename T>
static __device__ __forceinline__ void tile_coords(const GemmParams<T> &p, bool tri, int bm, int bn, int tile, int &tm,
                                                   int &tn) {
    if (tri && p.tri_c) {
        tm = 0;
        tn = 0;
        bool found = false;
        for (int r0 = 0; r0 < p.tiles_m && !found; r0 += p.group_m) {
            const int r1 = r0 + p.group_m < p.tiles_m ? r0 + p.group_m : p.tiles_m;
            int in_group = 0;
            for (int r = r0; r < r1; ++r) {
                if (p.tri_c == 1) {
                    const int last = (r * bm + bm - 1) / bn;
                    in_group += last + 1 < p.tiles_n ? last + 1 : p.tiles_n;
                } else {
                    const int first = (r * bm) / bn;
                    in_group += first < p.tiles_n ? p.tiles_n - first : 0;
                }
            }
            if (tile >= in_group) { tile -= in_group; continue; }
            for (int c = 0; c < p.tiles_n; ++c) {
                int lo = r0, hi = r1;  // rows [lo, hi) of the group hold column c
                if (p.tri_c == 1) {
                    const int need = c * bn - bm + 1;  // first row index that reaches column c
                    const int rmin = need <= 0 ? 0 : (need + bm - 1) / bm;
                    lo = rmin > r0 ? rmin : r0;
                } else {
                    const int rmax = (c * bn + bn - 1) / bm;
                    hi = rmax + 1 < r1 ? rmax + 1 : r1;
                }
                const int cnt = hi > lo ? hi - lo : 0;
                if (tile < cnt) { tm = lo + tile; tn = c; found = true; break; }
                tile -= cnt;
            }
        }
    } else {
        const int per_group = p.group_m * p.tiles_n;
        const int grp = tile / per_group;
        const int first_m = grp * p.group_m;
        const int gm = (p.tiles_m - first_m) < p.group_m ? (p.tiles_m - first_m) : p.group_m;
        const int r = tile - grp * per_group;
        tm = first_m + r % gm;
        tn = r / gm;
        if (tri && p.rev_m) tm = p.tiles_m - 1 - tm;
        if (tri && p.rev_n) tn = p.tiles_n - 1 - tn;
    }
}

static __device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, int64_t bytes_left) {
    // Descriptors address at most 2 GiB from their base; tiles are re-based so that every
    // legitimate offset is below that.  A non-positive remainder yields an empty buffer.
    uint32_t n = bytes_left <= 0 ? 0u : (bytes_left > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)bytes_left);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)n, 0x00020000);
}

typedef __attribute__((address_space(3))) void lds_void_t;

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4, lgkmcnt 11:8; the other counters are left at "don't wait").
#define CBA_VMCNT_ONLY(n) ((((n) & 0xf) | ((((n) >> 4) & 0x3) << 14) | (0x7 << 4) | (0xf << 8)))

// How an operand panel gets from memory into LDS (always `buffer_load_dwordx4 ... lds`).
//   LM_DMA_X: memory contiguous along the tile edge x; LDS image [k][x], pitch BX.
//   LM_DMA_K: memory contiguous along k; LDS image [x'][k], pitch BK, 16-byte slots of row x'
//             stored at slot ^ swz(x').  Row x' of the image holds tile row perm(x'): with
//             interleave IL and block edge MBLK, image rows [e*MBLK, (e+1)*MBLK) of every
//             span of IL*MBLK rows hold the tile rows j*IL + e (IL == 1: identity).
enum LoadMode { LM_DMA_X = 0, LM_DMA_K = 1 };

// Where a panel is read from: the operand's memory from the panel's first element on.  The plain
// loaders turn it into one buffer descriptor per panel; the WIDE loaders keep pointer and length
// and make a descriptor per row.
struct PanelSrc {
    __amdgpu_buffer_rsrc_t rsrc;  // the whole remainder from `base` on (what the plain loaders use)
    const void *base;
    int64_t bytes_left;
    __device__ __forceinline__ PanelSrc() : base(nullptr), bytes_left(0) {}
    __device__ __forceinline__ PanelSrc(const void *b, int64_t n) : rsrc(make_rsrc(b, n)), base(b), bytes_left(n) {}
};

// WIDE: for leading dimensions so large that the rows of a panel are further apart than the 32-bit
// offset of a buffer load reaches (2 GiB).  Every row of the panel then gets its own descriptor,
// based at the row's first element, and the lanes that hold other rows sit the load out; the
// offsets inside a row stay below the row's length in the panel (at most 1 KiB).  One load
// instruction per row instead of one per 64 lanes: slower, and only instantiated for the smallest
// tile of each type, but there is no leading dimension it cannot serve.
// GRP: lanes that read one k row together in a fragment read (the block edge of the MFMA: 32, or 16).
template <typename T, int BX, int BK, int NT, int MODE, int IL = 1, int MBLK = 1, bool WIDE = false, int GRP = 32> struct PanelLoader {
    static constexpr int VEC = 16 / (int)sizeof(T);
    static constexpr int NVEC = BX * BK / VEC;
    static constexpr int PER = NVEC / NT;  // 16-byte vectors per thread = wave-wide loads per wave
    static_assert(NVEC % NT == 0 && PER >= 1, "panel does not divide over the workgroup");
    static constexpr int NW = NT / 64;
    static constexpr int CHUNK = 64 * VEC;  // elements written by one wave-wide LDS load (1 KiB)
    // LM_DMA_X: every 1 KiB chunk (CHUNK / BX rows of the [k][x] image) is followed by a small
    // gap, sized so that the rows read together by the lane groups of one fragment read
    // (VEC rows apart) start 64 bytes = 16 banks apart.
    static constexpr int ROWS_PER_CHUNK = CHUNK / BX > 0 ? CHUNK / BX : 1;
    static constexpr int CHUNKS_APART = VEC / ROWS_PER_CHUNK > 0 ? VEC / ROWS_PER_CHUNK : 1;
    // That is for the 32-lane groups of the FP32 MFMAs (512 contiguous bytes per group).  The
    // FP64 MFMAs read in 16-lane groups of 256 bytes, and those are conflict-free exactly when
    // all groups start in the same bank (measured: any stagger costs half of the LDS cycles),
    // which the unpadded image gives (rows are multiples of 256 bytes apart).
    static constexpr bool FP64_GROUPS = sizeof(typename Elem<T>::Real) == 8;
    // FP32 and complex FP32 on the 16x16x4 MFMA: four groups of 16 lanes read four rows VEC apart.  Measured
    // (SQ_LDS_BANK_CONFLICT over SQ_LDS_IDX_ACTIVE, 19-50 % with the layout of the 32-lane groups, 0 % with this):
    // with 16 bytes per lane a group fills a pass by itself and, as for FP64, all groups start in the same bank (no
    // gap); with 8 or 4 bytes per lane two groups are read together and have to lie next to each other, one group's
    // bytes (16 lanes) apart.  Rows VEC apart in different chunks: the gap after a chunk does it.  Rows VEC apart in
    // the same chunk (panels 32 wide, a row being two groups long): every other set of VEC rows is stored with its
    // two halves exchanged - the loads name their source freely.
    static constexpr bool SMALL_GROUPS = GRP == 16 && !FP64_GROUPS && MODE == LM_DMA_X;
    static constexpr int LANE_BYTES = IL * (int)sizeof(T);
    static constexpr int GROUP_ELEMS = 16 * IL;
    static constexpr bool NEED_STAGGER = SMALL_GROUPS && LANE_BYTES < 16;
    static constexpr bool FLIP_HALVES = NEED_STAGGER && ROWS_PER_CHUNK > VEC;
    static_assert(!FLIP_HALVES || (BX == 2 * GROUP_ELEMS && !WIDE), "exchanged halves: a row is two groups long");
    static constexpr int CHUNK_PAD =
        MODE != LM_DMA_X || FP64_GROUPS ? 0
        : SMALL_GROUPS ? ((NEED_STAGGER && !FLIP_HALVES) ? GROUP_ELEMS / CHUNKS_APART : 0)
                       : (64 / (int)sizeof(T)) / CHUNKS_APART;  // elements
    static constexpr int CHUNK_PITCH = CHUNK + CHUNK_PAD;
    static constexpr int LDS_PITCH = MODE == LM_DMA_X ? BX : BK;
    static constexpr int LDS_ELEMS = (NVEC / 64) * CHUNK_PITCH;
    // LM_DMA_X: column of the image that holds column x of k row k (and the other way round).
    static __device__ __forceinline__ int image_col(int k, int x) {
        return FLIP_HALVES ? x ^ (((k / VEC) & 1) * GROUP_ELEMS) : x;
    }
    // LM_DMA_X: LDS element offset of image element (k, x).
    static __device__ __forceinline__ int lds_at(int k, int x) {
        const int e = k * BX + image_col(k, x);
        return e + (e / CHUNK) * CHUNK_PAD;
    }
    // LM_DMA_K swizzle: S slots per row; rows x and x + 16/S start in the same bank.
    static constexpr int S = BK / VEC;
    static_assert(MODE != LM_DMA_K || (S <= 16 && 16 % S == 0), "swizzle needs S | 16");
    static_assert(MODE != LM_DMA_K || BX % (IL * MBLK) == 0, "row interleave must tile the panel");
    static __device__ __forceinline__ int swz(int x) { return (x / (16 / S)) % S; }
    // LM_DMA_K: tile row held by image row x.
    static __device__ __forceinline__ int perm(int x) {
        if (IL == 1) return x;
        const int span = IL * MBLK, r = x % span;
        return (x / span) * span + (r % MBLK) * IL + r / MBLK;
    }

    // Rows (of stride ld) that one wave-wide load covers.
    static constexpr int ROWS_PER_LOAD = MODE == LM_DMA_X ? (CHUNK / BX > 0 ? CHUNK / BX : 1) : 64 / S;
    static_assert(!WIDE || MODE != LM_DMA_X || BX <= CHUNK, "WIDE: a row of the [k][x] image must not exceed one load");

    uint32_t voff[PER];  // plain: byte offset of this lane's 16 bytes from the panel's first element; WIDE: from its row's
    int64_t ld_bytes;    // WIDE only
    int my_row;          // WIDE only: which of the ROWS_PER_LOAD rows of a load this lane holds

    __device__ __forceinline__ void init(int tid, int64_t ld) {
        const int lane = tid & 63, wave = tid >> 6;
        ld_bytes = ld * (int64_t)sizeof(T);
        my_row = 0;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            if (MODE == LM_DMA_X) {
                const int e = (wave + i * NW) * CHUNK + lane * VEC;  // element index in the [k][x] image
                const int k = e / BX, x = image_col(k, e % BX);
                if (WIDE) {
                    voff[i] = (uint32_t)(x * (int)sizeof(T));
                    my_row = k - ((wave + i * NW) * CHUNK) / BX;  // the same for every i
                } else {
                    voff[i] = (uint32_t)(((int64_t)k * ld + x) * (int64_t)sizeof(T));
                }
            } else {
                const int x = (wave + i * NW) * (64 / S) + lane / S;
                const int slot = (lane % S) ^ swz(x);  // logical slot stored in this lane's place
                if (WIDE) {
                    voff[i] = (uint32_t)(slot * VEC * (int)sizeof(T));
                    my_row = lane / S;
                } else {
                    voff[i] = (uint32_t)(((int64_t)perm(x) * ld + slot * VEC) * (int64_t)sizeof(T));
                }
            }
        }
    }

    // WIDE: row (in units of ld from the panel's first element) that row r of load i of wave `wave_u` holds.
    static __device__ __forceinline__ int wide_row(int wave_u, int i, int r) {
        if (MODE == LM_DMA_X) return ((wave_u + i * NW) * CHUNK) / BX + r;
        return perm((wave_u + i * NW) * (64 / S) + r);
    }

    // Starts the transfer of one panel.  base: first element of the panel; bytes_left:
    // footprint bytes from `base` on; lds: this operand's image in the receiving stage.
    __device__ __forceinline__ void issue(const T *base, int64_t bytes_left, T *lds, int wave_u) const {
        const PanelSrc src(base, bytes_left);
#pragma unroll
        for (int i = 0; i < PER; ++i) issue_one(src, lds, wave_u, i);
    }

    // One of the PER wave-wide loads of a panel.
    __device__ __forceinline__ void issue_one(const PanelSrc &src, T *lds, int wave_u, int i) const {
        lds_void_t *dst = (lds_void_t *)(lds + (wave_u + i * NW) * CHUNK_PITCH);
        if (!WIDE) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src.rsrc, dst, 16, (int)voff[i], 0, 0, 0);
        } else {
#pragma nounroll  // (unrolled, the descriptors of all rows are kept live at once and registers spill)
            for (int r = 0; r < ROWS_PER_LOAD; ++r) {
                const int64_t off = (int64_t)wide_row(wave_u, i, r) * ld_bytes;
                __amdgpu_buffer_rsrc_t rs = make_rsrc((const char *)src.base + off, src.bytes_left - off);
                if (my_row == r) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, (int)voff[i], 0, 0, 0);
            }
        }
    }

    // Triangular operand: in the 16 bytes each of this thread's loads delivered, zeroes the
    // elements outside the triangle (mode 1 keeps k <= x, mode 2 keeps k >= x; x0, k0: global
    // coordinates of the panel's first element); unit == 1 sets the diagonal to one, 2 to zero.
    // Call after waiting for the thread's own loads.
    __device__ __forceinline__ void mask_tri(T *lds, int tid, int x0, int k0, int mode, int unit) const {
        const int lane = tid & 63, wave = tid >> 6;
        auto fix = [&](T &v, int xg, int kg) {
            const bool keep = mode == 1 ? kg <= xg : kg >= xg;
            if (!keep || (unit == 2 && kg == xg)) v = T();
            else if (unit == 1 && kg == xg) v = el_one<T>();
            else if (unit == 3 && kg == xg) v = el_real_only(v);
        };
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            if (MODE == LM_DMA_X) {
                const int e0 = (wave + i * NW) * CHUNK + lane * VEC;
                const int k = e0 / BX, x = image_col(k, e0 % BX);
                T *q = lds + (wave + i * NW) * CHUNK_PITCH + lane * VEC;
#pragma unroll
                for (int e = 0; e < VEC; ++e) fix(q[e], x0 + x + e, k0 + k);
            } else {
                const int ximg = (wave + i * NW) * (64 / S) + lane / S;
                const int place = lane % S, slot = place ^ swz(ximg);
                const int xg = x0 + perm(ximg);
#pragma unroll
                for (int e = 0; e < VEC; ++e) fix(lds[ximg * BK + place * VEC + e], xg, k0 + slot * VEC + e);
            }
        }
    }

    // LM_DMA_K: clears the elements past K of a partial panel, each thread in the 16 bytes
    // its own loads delivered (call after waiting for those loads).
    __device__ __forceinline__ void clear_k_tail(T *lds, int tid, int k_valid) const {
        if (MODE != LM_DMA_K) return;
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int x = (wave + i * NW) * (64 / S) + lane / S;
            const int place = lane % S, slot = place ^ swz(x);
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (slot * VEC + e >= k_valid) lds[x * BK + place * VEC + e] = T();
        }
    }
};

template <typename T, int BM, int BN, int BK, int WM, int WN, bool A_KC, bool B_KC, bool WIDE = false> struct GemmCfg {
    typedef typename MmaFor<typename Elem<T>::Real, WM, WN>::type M;
    static constexpr bool CPLX = Elem<T>::CPLX;
    static constexpr int VEC = 16 / (int)sizeof(T);
    static constexpr int MB = M::MB, KS = M::KS, NACC = M::NACC;
    static constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    static constexpr int NT = 64 * WAVES_M * WAVES_N;
    static constexpr int TM = WM / MB, TN = WN / MB;
    static constexpr int VM = TM < VEC ? TM : VEC;
    static constexpr int VN = TN < VEC ? TN : VEC;
    static_assert(BM % WM == 0 && BN % WN == 0 && WM % MB == 0 && WN % MB == 0, "tile shape");
    static_assert(TM % VM == 0 && TN % VN == 0 && BK % KS == 0, "tile shape");
    // k-contiguous panels (transA == T, transB == N) are kept as As[m][k] / Bs[n][k].  The m
    // interleave of the C mapping is the same for both A layouts (the [m][k] image permutes
    // its rows instead); n is interleaved only for a k-major B panel.
    static constexpr bool A_KLAY = A_KC, B_KLAY = B_KC;
    static constexpr int VNM = B_KLAY ? 1 : VN;  // n interleave used by the fragment/epilogue mapping
    static constexpr int NG = KS;                // lane groups along k
    static_assert(BK % (VEC * NG) == 0, "panel depth must hold whole k groups");
    typedef PanelLoader<T, BM, BK, NT, A_KC ? LM_DMA_K : LM_DMA_X, VM, MB, WIDE, MB> LoaderA;
    typedef PanelLoader<T, BN, BK, NT, B_KC ? LM_DMA_K : LM_DMA_X, 1, 1, WIDE, MB> LoaderB;
    static constexpr int PITCH_A = LoaderA::LDS_PITCH, PITCH_B = LoaderB::LDS_PITCH;
    static constexpr int A_ELEMS = LoaderA::LDS_ELEMS;
    static constexpr int STAGE = LoaderA::LDS_ELEMS + LoaderB::LDS_ELEMS;  // elements per LDS stage
    // Two stages: the loads of panel p+1 are issued during panel p.  Deeper rings (three,
    // four and six stages) were measured slower on large problems and on small ones alike.
    static constexpr int NSTAGE = 2;
    static constexpr size_t SMEM = (size_t)NSTAGE * STAGE * sizeof(T);
};

template <typename T, int BM, int BN, int BK, int WM, int WN, bool A_KC, bool B_KC, bool SPLITK, int MINW,
          bool TRI = false, bool WIDE = false>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64, MINW)
gemm_mfma_kernel(const GemmParams<T> p) {
    static_assert(!(SPLITK && TRI), "triangular variants do not split K");
    typedef GemmCfg<T, BM, BN, BK, WM, WN, A_KC, B_KC, WIDE> Cfg;
    typedef typename Elem<T>::Real R;
    typedef typename Cfg::M M;
    constexpr bool CPLX = Cfg::CPLX;
    constexpr int NP = CPLX ? 2 : 1;  // MFMA accumulator blocks per C block (re, im)
    constexpr int MB = Cfg::MB, KS = Cfg::KS, NACC = Cfg::NACC;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, VM = Cfg::VM, VN = Cfg::VN;
    constexpr int PITCH_A = Cfg::PITCH_A, PITCH_B = Cfg::PITCH_B, STAGE = Cfg::STAGE;
    constexpr int VEC = Cfg::VEC, NG = Cfg::NG, A_ELEMS = Cfg::A_ELEMS, VNM = Cfg::VNM;
    constexpr int NSTAGE = Cfg::NSTAGE;
    constexpr bool A_KLAY = Cfg::A_KLAY, B_KLAY = Cfg::B_KLAY;

    // Two workgroups that share a CU from the start run in lockstep and finish together; both
    // of their slots then go to two later workgroups at once, and at the end of a launch that
    // is not a whole number of rounds some CUs hold two workgroups while others idle.  So the
    // workgroups that took the second wave slot of their SIMD in the first round start late,
    // by about a quarter of the time two of them take for a tile.  (First thing in the kernel:
    // nothing is live yet.)
    if (p.stagger && blockIdx.x < 512) {
        const unsigned slot = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (3 << 11));  // HW_ID.WAVE_ID
        if (slot & 1) {
            // MFMA time of one wavefront for one panel, in cycles
            constexpr int PANEL_CYCLES = Cfg::TM * Cfg::TN * (BK / Cfg::KS) * (Cfg::CPLX ? 4 : 1) * 64;
            const int panels = (SPLITK ? p.k_per_split : p.K) / BK;
            const int n = (int)(((int64_t)panels * PANEL_CYCLES / 2) >> 12);
            for (int i = 0; i < n; ++i) __builtin_amdgcn_s_sleep(64);  // ~4096 cycles each
        }
    }

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *smem = reinterpret_cast<T *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // same value, known to be wave-uniform
    const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
    const int j = lane % MB;  // position along the block edge
    const int g = lane / MB;  // k sub-step supplied by this lane
    // Complex product with sA, sB = -1 where op(A), op(B) are conjugated, t = sA*sB:
    //   Re  = sum ar*br + ai*(-t*bi)
    //   Im' = sum ar*bi + ai*( t*br),   Im = sB * Im'
    // so exactly one of bi, br is sign-flipped per B element (masks below; the other mask
    // is zero) and Im' is negated in the epilogue when B is conjugated.
    const bool t_pos = CPLX && (p.conj_a == p.conj_b);
    const uint32_t sgn_bi = (CPLX && t_pos) ? 0x80000000u : 0u;
    const uint32_t sgn_br = (CPLX && !t_pos) ? 0x80000000u : 0u;
    auto flip = [](R x, uint32_t m) -> R {
        if constexpr (sizeof(R) == 4) return __builtin_bit_cast(R, __builtin_bit_cast(uint32_t, x) ^ m);
        else return __builtin_bit_cast(R, __builtin_bit_cast(uint64_t, x) ^ ((uint64_t)m << 32));
    };

    // ---- tile assignment: each XCD takes a contiguous chunk of the tile list (see
    //      tile_coords for the order of that list); slices of the tail come last and are
    //      dealt round-robin. ----
    int tile, slice = -1;
    {
        const int sliced = (TRI && p.tail_slices > 1) ? 1 : 0;
        const int nwg = sliced ? p.tail_first : (int)gridDim.x;  // whole tiles
        const int id = blockIdx.x;
        if (sliced && id >= nwg) {
            const int u = id - nwg;
            tile = nwg + u / p.tail_slices;
            slice = u % p.tail_slices;
        } else {
            const int xcd = id & 7, q = id >> 3;
            const int per = nwg >> 3, rem = nwg & 7;
            tile = p.xcd_remap ? xcd * per + (xcd < rem ? xcd : rem) + q : id;
        }
    }
    int tm, tn;
    tile_coords(p, TRI, BM, BN, tile, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- K range of this workgroup ----
    int k_begin = 0, k_end = p.K;
    if (SPLITK) {
        k_begin = blockIdx.y * p.k_per_split;
        k_end = k_begin + p.k_per_split < p.K ? k_begin + p.k_per_split : p.K;
    }
    if (TRI && slice >= 0) {
        k_begin = slice * p.tail_kps;
        k_end = k_begin + p.tail_kps < p.K ? k_begin + p.tail_kps : p.K;
    }
    if (TRI) {
        // Panels that lie wholly in the zero part of a triangular operand are skipped.
        if (p.tri_a == 1 && m0 + BM < k_end) k_end = m0 + BM;
        if (p.tri_b == 1 && n0 + BN < k_end) k_end = n0 + BN;
        if (p.tri_a == 2 && (m0 / BK) * BK > k_begin) k_begin = (m0 / BK) * BK;
        if (p.tri_b == 2 && (n0 / BK) * BK > k_begin) k_begin = (n0 / BK) * BK;
    }
    const int n_panels = k_end > k_begin ? (k_end - k_begin + BK - 1) / BK : 0;

    typename Cfg::LoaderA la;
    typename Cfg::LoaderB lb;
    la.init(tid, p.lda);
    lb.init(tid, p.ldb);

    // Element offset of panel `kp` of this tile from the operand base.
    auto a_off = [&](int k0) -> int64_t { return A_KC ? (int64_t)m0 * p.lda + k0 : (int64_t)k0 * p.lda + m0; };
    auto b_off = [&](int k0) -> int64_t { return B_KC ? (int64_t)n0 * p.ldb + k0 : (int64_t)k0 * p.ldb + n0; };

    typename M::Acc acc[TN][TM][NP];
#pragma unroll
    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
        for (int bm = 0; bm < TM; ++bm)
#pragma unroll
            for (int pp = 0; pp < NP; ++pp)
#pragma unroll
                for (int v = 0; v < NACC; ++v) acc[bn][bm][pp][v] = (R)0;

    if (n_panels > 0) {
        // Software pipeline over panels: two LDS stages, panel kp lives in stage kp % 2.  The
        // loads of panel kp+1 go out during panel kp into the stage whose last readers finished
        // before the barrier that ended panel kp-1.  Before the barrier that ends panel kp,
        // each wave waits for its own loads of panel kp+1.
        typedef typename Cfg::LoaderA LA;
        typedef typename Cfg::LoaderB LB;

        auto stage_ptr = [&](int kp) -> T * { return smem + (kp % NSTAGE) * STAGE; };
        auto issue_panel = [&](int kp) __attribute__((always_inline)) {
            const int k0 = k_begin + kp * BK;
            const int64_t ao = a_off(k0), bo = b_off(k0);
            T *dst = stage_ptr(kp);
            la.issue(p.A + ao, p.a_bytes - ao * (int64_t)sizeof(T), dst, wave_u);
            lb.issue(p.B + bo, p.b_bytes - bo * (int64_t)sizeof(T), dst + A_ELEMS, wave_u);
        };
        // Makes panel kp (already requested) readable by the whole workgroup: own loads
        // complete, K tail cleared, barrier.
        // full_depth: the caller knows that the panel is not the last one of its K range, so
        // it has no tail.
        // masks: an operand is triangular (TRI kernels only).
        auto publish_panel = [&](int kp, bool full_depth, bool masks) __attribute__((always_inline)) {
            T *dst = stage_ptr(kp);
            const int k_valid = k_end - (k_begin + kp * BK);
            __builtin_amdgcn_s_waitcnt(CBA_VMCNT_ONLY(0));
            if (!full_depth && k_valid < BK) {
                la.clear_k_tail(dst, tid, k_valid);
                lb.clear_k_tail(dst + A_ELEMS, tid, k_valid);
            }
            if (TRI && masks) {
                // Only the panels that meet the diagonal (or the zero side of it) need the fix-up.
                const int k0 = k_begin + kp * BK;
                if ((p.tri_a == 1 && k0 + BK > m0) || (p.tri_a == 2 && k0 < m0 + BM))
                    la.mask_tri(dst, tid, m0, k0, p.tri_a, p.unit_a);
                if ((p.tri_b == 1 && k0 + BK > n0) || (p.tri_b == 2 && k0 < n0 + BN))
                    lb.mask_tri(dst + A_ELEMS, tid, n0, k0, p.tri_b, p.unit_b);
            }
            __syncthreads();
        };

        issue_panel(0);
        publish_panel(0, false, true);

        const int a_frag = wm * WM + j * VM;
        const int b_frag = wn * WN + j * VN;
        constexpr int STEPS = BK / KS;

        // steady_tag: panel kp+1 exists and is not the last one - true for all
        // but the last few panels, which lets the body run without a single branch.
        auto do_panel = [&](int kp, auto steady_tag, auto masks_tag) __attribute__((always_inline)) {
            constexpr bool steady = decltype(steady_tag)::value;
            constexpr bool masks = decltype(masks_tag)::value;
            const bool issued = steady || kp + 1 < n_panels;
            // The loads of panel kp+1 are not issued here, all at once, but one by one behind
            // the MFMAs of the first steps below, where their issue does not hold up this
            // wavefront's MFMAs (8192^3: FP32 144 -> 149 TFLOP/s, FP64 70.5 -> 74; 1024^3 FP32
            // 75 -> 81).  Only the descriptors are made here.
            PanelSrc ra, rb;
            T *dst_next = stage_ptr(kp + 1);
            if (issued) {
                const int k0n = k_begin + (kp + 1) * BK;
                const int64_t ao = a_off(k0n), bo = b_off(k0n);
                ra = PanelSrc(p.A + ao, p.a_bytes - ao * (int64_t)sizeof(T));
                rb = PanelSrc(p.B + bo, p.b_bytes - bo * (int64_t)sizeof(T));
            }
            // (Complex FP64, with two long steps per panel, is the exception: 73.8 TFLOP/s at
            // 8192^3 with all loads up front, 72.7 with them behind the first step.)
            constexpr bool LOADS_UP_FRONT = sizeof(T) == 16;
            auto issue_behind_step = [&](int s) __attribute__((always_inline)) {
                constexpr int L = LA::PER + LB::PER;
                // over the first quarter of the steps: as good as over all of them where
                // workgroups share a CU, and the loads keep most of the panel to complete in
                constexpr int SP = STEPS / 4 > 0 ? STEPS / 4 : 1;
#pragma unroll
                for (int i = 0; i < L; ++i)
                    if ((LOADS_UP_FRONT ? -1 : i * SP / L) == s) {
                        if (i < LA::PER) la.issue_one(ra, dst_next, wave_u, i);
                        else lb.issue_one(rb, dst_next + A_ELEMS, wave_u, i - LA::PER);
                    }
            };

            const T *As = stage_ptr(kp);
            const T *Bs = As + A_ELEMS;
            // MFMA step s of a panel consumes, in lane group g, the k index
            //   kmap(s,g) = (s / VEC) * VEC * NG + g * VEC + s % VEC,
            // i.e. VEC consecutive steps walk VEC consecutive k: a k-major panel row is read
            // per step, a [x][k] panel is read as one 16-byte vector per VEC steps.
            // Fragments are read one step (one VEC-step group for [x][k]) ahead of their use.
            T a[2][TM], b[2][TN], ak[2][TM][VEC], bk[2][TN][VEC];
            auto kmap = [&](int s) { return (s / VEC) * (VEC * NG) + g * VEC + (s % VEC); };
            auto read_a = [&](int s, T (&af)[TM]) {  // k-major A panel
                const int krow = kmap(s);
#pragma unroll
                for (int ga = 0; ga < TM / VM; ++ga) {
                    typename Vec<T, VM>::type av =
                        *reinterpret_cast<const typename Vec<T, VM>::type *>(&As[LA::lds_at(krow, a_frag + ga * MB * VM)]);
#pragma unroll
                    for (int e = 0; e < VM; ++e) af[ga * VM + e] = Vec<T, VM>::get(av, e);
                }
            };
            auto read_b = [&](int s, T (&bf)[TN]) {  // k-major B panel
                const int krow = kmap(s);
#pragma unroll
                for (int gb = 0; gb < TN / VN; ++gb) {
                    typename Vec<T, VN>::type bv =
                        *reinterpret_cast<const typename Vec<T, VN>::type *>(&Bs[LB::lds_at(krow, b_frag + gb * MB * VN)]);
#pragma unroll
                    for (int e = 0; e < VN; ++e) bf[gb * VN + e] = Vec<T, VN>::get(bv, e);
                }
            };
            auto read_ak = [&](int grp, T (&af)[TM][VEC]) {  // [m'][k] A panel, VEC steps at once
#pragma unroll
                for (int bm = 0; bm < TM; ++bm) {
                    const int m_img = wm * WM + bm * MB + j;  // image row of block bm, lane j
                    const int place = (grp * NG + g) ^ LA::swz(m_img);
                    typename Vec<T, VEC>::type av =
                        *reinterpret_cast<const typename Vec<T, VEC>::type *>(&As[m_img * PITCH_A + place * VEC]);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) af[bm][e] = Vec<T, VEC>::get(av, e);
                }
            };
            auto read_bk = [&](int grp, T (&bf)[TN][VEC]) {  // [n][k] B panel, VEC steps at once
#pragma unroll
                for (int bn = 0; bn < TN; ++bn) {
                    const int n_loc = wn * WN + bn * MB + j;
                    const int place = (grp * NG + g) ^ LB::swz(n_loc);
                    typename Vec<T, VEC>::type bv =
                        *reinterpret_cast<const typename Vec<T, VEC>::type *>(&Bs[n_loc * PITCH_B + place * VEC]);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) bf[bn][e] = Vec<T, VEC>::get(bv, e);
                }
            };
            if (LOADS_UP_FRONT && issued) issue_behind_step(-1);
            if constexpr (A_KLAY) read_ak(0, ak[0]); else read_a(0, a[0]);
            if constexpr (B_KLAY) read_bk(0, bk[0]); else read_b(0, b[0]);
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                if (s + 1 < STEPS) {
                    if constexpr (A_KLAY) {
                        if ((s + 1) % VEC == 0) read_ak((s + 1) / VEC, ak[((s + 1) / VEC) & 1]);
                    } else {
                        read_a(s + 1, a[(s + 1) & 1]);
                    }
                    if constexpr (B_KLAY) {
                        if ((s + 1) % VEC == 0) read_bk((s + 1) / VEC, bk[((s + 1) / VEC) & 1]);
                    } else {
                        read_b(s + 1, b[(s + 1) & 1]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                auto a_of = [&](int bm) -> T { return A_KLAY ? ak[(s / VEC) & 1][bm][s % VEC] : a[s & 1][bm]; };
                auto b_of = [&](int bn) -> T { return B_KLAY ? bk[(s / VEC) & 1][bn][s % VEC] : b[s & 1][bn]; };
                if constexpr (!CPLX) {
#pragma unroll
                    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
                        for (int bm = 0; bm < TM; ++bm) acc[bn][bm][0] = M::run(b_of(bn), a_of(bm), acc[bn][bm][0]);
                } else {
                    // Four sweeps over the blocks, so that the two MFMAs into one accumulator
                    // are TM*TN*2 instructions apart.
                    R bre[TN], bim[TN], bre_x[TN], bim_x[TN];
#pragma unroll
                    for (int bn = 0; bn < TN; ++bn) {
                        const T bv = b_of(bn);
                        bre[bn] = bv.re;
                        bim[bn] = bv.im;
                        bim_x[bn] = flip(bv.im, sgn_bi);  // -t*bi up to the zero mask
                        bre_x[bn] = flip(bv.re, sgn_br);  //  t*br
                    }
#pragma unroll
                    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
                        for (int bm = 0; bm < TM; ++bm) acc[bn][bm][0] = M::run(bre[bn], a_of(bm).re, acc[bn][bm][0]);
#pragma unroll
                    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
                        for (int bm = 0; bm < TM; ++bm) acc[bn][bm][1] = M::run(bim[bn], a_of(bm).re, acc[bn][bm][1]);
#pragma unroll
                    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
                        for (int bm = 0; bm < TM; ++bm) acc[bn][bm][0] = M::run(bim_x[bn], a_of(bm).im, acc[bn][bm][0]);
#pragma unroll
                    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
                        for (int bm = 0; bm < TM; ++bm) acc[bn][bm][1] = M::run(bre_x[bn], a_of(bm).im, acc[bn][bm][1]);
                }
                if (!LOADS_UP_FRONT && issued) issue_behind_step(s);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (steady || kp + 1 < n_panels) publish_panel(kp + 1, steady, masks);
            else __syncthreads();
        };
        // Two panels per trip, so that the stage addresses of each copy are loop-invariant.
        // Taken branches cost a wavefront tens of cycles of instruction fetch, which shows as
        // idle MFMA time when only two wavefronts share a SIMD: the steady part of the loop is
        // straight-line code, and the last panels (at most three) run a general copy.
        auto k_loop = [&](auto masks_tag) __attribute__((always_inline)) {
            const int n_steady = n_panels > 2 ? ((n_panels - 2) & ~1) : 0;
            int kp = 0;
            for (; kp < n_steady; kp += 2) {
                do_panel(kp, std::true_type(), masks_tag);
                do_panel(kp + 1, std::true_type(), masks_tag);
            }
            for (; kp < n_panels; ++kp) do_panel(kp, std::false_type(), masks_tag);
        };
        // A triangular operand puts tests (and now and then a fix-up) between the panels; the
        // other users of the TRI kernels - a triangle of C, sliced tails - keep the straight line.
        if (TRI && (p.tri_a || p.tri_b)) k_loop(std::true_type());
        else k_loop(std::false_type());
    }

    // ---- epilogue ----
    T *Cout = p.C;
    int64_t ldc = p.ldc;
    T alpha = p.alpha, beta = p.beta;
    if (SPLITK) {
        Cout = p.ws + (int64_t)blockIdx.y * p.ws_slice;
        ldc = p.ws_ld;
        alpha = el_one<T>();
        beta = T();
    }
    int tri_c = TRI ? p.tri_c : 0;
    bool herm_c = TRI && p.herm_c;  // Hermitian C: diagonal elements are stored with a zero imaginary part
    if (TRI && slice >= 0) {
        // partial tile, tile-local coordinates, finished by tail_reduce_kernel
        const int u = (int)blockIdx.x - p.tail_first;
        const int64_t shift = (int64_t)u * (BM * BN) - ((int64_t)n0 * BM + m0);  // may be negative
        Cout = reinterpret_cast<T *>(reinterpret_cast<uintptr_t>(p.ws) + (uintptr_t)(shift * (int64_t)sizeof(T)));
        ldc = BM;
        alpha = el_one<T>();
        beta = T();
        tri_c = 0;
        herm_c = false;
    }
    const bool read_c = !el_is_zero(beta);
    const bool neg_im = CPLX && p.conj_b;  // Im = sB * Im'
    auto acc_elem = [&](int bn, int bm, int v) -> T {
        if constexpr (CPLX) return T{acc[bn][bm][0][v], neg_im ? -acc[bn][bm][1][v] : acc[bn][bm][1][v]};
        else return acc[bn][bm][0][v];
    };

    // C is read in batches of CH accumulator rows per lane before any of them is written
    // back, so that the load latencies of a batch overlap instead of queueing behind each
    // store (loads and stores go to the same array, so the compiler keeps their order).
    typedef Vec<T, VM> VC;
    typedef typename VC::utype UV;
    constexpr int CH = NACC < 8 ? NACC : 8;
#pragma unroll
    for (int bn = 0; bn < TN; ++bn) {
#pragma unroll
        for (int v0 = 0; v0 < NACC; v0 += CH) {
            UV cold[CH][TM / VM];
            if (read_c) {
#pragma unroll
                for (int dv = 0; dv < CH; ++dv) {
                    const int n = n0 + wn * WN + (bn / VNM) * (MB * VNM) + M::row(v0 + dv, lane) * VNM + (bn % VNM);
                    const T *col = Cout + (int64_t)n * ldc;
#pragma unroll
                    for (int ga = 0; ga < TM / VM; ++ga) {
                        const int m = m0 + wm * WM + ga * (MB * VM) + j * VM;
                        if (n < p.N && m + VM <= p.M) cold[dv][ga] = *reinterpret_cast<const UV *>(col + m);
                    }
                }
            }
#pragma unroll
            for (int dv = 0; dv < CH; ++dv) {
                const int v = v0 + dv;
                const int n = n0 + wn * WN + (bn / VNM) * (MB * VNM) + M::row(v, lane) * VNM + (bn % VNM);
                if (n >= p.N) continue;
                T *col = Cout + (int64_t)n * ldc;
#pragma unroll
                for (int ga = 0; ga < TM / VM; ++ga) {
                    const int m = m0 + wm * WM + ga * (MB * VM) + j * VM;
                    bool whole = true;  // all VM rows of this vector are stored
                    if (TRI && tri_c) {
                        if (tri_c == 1 ? m + VM - 1 < n : m > n) continue;  // none of them is
                        whole = tri_c == 1 ? m >= n : m + VM - 1 <= n;
                    }
                    if (m + VM <= p.M && whole) {
                        UV ov;
#pragma unroll
                        for (int e = 0; e < VM; ++e) {
                            T r = el_scale(alpha, acc_elem(bn, ga * VM + e, v));
                            if (TRI && CPLX && herm_c && m + e == n) {
                                // the stored imaginary part of a Hermitian diagonal is not part of the matrix
                                if (read_c) r = el_axpy(beta, el_real_only(VC::get(cold[dv][ga], e)), r);
                                r = el_real_only(r);
                            } else if (read_c) {
                                r = el_axpy(beta, VC::get(cold[dv][ga], e), r);
                            }
                            VC::set(ov, e, r);
                        }
                        *reinterpret_cast<UV *>(col + m) = ov;
                    } else {
#pragma unroll
                        for (int e = 0; e < VM; ++e) {
                            const bool kept = !(TRI && tri_c) || (tri_c == 1 ? m + e >= n : m + e <= n);
                            if (m + e < p.M && kept) {
                                T r = el_scale(alpha, acc_elem(bn, ga * VM + e, v));
                                if (TRI && CPLX && herm_c && m + e == n) {
                                    if (read_c) r = el_axpy(beta, el_real_only(col[m + e]), r);
                                    r = el_real_only(r);
                                } else if (read_c) {
                                    r = el_axpy(beta, col[m + e], r);
                                }
                                col[m + e] = r;
                            }
                        }
                    }
                }
            }
        }
    }
}

// Sums the split-K partials in a fixed order and applies alpha / beta once.
// 1-D grid: block b covers rows [256*(b % m_blocks), +256) of column b / m_blocks.
template <typename T>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const T *ws, int64_t ws_ld, int64_t ws_slice, int splits, int M, int N, int m_blocks,
                     T alpha, T beta, T *C, int64_t ldc) {
    const int m = (blockIdx.x % m_blocks) * 256 + threadIdx.x;
    const int n = blockIdx.x / m_blocks;
    if (m >= M || n >= N) return;
    // partials are fetched eight at a time (independent loads) and added in split order
    const T *w = ws + (int64_t)n * ws_ld + m;
    T s = T();
    int i = 0;
    for (; i + 8 <= splits; i += 8) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = w[(int64_t)(i + u) * ws_slice];
#pragma unroll
        for (int u = 0; u < 8; ++u) s = el_add(s, v[u]);
    }
    for (; i < splits; ++i) s = el_add(s, w[(int64_t)i * ws_slice]);
    T *c = C + (int64_t)n * ldc + m;
    T r = el_scale(alpha, s);
    if (!el_is_zero(beta)) r = el_axpy(beta, *c, r);
    *c = r;
}

// The same for many K ranges over a small C (deep K, few tiles), where the pass above is a chain of
// dependent load batches on too few threads: 8 threads share an element, thread part l fetches ranges
// l, l + 8, l + 16, ... at once (up to 8 independent loads) and adds them in that order, and the
// 8 part sums are added in part order.  A fixed order, so the result is reproducible bit for bit;
// it differs from the order of the pass above only in which roundings happen.
// Block b covers rows [32 * (b % m_blocks), +32) of column b / m_blocks; thread t: part t / 32, row t % 32.
template <typename T>
__global__ void __launch_bounds__(256)
splitk_reduce_wide_kernel(const T *ws, int64_t ws_ld, int64_t ws_slice, int splits, int M, int N, int m_blocks,
                          T alpha, T beta, T *C, int64_t ldc) {
    __shared__ T part_sum[8][33];
    const int part = threadIdx.x >> 5, row = threadIdx.x & 31;
    const int m = (blockIdx.x % m_blocks) * 32 + row;
    const int n = blockIdx.x / m_blocks;
    T s = T();
    if (m < M) {
        const T *w = ws + (int64_t)n * ws_ld + m;
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (part + 8 * u < splits) v[u] = w[(int64_t)(part + 8 * u) * ws_slice];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (part + 8 * u < splits) s = u == 0 ? v[0] : el_add(s, v[u]);
    }
    part_sum[part][row] = s;
    __syncthreads();
    if (part == 0 && m < M) {
        T t = part_sum[0][row];
        const int parts = splits < 8 ? splits : 8;
        for (int l = 1; l < parts; ++l) t = el_add(t, part_sum[l][row]);
        T *c = C + (int64_t)n * ldc + m;
        T r = el_scale(alpha, t);
        if (!el_is_zero(beta)) r = el_axpy(beta, *c, r);
        *c = r;
    }
}

// Finishes the tiles whose K range was cut into slices (see GemmParams::tail_*): sums the
// slices in a fixed order, applies alpha / beta once and honours tri_c.  Block (x, r) covers
// elements [256 x, 256 x + 256) of sliced tile r (tile-local, column-major, pitch bm).
template <typename T>
__global__ void __launch_bounds__(256) tail_reduce_kernel(const GemmParams<T> p, int bm, int bn) {
    const int r = blockIdx.y;
    int tm, tn;
    tile_coords(p, true, bm, bn, p.tail_first + r, tm, tn);
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= bm * bn) return;
    const int m = tm * bm + e % bm, n = tn * bn + e / bm;
    if (m >= p.M || n >= p.N) return;
    if (p.tri_c && (p.tri_c == 1 ? m < n : m > n)) return;
    const T *w = p.ws + (int64_t)r * p.tail_slices * (bm * bn) + e;
    T s = T();
    int i = 0;
    for (; i + 4 <= p.tail_slices; i += 4) {  // four independent loads at a time, added in slice order
        T v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = w[(int64_t)(i + u) * (bm * bn)];
#pragma unroll
        for (int u = 0; u < 4; ++u) s = el_add(s, v[u]);
    }
    for (; i < p.tail_slices; ++i) s = el_add(s, w[(int64_t)i * (bm * bn)]);
    T *c = p.C + (int64_t)n * p.ldc + m;
    T v = el_scale(p.alpha, s);
    const bool herm_diag = p.herm_c && m == n;
    if (!el_is_zero(p.beta)) v = el_axpy(p.beta, herm_diag ? el_real_only(*c) : *c, v);
    if (herm_diag) v = el_real_only(v);
    *c = v;
}

// C <- beta * C (K == 0); beta == 0 stores zeros without reading C.
template <typename T>
__global__ void __launch_bounds__(256) scale_c_kernel(int M, int N, int m_blocks, T beta, T *C, int64_t ldc) {
    const int m = (blockIdx.x % m_blocks) * 256 + threadIdx.x;
    const int n = blockIdx.x / m_blocks;
    if (m >= M || n >= N) return;
    T *c = C + (int64_t)n * ldc + m;
    *c = el_is_zero(beta) ? T() : el_scale(beta, *c);
}

}  // namespace cba
