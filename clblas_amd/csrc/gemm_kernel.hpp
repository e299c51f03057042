// MFMA GEMM kernel for gfx950 (CDNA4), FP32 and FP64, all four transpose combinations.
//
// Computes (column-major, after the host has folded row-major calls)
//     C(m,n) <- alpha * sum_k opA(m,k) * opB(k,n) + beta * C(m,n)
// which is the contract of the reference's AutoGemm kernels
// (src/library/blas/AutoGemm/KernelOpenCL.py:311-452): one accumulator per C element,
// alpha/beta applied once in the epilogue, beta == 0 never reads C.
//
// Structure of one workgroup (BM x BN macro tile of C, waves arranged WAVES_M x WAVES_N):
//   * A and B panels of depth BK are fetched with 16-byte raw buffer loads into registers
//     while the MFMAs of the previous panel run, then written to one of two LDS stages
//     (double buffering, one barrier per panel).  Buffer descriptors are re-based every
//     panel and sized to the exact footprint of the operand, so the hardware range check
//     turns every access past the end of the matrix into a zero: no extra launch and no
//     per-element branch is needed for M/N/K remainders.
//   * LDS always holds the panels "k-major": As[k][m], Bs[k][n].  Operands whose
//     contiguous direction in memory is k (transA == T, transB == N) are transposed on the
//     way into LDS; a row pitch of tile+4 elements makes both the transposing scalar
//     writes and the 16-byte fragment reads bank-conflict free.
//   * Each wave owns a WM x WN sub-tile as TM x TN MFMA blocks
//     (v_mfma_f32_32x32x2_f32 / v_mfma_f64_16x16x4_f64).  The MFMA "B" operand carries the
//     A matrix and the "A" operand carries the B matrix, so that the lane index of the
//     result runs along m, the contiguous direction of C.  The m (and n) coordinates are
//     interleaved between blocks so that one 16-byte LDS read feeds VM blocks and one
//     16-byte global store writes VM consecutive rows of C.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace cba {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Vector of N elements of T with only element alignment (global C may be misaligned by
// offC / ldc) and with natural alignment (LDS).
template <typename T, int N> struct Vec;
template <> struct Vec<float, 1> { typedef float type; typedef float utype; };
template <> struct Vec<float, 2> { typedef f32x2 type; typedef float utype __attribute__((ext_vector_type(2), aligned(4))); };
template <> struct Vec<float, 4> { typedef f32x4 type; typedef float utype __attribute__((ext_vector_type(4), aligned(4))); };
template <> struct Vec<double, 1> { typedef double type; typedef double utype; };
template <> struct Vec<double, 2> { typedef f64x2 type; typedef double utype __attribute__((ext_vector_type(2), aligned(8))); };

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

template <typename T> struct GemmParams {
    const T *A;
    const T *B;
    T *C;
    int64_t lda, ldb, ldc;
    int64_t a_bytes, b_bytes;  // exact footprint of op-A / op-B storage, from A / B
    int M, N, K;
    T alpha, beta;
    int tiles_m, tiles_n;
    int group_m;      // tile rows walked together (L2 locality)
    int xcd_remap;    // 1: give each XCD a contiguous chunk of the tile list
    int k_per_split;  // multiple of BK; >= K when the K loop is not split
    T *ws;            // split-K partial sums: ws[split * ws_slice + n * ws_ld + m]
    int64_t ws_ld, ws_slice;
};

static __device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, int64_t bytes_left) {
    // Descriptors address at most 2 GiB from their base; tiles are re-based so that every
    // legitimate offset is below that.  A non-positive remainder yields an empty buffer.
    uint32_t n = bytes_left <= 0 ? 0u : (bytes_left > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)bytes_left);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)n, 0x00020000);
}

// Fetches one BX x BK operand panel.  KC == true: memory is contiguous along k
// (element (x,k) at x*ld + k); KC == false: contiguous along x (element at k*ld + x).
// KLAY selects the LDS layout: false: [k][x] (row pitch BX+4); true (only with KC): [x][k]
// (row pitch BK + one 16-byte vector), written with one 16-byte store per loaded vector.
template <typename T, int BX, int BK, int NT, bool KC, bool KLAY> struct PanelLoader {
    static_assert(!KLAY || KC, "[x][k] layout is for k-contiguous operands");
    static constexpr int VEC = 16 / (int)sizeof(T);
    static constexpr int NVEC = BX * BK / VEC;
    static constexpr int PER = NVEC / NT;
    static_assert(NVEC % NT == 0 && PER >= 1, "panel does not divide over the workgroup");
    static constexpr int LDS_PITCH = KLAY ? BK + VEC : BX + 4;
    static constexpr int LDS_ELEMS = KLAY ? BX * LDS_PITCH : BK * LDS_PITCH;

    struct Regs { u32x4 v[PER]; };  // one panel's worth of data in flight
    uint32_t voff[PER];

    __device__ __forceinline__ void init(int tid, int64_t ld) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int idx = tid + i * NT;
            if (KC) {
                int x = idx / (BK / VEC), kv = (idx % (BK / VEC)) * VEC;
                voff[i] = (uint32_t)(((int64_t)x * ld + kv) * (int64_t)sizeof(T));
            } else {
                int k = idx / (BX / VEC), x = (idx % (BX / VEC)) * VEC;
                voff[i] = (uint32_t)(((int64_t)k * ld + x) * (int64_t)sizeof(T));
            }
        }
    }

    // base: first element of the panel; bytes_left: footprint bytes from `base` on.
    __device__ __forceinline__ void fetch(const T *base, int64_t bytes_left, Regs &reg) const {
        __amdgpu_buffer_rsrc_t r = make_rsrc(base, bytes_left);
#pragma unroll
        for (int i = 0; i < PER; ++i) reg.v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff[i], 0, 0);
    }

    // k_valid: number of valid k rows in this panel (>= BK for a full panel).
    __device__ __forceinline__ void store(T *lds, int tid, int k_valid, const Regs &reg) const {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int idx = tid + i * NT;
            if (KC) {
                int x = idx / (BK / VEC), kv = (idx % (BK / VEC)) * VEC;
                union { u32x4 u; T e[VEC]; } cv;
                cv.u = reg.v[i];
                // Past-K elements of a k-contiguous operand are real memory (the next
                // column), not out of range, so they are cleared here.
#pragma unroll
                for (int e = 0; e < VEC; ++e) cv.e[e] = (kv + e < k_valid) ? cv.e[e] : (T)0;
                if (KLAY) {
                    *reinterpret_cast<u32x4 *>(&lds[x * LDS_PITCH + kv]) = cv.u;
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) lds[(kv + e) * LDS_PITCH + x] = cv.e[e];
                }
            } else {
                int k = idx / (BX / VEC), x = (idx % (BX / VEC)) * VEC;
                // Rows k >= K lie past the operand's footprint: the range check already
                // returned zeros for them.
                *reinterpret_cast<u32x4 *>(&lds[k * LDS_PITCH + x]) = reg.v[i];
            }
        }
    }
};

template <typename T, int BM, int BN, int BK, int WM, int WN, bool A_KC, bool B_KC> struct GemmCfg {
    typedef Mma<T> M;
    static constexpr int VEC = 16 / (int)sizeof(T);
    static constexpr int MB = M::MB, KS = M::KS, NACC = M::NACC;
    static constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    static constexpr int NT = 64 * WAVES_M * WAVES_N;
    static constexpr int TM = WM / MB, TN = WN / MB;
    static constexpr int VM = TM < VEC ? TM : VEC;
    static constexpr int VN = TN < VEC ? TN : VEC;
    static_assert(BM % WM == 0 && BN % WN == 0 && WM % MB == 0 && WN % MB == 0, "tile shape");
    static_assert(TM % VM == 0 && TN % VN == 0 && BK % KS == 0, "tile shape");
    // A k-contiguous B panel (transB == N) is kept as Bs[n][k]; a k-contiguous A panel is
    // still transposed into As[k][m] so that C keeps its 16-byte row-interleaved stores.
    static constexpr bool B_KLAY = B_KC;
    static constexpr int VNM = B_KLAY ? 1 : VN;  // n interleave used by the fragment/epilogue mapping
    static constexpr int NG = 64 / MB;           // lane groups along k
    static_assert(BK % (VEC * NG) == 0, "panel depth must hold whole k groups");
    typedef PanelLoader<T, BM, BK, NT, A_KC, false> LoaderA;
    typedef PanelLoader<T, BN, BK, NT, B_KC, B_KLAY> LoaderB;
    static constexpr int PITCH_A = LoaderA::LDS_PITCH, PITCH_B = LoaderB::LDS_PITCH;
    static constexpr int A_ELEMS = LoaderA::LDS_ELEMS;
    static constexpr int STAGE = LoaderA::LDS_ELEMS + LoaderB::LDS_ELEMS;  // elements per LDS stage
    // Panels in flight from HBM (register sets).  Two everywhere except FP64 with a [n][k] B
    // panel, where the second set would push the kernel over 256 VGPRs.
    static constexpr int DEPTH = (sizeof(T) == 8 && B_KLAY && TM * TN >= 16) ? 1 : 2;
    static constexpr size_t SMEM = 2 * (size_t)STAGE * sizeof(T);
};

template <typename T, int BM, int BN, int BK, int WM, int WN, bool A_KC, bool B_KC, bool SPLITK, int MINW>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64, MINW)
gemm_mfma_kernel(const GemmParams<T> p) {
    typedef GemmCfg<T, BM, BN, BK, WM, WN, A_KC, B_KC> Cfg;
    typedef Mma<T> M;
    constexpr int MB = Cfg::MB, KS = Cfg::KS, NACC = Cfg::NACC;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, VM = Cfg::VM, VN = Cfg::VN;
    constexpr int PITCH_A = Cfg::PITCH_A, PITCH_B = Cfg::PITCH_B, STAGE = Cfg::STAGE;
    constexpr int VEC = Cfg::VEC, NG = Cfg::NG, A_ELEMS = Cfg::A_ELEMS, VNM = Cfg::VNM;
    constexpr bool B_KLAY = Cfg::B_KLAY;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *smem = reinterpret_cast<T *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
    const int j = lane % MB;  // position along the block edge
    const int g = lane / MB;  // k sub-step supplied by this lane

    // ---- tile assignment: contiguous chunk of the tile list per XCD, then walk
    //      `group_m` tile rows at a time so that concurrently running workgroups of one
    //      XCD share A and B panels in that XCD's L2. ----
    int tile;
    {
        const int nwg = p.tiles_m * p.tiles_n;
        const int id = blockIdx.x;
        const int xcd = id & 7, q = id >> 3;
        const int per = nwg >> 3, rem = nwg & 7;
        tile = p.xcd_remap ? xcd * per + (xcd < rem ? xcd : rem) + q : id;
    }
    int tm, tn;
    {
        const int per_group = p.group_m * p.tiles_n;
        const int grp = tile / per_group;
        const int first_m = grp * p.group_m;
        const int gm = (p.tiles_m - first_m) < p.group_m ? (p.tiles_m - first_m) : p.group_m;
        const int r = tile - grp * per_group;
        tm = first_m + r % gm;
        tn = r / gm;
    }
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- K range of this workgroup ----
    int k_begin = 0, k_end = p.K;
    if (SPLITK) {
        k_begin = blockIdx.y * p.k_per_split;
        k_end = k_begin + p.k_per_split < p.K ? k_begin + p.k_per_split : p.K;
    }
    const int n_panels = (k_end - k_begin + BK - 1) / BK;

    typename Cfg::LoaderA la;
    typename Cfg::LoaderB lb;
    la.init(tid, p.lda);
    lb.init(tid, p.ldb);

    // Element offset of panel `kp` of this tile from the operand base.
    auto a_off = [&](int k0) -> int64_t { return A_KC ? (int64_t)m0 * p.lda + k0 : (int64_t)k0 * p.lda + m0; };
    auto b_off = [&](int k0) -> int64_t { return B_KC ? (int64_t)n0 * p.ldb + k0 : (int64_t)k0 * p.ldb + n0; };

    typename M::Acc acc[TN][TM];
#pragma unroll
    for (int bn = 0; bn < TN; ++bn)
#pragma unroll
        for (int bm = 0; bm < TM; ++bm)
#pragma unroll
            for (int v = 0; v < NACC; ++v) acc[bn][bm][v] = (T)0;

    if (n_panels > 0) {
        // Software pipeline over panels.  DEPTH register sets hold panels in flight from HBM.
        // DEPTH 2: at the top of panel kp the loads of panel kp+2 are issued, in the middle of
        // its MFMAs panel kp+1 (issued a whole panel earlier) is written into the idle LDS
        // stage, and the single barrier at the end publishes it.  DEPTH 1: panel kp+1 is
        // requested at the top of panel kp and written after its last MFMA.
        constexpr int DEPTH = Cfg::DEPTH;
        typename Cfg::LoaderA::Regs ra[DEPTH];
        typename Cfg::LoaderB::Regs rb[DEPTH];
        auto fetch_panel = [&](int kp, typename Cfg::LoaderA::Regs &xa, typename Cfg::LoaderB::Regs &xb) {
            const int k0 = k_begin + kp * BK;
            const int64_t ao = a_off(k0), bo = b_off(k0);
            la.fetch(p.A + ao, p.a_bytes - ao * (int64_t)sizeof(T), xa);
            lb.fetch(p.B + bo, p.b_bytes - bo * (int64_t)sizeof(T), xb);
        };
        auto store_panel = [&](int kp, const typename Cfg::LoaderA::Regs &xa, const typename Cfg::LoaderB::Regs &xb) {
            T *dst = smem + (kp & 1) * STAGE;
            const int k_valid = k_end - (k_begin + kp * BK);
            la.store(dst, tid, k_valid, xa);
            lb.store(dst + A_ELEMS, tid, k_valid, xb);
        };

        fetch_panel(0, ra[0], rb[0]);
        if (DEPTH == 2 && n_panels > 1) fetch_panel(1, ra[DEPTH - 1], rb[DEPTH - 1]);
        store_panel(0, ra[0], rb[0]);
        __syncthreads();

        const int a_frag = wm * WM + j * VM;
        const int b_frag = wn * WN + j * VN;
        constexpr int STEPS = BK / KS;
        // MFMA step after which the next panel goes to LDS: mid-way when it was requested a
        // whole panel earlier, at the end when it was requested at the top of this panel.
        constexpr int STORE_AT = DEPTH == 2 ? STEPS / 2 : STEPS;

        // One panel: `par` is kp & 1, known at compile time so that the register sets are
        // addressed statically.
        auto do_panel = [&](int kp, auto par_tag) {
            constexpr int PAR = decltype(par_tag)::value;
            constexpr int R_IN = DEPTH == 2 ? PAR : 0;       // set receiving the new loads
            constexpr int R_OUT = DEPTH == 2 ? PAR ^ 1 : 0;  // set written to LDS during this panel
            if (kp + DEPTH < n_panels) fetch_panel(kp + DEPTH, ra[R_IN], rb[R_IN]);

            const T *As = smem + PAR * STAGE;
            const T *Bs = As + A_ELEMS;
            // MFMA step s of a panel consumes, in lane group g, the k index
            //   kmap(s,g) = (s / VEC) * VEC * NG + g * VEC + s % VEC,
            // i.e. VEC consecutive steps walk VEC consecutive k: a k-major panel row is read
            // per step, a [n][k] panel is read as one 16-byte vector per VEC steps.
            // Fragments are read one step (one VEC-step group for [n][k]) ahead of their use.
            T a[2][TM], b[2][TN], bk[2][TN][VEC];
            auto kmap = [&](int s) { return (s / VEC) * (VEC * NG) + g * VEC + (s % VEC); };
            auto read_a = [&](int s, T (&af)[TM]) {
                const int krow = kmap(s);
#pragma unroll
                for (int ga = 0; ga < TM / VM; ++ga) {
                    typename Vec<T, VM>::type av =
                        *reinterpret_cast<const typename Vec<T, VM>::type *>(&As[krow * PITCH_A + a_frag + ga * MB * VM]);
                    if constexpr (VM == 1) af[ga] = av;
                    else {
#pragma unroll
                        for (int e = 0; e < VM; ++e) af[ga * VM + e] = av[e];
                    }
                }
            };
            auto read_b = [&](int s, T (&bf)[TN]) {  // k-major B panel
                const int krow = kmap(s);
#pragma unroll
                for (int gb = 0; gb < TN / VN; ++gb) {
                    typename Vec<T, VN>::type bv =
                        *reinterpret_cast<const typename Vec<T, VN>::type *>(&Bs[krow * PITCH_B + b_frag + gb * MB * VN]);
                    if constexpr (VN == 1) bf[gb] = bv;
                    else {
#pragma unroll
                        for (int e = 0; e < VN; ++e) bf[gb * VN + e] = bv[e];
                    }
                }
            };
            auto read_bk = [&](int grp, T (&bf)[TN][VEC]) {  // [n][k] B panel, VEC steps at once
#pragma unroll
                for (int bn = 0; bn < TN; ++bn) {
                    typename Vec<T, VEC>::type bv = *reinterpret_cast<const typename Vec<T, VEC>::type *>(
                        &Bs[(wn * WN + bn * MB + j) * PITCH_B + grp * (VEC * NG) + g * VEC]);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) bf[bn][e] = bv[e];
                }
            };
            read_a(0, a[0]);
            if constexpr (B_KLAY) read_bk(0, bk[0]); else read_b(0, b[0]);
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                if (s + 1 < STEPS) {
                    read_a(s + 1, a[(s + 1) & 1]);
                    if constexpr (B_KLAY) {
                        if ((s + 1) % VEC == 0) read_bk((s + 1) / VEC, bk[((s + 1) / VEC) & 1]);
                    } else {
                        read_b(s + 1, b[(s + 1) & 1]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int bn = 0; bn < TN; ++bn) {
                    const T bval = B_KLAY ? bk[(s / VEC) & 1][bn][s % VEC] : b[s & 1][bn];
#pragma unroll
                    for (int bm = 0; bm < TM; ++bm) acc[bn][bm] = M::run(bval, a[s & 1][bm], acc[bn][bm]);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (s + 1 == STORE_AT) {
                    if (kp + 1 < n_panels) store_panel(kp + 1, ra[R_OUT], rb[R_OUT]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __syncthreads();
        };

        for (int kp = 0; kp < n_panels; kp += 2) {
            do_panel(kp, std::integral_constant<int, 0>());
            if (kp + 1 < n_panels) do_panel(kp + 1, std::integral_constant<int, 1>());
        }
    }

    // ---- epilogue ----
    T *Cout = p.C;
    int64_t ldc = p.ldc;
    T alpha = p.alpha, beta = p.beta;
    if (SPLITK) {
        Cout = p.ws + (int64_t)blockIdx.y * p.ws_slice;
        ldc = p.ws_ld;
        alpha = (T)1;
        beta = (T)0;
    }
    const bool read_c = !(beta == (T)0);

#pragma unroll
    for (int bn = 0; bn < TN; ++bn) {
#pragma unroll
        for (int v = 0; v < NACC; ++v) {
            const int n = n0 + wn * WN + (bn / VNM) * (MB * VNM) + M::row(v, lane) * VNM + (bn % VNM);
            if (n >= p.N) continue;
            T *col = Cout + (int64_t)n * ldc;
#pragma unroll
            for (int ga = 0; ga < TM / VM; ++ga) {
                const int m = m0 + wm * WM + ga * (MB * VM) + j * VM;
                if (m + VM <= p.M) {
                    typedef typename Vec<T, VM>::utype UV;
                    T r[VM];
                    if (read_c) {
                        UV cv = *reinterpret_cast<const UV *>(col + m);
#pragma unroll
                        for (int e = 0; e < VM; ++e) {
                            T c_old;
                            if constexpr (VM == 1) c_old = cv; else c_old = cv[e];
                            r[e] = alpha * acc[bn][ga * VM + e][v] + beta * c_old;
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < VM; ++e) r[e] = alpha * acc[bn][ga * VM + e][v];
                    }
                    UV ov;
                    if constexpr (VM == 1) ov = r[0];
                    else {
#pragma unroll
                        for (int e = 0; e < VM; ++e) ov[e] = r[e];
                    }
                    *reinterpret_cast<UV *>(col + m) = ov;
                } else {
#pragma unroll
                    for (int e = 0; e < VM; ++e) {
                        if (m + e < p.M) {
                            T r = alpha * acc[bn][ga * VM + e][v];
                            if (read_c) r += beta * col[m + e];
                            col[m + e] = r;
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
    T s = (T)0;
    for (int i = 0; i < splits; ++i) s += ws[(int64_t)i * ws_slice + (int64_t)n * ws_ld + m];
    T *c = C + (int64_t)n * ldc + m;
    T r = alpha * s;
    if (!(beta == (T)0)) r += beta * *c;
    *c = r;
}

// C <- beta * C (K == 0); beta == 0 stores zeros without reading C.
template <typename T>
__global__ void __launch_bounds__(256) scale_c_kernel(int M, int N, int m_blocks, T beta, T *C, int64_t ldc) {
    const int m = (blockIdx.x % m_blocks) * 256 + threadIdx.x;
    const int n = blockIdx.x / m_blocks;
    if (m >= M || n >= N) return;
    T *c = C + (int64_t)n * ldc + m;
    *c = (beta == (T)0) ? (T)0 : beta * *c;
}

// Plain kernel with 64-bit indexing for leading dimensions too large for the 32-bit
// panel offsets of the MFMA kernel.  Same contract; one thread per C element.
template <typename T>
__global__ void __launch_bounds__(256)
gemm_wide_ld_kernel(int transA, int transB, int M, int N, int K, int m_blocks, T alpha, const T *A, int64_t lda,
                    const T *B, int64_t ldb, T beta, T *C, int64_t ldc) {
    const int64_t m = (int64_t)(blockIdx.x % m_blocks) * 256 + threadIdx.x;
    const int64_t n = blockIdx.x / m_blocks;
    if (m >= M || n >= N) return;
    T s = (T)0;
    for (int64_t k = 0; k < K; ++k) {
        T a = transA ? A[k + m * lda] : A[m + k * lda];
        T b = transB ? B[n + k * ldb] : B[k + n * ldb];
        s = fma(a, b, s);
    }
    T *c = C + n * ldc + m;
    T r = alpha * s;
    if (!(beta == (T)0)) r += beta * *c;
    *c = r;
}

}  // namespace cba
