// Host-side launch plumbing shared by the FP32 and FP64 GEMM translation units:
// one table entry per (tile shape), each holding the 4 transpose x {plain, split-K}
// kernel instantiations.  Takes the place of the reference's generated
// gemmSelectKernel<T>() / makeGemmKernel / enqueueGemmKernel
// (src/library/blas/xgemm.cc:160-313, AutoGemm/KernelSelection.py:101-305): kernels are
// compiled ahead of time, so "selection" is only a table lookup.
#pragma once

#include <cstdio>

#include "gemm_kernel.hpp"
#include "internal.h"

namespace cba {

template <typename T> struct TileEntry {
    int bm, bn, bk, threads;
    // The same tile with deeper panels (bk_deep; 0: none), for workgroups with a long K range: half
    // the barriers and loop overhead per flop (FP32 64x64 with depth 64 instead of 32: 1024 x 1024 x 4096
    // 70.6 -> 66.5 us, 960 x 960 x 2048 38.0 -> 35.8, 1024^3 22.3 -> 21.7), but a first panel twice as
    // long to fetch before the first MFMA (512^3: 11.4 -> 12.9 us), so only from 1024 deep (512 for a single
    // round of workgroups: see where the variant is chosen).
    int bk_deep;
    double deep_gain;  // factor on `eff` where the deep form runs (plain products, K range from 1024)
    double streamed_gain;  // factor on `eff` where the operands are streamed from HBM (beyond the memory-side cache): the
                           // tiles of 32 rows or columns read a streamed operand more often than the larger ones
    bool slices_tail;  // a last, partly filled round of tiles may be cut into K slices (tiles with triangular forms only)
    double split_gain; // factor on `eff` in a launch that cuts K into ranges (the 64x128 FP32 tile: 4-6 % ahead of 128x64 there, behind it everywhere else)
    size_t smem_deep[4];
    void (*plain_deep[4])(const GemmParams<T>);
    void (*splitk_deep[4])(const GemmParams<T>);
    size_t smem;     // largest of the four variants (for the residency estimate)
    size_t smem_of[4];
    bool has_splitk;
    // Tile choice model: fraction of MFMA peak the tile is credited with.  Fitted to the choices that
    // measure best at 1000..5000, where the short K loops cost the small tiles more than at 8192^3
    // (there the five FP32 tiles run at .953 / .943 / .93 / .915 / .88; crediting them with those
    // figures moved 3000 x 1500 x 1000 from 105 to 98 TFLOP/s and 4097 x 4095 x 1031 from 125 to 122).
    double eff;
    double alone;    // further factor when a workgroup has its CU to itself (at most 256 tiles)
    double eff_tri;  // `eff` for products with a triangular A or B (TRMM, SYMM passes); 0: not offered
    // Fixed time of a workgroup (first loads, write-back of C) as a depth: the cost of a tile is taken
    // times (1 + k0 / K).  On large C with short K the write-back is what bounds the rate, and the
    // small tiles, more of them per CU, overlap it better (8192 x 8192 x 64 FP64: 35.7 TFLOP/s with 64x64 tiles,
    // 31.6 with 128x128; rates over K fit T(K) = T_inf K / (K + k0) with k0 = 68 and 95).  0: no such term.
    double eff_tri_c;  // `eff` for products that store one triangle of C (SYRK, HERK, ...); default: eff
    double k0;
    double tail_extra;  // rounds that a sliced tail adds on top of 1 / slices (reduction pass, uneven slices)
    // index: (transA ? 2 : 0) | (transB ? 1 : 0)
    void (*plain[4])(const GemmParams<T>);
    void (*splitk[4])(const GemmParams<T>);
    void (*tri[4])(const GemmParams<T>);  // variants that honour the triangular fields (or null)
    // Variants for leading dimensions beyond the reach of a panel-wide buffer descriptor (one descriptor
    // per row, see PanelLoader); built for the smallest tile of each type only.
    void (*plain_wide[4])(const GemmParams<T>);
    void (*splitk_wide[4])(const GemmParams<T>);
    void (*tri_wide[4])(const GemmParams<T>);
};


template <typename T, int BM, int BN, int BK, int WM, int WN, int MINW, bool WITH_SPLITK, bool WITH_TRI = false, int BK_DEEP = 0, bool WITH_WIDE = false>
TileEntry<T> make_tile_entry(double eff, double alone = 0.85, double eff_tri = -1.0, double k0 = 0.0,
                             double tail_extra = 0.05, double eff_tri_c = -1.0) {
    typedef GemmCfg<T, BM, BN, BK, WM, WN, false, false> Cfg;
    TileEntry<T> e;
    e.bm = BM; e.bn = BN; e.bk = BK; e.threads = Cfg::NT; e.has_splitk = WITH_SPLITK;
    e.split_gain = 1.0;
    e.streamed_gain = 1.0;
    e.slices_tail = WITH_TRI;
    e.eff = eff; e.alone = alone; e.eff_tri = eff_tri < 0 ? eff : eff_tri; e.k0 = k0; e.tail_extra = tail_extra;
    e.eff_tri_c = eff_tri_c < 0 ? eff : eff_tri_c;
    // LDS need depends on the layout of the B panel (transB): index as plain[].
    e.smem_of[0] = GemmCfg<T, BM, BN, BK, WM, WN, false, true>::SMEM;
    e.smem_of[1] = GemmCfg<T, BM, BN, BK, WM, WN, false, false>::SMEM;
    e.smem_of[2] = GemmCfg<T, BM, BN, BK, WM, WN, true, true>::SMEM;
    e.smem_of[3] = GemmCfg<T, BM, BN, BK, WM, WN, true, false>::SMEM;
    e.smem = e.smem_of[0];
    for (int i = 1; i < 4; ++i) e.smem = e.smem_of[i] > e.smem ? e.smem_of[i] : e.smem;
    // A is k-contiguous when transposed; B is k-contiguous when NOT transposed.
    e.plain[0] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, true, false, MINW>;   // NN
    e.plain[1] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, false, false, MINW>;  // NT
    e.plain[2] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, true, false, MINW>;    // TN
    e.plain[3] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, false, false, MINW>;   // TT
    if constexpr (WITH_SPLITK) {
        e.splitk[0] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, true, true, MINW>;
        e.splitk[1] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, false, true, MINW>;
        e.splitk[2] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, true, true, MINW>;
        e.splitk[3] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, false, true, MINW>;
    } else {
        for (int i = 0; i < 4; ++i) e.splitk[i] = nullptr;
    }
    if constexpr (WITH_WIDE) {
        static_assert(WITH_SPLITK && WITH_TRI, "the wide-ld tile serves every kind of launch");
        e.plain_wide[0] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, true, false, MINW, false, true>;
        e.plain_wide[1] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, false, false, MINW, false, true>;
        e.plain_wide[2] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, true, false, MINW, false, true>;
        e.plain_wide[3] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, false, false, MINW, false, true>;
        e.splitk_wide[0] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, true, true, MINW, false, true>;
        e.splitk_wide[1] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, false, true, MINW, false, true>;
        e.splitk_wide[2] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, true, true, MINW, false, true>;
        e.splitk_wide[3] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, false, true, MINW, false, true>;
        e.tri_wide[0] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, true, false, MINW, true, true>;
        e.tri_wide[1] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, false, false, MINW, true, true>;
        e.tri_wide[2] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, true, false, MINW, true, true>;
        e.tri_wide[3] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, false, false, MINW, true, true>;
    } else {
        for (int i = 0; i < 4; ++i) { e.plain_wide[i] = nullptr; e.splitk_wide[i] = nullptr; e.tri_wide[i] = nullptr; }
    }
    // The same tile with panels of depth BK_DEEP (see TileEntry::bk_deep).
    if constexpr (BK_DEEP > 0) {
        e.bk_deep = BK_DEEP;
        e.deep_gain = 1.05;
        e.smem_deep[0] = GemmCfg<T, BM, BN, BK_DEEP, WM, WN, false, true>::SMEM;
        e.smem_deep[1] = GemmCfg<T, BM, BN, BK_DEEP, WM, WN, false, false>::SMEM;
        e.smem_deep[2] = GemmCfg<T, BM, BN, BK_DEEP, WM, WN, true, true>::SMEM;
        e.smem_deep[3] = GemmCfg<T, BM, BN, BK_DEEP, WM, WN, true, false>::SMEM;
        e.plain_deep[0] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, false, true, false, MINW>;
        e.plain_deep[1] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, false, false, false, MINW>;
        e.plain_deep[2] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, true, true, false, MINW>;
        e.plain_deep[3] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, true, false, false, MINW>;
        if constexpr (WITH_SPLITK) {
            e.splitk_deep[0] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, false, true, true, MINW>;
            e.splitk_deep[1] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, false, false, true, MINW>;
            e.splitk_deep[2] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, true, true, true, MINW>;
            e.splitk_deep[3] = gemm_mfma_kernel<T, BM, BN, BK_DEEP, WM, WN, true, false, true, MINW>;
        } else {
            for (int i = 0; i < 4; ++i) e.splitk_deep[i] = nullptr;
        }
    } else {
        e.bk_deep = 0;
        e.deep_gain = 1.0;
        for (int i = 0; i < 4; ++i) { e.smem_deep[i] = 0; e.plain_deep[i] = nullptr; e.splitk_deep[i] = nullptr; }
    }
    if constexpr (WITH_TRI) {
        e.tri[0] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, true, false, MINW, true>;
        e.tri[1] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, false, false, false, MINW, true>;
        e.tri[2] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, true, false, MINW, true>;
        e.tri[3] = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, true, false, false, MINW, true>;
    } else {
        for (int i = 0; i < 4; ++i) e.tri[i] = nullptr;
    }
    return e;
}

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// 1-D grids are built from 64-bit products; HIP takes 32-bit block counts.
static const int64_t kMaxGrid = 0x7fffffffLL;

template <typename T> static char type_letter() {
    return Elem<T>::CPLX ? (sizeof(T) == 8 ? 'c' : 'z') : (sizeof(T) == 4 ? 's' : 'd');
}

// Records the launch for clblasAmdLastDispatch and, with CLBLAS_AMD_LOG=1, prints it.
template <typename T>
static DispatchRecord &note_launch(const char *kernel, int bm, int bn, int bk, int threads, bool tA, bool tB, int M,
                                   int N, int K, unsigned gx, unsigned gy) {
    DispatchRecord &r = dispatch_record();
    r.type = type_letter<T>(); r.kernel = kernel;
    r.bm = bm; r.bn = bn; r.bk = bk; r.threads = threads;
    r.trans_a = tA; r.trans_b = tB; r.M = M; r.N = N; r.K = K;
    r.splits = 1; r.tail_slices = 1; r.tri = 0;
    r.grid_x = gx; r.grid_y = gy;
    r.launches++;
    return r;
}
static inline void log_dispatch(const DispatchRecord &r) {
    if (knobs().log)
        fprintf(stderr, "clblas_amd: %s<%c,%dx%dx%d> %c%c M=%d N=%d K=%d grid=(%u,%u) block=%d splits=%d tail_slices=%d tri=%d\n",
                r.kernel, r.type, r.bm, r.bn, r.bk, r.trans_a ? 'T' : 'N', r.trans_b ? 'T' : 'N', r.M, r.N, r.K, r.grid_x,
                r.grid_y, r.threads, r.splits, r.tail_slices, r.tri);
}

// Scratch for this call: the caller's fixed buffer if there is one, else the per-stream cache.
static inline hipError_t scratch_for(hipStream_t stream, size_t bytes, const FixedScratch *fixed, void **out) {
    if (fixed) {
        *out = nullptr;
        if (bytes > fixed->bytes) return hipErrorOutOfMemory;
        *out = fixed->ptr;
        return hipSuccess;
    }
    return workspace_get(stream, bytes, 0, out);
}

// Chooses tile and split count.  The reference keys its choice on M*N brackets and
// divisibility (AutoGemmParameters.py:8-55); here remainders are handled in-kernel, so the
// question is only how well a tile shape fills 256 CUs.  Workgroups that share a CU share
// its MFMA pipes, so time is quantised per CU, not per resident workgroup:
//     time ~ ceil(tiles / 256) * BM * BN / eff
// with eff the measured MFMA efficiency of that tile shape on large problems (padding is
// paid for automatically because whole tiles are counted; for SYRK only the tiles of the
// stored triangle count).  The smallest tile adds a K
// split when even it cannot give every CU a workgroup.
// Number of bm x bn tiles of an M x N matrix that touch its lower (tri_c == 1) or upper (2)
// triangle; all of them for tri_c == 0.  Row r holds the columns [0, last] resp. [first, end).
static inline int64_t active_tiles(int M, int N, int bm, int bn, int tri_c) {
    const int64_t tiles_m = ceil_div64(M, bm), tiles_n = ceil_div64(N, bn);
    if (!tri_c) return tiles_m * tiles_n;
    int64_t total = 0;
    for (int64_t r = 0; r < tiles_m; ++r) {
        if (tri_c == 1) {
            const int64_t last = (r * bm + bm - 1) / bn;
            total += last + 1 < tiles_n ? last + 1 : tiles_n;
        } else {
            const int64_t first = (r * bm) / bn;
            total += first < tiles_n ? tiles_n - first : 0;
        }
    }
    return total;
}

// Sliced tail: with `t` equally long tiles over 256 CUs the last round holds r = t mod 256
// tiles and leaves the other CUs idle.  Cutting each of those r tiles into s = 256 / r K
// ranges fills the round and shortens it to 1/s (plus a small reduction pass).  Returns s, or
// 1 where that does not apply or does not pay: fewer than one full round (split-K covers
// that case), more than 24 rounds (the tail is a few percent), slices under 8 panels.
static inline int tail_slices_for(int64_t t, int K, int bk, bool allowed) {
    const int64_t kCUs = 256;
    if (!allowed || t <= kCUs || t / kCUs > 24) return 1;
    const int64_t r = t % kCUs;
    if (r == 0) return 1;
    int64_t s = kCUs / r;
    const int64_t by_k = K / (8 * bk);
    if (s > by_k) s = by_k;
    if (s > 16) s = 16;
    return s < 2 ? 1 : (int)s;
}

// K split of a tile shape that cannot give every CU a workgroup: about two workgroups per CU,
// at least four panels per range.
static inline int splits_for(int64_t t, int K, int bk) {
    const int64_t kCUs = 256;
    if (t >= kCUs || K < 8 * bk) return 1;
    int64_t want = (2 * kCUs) / t;
    const int64_t max_by_k = K / (4 * bk);
    if (want > max_by_k) want = max_by_k;
    // (up to 512 ranges: a single tile with a depth in the millions still gets a workgroup on every CU;
    // DGEMM TN 64 x 64 x 2^21 in 64 ranges 6.1 ms, in 512 ranges see the tile comments)
    if (want > 512) want = 512;
    return want < 1 ? 1 : (int)want;
}

// Cost of the pass that adds up the K ranges, in the tile model's unit (elements of C per CU at
// the MFMA peak over the whole depth K): a dependent launch of about 5 us plus the partial sums
// written and read back at about 4 TB/s.  Fitted to FP64 with 64x64 tiles, us by ranges (model):
// 512^3 1: 21 (22), 4: 15 (16), 8: 18 (17.5); 960 x 960 x 256 1: 14 (13), 2: 22 (22); 640 x 640 x 512
// 1: 20.9 (21.9), 5: 19.1 (20), each with 4 us for the first launch.
template <typename T> static double split_overhead_cost(int M, int N, int K, int splits) {
    const double peak_per_cu = (sizeof(typename Elem<T>::Real) == 4 ? 157.3e12 : 78.6e12) / 256.0;
    const double flops_per_step = Elem<T>::CPLX ? 8.0 : 2.0;
    const double seconds = 5e-6 + (double)(splits + 1) * M * N * sizeof(T) / 4e12;
    return seconds * peak_per_cu / (flops_per_step * K);
}

template <typename T>
static void choose_tile(const TileEntry<T> *tab, int ntab, int M, int N, int K, int force, bool need_tri, int tri_c,
                        bool tri_operand, bool tail_ok, int *tile_out, int *splits_out, double *costs_out = nullptr,
                        double *chosen_cost = nullptr) {
    const int64_t kCUs = 256;
    int pick = ntab - 1;  // table is ordered large -> small
    bool pick_split = true;
    int model_splits = -1;  // ranges chosen by the cost model for the smallest tile (-1: none)
    if (force >= 0 && force < ntab && (!need_tri || tab[force].tri[0])) {
        pick = force;
    } else {
        // Cost of tile i with its depth cut into s ranges: the ranges fill the CUs that the tiles
        // alone leave idle, at the price of the pass that adds them up.
        // Operands beyond the 256 MB of the memory-side cache are streamed from HBM, and a workgroup alone on
        // its CU then has too few loads in flight for the latency: SGEMM 16384 x 64 x 10000 (655 MB of A, one
        // 64x64 tile per CU) runs at 105 TFLOP/s where 1024 x 1024 x 8192 (64 MB, the same 256 tiles) runs at 125.
        const bool streamed = ((double)M * K + (double)K * N) * sizeof(T) > 256e6;
        const double lone_stream = streamed ? 0.85 : 1.0;
        auto split_cost = [&](int i, int64_t t, int s) {
            const double alone = t * s <= kCUs ? tab[i].alone * lone_stream : 1.0;
            const double deep = (tab[i].bk_deep > 0 && (K / s >= 1024 || (K / s >= 512 && t * s <= kCUs))) ? tab[i].deep_gain : 1.0;
            return (double)ceil_div64(t * s, kCUs) * tab[i].bm * tab[i].bn / (s * tab[i].eff * tab[i].split_gain * deep * alone) +
                   split_overhead_cost<T>(M, N, K, s);
        };
        const bool split_model = knobs().split_model != 0 && !need_tri;
        double best = 0, best_split = 0, cost_last = 0;
        int pick_of_split = -1;
        bool have = false;
        for (int i = 0; i < ntab; ++i) {
            if (need_tri && !tab[i].tri[0]) continue;
            if (tri_operand && tab[i].eff_tri <= 0) continue;
            const int64_t t = active_tiles(M, N, tab[i].bm, tab[i].bn, tri_c);
            double rounds = (double)ceil_div64(t, kCUs);
            const int ts = tail_slices_for(t, K, tab[i].bk, tail_ok && tab[i].tri[0] && tab[i].slices_tail);
            // A sliced tail round lasts 1 / ts of a round plus what does not shrink with the depth of a slice
            // (its first loads, the partial tiles written and added up by a second pass): about 120 deep.
            if (ts > 1) {
                // With a single whole round every CU holds one whole tile next to its slice, and once the slice
                // is done that tile runs at the rate of a workgroup alone - which matters where the operands are
                // streamed: SGEMM 10000 x 100 x 10000 on 64x64 tiles, 256 whole + 58 x 4 slices, takes 1.25 x the
                // 0.199 ms of 16384 x 64 x 10000 (one tile per CU), 1.7 rounds at the pair rate, not 1.3;
                // 5000 x 200 x 8192 (164 MB, each panel of A used by four tiles) takes the 1.3.
                const double lone = (streamed && t / kCUs == 1) ? (tab[i].alone < 0.8 ? tab[i].alone : 0.8) : 1.0;
                rounds = ((double)(t / kCUs) + 1.0 / ts) / lone + tab[i].tail_extra + 120.0 / K;
            }
            // A triangular operand makes the tiles differ in depth (half of the full depth on
            // average, started deepest first): the CUs share the total evenly up to a fraction
            // of one full-depth tile, fitted to STRMM / DTRMM 4096 and 8192 (STRMM 4096: 256x128
            // tiles 0.77 ms, 128x128 0.60 ms, 64x64 0.67 ms).
            if (tri_operand) rounds = (double)t / (2.0 * kCUs) + 0.4;
            double eff = tri_operand ? tab[i].eff_tri : tri_c ? tab[i].eff_tri_c : tab[i].eff;
            if (streamed) eff *= tab[i].streamed_gain;
            // (credited up to three rounds of tiles: beyond that the small tile's memory traffic costs more
            // than the deeper panels gain - 2000^3 FP32 128 TFLOP/s with 128x64 tiles, 119 with 64x64)
            if (!need_tri && ts <= 1 && tab[i].bk_deep > 0 && ((K >= 1024 && t <= 3 * kCUs) || (K >= 512 && t <= kCUs))) eff *= tab[i].deep_gain;
            double cost = rounds * tab[i].bm * tab[i].bn / eff;
            if (t <= kCUs) cost /= tab[i].alone * lone_stream;  // a workgroup alone on its CU cannot keep the MFMA pipes full
            cost *= 1.0 + tab[i].k0 / K;
            if (costs_out) costs_out[i] = cost;
            if (i == ntab - 1) cost_last = cost;
            if (!have || cost < best) { best = cost; pick = i; have = true; }
            // Small C, deep K: the larger tiles with a K split, ranges of at least 512 and 32 panels.
            if (split_model && tab[i].has_splitk && i != ntab - 1) {
                const int s = splits_for(t, K, tab[i].bk);
                if (s > 1 && K / s >= 512 && K / s >= 32 * tab[i].bk) {
                    const double c = split_cost(i, t, s);
                    if (pick_of_split < 0 || c < best_split) { best_split = c; pick_of_split = i; }
                }
            }
        }
        // The smallest tile, when even it cannot give every CU a workgroup, takes the number of ranges
        // that the same model prices lowest, one range included (short K: the pass that adds the
        // ranges up costs more than the idle CUs; 960 x 960 x 256 FP64 22 -> 14 us, 512^3 18 -> 15 us).
        // A larger tile is split only where the model puts it 10 % ahead of what would run otherwise (the model
        // is hard on one round of unsplit small tiles over a deep K: DGEMM 1024 x 1024 x 8192 and 2048 x 512 x 8192
        // run 69.1 TFLOP/s on 256 tiles of 64x64 and 66.6 on 128x128 tiles in 8 ranges, which it had 7 % ahead;
        // 896 x 896 x 8192, 60.4 against 53.1 the other way, it has further ahead than that).
        // Tiles below it in size (listed before it, without K ranges of their own) fill the CUs of a small product
        // in one launch; against them the last tile is priced with its best number of ranges as well.
        const int last = ntab - 1;
        int last_splits = -1;  // -1: the rule without the model
        const bool below_last = pick != last && tab[pick].bm * tab[pick].bn < tab[last].bm * tab[last].bn;
        if (split_model && (pick == last || below_last) && tab[last].has_splitk) {
            const int64_t t = active_tiles(M, N, tab[last].bm, tab[last].bn, 0);
            const int s_max = splits_for(t, K, tab[last].bk);
            if (s_max > 1) {
                static const int kCand[] = {2, 3, 4, 5, 6, 8, 10, 12, 16, 20, 24, 32, 40, 48, 64, 96, 128, 192, 256, 384};
                double c_best = cost_last;  // the cost of one range
                int s_best = 1;
                for (int s : kCand) {
                    if (s >= s_max) break;
                    const double c = split_cost(last, t, s);
                    if (c < c_best) { c_best = c; s_best = s; }
                }
                const double c = split_cost(last, t, s_max);
                if (c < c_best) { c_best = c; s_best = s_max; }
                if (pick == last || c_best < best) { pick = last; best = c_best; last_splits = s_best; }
            }
        }
        if (pick_of_split >= 0) {
            // (the margin is for a split against an unsplit launch; where the smallest tile is itself cut into
            // ranges both pay the pass that adds them up, and the prices are compared as they are)
            const double margin = (pick == last && last_splits > 1) ? 1.0 : 1.10;
            if (best_split * margin < best) { pick = pick_of_split; best = best_split; }
            else pick_of_split = -1;
        }
        if (chosen_cost) *chosen_cost = best;
        pick_split = pick == last || pick == pick_of_split;
        if (pick == last) model_splits = last_splits;
    }
    int splits = 1;
    if (tab[pick].has_splitk && !need_tri) {
        const int by_rule = splits_for(ceil_div64(M, tab[pick].bm) * ceil_div64(N, tab[pick].bn), K, tab[pick].bk);
        if (model_splits >= 0) splits = model_splits;
        else if (pick_split) splits = by_rule;
        const int forced = knobs().splits;  // debug: number of K ranges
        const int most = K / (4 * tab[pick].bk) > 0 ? K / (4 * tab[pick].bk) : 1;  // 4 panels per range
        if (forced > 0) splits = forced < most ? forced : most;
    }
    *tile_out = pick;
    *splits_out = splits;
}

template <typename T>
static hipError_t run_gemm_whole(const TileEntry<T> *tab, int ntab, bool tA, bool tB, bool cA, bool cB, int M,
                                 int N, int K, T alpha, const T *A, int64_t lda, const T *B, int64_t ldb,
                                 T beta, T *C, int64_t ldc, hipStream_t stream, const GemmTri *tri = nullptr,
                                 const FixedScratch *fixed = nullptr) {
    const bool need_tri = tri && tri->any();
    if (need_tri && K == 0) return hipErrorInvalidValue;  // callers reject empty products earlier
    if (K == 0) {
        int mb = (int)ceil_div64(M, 256);
        if ((int64_t)mb * N > kMaxGrid) return hipErrorInvalidValue;
        log_dispatch(note_launch<T>("scale_c_kernel", 0, 0, 0, 256, tA, tB, M, N, K, (unsigned)((int64_t)mb * N), 1));
        return launch_kernel(scale_c_kernel<T>, dim3((unsigned)((int64_t)mb * N)), dim3(256), 0, stream, M, N, mb,
                             beta, C, ldc);
    }
    // 32-bit panel offsets: (tile edge or panel depth) * ld * sizeof(T) must stay < 2^31.  Beyond
    // that the smallest tile's wide-ld kernels take over (one buffer descriptor per panel row).
    const int64_t max_edge = 256;
    const int64_t ld_limit = (int64_t)0x7fffffff / (max_edge * (int64_t)sizeof(T)) - 8;
    const bool wide = lda > ld_limit || ldb > ld_limit || knobs().wide_ld != 0;
    if (wide && !tab[ntab - 1].plain_wide[0]) return hipErrorNotSupported;

    int tile, splits;
    // The tail may be sliced unless tiles differ in depth (triangular operands).
    const bool tail_ok = !(need_tri && (tri->tri_a || tri->tri_b)) && knobs().tail != 0;
    choose_tile(tab, ntab, M, N, K, wide ? ntab - 1 : knobs().gemm_tile, need_tri, need_tri ? tri->tri_c : 0,
                need_tri && (tri->tri_a || tri->tri_b), tail_ok, &tile, &splits);
    const TileEntry<T> &e = tab[tile];

    GemmParams<T> p;
    p.A = A; p.B = B; p.C = C;
    p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    // op(A) is M x K: stored M x K (ld rows = M) when not transposed, K x M when transposed.
    p.a_bytes = (tA ? ((int64_t)(M - 1) * lda + K) : ((int64_t)(K - 1) * lda + M)) * (int64_t)sizeof(T);
    p.b_bytes = (tB ? ((int64_t)(K - 1) * ldb + N) : ((int64_t)(N - 1) * ldb + K)) * (int64_t)sizeof(T);
    p.M = M; p.N = N; p.K = K;
    p.conj_a = cA ? 1 : 0; p.conj_b = cB ? 1 : 0;
    p.alpha = alpha; p.beta = beta;
    p.tiles_m = (int)ceil_div64(M, e.bm);
    p.tiles_n = (int)ceil_div64(N, e.bn);
    // Tile rows walked together: the workgroups resident on one XCD should cover a roughly
    // square block of C (measured L2-miss traffic at 8192^3 FP32, 128x128 tiles: 9.3 GB with
    // 4 rows, 7.4 GB with 8, 11.4 GB with 16).
    // With R workgroups resident per XCD that block is group_m x R/group_m tiles:
    // group_m ~ sqrt(R * BN / BM), R = 32 CUs x (2 or 4 workgroups, by LDS use).  ZGEMM with
    // its 128x64 tiles fetched 61 GB with 4 rows and 108 GB with 8.
    int gm_default = 1;
    {
        const double resident = e.smem_of[0] > 40 * 1024 ? 64.0 : 128.0;
        while ((double)(2 * gm_default) * (2 * gm_default) <= resident * e.bn / e.bm && gm_default < 16) gm_default *= 2;
    }
    p.group_m = knobs().group_m > 0 ? knobs().group_m : gm_default;
    if (p.group_m > p.tiles_m) p.group_m = p.tiles_m;
    if (p.group_m < 1) p.group_m = 1;
    p.xcd_remap = knobs().xcd;
    p.stagger = 0;
    p.ws = nullptr; p.ws_ld = 0; p.ws_slice = 0;
    p.k_per_split = K;
    p.tri_c = p.tri_a = p.tri_b = p.unit_a = p.unit_b = p.rev_m = p.rev_n = p.herm_c = 0;
    p.tail_first = 0; p.tail_slices = 1; p.tail_kps = K;
    const int idx = (tA ? 2 : 0) | (tB ? 1 : 0);
    int64_t ntiles = (int64_t)p.tiles_m * p.tiles_n;
    if (ntiles > 0x7fffffffLL) return hipErrorInvalidValue;

    auto fn = wide ? e.plain_wide[idx] : e.plain[idx];
    int bk_used = e.bk;
    if (need_tri) {
        if (!e.tri[idx]) return hipErrorNotSupported;
        fn = wide ? e.tri_wide[idx] : e.tri[idx];
        p.tri_c = tri->tri_c; p.tri_a = tri->tri_a; p.tri_b = tri->tri_b;
        p.unit_a = tri->unit_a; p.unit_b = tri->unit_b;
        p.herm_c = tri->herm_c;
        if (p.tri_c) ntiles = active_tiles(M, N, e.bm, e.bn, p.tri_c);  // the kernel enumerates the same set
        if (p.tri_a || p.tri_b) {
            // Tiles differ in depth (by tile row for a triangular A, by tile column for B):
            // start them strictly deepest first - row by row resp. column by column - and deal
            // consecutive tiles to different XCDs so that every XCD gets the same mix.
            p.rev_m = p.tri_a == 1;
            p.rev_n = p.tri_b == 1;
            p.group_m = p.tri_a ? 1 : p.tiles_m;
            p.xcd_remap = 0;
        }
    }
    int64_t grid_x = ntiles;
    if (splits <= 1 && e.tri[idx] && e.slices_tail) {
        const int ts = tail_slices_for(ntiles, K, e.bk, tail_ok);
        if (ts > 1) {
            const int64_t kps = ceil_div64(ceil_div64(K, ts), e.bk) * e.bk;
            const int slices = (int)ceil_div64(K, kps);
            const int64_t r = ntiles % 256;
            void *w = nullptr;
            const size_t need = (size_t)(r * slices) * e.bm * e.bn * sizeof(T);
            if (slices > 1) {
                hipError_t we = scratch_for(stream, need, fixed, &w);
                // A caller that must not allocate gets an error rather than another schedule (its
                // results then never depend on what happens to be allocated); so does a stream
                // under capture.  Plain out-of-memory falls back to the unsliced schedule.
                if (we != hipSuccess && (fixed || we != hipErrorOutOfMemory)) return we;
            }
            if (slices > 1 && w) {
                fn = wide ? e.tri_wide[idx] : e.tri[idx];
                p.tail_first = (int)(ntiles - r);
                p.tail_slices = slices;
                p.tail_kps = (int)kps;
                p.ws = (T *)w;
                grid_x = (ntiles - r) + r * slices;
            }
        }
    }
    if (splits > 1) {
        int64_t kps = ceil_div64(ceil_div64(K, splits), e.bk) * e.bk;
        splits = (int)ceil_div64(K, kps);
        if (splits > 1) {
            p.k_per_split = (int)kps;
            p.ws_ld = ((int64_t)M + 63) / 64 * 64;
            p.ws_slice = p.ws_ld * N;
            void *w = nullptr;
            hipError_t we = scratch_for(stream, (size_t)(p.ws_slice * splits) * sizeof(T), fixed, &w);
            if (we != hipSuccess) return we;
            p.ws = (T *)w;
            fn = wide ? e.splitk_wide[idx] : e.splitk[idx];
        }
    }
    // The late start that keeps the workgroups of a CU out of lockstep (see the kernel).  It was needed
    // where a launch is not a whole number of rounds of 2 x 256 workgroups (3584^3 FP64: 54 -> 69 TFLOP/s)
    // until the sliced tail took that case over; what is left of it is the gain with short K ranges, where
    // the epilogue of one workgroup overlaps the K loop of its neighbour (8192 x 8192 x 512 FP64: 66.6 -> 68.2).
    {
        const int64_t wgs = grid_x * (splits > 1 ? splits : 1);
        const int mode = knobs().stagger;  // 0: never, 2: whatever the type
        // FP64 only: with the sliced tail in place the FP32 kernels gain nothing from it any more (35 shapes, on
        // against off: within 0.5 % either way) and the 128x64 tile loses 8-10 % with it on TN operands
        // (3000^3 120 against 131 TFLOP/s, 3072^3 127 against 138, 3328^3 124 against 139), while DGEMM still takes
        // + 2.4 % at 8192 x 8192 x 512, + 1.3 % at 12000 x 12000 x 512 and + 7 % at 4200 x 1700 x 900 from it.
        const bool type_gains = sizeof(typename Elem<T>::Real) == 8 || mode == 2;
        // ... and only with K ranges of up to 2048: beyond that it is neutral or costs a percent (DGEMM 3072^3
        // 71.4 -> 70.5, 2560^3 68.6 -> 68.0; 3584^3, 3700^3, 5000^3, 6000^3, 6144^3 within 0.3 %).
        p.stagger = mode != 0 && type_gains && wgs > 512 && !(p.tri_a || p.tri_b) && p.k_per_split <= 2048;
    }
    size_t smem = e.smem_of[idx];
    const int threads = e.threads;
    if (e.bk_deep > 0 && !wide && !need_tri && p.tail_slices <= 1 && knobs().deep_panels != 0) {
        // A long K range per workgroup: the variant with deeper panels (K ranges are cut at multiples
        // of the tile's own depth, so they have to be multiples of the deeper one too).
        const int krange = splits > 1 ? p.k_per_split : K;
        // From 1024 deep; from 512 where the launch is a single round of workgroups (there the shorter loop
        // wins - DGEMM 512 x 2048 x 512 22.2 -> 21.0 us, 1024 x 1024 x 768 31.1 -> 29.3 - while launches of
        // several rounds lose the workgroups per CU that the larger LDS stage costs: 4096 x 4096 x 512 +3 %).
        const int64_t wgs = grid_x * (splits > 1 ? splits : 1);
        const int deep_from = knobs().deep_panels > 2 ? knobs().deep_panels : (wgs <= 256 ? 512 : 1024);  // (knob above 2: that threshold)
        if ((krange >= deep_from || knobs().deep_panels == 2) && (splits <= 1 || p.k_per_split % e.bk_deep == 0)) {
            fn = splits > 1 ? e.splitk_deep[idx] : e.plain_deep[idx];
            smem = e.smem_deep[idx];
            bk_used = e.bk_deep;
        }
    }
    if (smem > 64 * 1024) {
        hipError_t err = ensure_dynamic_lds((const void *)fn, smem);
        if (err != hipSuccess) return err;
    }
    if (grid_x > kMaxGrid) return hipErrorInvalidValue;
    {
        DispatchRecord &rec = note_launch<T>(wide ? "gemm_mfma_kernel(wide ld)" : "gemm_mfma_kernel", e.bm, e.bn, bk_used, threads, tA, tB, M, N, K,
                                             (unsigned)grid_x, (unsigned)splits);
        rec.splits = splits; rec.tail_slices = p.tail_slices; rec.tri = need_tri ? 1 : 0;
        log_dispatch(rec);
    }
    hipError_t err = launch_kernel(fn, dim3((unsigned)grid_x, (unsigned)splits), dim3(threads), smem, stream, p);
    if (err != hipSuccess) return err;
    if (p.tail_slices > 1) {
        const int64_t r = ntiles - p.tail_first;
        dispatch_record().launches++;
        err = launch_kernel(tail_reduce_kernel<T>, dim3((unsigned)ceil_div64((int64_t)e.bm * e.bn, 256), (unsigned)r),
                            dim3(256), 0, stream, p, e.bm, e.bn);
        if (err != hipSuccess) return err;
    }
    if (splits > 1) {
        dispatch_record().launches++;
        // Many ranges over a small C: the pass with eight threads per element (all loads of an element in
        // flight at once; SGEMM 127 x 129 x 8192 in 37 ranges: 13.7 -> 12.4 us per call); otherwise one
        // thread per element.
        if (splits > 8 && splits <= 64 && (int64_t)M * N <= (1 << 20)) {
            int mb = (int)ceil_div64(M, 32);
            err = launch_kernel(splitk_reduce_wide_kernel<T>, dim3((unsigned)((int64_t)mb * N)), dim3(256), 0, stream,
                                p.ws, p.ws_ld, p.ws_slice, splits, M, N, mb, alpha, beta, C, ldc);
        } else {
            int mb = (int)ceil_div64(M, 256);
            if ((int64_t)mb * N > kMaxGrid) return hipErrorInvalidValue;
            err = launch_kernel(splitk_reduce_kernel<T>, dim3((unsigned)((int64_t)mb * N)), dim3(256), 0, stream, p.ws,
                                p.ws_ld, p.ws_slice, splits, M, N, mb, alpha, beta, C, ldc);
        }
    }
    return err;
}

// A dimension that is a few rows or columns more than a whole number of tiles costs a whole extra row or
// column of tiles that compute on padding (SGEMM 8193^3: 138 TFLOP/s against 148 at 8192^3; 10000 = 39 x 256 + 16).
// Where the model prices it lower, the product is made in two launches instead: the part up to the last
// multiple of 128, and the strip of at most 64 rows (or columns: one row of the smallest tile) as a product of
// its own - a skinny one, which gets small tiles and a K split.  Both write disjoint parts of C with the same
// alpha and beta.  The parts are priced by the same model as the whole (same K, so the costs add); a launch
// costs about 3 us on top.  Plain products only (no triangular structure, no forced tile, no wide leading
// dimensions).  (depth: 0 the caller's product, 1 a main part - it may lose a strip of the other dimension -,
// 2 a strip: made whole.)
template <typename T>
static hipError_t run_gemm_colmajor(const TileEntry<T> *tab, int ntab, bool tA, bool tB, bool cA, bool cB, int M,
                                    int N, int K, T alpha, const T *A, int64_t lda, const T *B, int64_t ldb,
                                    T beta, T *C, int64_t ldc, hipStream_t stream, const GemmTri *tri = nullptr,
                                    const FixedScratch *fixed = nullptr, int depth = 0) {
    const int mode = knobs().peel;  // 0: never, 1: where the model prices it lower, 2: wherever a strip exists (tests)
    const bool plain = !(tri && tri->any()) && K > 0 && knobs().gemm_tile < 0 && knobs().wide_ld == 0;
    if (mode != 0 && plain && depth < 2) {
        const int64_t ld_limit = (int64_t)0x7fffffff / (256 * (int64_t)sizeof(T)) - 8;
        const int kStrip = 64, kEdge = 128, kLeast = 1024;
        const int rm = M % kEdge, rn = N % kEdge;
        const bool can_m = rm > 0 && rm <= kStrip && M - rm >= kLeast, can_n = rn > 0 && rn <= kStrip && N - rn >= kLeast;
        if ((can_m || can_n) && lda <= ld_limit && ldb <= ld_limit) {
            const bool tail_ok = knobs().tail != 0;
            auto price = [&](int m, int n) {
                int t, sp;
                double c = 0;
                choose_tile(tab, ntab, m, n, K, -1, false, 0, false, tail_ok, &t, &sp, nullptr, &c);
                return c;
            };
            const double peak_per_cu = (sizeof(typename Elem<T>::Real) == 4 ? 157.3e12 : 78.6e12) / 256.0;
            const double launch = 3e-6 * peak_per_cu / ((Elem<T>::CPLX ? 8.0 : 2.0) * K);
            const double whole = price(M, N);
            // the dimension whose strip saves more goes first; the main part is asked again about the other
            double gain_m = -2e300, gain_n = -2e300;
            if (can_m) gain_m = whole - (price(M - rm, N) + price(rm, N) + launch);
            if (can_n) gain_n = whole - (price(M, N - rn) + price(M, rn) + launch);
            const double least = mode == 2 ? -1e300 : 0.005 * whole;
            const bool peel_m = can_m && gain_m > least && gain_m >= gain_n;
            const bool peel_n = !peel_m && can_n && gain_n > least;
            if (peel_m) {
                const int m0 = M - rm;
                hipError_t e = run_gemm_colmajor(tab, ntab, tA, tB, cA, cB, m0, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream,
                                                 tri, fixed, depth + 1);
                if (e != hipSuccess) return e;
                const T *As = tA ? A + (int64_t)m0 * lda : A + m0;  // rows m0.. of op(A)
                return run_gemm_colmajor(tab, ntab, tA, tB, cA, cB, rm, N, K, alpha, As, lda, B, ldb, beta, C + m0, ldc, stream,
                                         tri, fixed, 2);
            }
            if (peel_n) {
                const int n0 = N - rn;
                hipError_t e = run_gemm_colmajor(tab, ntab, tA, tB, cA, cB, M, n0, K, alpha, A, lda, B, ldb, beta, C, ldc, stream,
                                                 tri, fixed, depth + 1);
                if (e != hipSuccess) return e;
                const T *Bs = tB ? B + n0 : B + (int64_t)n0 * ldb;  // columns n0.. of op(B)
                return run_gemm_colmajor(tab, ntab, tA, tB, cA, cB, M, rn, K, alpha, A, lda, Bs, ldb, beta,
                                         C + (int64_t)n0 * ldc, ldc, stream, tri, fixed, 2);
            }
        }
    }
    return run_gemm_whole(tab, ntab, tA, tB, cA, cB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, tri, fixed);
}

// The tile choice as a function of the shape alone (plain product, no forced tile), with the cost the
// model puts on every tile in one range (negative where a tile is not offered): what
// clblasAmdTileModelQuery reports and the fitting script (clblas_amd/fit_tile_model.py) evaluates.
template <typename T>
static void model_query(const TileEntry<T> *tab, int ntab, int M, int N, int K, int *tile, int *splits, int *tail_slices,
                        double *costs, int max_costs) {
    double c[16];
    for (int i = 0; i < 16; ++i) c[i] = -1.0;
    choose_tile(tab, ntab, M, N, K, -1, false, 0, false, knobs().tail != 0, tile, splits, c);
    for (int i = 0; i < max_costs && i < ntab && i < 16; ++i) costs[i] = c[i];
    const TileEntry<T> &e = tab[*tile];
    const int64_t ntiles = ceil_div64(M, e.bm) * ceil_div64(N, e.bn);
    *tail_slices = (*splits <= 1 && e.tri[0] && e.slices_tail) ? tail_slices_for(ntiles, K, e.bk, knobs().tail != 0) : 1;
}

// A table entry with its credit in launches that cut K set (see TileEntry::split_gain).
template <typename T> static TileEntry<T> with_split_gain(TileEntry<T> e, double g) {
    e.split_gain = g;
    return e;
}

// A table entry with its credit on streamed operands set (see TileEntry::streamed_gain), as the tiles below
// 64x64 are entered: their last round is never cut into K slices (they are for products of few tiles).
template <typename T> static TileEntry<T> with_streamed_gain(TileEntry<T> e, double g) {
    e.streamed_gain = g;
    e.slices_tail = false;
    return e;
}

// One parameter of the choice model of tile `i`: 0 eff, 1 alone, 2 k0, 3 tail_extra, 4 deep_gain, 5 split_gain,
// 6 streamed_gain.
template <typename T> static double *model_param(TileEntry<T> *tab, int ntab, int i, int which) {
    if (i < 0 || i >= ntab) return nullptr;
    switch (which) {
        case 0: return &tab[i].eff;
        case 1: return &tab[i].alone;
        case 2: return &tab[i].k0;
        case 3: return &tab[i].tail_extra;
        case 4: return &tab[i].deep_gain;
        case 5: return &tab[i].split_gain;
        case 6: return &tab[i].streamed_gain;
        default: return nullptr;
    }
}

}  // namespace cba
