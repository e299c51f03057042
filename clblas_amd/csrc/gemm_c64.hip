// Complex FP64 GEMM: tile table and entry point.
#include "gemm_launch.hpp"

namespace cba {

// Ordered from the largest tile to the smallest.
//   0: 128x64x8, wave 64x32 (2 workgroups of 4 waves per CU), split-K capable for small C with deep K
//      (1024 x 1024 x 8192: 64 -> 71 TFLOP/s, 768 x 768 x 16384 59 -> 70)
//   1:  64x32x16, wave 32x16, and
//   2:  32x32x16, wave 16x16: for small products, which they cover in one launch where the 64x64 tiles leave CUs
//      idle or cut K and pay a second, dependent launch (ZGEMM 512^3 28.2 -> 23.6 us, 800 x 600 x 400 45.6 -> 31.7,
//      640 x 640 x 128 21.7 -> 12.9, 1024^3 141 -> 131, 9000 x 130 x 9000 2.14 -> 1.63 ms); no K ranges; triangular forms without sliced tails.
//   3:  64x64x8, wave 32x32, split-K capable
//   On large C the 64x64 tiles are the faster ones at every depth (8192^3: 73.2 against 72.0 TFLOP/s, 8192 x 8192 x
//   2048 72.8 / 71.4, x 512 71.6 / 69.4, x 64 53.3 / 48.8, 4096 x 4096 x 32 38.5 / 32.4), so they are credited with
//   .945 against .93 and with the smaller fixed time (k0 = 35 and 44 from T(K) = T_inf K / (K + k0)); the 128x64
//   tiles keep the cases where they fill the rounds better.  Products with a triangular operand or a triangular C are
//   credited .86 with the 64x64 tiles and .84 (operand) / .86 (C) with the 128x64 ones, from runs with each tile
//   forced: ZTRMM 3000 60.3 / 64.2 TFLOP/s (128x64 / 64x64), 5000 63.8 / 66.9, 6000 67.7 / 69.0, 8192 69.6 / 70.4;
//   ZSYRK 3000 50.1 / 65.2, 5000 64.8 / 67.4, 6000 67.9 / 69.6 and only at 8192 70.3 / 69.3, where the equal
//   credits leave the choice to the count of rounds.
//   A sliced tail costs these tiles more than the others (3000 x 1500 x 1000, 1128 tiles with 104 in the tail
//   round: 60.4 TFLOP/s against 64.4 with the 128x64 tiles), so it is priced at 0.35 rounds instead of 0.05.
static TileEntry<Cx<double>> *c64_tiles(int *n) {
    static TileEntry<Cx<double>> tab[] = {
        make_tile_entry<Cx<double>, 128, 64, 8, 64, 32, 2, true, true>(0.93, 0.85, 0.84, 44.0, 0.05, 0.86),
        with_streamed_gain(make_tile_entry<Cx<double>, 64, 32, 16, 32, 16, 2, false, true>(0.86, 0.8, -1.0, 30.0), 0.95),
        with_streamed_gain(make_tile_entry<Cx<double>, 32, 32, 16, 16, 16, 2, false, true>(0.82, 0.9, -1.0, 30.0), 0.75),
        make_tile_entry<Cx<double>, 64, 64, 8, 32, 32, 2, true, true, 0, true>(0.945, 0.85, 0.86, 35.0, 0.35, 0.86),
    };
    *n = (int)(sizeof(tab) / sizeof(tab[0]));
    return tab;
}

hipError_t zgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<double> alpha,
                          const Cx<double> *A, int64_t lda, const Cx<double> *B, int64_t ldb, Cx<double> beta,
                          Cx<double> *C, int64_t ldc, hipStream_t stream, const GemmTri *tri) {
    int n;
    const TileEntry<Cx<double>> *tab = c64_tiles(&n);
    return run_gemm_colmajor<Cx<double>>(tab, n, transA, transB, conjA, conjB, M, N, K, alpha, A, lda, B, ldb, beta,
                                         C, ldc, stream, tri);
}

int zgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims) {
    int n;
    const TileEntry<Cx<double>> *tab = c64_tiles(&n);
    model_query<Cx<double>>(tab, n, M, N, K, tile, splits, tail_slices, costs, max_costs);
    for (int i = 0; i < n && i < max_costs; ++i) { dims[3 * i] = tab[i].bm; dims[3 * i + 1] = tab[i].bn; dims[3 * i + 2] = tab[i].bk; }
    return n;
}
double *zgemm_model_param(int tile, int which) {
    int n;
    return model_param<Cx<double>>(c64_tiles(&n), n, tile, which);
}

}  // namespace cba
