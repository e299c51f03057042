// Complex FP32 GEMM: tile table and entry point.
#include "gemm_launch.hpp"

namespace cba {

// Ordered from the largest tile to the smallest.  A complex element carries four times the
// flops of a real one for twice the bytes, so these tiles match the real 256x128 / 128x128
// ones in arithmetic intensity.
//   0: 128x128x16, wave 64x64 (2 workgroups of 4 waves per CU), split-K capable for small C with deep K
//      (1024 x 1024 x 8192: 116 -> 139 TFLOP/s, 1280 x 1280 x 16384 105 -> 142)
//   1:  64x32x32, wave 32x16, and
//   2:  32x32x32, wave 16x16, both on the 16x16x4 MFMA: for small products, which they cover in one launch where
//      the 64x64 tiles leave CUs idle or cut K and pay a second, dependent launch (CGEMM 512^3 20.4 -> 14.4 us,
//      1024^3 79 -> 68, 512 x 1024 x 512 30.4 -> 21.7, 896^3 69.5 -> 59.7); no K ranges; triangular forms without sliced tails.
//   3:  64x64x8,  wave 32x32, split-K capable (credited with .90; .84 where an operand is triangular:
//      3328^3 127 -> 135 TFLOP/s, 3000 x 1500 x 1000 120 -> 126, CSYRK 6144 130 -> 139 against .84 for all)
static TileEntry<Cx<float>> *c32_tiles(int *n) {
    static TileEntry<Cx<float>> tab[] = {
        make_tile_entry<Cx<float>, 128, 128, 16, 64, 64, 2, true, true>(0.93),
        with_streamed_gain(make_tile_entry<Cx<float>, 64, 32, 32, 32, 16, 2, false, true>(0.88, 1.0, -1.0, 10.0), 0.9),
        with_streamed_gain(make_tile_entry<Cx<float>, 32, 32, 32, 16, 16, 2, false, true>(0.86, 0.7, -1.0, 10.0), 0.75),
        make_tile_entry<Cx<float>, 64, 64, 8, 32, 32, 2, true, true, 0, true>(0.90, 0.85, 0.84),
    };
    *n = (int)(sizeof(tab) / sizeof(tab[0]));
    return tab;
}

hipError_t cgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<float> alpha,
                          const Cx<float> *A, int64_t lda, const Cx<float> *B, int64_t ldb, Cx<float> beta,
                          Cx<float> *C, int64_t ldc, hipStream_t stream, const GemmTri *tri) {
    int n;
    const TileEntry<Cx<float>> *tab = c32_tiles(&n);
    return run_gemm_colmajor<Cx<float>>(tab, n, transA, transB, conjA, conjB, M, N, K, alpha, A, lda, B, ldb, beta,
                                        C, ldc, stream, tri);
}

int cgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims) {
    int n;
    const TileEntry<Cx<float>> *tab = c32_tiles(&n);
    model_query<Cx<float>>(tab, n, M, N, K, tile, splits, tail_slices, costs, max_costs);
    for (int i = 0; i < n && i < max_costs; ++i) { dims[3 * i] = tab[i].bm; dims[3 * i + 1] = tab[i].bn; dims[3 * i + 2] = tab[i].bk; }
    return n;
}
double *cgemm_model_param(int tile, int which) {
    int n;
    return model_param<Cx<float>>(c32_tiles(&n), n, tile, which);
}

}  // namespace cba
