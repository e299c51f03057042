// FP64 GEMM: tile table and entry point.
#include "gemm_launch.hpp"

namespace cba {

// Ordered from the largest tile to the smallest.
//   0: 128x128x16, wave 64x64 (2 workgroups of 4 waves per CU), split-K capable for small C with deep K
//      (1024 x 1024 x 16384: 50 -> 69 TFLOP/s, 1280 x 1280 x 8192 54 -> 66, 256 x 4096 x 8192 46 -> 66)
//   1:  64x32x32,  wave 32x16, and
//   2:  32x32x32,  wave 16x16: for products of up to a few hundred tiles of 64x64, which they cover with one
//      workgroup or more per CU in a single launch, where the 64x64 tiles leave CUs idle or cut K and pay a second,
//      dependent launch (DGEMM 512^3 14.7 -> 8.6 us, the vendor library 11.6; 448^3 13.4 -> 7.8, 704^3 21.1 -> 15.6,
//      800 x 600 x 400 17.2 -> 11.0, 512 x 1024 x 512 - an update of DTRSM 1024 - 19.2 -> 12.1; from 900^3 on and
//      for deep K the 64x64 tiles are ahead again).  No K ranges; with
//      the triangular forms (DSYRK 512 25 -> 12 us, DTRMM 1024 52 -> 37), whose last round is never sliced.  A
//      workgroup of 32x32 alone on its CU runs at 0.44 of the CU's peak, two at 0.61, three or more at 0.7; one of
//      64x32 at 0.79 alone, 0.83-0.85 in company, with about 3 us before its first MFMA: eff / alone / k0 below.
//   3:  64x64x16,  wave 32x32, split-K capable.  Credited with .90 for plain and triangular-C
//      products (2304^3 64.7 -> 67.9 TFLOP/s, 3328^3 64.5 -> 68.6, 3000 x 1500 x 1000 56.6 -> 61.1 against
//      .84) and with .84 where an operand is triangular (DTRMM / DSYMM 6144 lose 2-3 % with .90).
//      With panels of depth 32 where a workgroup's K range is at least 1024 (1024^3 54.9 -> 58.5 TFLOP/s,
//      1024 x 1024 x 2048 59.8 -> 64.2, 960 x 960 x 2048 50.9 -> 53.4).
//   Last refit (clblas_amd/fit_tile_model.py on bench.py --only tilemodel): k0 of the 128x128 tile 95 -> 85, a
//   sliced tail of the 64x64 tiles priced at 0.35 rounds instead of 0.05 (4480 x 4480 x 2000, 2500 x 7000 x 1200,
//   8192 x 8192 x 512: the 128x128 tile 0.5-0.9 % ahead).
//   Short K on large C goes to the 64x64 tiles through the fixed-time term (k0 = 85 and 68):
//   4096 x 4096 x 64 31.9 -> 38.9 TFLOP/s, x 128 45.5 -> 52.2, x 256 57.5 -> 61.6, 3000 x 3000 x 640 59.2 -> 64.3.
// (Not const: clblasAmdTileModelParam lets the fitting script vary the model's parameters; the launch path only reads.)
static TileEntry<double> *f64_tiles(int *n) {
    static TileEntry<double> tab[] = {
        make_tile_entry<double, 128, 128, 16, 64, 64, 2, true, true>(0.94, 0.85, -1.0, 85.0),
        with_streamed_gain(make_tile_entry<double, 64, 32, 32, 32, 16, 2, false, true>(0.77, 1.0, -1.0, 100.0), 0.95),
        with_streamed_gain(make_tile_entry<double, 32, 32, 32, 16, 16, 2, false, true>(0.80, 0.62, -1.0, 200.0), 0.75),
        // (in launches that cut K it is credited 4 % less: DGEMM 100 x 5000 x 20000 ran 5.6 % behind the 128x128
        // tile in twelve ranges with it)
        with_split_gain(make_tile_entry<double, 64, 64, 16, 32, 32, 2, true, true, 32, true>(0.90, 0.85, 0.84, 68.0, 0.35), 0.96),
    };
    *n = (int)(sizeof(tab) / sizeof(tab[0]));
    return tab;
}

hipError_t dgemm_colmajor(bool transA, bool transB, int M, int N, int K, double alpha, const double *A,
                          int64_t lda, const double *B, int64_t ldb, double beta, double *C, int64_t ldc,
                          hipStream_t stream, const GemmTri *tri) {
    int n;
    const TileEntry<double> *tab = f64_tiles(&n);
    return run_gemm_colmajor<double>(tab, n, transA, transB, false, false, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, tri);
}

int dgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims) {
    int n;
    const TileEntry<double> *tab = f64_tiles(&n);
    model_query<double>(tab, n, M, N, K, tile, splits, tail_slices, costs, max_costs);
    for (int i = 0; i < n && i < max_costs; ++i) { dims[3 * i] = tab[i].bm; dims[3 * i + 1] = tab[i].bn; dims[3 * i + 2] = tab[i].bk; }
    return n;
}
double *dgemm_model_param(int tile, int which) {
    int n;
    return model_param<double>(f64_tiles(&n), n, tile, which);
}

}  // namespace cba
