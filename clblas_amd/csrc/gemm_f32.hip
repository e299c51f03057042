// FP32 GEMM: tile table and entry point.
#include "gemm_launch.hpp"

namespace cba {

// Ordered from the largest tile to the smallest.
//   0: 256x128x16, wave 128x64 (2 workgroups of 4 waves per CU)
//   1: 128x128x16, wave 64x64, split-K capable; its sliced tail is priced at 0.12 rounds (2304^3, 324 tiles with 68
//      in the tail round: 119 TFLOP/s, where the 64x64 tiles reach 127; 3700^3 stays with this tile, 137.8
//      against 134.5)
//   2: 128x64x32,  wave 64x32 (narrow C: 65536 x 64 x 4096 runs at 119 TFLOP/s with it, 107 with 64x64).
//      Panels of depth 32 keep twice the bytes in flight, which is what a product that streams A
//      from HBM needs (depth 16: 114.6), and let a workgroup that is alone on its CU run at full rate
//      (16384 x 128 x 2048: 126 against 117 with depth 16); the larger tiles lose residency with them.
//   3:  64x128x32, wave 32x64: the mirror image for wide C (64 x 65536 x 4096: 116 against 107)
//      Tiles 1 to 3 are split-K capable for small C with deep K, where the 64x64 tile (split or not) loses to
//      them: 1024 x 1024 x 65536 98 -> 141 TFLOP/s, 1280 x 1280 x 8192 108 -> 125, 768 x 768 x 16384 109 -> 128,
//      3000 x 200 x 6000 72 -> 87.
//      Products with a triangular operand (TRMM, SYMM) are offered tile 3 but not tile 2 (STRMM 4000: 120.6
//      TFLOP/s with 64x128, 111.8 with 128x64, 113.7 with 64x64), and the credits for them were set from STRMM /
//      SSYMM at 2000 .. 10000 with every tile forced: 64x64 .83 and 64x128 .885 beside .92 and .942 of the two
//      large tiles, so that 64x64 is taken up to 3000, 64x128 at 4000 .. 6000, 128x128 from there (STRMM 5000
//      116 -> 124, 6000 116 -> 123, 7000 117 -> 127; SSYMM 5000 118 -> 128, 7000 120 -> 131).
//   The parameters of the choice model (efficiency, fixed time per workgroup as a depth k0, price of a sliced
//   tail) were last refitted with clblas_amd/fit_tile_model.py on bench.py --only tilemodel: the 256x128 tile
//   has a k0 (on large C with K of a few hundred the 128x128 tile is ahead: 8192 x 8192 x 128 +3.5 %,
//   4096 x 4096 x 64 +1.3 %), the 128x128 tile's sliced tail 0.12 -> 0.07, the 64x64 tile .86 -> .88
//   (5000 x 1000 x 1000 +7 %, 4200 x 1700 x 900 +3 %).  With shapes beyond 8192 in the set (tens of rounds of
//   tiles, edges that are no multiples of a tile) the 256x128 tile went from (.942, k0 80, tail .05) to
//   (.952, 40, .03): 10000^3, 16000 x 16000 x 2048 and 20000 x 20000 x 8192 had been given 128x64 tiles
//   and ran 8-11 % behind (its credit for plain products only: the triangular forms keep .942); and the
//   128x64 / 64x128 tiles got k0 = 10 (20000 x 20000 x 256 and 16000 x 16000 x 128 ran 3.5 and 8 % behind the
//   128x128 tile with them, 6000 x 6000 x 640 2.8 %).  With one or two rows / columns of tiles over a deep K in
//   the set (10000 x 100 x 10000, 16384 x 64 x 10000, ...: the streamed operand comes from HBM and a workgroup
//   alone on its CU reaches two thirds of the MFMA rate) `alone` of the 64x64 tile went .95 -> .85 and that of
//   the 128x64 pair .97 -> .9 (16384 x 64 x 10000: 128x64 in four K ranges, +10 %), the 64x64 tile's sliced
//   tail .05 -> .02; and the 64x128 tile is credited
//   2 % more than its twin in launches that cut K, where it is 4-6 % ahead of it whichever dimension is the short
//   one (10000 x 100 x 10000, 100 x 10000 x 10000, 200 x 3000 x 6000, 768 x 768 x 16384), while it is behind
//   it in every launch of whole tiles.
//   4:  64x32x64,  wave 32x16, and
//   5:  32x32x64,  wave 16x16, both on the 16x16x4 MFMA (workgroups of four wavefronts on tiles below 64x64): for
//      products of up to a few hundred 64x64 tiles, which they cover with one workgroup or more per CU in a single
//      launch where the 64x64 tiles leave CUs idle or cut K and pay a second, dependent launch (SGEMM 448^3 11.9 ->
//      7.1 us, 512^3 10.4 -> 7.1, 704^3 16.0 -> 9.9, 800 x 600 x 400 11.7 -> 7.9, 512 x 1024 x 512 12.6 -> 8.0,
//      1024^3 21.1-21.9 -> 20.2-20.4 in all four transpose cases, 9000 x 130 x 9000 290 -> 228; from about 1100^3 on
//      and for deep K the larger tiles are ahead again).  No K ranges; with the triangular
//      forms (SSYRK 512 17 -> 10 us, STRMM 1024 33 -> 25), whose last round is never sliced, credited .74 / .72
//      where an operand is triangular (with the plain credits STRMM / SSYMM 3000 took them and ran 17-20 % slower).
//      Parameters from runs with every tile forced on 23 shapes, fitted through the model query; checked against
//      the library without them on 63 further shapes (nothing more than 1.1 % slower).  Tiles 32 wide read a
//      streamed operand more often: credited .88 / .75 there (16384 x 64 x 10000 stays with 128x64 in four ranges).
//   6:  64x64x32,  wave 32x32, split-K capable (small / deep-K problems; 1024^3: 94 against 86 with
//      depth 16, 8192 x 64 x 8192: 106-112 against 91-94); with panels of depth 64 where a workgroup's K
//      range is at least 1024 (1024^3 95.4 -> 99.0 TFLOP/s, 1024 x 1024 x 2048 109 -> 115, 960 x 960 x 2048
//      96 -> 101, 512 x 512 x 4096 85 -> 90)
// (Not const: clblasAmdTileModelParam lets the fitting script vary the model's parameters; the launch path only reads.)
static TileEntry<float> *f32_tiles(int *n) {
    static TileEntry<float> tab[] = {
        make_tile_entry<float, 256, 128, 16, 128, 64, 2, false, true>(0.952, 0.85, 0.942, 40.0, 0.03, 0.942),
        make_tile_entry<float, 128, 128, 16, 64, 64, 2, true, true>(0.920, 0.85, -1.0, 0.0, 0.07),
        make_tile_entry<float, 128, 64, 32, 64, 32, 2, true, true>(0.92, 0.9, 0.0, 10.0),
        with_split_gain(make_tile_entry<float, 64, 128, 32, 32, 64, 2, true, true>(0.92, 0.9, 0.885, 10.0), 1.02),
        with_streamed_gain(make_tile_entry<float, 64, 32, 64, 32, 16, 2, false, true>(0.85, 1.0, 0.74, 10.0), 0.88),
        with_streamed_gain(make_tile_entry<float, 32, 32, 64, 16, 16, 2, false, true>(0.84, 0.6, 0.72, 30.0), 0.75),
        make_tile_entry<float, 64, 64, 32, 32, 32, 2, true, true, 64, true>(0.88, 0.85, 0.83, 0.0, 0.02),
    };
    *n = (int)(sizeof(tab) / sizeof(tab[0]));
    return tab;
}

hipError_t sgemm_colmajor(bool transA, bool transB, int M, int N, int K, float alpha, const float *A, int64_t lda,
                          const float *B, int64_t ldb, float beta, float *C, int64_t ldc, hipStream_t stream, const GemmTri *tri,
                          const FixedScratch *fixed) {
    int n;
    const TileEntry<float> *tab = f32_tiles(&n);
    return run_gemm_colmajor<float>(tab, n, transA, transB, false, false, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, tri, fixed);
}

int sgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims) {
    int n;
    const TileEntry<float> *tab = f32_tiles(&n);
    model_query<float>(tab, n, M, N, K, tile, splits, tail_slices, costs, max_costs);
    for (int i = 0; i < n && i < max_costs; ++i) { dims[3 * i] = tab[i].bm; dims[3 * i + 1] = tab[i].bn; dims[3 * i + 2] = tab[i].bk; }
    return n;
}
double *sgemm_model_param(int tile, int which) {
    int n;
    return model_param<float>(f32_tiles(&n), n, tile, which);
}

}  // namespace cba
