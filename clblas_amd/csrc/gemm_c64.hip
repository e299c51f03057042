// Complex FP64 GEMM: tile table and entry point.
#include "gemm_launch.hpp"

namespace cba {

// Ordered from the largest tile to the smallest.
//   0: 128x64x8, wave 64x32 (2 workgroups of 4 waves per CU), split-K capable for small C with deep K
//      (1024 x 1024 x 8192: 64 -> 71 TFLOP/s, 768 x 768 x 16384 59 -> 70)
//   1:  64x64x8, wave 32x32, split-K capable
static const TileEntry<Cx<double>> *c64_tiles(int *n) {
    static const TileEntry<Cx<double>> tab[] = {
        make_tile_entry<Cx<double>, 128, 64, 8, 64, 32, 2, true, true>(0.93),
        make_tile_entry<Cx<double>, 64, 64, 8, 32, 32, 2, true, true>(0.86),
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

}  // namespace cba
