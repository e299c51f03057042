// Drives every argument-validation path of the C ABI in a CPU build of clblas_amd/csrc/api.cpp
// with AddressSanitizer / UBSan.  The launchers that api.cpp hands valid problems to are
// replaced by stubs that abort: a call that gets past validation here is a test failure.
#include <cstdio>
#include <cstdlib>

#include "../../clblas_amd/csrc/internal.h"
#include "../../include/clblas_amd.h"

namespace cba {
[[noreturn]] static void reached(const char *what) {
    std::fprintf(stderr, "launcher %s reached: validation let an invalid call through\n", what);
    std::abort();
}
template <typename T>
hipError_t launch_gemm(bool, bool, bool, bool, int, int, int, T, const T *, int64_t, const T *, int64_t, T, T *, int64_t,
                       hipStream_t, const GemmTri *) { reached("gemm"); }
template <typename T>
hipError_t syrk_colmajor(bool, bool, int, int, T, const T *, int64_t, T, T *, int64_t, hipStream_t) { reached("syrk"); }
template <typename T>
hipError_t trmm_colmajor(bool, bool, bool, bool, bool, int, int, T, const T *, int64_t, T *, int64_t, hipStream_t) { reached("trmm"); }
template <typename T>
hipError_t symm_colmajor(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *, int64_t, hipStream_t) { reached("symm"); }
template <typename T>
hipError_t syr2k_colmajor(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *, int64_t, hipStream_t) { reached("syr2k"); }
template <typename R>
hipError_t herk_colmajor(bool, bool, int, int, R, const Cx<R> *, int64_t, R, Cx<R> *, int64_t, hipStream_t) { reached("herk"); }
template <typename R>
hipError_t her2k_colmajor(bool, bool, int, int, Cx<R>, const Cx<R> *, int64_t, const Cx<R> *, int64_t, R, Cx<R> *, int64_t,
                          hipStream_t) { reached("her2k"); }
template <typename T>
hipError_t hemm_colmajor(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *, int64_t, hipStream_t) { reached("hemm"); }
template <typename T>
hipError_t trsm_colmajor(bool, bool, bool, bool, bool, int, int, T, const T *, int64_t, T *, int64_t, hipStream_t) { reached("trsm"); }
hipError_t sgemm_colmajor_noalloc(bool, bool, int, int, int, float, const float *, int64_t, const float *, int64_t, float,
                                  float *, int64_t, hipStream_t) { reached("sgemm_noalloc"); }
hipError_t noalloc_scratch(void **) { return hipErrorNoDevice; }
hipError_t trsm_poll_timeouts_read(unsigned int *count, bool) { if (count) *count = 0; return hipSuccess; }
int sgemm_model_query(int, int, int, int *, int *, int *, double *, int, int *) { return 0; }
int dgemm_model_query(int, int, int, int *, int *, int *, double *, int, int *) { return 0; }
double *sgemm_model_param(int, int) { return nullptr; }
double *dgemm_model_param(int, int) { return nullptr; }
int cgemm_model_query(int, int, int, int *, int *, int *, double *, int, int *) { return 0; }
int zgemm_model_query(int, int, int, int *, int *, int *, double *, int, int *) { return 0; }
double *cgemm_model_param(int, int) { return nullptr; }
double *zgemm_model_param(int, int) { return nullptr; }

#define INST(T)                                                                                                         \
    template hipError_t launch_gemm<T>(bool, bool, bool, bool, int, int, int, T, const T *, int64_t, const T *, int64_t, T, \
                                       T *, int64_t, hipStream_t, const GemmTri *);                                     \
    template hipError_t syrk_colmajor<T>(bool, bool, int, int, T, const T *, int64_t, T, T *, int64_t, hipStream_t);    \
    template hipError_t trmm_colmajor<T>(bool, bool, bool, bool, bool, int, int, T, const T *, int64_t, T *, int64_t,   \
                                         hipStream_t);                                                                  \
    template hipError_t symm_colmajor<T>(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *,       \
                                         int64_t, hipStream_t);                                                         \
    template hipError_t syr2k_colmajor<T>(bool, bool, int, int, T, const T *, int64_t, const T *, int64_t, T, T *,      \
                                          int64_t, hipStream_t);                                                        \
    template hipError_t trsm_colmajor<T>(bool, bool, bool, bool, bool, int, int, T, const T *, int64_t, T *, int64_t,   \
                                         hipStream_t);
INST(float)
INST(double)
INST(Cx<float>)
INST(Cx<double>)
template hipError_t herk_colmajor<float>(bool, bool, int, int, float, const Cx<float> *, int64_t, float, Cx<float> *, int64_t, hipStream_t);
template hipError_t herk_colmajor<double>(bool, bool, int, int, double, const Cx<double> *, int64_t, double, Cx<double> *, int64_t, hipStream_t);
template hipError_t her2k_colmajor<float>(bool, bool, int, int, Cx<float>, const Cx<float> *, int64_t, const Cx<float> *, int64_t, float, Cx<float> *, int64_t, hipStream_t);
template hipError_t her2k_colmajor<double>(bool, bool, int, int, Cx<double>, const Cx<double> *, int64_t, const Cx<double> *, int64_t, double, Cx<double> *, int64_t, hipStream_t);
template hipError_t hemm_colmajor<Cx<float>>(bool, bool, int, int, Cx<float>, const Cx<float> *, int64_t, const Cx<float> *, int64_t, Cx<float>, Cx<float> *, int64_t, hipStream_t);
template hipError_t hemm_colmajor<Cx<double>>(bool, bool, int, int, Cx<double>, const Cx<double> *, int64_t, const Cx<double> *, int64_t, Cx<double>, Cx<double> *, int64_t, hipStream_t);
}  // namespace cba

static int failures = 0;
#define EXPECT(call, want)                                                                        \
    do {                                                                                          \
        const int got_ = (int)(call);                                                             \
        if (got_ != (int)(want)) { std::printf("line %d: %s = %d, expected %d\n", __LINE__, #call, got_, (int)(want)); ++failures; } \
    } while (0)

int main() {
    float *F = reinterpret_cast<float *>(0x1000);  // non-null "device pointers": never dereferenced
    double *D = reinterpret_cast<double *>(0x1000);
    FloatComplex *C = reinterpret_cast<FloatComplex *>(0x1000);
    DoubleComplex *Z = reinterpret_cast<DoubleComplex *>(0x1000);
    const FloatComplex c1 = {{1.f, 0.f}};
    const DoubleComplex z1 = {{1.0, 0.0}};
    const clblasOrder orders[] = {clblasRowMajor, clblasColumnMajor};
    const clblasTranspose transes[] = {clblasNoTrans, clblasTrans, clblasConjTrans};
    unsigned a = 9, b = 9, c = 9;
    EXPECT(clblasGetVersion(&a, &b, &c), clblasSuccess);
    EXPECT(clblasGetVersion(nullptr, nullptr, nullptr), clblasSuccess);
    size_t ns = 7, nb = 7;
    clblasAmdWorkspaceStats(&ns, &nb);
    EXPECT(ns, 0);
    EXPECT(nb, 0);
    char text[64];
    EXPECT(clblasAmdLastDispatch(text, sizeof text), 0);
    EXPECT(clblasAmdLastDispatch(nullptr, 0), 0);
    clblasAmdReloadDebugEnv();
    for (clblasOrder o : orders)
        for (clblasTranspose ta : transes)
            for (clblasTranspose tb : transes) {
                // null objects in A, B, C order; zero and oversize dimensions; short leading dimensions
                EXPECT(clblasSgemm(o, ta, tb, 4, 4, 4, 1.f, nullptr, 0, 4, F, 0, 4, 0.f, F, 0, 4, nullptr), clblasInvalidMatA);
                EXPECT(clblasDgemm(o, ta, tb, 4, 4, 4, 1.0, D, 0, 4, nullptr, 0, 4, 0.0, D, 0, 4, nullptr), clblasInvalidMatB);
                EXPECT(clblasCgemm(o, ta, tb, 4, 4, 4, c1, C, 0, 4, C, 0, 4, c1, nullptr, 0, 4, nullptr), clblasInvalidMatC);
                EXPECT(clblasZgemm(o, ta, tb, 0, 4, 4, z1, Z, 0, 4, Z, 0, 4, z1, Z, 0, 4, nullptr), clblasInvalidDim);
                EXPECT(clblasSgemm(o, ta, tb, 4, 0, 4, 1.f, F, 0, 4, F, 0, 4, 0.f, F, 0, 4, nullptr), clblasInvalidDim);
                EXPECT(clblasSgemm(o, ta, tb, 5, 6, 7, 1.f, F, 0, 4, F, 0, 9, 0.f, F, 0, 9, nullptr), clblasInvalidLeadDimA);
                EXPECT(clblasDgemm(o, ta, tb, 5, 6, 7, 1.0, D, 0, 9, D, 0, 5, 0.0, D, 0, 9, nullptr), clblasInvalidLeadDimB);
                EXPECT(clblasSgemm(o, ta, tb, 7, 7, 7, 1.f, F, 0, 9, F, 0, 9, 0.f, F, 0, 4, nullptr), clblasInvalidLeadDimC);
                EXPECT(clblasSgemmNoAlloc(o, ta, tb, 7, 7, 7, 1.f, F, 0, 9, F, 0, 9, 0.f, F, 0, 4, nullptr), clblasInvalidLeadDimC);
                const size_t huge = (size_t)1 << 31;
                EXPECT(clblasSgemm(o, ta, tb, huge, 2, 2, 1.f, F, 0, huge, F, 0, huge, 0.f, F, 0, huge, nullptr), clblasNotImplemented);
                EXPECT(clblasDgemm(o, ta, tb, 2, 2, (size_t)-1, 1.0, D, 0, (size_t)-1, D, 0, (size_t)-1, 0.0, D, 0, 2, nullptr), clblasNotImplemented);
            }
    EXPECT(clblasSgemm((clblasOrder)7, clblasNoTrans, clblasNoTrans, 4, 4, 4, 1.f, F, 0, 4, F, 0, 4, 0.f, F, 0, 4, nullptr), clblasInvalidValue);
    EXPECT(clblasSgemm(clblasColumnMajor, (clblasTranspose)3, clblasNoTrans, 4, 4, 4, 1.f, F, 0, 4, F, 0, 4, 0.f, F, 0, 4, nullptr), clblasInvalidValue);
    for (clblasOrder o : orders)
        for (int side = 0; side < 2; ++side)
            for (clblasTranspose ta : transes) {
                const clblasSide sd = (clblasSide)side;
                EXPECT(clblasStrsm(o, sd, clblasLower, ta, clblasNonUnit, 4, 4, 1.f, nullptr, 0, 4, F, 0, 4, nullptr), clblasInvalidMatA);
                EXPECT(clblasDtrsm(o, sd, clblasLower, ta, clblasNonUnit, 4, 4, 1.0, D, 0, 4, nullptr, 0, 4, nullptr), clblasInvalidMatB);
                EXPECT(clblasCtrsm(o, sd, clblasUpper, ta, clblasUnit, 0, 4, c1, C, 0, 8, C, 0, 8, nullptr), clblasInvalidDim);
                EXPECT(clblasZtrsm(o, sd, clblasUpper, ta, clblasUnit, 6, 6, z1, Z, 0, 5, Z, 0, 8, nullptr), clblasInvalidLeadDimA);
                EXPECT(clblasDtrsm(o, sd, clblasUpper, ta, clblasUnit, 6, 6, 1.0, D, 0, 8, D, 0, 5, nullptr), clblasInvalidLeadDimB);
                EXPECT(clblasStrmm(o, sd, clblasLower, ta, clblasNonUnit, 6, 6, 1.f, F, 0, 5, F, 0, 8, nullptr), clblasInvalidLeadDimA);
                EXPECT(clblasZtrmm(o, sd, clblasLower, ta, (clblasDiag)5, 6, 6, z1, Z, 0, 8, Z, 0, 8, nullptr), clblasInvalidValue);
                EXPECT(clblasDsymm(o, sd, clblasLower, 6, 6, 1.0, D, 0, 8, D, 0, 8, 0.0, D, 0, 5, nullptr), clblasInvalidLeadDimC);
                EXPECT(clblasChemm(o, sd, clblasLower, 6, 6, c1, C, 0, 8, nullptr, 0, 8, c1, C, 0, 8, nullptr), clblasInvalidMatB);
                EXPECT(clblasZhemm(o, sd, (clblasUplo)4, 6, 6, z1, Z, 0, 8, Z, 0, 8, z1, Z, 0, 8, nullptr), clblasInvalidValue);
            }
    for (clblasOrder o : orders) {
        EXPECT(clblasSsyrk(o, clblasLower, clblasNoTrans, 6, 0, 1.f, F, 0, 8, 0.f, F, 0, 8, nullptr), clblasInvalidDim);
        EXPECT(clblasDsyrk(o, clblasLower, clblasNoTrans, 6, 4, 1.0, D, 0, 8, 0.0, D, 0, 5, nullptr), clblasInvalidLeadDimC);
        EXPECT(clblasCsyrk(o, clblasLower, clblasConjTrans, 6, 4, c1, C, 0, 8, c1, C, 0, 8, nullptr), clblasInvalidValue);
        EXPECT(clblasZsyrk(o, clblasLower, clblasTrans, 6, 4, z1, nullptr, 0, 8, z1, Z, 0, 8, nullptr), clblasInvalidMatA);
        EXPECT(clblasSsyr2k(o, clblasUpper, clblasNoTrans, 6, 4, 1.f, F, 0, 8, nullptr, 0, 8, 0.f, F, 0, 8, nullptr), clblasInvalidMatB);
        EXPECT(clblasZsyr2k(o, clblasUpper, clblasConjTrans, 6, 4, z1, Z, 0, 8, Z, 0, 8, z1, Z, 0, 8, nullptr), clblasInvalidValue);
        EXPECT(clblasCherk(o, clblasUpper, clblasTrans, 6, 4, 1.f, C, 0, 8, 0.f, C, 0, 8, nullptr), clblasInvalidValue);
        EXPECT(clblasZherk(o, clblasUpper, clblasNoTrans, 6, 4, 1.0, Z, 0, 8, 0.0, nullptr, 0, 8, nullptr), clblasInvalidMatC);
        EXPECT(clblasCher2k(o, clblasUpper, clblasNoTrans, 6, 0, c1, C, 0, 8, C, 0, 8, 0.f, C, 0, 8, nullptr), clblasInvalidDim);
        EXPECT(clblasZher2k(o, clblasUpper, clblasConjTrans, 6, 4, z1, Z, 0, 3, Z, 0, 8, 0.0, Z, 0, 8, nullptr), clblasInvalidLeadDimA);
    }
    // CLBLAS_AMD_CHECK_MEM=1: the allocation behind every operand is looked up and the reference's rule
    // (generic/common.c:644-684; src/tests/functional/func-error.cpp:58-104 makes a matrix larger than its
    // buffer and expects clblasInsufficientMemMatA / MatB) applies: offset + footprint beyond the buffer.
    // The lookup is replaced by a table: F holds 64 floats, D2 64 doubles, anything else is unknown.
    setenv("CLBLAS_AMD_CHECK_MEM", "1", 1);
    clblasAmdReloadDebugEnv();
    double *D2 = reinterpret_cast<double *>(0x3000);  // (F and D2 above are one address)
    static const void *known_f = F, *known_d = D2;
    cba::set_mem_probe([](const void *ptr) -> size_t {
        if (ptr == known_f) return 64 * sizeof(float);
        if (ptr == known_d) return 64 * sizeof(double);
        return 0;
    });
    float *G = reinterpret_cast<float *>(0x2000);  // no allocation holds it
    for (clblasOrder o : orders)
        for (clblasTranspose ta : transes)
            for (clblasTranspose tb : transes) {
                // 9 x 8 elements with ld 9 need 72 > 64; 8 x 8 fits exactly until an offset of one pushes it out
                EXPECT(clblasSgemm(o, ta, tb, 9, 8, 8, 1.f, F, 0, 9, F, 0, 9, 0.f, F, 0, 9, nullptr), clblasInsufficientMemMatA);
                EXPECT(clblasSgemm(o, ta, tb, 8, 8, 8, 1.f, F, 1, 8, F, 0, 8, 0.f, F, 0, 8, nullptr), clblasInsufficientMemMatA);
                EXPECT(clblasSgemm(o, ta, tb, 8, 8, 8, 1.f, F, 0, 8, F, 1, 8, 0.f, F, 0, 8, nullptr), clblasInsufficientMemMatB);
                EXPECT(clblasDgemm(o, ta, tb, 8, 8, 8, 1.0, D2, 0, 8, D2, 0, 8, 0.0, D2, 1, 8, nullptr), clblasInsufficientMemMatC);
                // a padded leading dimension counts up to the last element only: (7 - 1) 9 + 8 = 62 fits, + 3 does not
                EXPECT(clblasDgemm(o, ta, tb, 7, 7, 7, 1.0, D2, 0, 9, D2, 0, 9, 0.0, D2, 7, 9, nullptr), clblasInsufficientMemMatC);
                // the order of the checks is unchanged: leading dimension of A before the memory of B
                EXPECT(clblasSgemm(o, ta, tb, 8, 8, 8, 1.f, F, 0, 7, F, 9, 8, 0.f, F, 0, 8, nullptr), clblasInvalidLeadDimA);
                // a pointer that no allocation holds is no matrix at all
                EXPECT(clblasSgemm(o, ta, tb, 8, 8, 8, 1.f, F, 0, 8, G, 0, 8, 0.f, F, 0, 8, nullptr), clblasInvalidMatB);
                // an offset that wraps round 64 bits does not pass for a small one
                EXPECT(clblasSgemm(o, ta, tb, 8, 8, 8, 1.f, F, (size_t)-60, 8, F, 0, 8, 0.f, F, 0, 8, nullptr), clblasInsufficientMemMatA);
            }
    for (clblasOrder o : orders) {
        EXPECT(clblasStrsm(o, clblasLeft, clblasLower, clblasNoTrans, clblasNonUnit, 9, 4, 1.f, F, 0, 9, F, 0, 9, nullptr), clblasInsufficientMemMatA);
        EXPECT(clblasDtrsm(o, clblasRight, clblasUpper, clblasTrans, clblasUnit, 4, 8, 1.0, D2, 0, 8, D2, 40, 8, nullptr), clblasInsufficientMemMatB);
        EXPECT(clblasSsyrk(o, clblasLower, clblasNoTrans, 8, 8, 1.f, F, 0, 8, 0.f, F, 2, 8, nullptr), clblasInsufficientMemMatC);
        EXPECT(clblasDtrmm(o, clblasLeft, clblasLower, clblasNoTrans, clblasNonUnit, 8, 8, 1.0, D2, 0, 8, D2, 1, 8, nullptr), clblasInsufficientMemMatB);
        EXPECT(clblasSsymm(o, clblasLeft, clblasLower, 8, 8, 1.f, F, 1, 8, F, 0, 8, 0.f, F, 0, 8, nullptr), clblasInsufficientMemMatA);
    }
    cba::set_mem_probe(nullptr);
    unsetenv("CLBLAS_AMD_CHECK_MEM");
    clblasAmdReloadDebugEnv();
    clblasTeardown();
    if (failures) { std::printf("%d failures\n", failures); return 1; }
    std::puts("ok");
    return 0;
}
