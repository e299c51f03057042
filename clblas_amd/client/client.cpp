// clblas_amd-client: benchmark command line for libclblas_amd.so.
//
// Takes the place of the reference's clBLAS-client (src/client/client.cpp:80-112 for the
// option names, src/client/clfunc_x{gemm,trsm,trmm,syrk,symm,syr2k,herk,her2k,hemm}.hpp for the GFLOP/s
// formulas)
// for the function families this library implements, and prints the
// CSV schema of the reference's published benchmark files (doc/performance/**.csv):
//   m,n,k,lda,ldb,ldc,offa,offb,offc,alpha,beta,order,transa,transb,side,uplo,diag,
//   function,device,library,numQueues,label,GFLOPS
// so that results can sit beside the published Hawaii / Fiji curves.
//
// Example:  clblas_amd-client -f gemm -r s --sizes 1024:8192:1024 --transposeB 1 --label mi355x
#include "../../include/clblas_amd.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace {

struct Options {
    size_t m = 128, n = 128, k = 128, lda = 0, ldb = 0, ldc = 0, offA = 0, offBX = 0, offCY = 0;
    double alpha = 1.0, beta = 1.0;
    int order = 1, transA = 0, transB = 0, side = 0, uplo = 0, diag = 0;
    std::string function = "gemm", precision = "s", label = "mi355x", sizes;
    unsigned profile = 20, apiCallCount = 10;
    bool header = true;
};

void usage() {
    std::puts(
        "clblas_amd-client options (names follow clBLAS-client):\n"
        "  -m/--sizem N  -n/--sizen N  -k/--sizek N     problem size (default 128)\n"
        "  --sizes A:B:S                                 sweep m=n=k from A to B in steps of S\n"
        "  --lda N --ldb N --ldc N                       leading dimensions (0 = tight)\n"
        "  --offA N --offBX N --offCY N                  element offsets\n"
        "  --alpha X --beta X\n"
        "  -o/--order 0|1                                0 = row major, 1 = column major\n"
        "  --transposeA 0|1|2  --transposeB 0|1|2\n"
        "  --side 0|1  --uplo 0|1  --diag 0|1            0 = left/upper/unit\n"
        "  -f/--function gemm|trsm|trmm|syrk|symm|syr2k|herk|her2k|hemm   -r/--precision s|d|c|z\n"
        "  -p/--profile N                                timed samples (default 20)\n"
        "  --apiCallCount N                              calls per sample (default 10)\n"
        "  --label TEXT  --noheader");
}

bool parse(int argc, char **argv, Options &o) {
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto val = [&]() -> const char * {
            if (i + 1 >= argc) { std::fprintf(stderr, "missing value for %s\n", a.c_str()); std::exit(2); }
            return argv[++i];
        };
        if (a == "-h" || a == "--help") return false;
        else if (a == "-m" || a == "--sizem") o.m = std::strtoull(val(), nullptr, 10);
        else if (a == "-n" || a == "--sizen") o.n = std::strtoull(val(), nullptr, 10);
        else if (a == "-k" || a == "--sizek") o.k = std::strtoull(val(), nullptr, 10);
        else if (a == "--sizes") o.sizes = val();
        else if (a == "--lda") o.lda = std::strtoull(val(), nullptr, 10);
        else if (a == "--ldb") o.ldb = std::strtoull(val(), nullptr, 10);
        else if (a == "--ldc") o.ldc = std::strtoull(val(), nullptr, 10);
        else if (a == "--offA") o.offA = std::strtoull(val(), nullptr, 10);
        else if (a == "--offBX") o.offBX = std::strtoull(val(), nullptr, 10);
        else if (a == "--offCY") o.offCY = std::strtoull(val(), nullptr, 10);
        else if (a == "--alpha") o.alpha = std::atof(val());
        else if (a == "--beta") o.beta = std::atof(val());
        else if (a == "-o" || a == "--order") o.order = std::atoi(val());
        else if (a == "--transposeA") o.transA = std::atoi(val());
        else if (a == "--transposeB") o.transB = std::atoi(val());
        else if (a == "--side") o.side = std::atoi(val());
        else if (a == "--uplo") o.uplo = std::atoi(val());
        else if (a == "--diag") o.diag = std::atoi(val());
        else if (a == "-f" || a == "--function") o.function = val();
        else if (a == "-r" || a == "--precision") o.precision = val();
        else if (a == "-p" || a == "--profile") o.profile = (unsigned)std::atoi(val());
        else if (a == "--apiCallCount") o.apiCallCount = (unsigned)std::atoi(val());
        else if (a == "--label") o.label = val();
        else if (a == "--noheader") o.header = false;
        else { std::fprintf(stderr, "unknown option %s\n", a.c_str()); return false; }
    }
    return true;
}

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); std::exit(1); } } while (0)

// Elements that must be addressable for a rows x cols op(X) (generic/common.c:606-644).
size_t footprint(int order, int trans, size_t rows, size_t cols, size_t off, size_t ld) {
    const bool rows_contig = (order == 1) == (trans == 0);
    const size_t inner = rows_contig ? rows : cols, outer = rows_contig ? cols : rows;
    return off + (outer - 1) * ld + inner;
}

// Fills `count` reals (matrix elements, or re/im pairs of them) with uniform values.
template <typename R> void fill(std::vector<R> &v, uint64_t seed, double scale) {
    uint64_t s = seed * 0x9e3779b97f4a7c15ULL + 1;
    for (auto &x : v) {
        s = s * 6364136223846793005ULL + 1442695040888963407ULL;
        x = (R)(((double)(s >> 40) / (double)(1 << 24) * 2.0 - 1.0) * scale);
    }
}

// One set of overloads per element type, so that run_case can be written once.
template <typename T> struct Type;
template <> struct Type<float> { typedef float Real; static const int NC = 1; static float scalar(double x) { return (float)x; } };
template <> struct Type<double> { typedef double Real; static const int NC = 1; static double scalar(double x) { return x; } };
template <> struct Type<FloatComplex> {
    typedef float Real; static const int NC = 2;
    static FloatComplex scalar(double x) { FloatComplex z; z.s[0] = (float)x; z.s[1] = 0.f; return z; }
};
template <> struct Type<DoubleComplex> {
    typedef double Real; static const int NC = 2;
    static DoubleComplex scalar(double x) { DoubleComplex z; z.s[0] = x; z.s[1] = 0.0; return z; }
};

#define CLIENT_OVERLOADS(T, L)                                                                                       \
    clblasStatus gemm(clblasOrder o, clblasTranspose ta, clblasTranspose tb, size_t m, size_t n, size_t k, T al,     \
                      const T *a, size_t oa, size_t lda, const T *b, size_t ob, size_t ldb, T be, T *c, size_t oc,   \
                      size_t ldc, hipStream_t s) {                                                                   \
        return clblas##L##gemm(o, ta, tb, m, n, k, al, a, oa, lda, b, ob, ldb, be, c, oc, ldc, s);                   \
    }                                                                                                                \
    clblasStatus syrk(clblasOrder o, clblasUplo u, clblasTranspose ta, size_t n, size_t k, T al, const T *a,         \
                      size_t oa, size_t lda, T be, T *c, size_t oc, size_t ldc, hipStream_t s) {                     \
        return clblas##L##syrk(o, u, ta, n, k, al, a, oa, lda, be, c, oc, ldc, s);                                   \
    }                                                                                                                \
    clblasStatus trmm(clblasOrder o, clblasSide sd, clblasUplo u, clblasTranspose ta, clblasDiag d, size_t m,        \
                      size_t n, T al, const T *a, size_t oa, size_t lda, T *b, size_t ob, size_t ldb,                \
                      hipStream_t s) {                                                                               \
        return clblas##L##trmm(o, sd, u, ta, d, m, n, al, a, oa, lda, b, ob, ldb, s);                                \
    }                                                                                                                \
    clblasStatus symm(clblasOrder o, clblasSide sd, clblasUplo u, size_t m, size_t n, T al, const T *a, size_t oa,   \
                      size_t lda, const T *b, size_t ob, size_t ldb, T be, T *c, size_t oc, size_t ldc,              \
                      hipStream_t s) {                                                                               \
        return clblas##L##symm(o, sd, u, m, n, al, a, oa, lda, b, ob, ldb, be, c, oc, ldc, s);                       \
    }                                                                                                                \
    clblasStatus syr2k(clblasOrder o, clblasUplo u, clblasTranspose t, size_t n, size_t k, T al, const T *a,         \
                       size_t oa, size_t lda, const T *b, size_t ob, size_t ldb, T be, T *c, size_t oc, size_t ldc,  \
                       hipStream_t s) {                                                                              \
        return clblas##L##syr2k(o, u, t, n, k, al, a, oa, lda, b, ob, ldb, be, c, oc, ldc, s);                       \
    }
CLIENT_OVERLOADS(float, S)
CLIENT_OVERLOADS(double, D)
CLIENT_OVERLOADS(FloatComplex, C)
CLIENT_OVERLOADS(DoubleComplex, Z)
#undef CLIENT_OVERLOADS
clblasStatus trsm(clblasOrder o, clblasSide sd, clblasUplo u, clblasTranspose ta, clblasDiag d, size_t m, size_t n,
                  float al, const float *a, size_t oa, size_t lda, float *b, size_t ob, size_t ldb, hipStream_t s) {
    return clblasStrsm(o, sd, u, ta, d, m, n, al, a, oa, lda, b, ob, ldb, s);
}
clblasStatus trsm(clblasOrder o, clblasSide sd, clblasUplo u, clblasTranspose ta, clblasDiag d, size_t m, size_t n,
                  double al, const double *a, size_t oa, size_t lda, double *b, size_t ob, size_t ldb, hipStream_t s) {
    return clblasDtrsm(o, sd, u, ta, d, m, n, al, a, oa, lda, b, ob, ldb, s);
}
clblasStatus trsm(clblasOrder o, clblasSide sd, clblasUplo u, clblasTranspose ta, clblasDiag d, size_t m, size_t n,
                  FloatComplex al, const FloatComplex *a, size_t oa, size_t lda, FloatComplex *b, size_t ob, size_t ldb,
                  hipStream_t s) {
    return clblasCtrsm(o, sd, u, ta, d, m, n, al, a, oa, lda, b, ob, ldb, s);
}
clblasStatus trsm(clblasOrder o, clblasSide sd, clblasUplo u, clblasTranspose ta, clblasDiag d, size_t m, size_t n,
                  DoubleComplex al, const DoubleComplex *a, size_t oa, size_t lda, DoubleComplex *b, size_t ob,
                  size_t ldb, hipStream_t s) {
    return clblasZtrsm(o, sd, u, ta, d, m, n, al, a, oa, lda, b, ob, ldb, s);
}

// Hermitian routines exist for the complex types only; alpha (HERK) and beta (HERK, HER2K) are real.
#define CLIENT_HERMITIAN(T, L)                                                                                       \
    clblasStatus herk(clblasOrder o, clblasUplo u, clblasTranspose t, size_t n, size_t k, T al, const T *a,          \
                      size_t oa, size_t lda, T be, T *c, size_t oc, size_t ldc, hipStream_t s) {                     \
        return clblas##L##herk(o, u, t, n, k, al.s[0], a, oa, lda, be.s[0], c, oc, ldc, s);                          \
    }                                                                                                                \
    clblasStatus her2k(clblasOrder o, clblasUplo u, clblasTranspose t, size_t n, size_t k, T al, const T *a,         \
                       size_t oa, size_t lda, const T *b, size_t ob, size_t ldb, T be, T *c, size_t oc, size_t ldc,  \
                       hipStream_t s) {                                                                              \
        return clblas##L##her2k(o, u, t, n, k, al, a, oa, lda, b, ob, ldb, be.s[0], c, oc, ldc, s);                  \
    }                                                                                                                \
    clblasStatus hemm(clblasOrder o, clblasSide sd, clblasUplo u, size_t m, size_t n, T al, const T *a, size_t oa,   \
                      size_t lda, const T *b, size_t ob, size_t ldb, T be, T *c, size_t oc, size_t ldc,              \
                      hipStream_t s) {                                                                               \
        return clblas##L##hemm(o, sd, u, m, n, al, a, oa, lda, b, ob, ldb, be, c, oc, ldc, s);                       \
    }
CLIENT_HERMITIAN(FloatComplex, C)
CLIENT_HERMITIAN(DoubleComplex, Z)
#undef CLIENT_HERMITIAN
// real types: rejected in main() before any call
template <typename T, typename... Rest> clblasStatus herk(clblasOrder, clblasUplo, clblasTranspose, size_t, size_t, T, Rest...) { return clblasNotImplemented; }
template <typename T, typename... Rest> clblasStatus her2k(clblasOrder, clblasUplo, clblasTranspose, size_t, size_t, T, Rest...) { return clblasNotImplemented; }
template <typename T, typename... Rest> clblasStatus hemm(clblasOrder, clblasSide, clblasUplo, size_t, size_t, T, Rest...) { return clblasNotImplemented; }

enum Fn { FN_GEMM, FN_TRSM, FN_TRMM, FN_SYRK, FN_SYMM, FN_SYR2K, FN_HERK, FN_HER2K, FN_HEMM, FN_COUNT };

template <typename T> double run_case(const Options &o, Fn fn, size_t m, size_t n, size_t k, hipStream_t stream, bool &ok) {
    typedef typename Type<T>::Real R;
    const int NC = Type<T>::NC;
    const bool tri = fn == FN_TRSM || fn == FN_TRMM;    // A triangular, B in place
    const size_t an = o.side == 0 ? m : n;                // order of the triangular / symmetric matrix
    auto tight = [&](int trans, size_t rows, size_t cols) { return ((o.order == 1) == (trans == 0)) ? rows : cols; };
    // shapes of A, B, C as the routine sees them
    size_t ar = m, ac = k, br = k, bc = n, cr = m, cc = n;
    int ta = o.transA, tb = o.transB;
    const bool rank_k = fn == FN_SYRK || fn == FN_HERK, rank_2k = fn == FN_SYR2K || fn == FN_HER2K;
    if (tri || fn == FN_SYMM || fn == FN_HEMM) { ar = ac = an; ta = 0; br = m; bc = n; tb = 0; }
    if (rank_k || rank_2k) { ar = n; ac = k; cr = cc = n; br = n; bc = k; tb = ta; }
    const size_t lda = o.lda ? o.lda : tight(ta, ar, ac);
    const size_t ldb = o.ldb ? o.ldb : tight(tb, br, bc);
    const size_t ldc = o.ldc ? o.ldc : tight(0, cr, cc);
    const size_t na = footprint(o.order, ta, ar, ac, o.offA, lda);
    const size_t nb = rank_k ? 1 : footprint(o.order, tb, br, bc, o.offBX, ldb);
    const size_t nc = (tri) ? 1 : footprint(o.order, 0, cr, cc, o.offCY, ldc);
    std::vector<R> ha(na * NC), hb(nb * NC), hc(nc * NC);
    fill(ha, 1, tri ? 1.0 / (double)an : 1.0);
    fill(hb, 2, 1.0);
    fill(hc, 3, 1.0);
    if (tri)  // well-conditioned triangle: diagonal in [1,2)
        for (size_t i = 0; i < an; ++i) {
            R &d = ha[(o.offA + i * lda + i) * NC];
            d = (R)(1.0 + std::fabs((double)d) * (double)an);
        }
    T *da, *db, *dc;
    HIP_OK(hipMalloc((void **)&da, na * sizeof(T)));
    HIP_OK(hipMalloc((void **)&db, nb * sizeof(T)));
    HIP_OK(hipMalloc((void **)&dc, nc * sizeof(T)));
    HIP_OK(hipMemcpy(da, ha.data(), na * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(db, hb.data(), nb * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dc, hc.data(), nc * sizeof(T), hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));

    const T alpha = Type<T>::scalar(o.alpha), beta = Type<T>::scalar(o.beta);
    const clblasOrder ord = (clblasOrder)o.order;
    const clblasTranspose tA = (clblasTranspose)o.transA, tB = (clblasTranspose)o.transB;
    const clblasSide side = (clblasSide)o.side;
    const clblasUplo uplo = (clblasUplo)o.uplo;
    const clblasDiag diag = (clblasDiag)o.diag;
    auto call = [&]() -> clblasStatus {
        switch (fn) {
        case FN_GEMM: return gemm(ord, tA, tB, m, n, k, alpha, da, o.offA, lda, db, o.offBX, ldb, beta, dc, o.offCY, ldc, stream);
        case FN_TRSM: return trsm(ord, side, uplo, tA, diag, m, n, alpha, (const T *)da, o.offA, lda, db, o.offBX, ldb, stream);
        case FN_TRMM: return trmm(ord, side, uplo, tA, diag, m, n, alpha, da, o.offA, lda, db, o.offBX, ldb, stream);
        case FN_SYRK: return syrk(ord, uplo, tA, n, k, alpha, da, o.offA, lda, beta, dc, o.offCY, ldc, stream);
        case FN_SYMM: return symm(ord, side, uplo, m, n, alpha, da, o.offA, lda, db, o.offBX, ldb, beta, dc, o.offCY, ldc, stream);
        case FN_SYR2K: return syr2k(ord, uplo, tA, n, k, alpha, da, o.offA, lda, db, o.offBX, ldb, beta, dc, o.offCY, ldc, stream);
        // (const pointers: an exact match, so that the complex overloads win over the catch-all templates)
        case FN_HERK: return herk(ord, uplo, tA, n, k, alpha, (const T *)da, o.offA, lda, beta, dc, o.offCY, ldc, stream);
        case FN_HER2K: return her2k(ord, uplo, tA, n, k, alpha, (const T *)da, o.offA, lda, (const T *)db, o.offBX, ldb, beta, dc, o.offCY, ldc, stream);
        default: return hemm(ord, side, uplo, m, n, alpha, (const T *)da, o.offA, lda, (const T *)db, o.offBX, ldb, beta, dc, o.offCY, ldc, stream);
        }
    };

    ok = true;
    clblasStatus st = call();  // warm-up sample, as in the reference methodology
    if (st != clblasSuccess) { std::fprintf(stderr, "%s returned %d\n", o.function.c_str(), (int)st); ok = false; }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<double> samples;
    for (unsigned p = 0; ok && p < std::max(1u, o.profile); ++p) {
        if (tri) HIP_OK(hipMemcpyAsync(db, hb.data(), nb * sizeof(T), hipMemcpyHostToDevice, stream));  // fresh B
        HIP_OK(hipEventRecord(e0, stream));
        for (unsigned c = 0; c < std::max(1u, o.apiCallCount); ++c) call();
        HIP_OK(hipEventRecord(e1, stream));
        HIP_OK(hipEventSynchronize(e1));
        float ms = 0;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        samples.push_back((double)ms * 1e6 / std::max(1u, o.apiCallCount));  // ns per call
    }
    double gflops = 0;
    if (ok) {
        std::sort(samples.begin(), samples.end());
        const double ns = samples[samples.size() / 2];
        // flop counts of the reference client: clfunc_xgemm.hpp:95-107,1199-1210, clfunc_xtrsm.hpp:70-92,
        // clfunc_xtrmm.hpp:85-95,757-784, clfunc_xsyrk.hpp:65-68,588-649, clfunc_xsymm.hpp:63-69,628-645,
        // clfunc_xsyr2k.hpp:70-73,754-757, clfunc_xherk.hpp:60-63, clfunc_xher2k.hpp:65-68, clfunc_xhemm.hpp:83-93
        const double cplx = NC == 2 ? 4.0 : 1.0, M = (double)m, N = (double)n, K = (double)k;
        double flop = 0;
        switch (fn) {
        case FN_GEMM: flop = 2.0 * cplx * M * N * K; break;
        case FN_TRSM:
        case FN_TRMM: flop = cplx * (o.side == 0 ? M * (M + 1) * N : M * (N + 1) * N); break;
        case FN_SYRK:
        case FN_HERK: flop = cplx * N * (N + 1) * K; break;
        case FN_SYR2K:
        case FN_HER2K: flop = 2.0 * cplx * K * N * N + (NC == 2 ? 2.0 : 1.0) * N; break;
        default: flop = 2.0 * cplx * (o.side == 0 ? M * M * N : N * N * M); break;
        }
        gflops = flop / ns;
    }
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    HIP_OK(hipFree(da));
    HIP_OK(hipFree(db));
    HIP_OK(hipFree(dc));
    return gflops;
}

const char *trans_name(int t) { return t == 0 ? "none" : (t == 1 ? "transpose" : "conj"); }

}  // namespace

int main(int argc, char **argv) {
    Options o;
    if (!parse(argc, argv, o)) { usage(); return 2; }
    const char *fnames[] = {"gemm", "trsm", "trmm", "syrk", "symm", "syr2k", "herk", "her2k", "hemm"};
    int fn = -1;
    for (int i = 0; i < FN_COUNT; ++i)
        if (o.function == fnames[i]) fn = i;
    const bool real = o.precision == "s" || o.precision == "d", cplx = o.precision == "c" || o.precision == "z";
    if (fn < 0 || !(real || cplx) || (real && fn >= FN_HERK)) {
        std::fprintf(stderr, "this library implements -f gemm|trsm|trmm|syrk|symm|syr2k with -r s|d|c|z and "
                             "-f herk|her2k|hemm with -r c|z\n");
        return 2;
    }
    if (clblasSetup() != clblasSuccess) { std::fprintf(stderr, "clblasSetup failed (needs a gfx950 device)\n"); return 1; }
    std::vector<size_t> sizes;
    if (!o.sizes.empty()) {
        size_t a = 0, b = 0, s = 1;
        if (std::sscanf(o.sizes.c_str(), "%zu:%zu:%zu", &a, &b, &s) < 2 || s == 0 || a == 0) { usage(); return 2; }
        for (size_t x = a; x <= b; x += s) sizes.push_back(x);
    }
    if (o.header)
        std::puts("m,n,k,lda,ldb,ldc,offa,offb,offc,alpha,beta,order,transa,transb,side,uplo,diag,function,device,"
                  "library,numQueues,label,GFLOPS");
    const size_t count = sizes.empty() ? 1 : sizes.size();
    int rc = 0;
    hipStream_t stream;  // one stream for the whole run: the library keeps its scratch buffers per stream
    HIP_OK(hipStreamCreate(&stream));
    for (size_t i = 0; i < count; ++i) {
        const size_t m = sizes.empty() ? o.m : sizes[i], n = sizes.empty() ? o.n : sizes[i], k = sizes.empty() ? o.k : sizes[i];
        bool ok = true;
        double g;
        if (o.precision == "s") g = run_case<float>(o, (Fn)fn, m, n, k, stream, ok);
        else if (o.precision == "d") g = run_case<double>(o, (Fn)fn, m, n, k, stream, ok);
        else if (o.precision == "c") g = run_case<FloatComplex>(o, (Fn)fn, m, n, k, stream, ok);
        else g = run_case<DoubleComplex>(o, (Fn)fn, m, n, k, stream, ok);
        if (!ok) { rc = 1; continue; }
        std::printf("%zu,%zu,%zu,%zu,%zu,%zu,%zu,%zu,%zu,%g,%g,%s,%s,%s,%s,%s,%s,%s%s,gpu,clblas_amd,1,%s,%g\n", m, n, k,
                    o.lda, o.ldb, o.ldc, o.offA, o.offBX, o.offCY, o.alpha, o.beta, o.order ? "column" : "row",
                    trans_name(o.transA), trans_name(o.transB), o.side ? "right" : "left", o.uplo ? "lower" : "upper",
                    o.diag ? "nonunit" : "unit", o.precision.c_str(), o.function.c_str(), o.label.c_str(), g);
        std::fflush(stdout);
    }
    HIP_OK(hipStreamSynchronize(stream));
    clblasAmdReleaseStream(stream);
    HIP_OK(hipStreamDestroy(stream));
    clblasTeardown();
    return rc;
}
