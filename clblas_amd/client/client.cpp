// clblas_amd-client: benchmark command line for libclblas_amd.so.
//
// Takes the place of the reference's clBLAS-client (src/client/client.cpp:80-112 for the
// option names, src/client/clfunc_xgemm.hpp:95-107 and clfunc_xtrsm.hpp:70-92 for the
// GFLOP/s formulas) for the two function families this library implements, and prints the
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
        "  -f/--function gemm|trsm   -r/--precision s|d\n"
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

template <typename T> void fill(std::vector<T> &v, uint64_t seed, double scale, double shift) {
    uint64_t s = seed * 0x9e3779b97f4a7c15ULL + 1;
    for (auto &x : v) {
        s = s * 6364136223846793005ULL + 1442695040888963407ULL;
        x = (T)(((double)(s >> 40) / (double)(1 << 24) * 2.0 - 1.0) * scale + shift);
    }
}

template <typename T> double run_case(const Options &o, size_t m, size_t n, size_t k, bool &ok) {
    const bool gemm = o.function == "gemm";
    const size_t an = o.side == 0 ? m : n;  // order of the triangular matrix
    auto tight = [&](int trans, size_t rows, size_t cols) { return ((o.order == 1) == (trans == 0)) ? rows : cols; };
    const size_t lda = o.lda ? o.lda : (gemm ? tight(o.transA, m, k) : an);
    const size_t ldb = o.ldb ? o.ldb : (gemm ? tight(o.transB, k, n) : tight(0, m, n));
    const size_t ldc = o.ldc ? o.ldc : tight(0, m, n);
    const size_t na = gemm ? footprint(o.order, o.transA, m, k, o.offA, lda) : footprint(o.order, 0, an, an, o.offA, lda);
    const size_t nb = gemm ? footprint(o.order, o.transB, k, n, o.offBX, ldb) : footprint(o.order, 0, m, n, o.offBX, ldb);
    const size_t nc = gemm ? footprint(o.order, 0, m, n, o.offCY, ldc) : 1;
    std::vector<T> ha(na), hb(nb), hc(nc);
    fill(ha, 1, gemm ? 1.0 : 1.0 / (double)an, 0.0);
    fill(hb, 2, 1.0, 0.0);
    fill(hc, 3, 1.0, 0.0);
    if (!gemm)  // well-conditioned triangle: diagonal in [1,2)
        for (size_t i = 0; i < an; ++i) ha[o.offA + i * lda + i] = (T)(1.0 + std::fabs((double)ha[o.offA + i * lda + i]) * (double)an);
    T *da, *db, *dc;
    HIP_OK(hipMalloc((void **)&da, na * sizeof(T)));
    HIP_OK(hipMalloc((void **)&db, nb * sizeof(T)));
    HIP_OK(hipMalloc((void **)&dc, nc * sizeof(T)));
    HIP_OK(hipMemcpy(da, ha.data(), na * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(db, hb.data(), nb * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dc, hc.data(), nc * sizeof(T), hipMemcpyHostToDevice));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));

    auto call = [&]() -> clblasStatus {
        if (gemm) {
            if (sizeof(T) == 4)
                return clblasSgemm((clblasOrder)o.order, (clblasTranspose)o.transA, (clblasTranspose)o.transB, m, n, k,
                                   (float)o.alpha, (const float *)da, o.offA, lda, (const float *)db, o.offBX, ldb,
                                   (float)o.beta, (float *)dc, o.offCY, ldc, stream);
            return clblasDgemm((clblasOrder)o.order, (clblasTranspose)o.transA, (clblasTranspose)o.transB, m, n, k,
                               o.alpha, (const double *)da, o.offA, lda, (const double *)db, o.offBX, ldb, o.beta,
                               (double *)dc, o.offCY, ldc, stream);
        }
        if (sizeof(T) == 4)
            return clblasStrsm((clblasOrder)o.order, (clblasSide)o.side, (clblasUplo)o.uplo, (clblasTranspose)o.transA,
                               (clblasDiag)o.diag, m, n, (float)o.alpha, (const float *)da, o.offA, lda, (float *)db,
                               o.offBX, ldb, stream);
        return clblasDtrsm((clblasOrder)o.order, (clblasSide)o.side, (clblasUplo)o.uplo, (clblasTranspose)o.transA,
                           (clblasDiag)o.diag, m, n, o.alpha, (const double *)da, o.offA, lda, (double *)db, o.offBX,
                           ldb, stream);
    };

    ok = true;
    clblasStatus st = call();  // warm-up sample, as in the reference methodology
    if (st != clblasSuccess) { std::fprintf(stderr, "%s returned %d\n", o.function.c_str(), (int)st); ok = false; }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<double> samples;
    for (unsigned p = 0; ok && p < std::max(1u, o.profile); ++p) {
        if (!gemm) HIP_OK(hipMemcpyAsync(db, hb.data(), nb * sizeof(T), hipMemcpyHostToDevice, stream));  // fresh right-hand sides
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
        const double flop = gemm ? 2.0 * m * n * k : (o.side == 0 ? (double)m * (m + 1) * n : (double)m * (n + 1) * n);
        gflops = flop / ns;
    }
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    HIP_OK(hipStreamDestroy(stream));
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
    if ((o.function != "gemm" && o.function != "trsm") || (o.precision != "s" && o.precision != "d")) {
        std::fprintf(stderr, "this library implements -f gemm|trsm with -r s|d\n");
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
    for (size_t i = 0; i < count; ++i) {
        const size_t m = sizes.empty() ? o.m : sizes[i], n = sizes.empty() ? o.n : sizes[i], k = sizes.empty() ? o.k : sizes[i];
        bool ok = true;
        const double g = o.precision == "s" ? run_case<float>(o, m, n, k, ok) : run_case<double>(o, m, n, k, ok);
        if (!ok) { rc = 1; continue; }
        std::printf("%zu,%zu,%zu,%zu,%zu,%zu,%zu,%zu,%zu,%g,%g,%s,%s,%s,%s,%s,%s,%s%s,gpu,clblas_amd,1,%s,%g\n", m, n, k,
                    o.lda, o.ldb, o.ldc, o.offA, o.offBX, o.offCY, o.alpha, o.beta, o.order ? "column" : "row",
                    trans_name(o.transA), trans_name(o.transB), o.side ? "right" : "left", o.uplo ? "lower" : "upper",
                    o.diag ? "nonunit" : "unit", o.precision.c_str(), o.function.c_str(), o.label.c_str(), g);
        std::fflush(stdout);
    }
    clblasTeardown();
    return rc;
}
