// C ABI of libclblas_amd.so: argument validation, row-major folding and dispatch.
//
// This is the host front end that stands where the reference has
//   src/library/blas/xgemm.cc:667-905  (clblasSgemm / clblasDgemm / clblasCgemm / clblasZgemm),
//   src/library/blas/xgemm.cc:341-383  (clblasGemm<T>: ConjTrans and row-major folding),
//   src/library/blas/xtrsm.cc:1600-1914 (clblasStrsm / clblasDtrsm / clblasCtrsm / clblasZtrsm),
//   src/library/blas/xsyrk.c:27-233, xtrmm.c:27-245, xsymm.c:33-429 (SYRK / TRMM / SYMM),
//   src/library/blas/xsyr2k.c:27-251, xherk.c:29-210, xher2k.c:30-245, xhemm.c:36-112
//   (SYR2K / HERK / HER2K / HEMM),
//   src/library/blas/functor/functor_xtrsm.cc:57-75 (doTrsm validation),
//   src/library/blas/generic/common.c:585-688 (checkMatrixSizes),
//   src/library/blas/init.c:33-263 (GetVersion / Setup / Teardown).
#include "../../include/clblas_amd.h"
#include "internal.h"
#include "workspace.hpp"

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

namespace cba {

namespace {
DebugKnobs g_knobs;
std::once_flag g_knobs_once;

int env_int(const char *name, int dflt) {
    const char *s = std::getenv(name);
    if (!s || !*s) return dflt;
    return std::atoi(s);
}

void read_knobs() {
    DebugKnobs k;
    k.gemm_tile = env_int("CLBLAS_AMD_GEMM_TILE", -1);
    k.split_model = env_int("CLBLAS_AMD_GEMM_SPLIT_MODEL", 1);
    k.splits = env_int("CLBLAS_AMD_GEMM_SPLITS", 0);
    k.tail = env_int("CLBLAS_AMD_GEMM_TAIL", 1);
    k.peel = env_int("CLBLAS_AMD_GEMM_PEEL", 1);
    k.group_m = env_int("CLBLAS_AMD_GEMM_GROUP_M", 0);
    k.xcd = env_int("CLBLAS_AMD_GEMM_XCD", 1);
    k.stagger = env_int("CLBLAS_AMD_GEMM_STAGGER", 1);
    k.deep_panels = env_int("CLBLAS_AMD_GEMM_DEEP", 1);
    k.wide_ld = env_int("CLBLAS_AMD_GEMM_WIDE_LD", 0);
    k.log = env_int("CLBLAS_AMD_LOG", 0);
    k.check_mem = env_int("CLBLAS_AMD_CHECK_MEM", 0);
    k.trsm_leaf = env_int("CLBLAS_AMD_TRSM_LEAF", 0);
    k.trsm_wide = env_int("CLBLAS_AMD_TRSM_WIDE", -1);
    k.trsm_poll_limit = env_int("CLBLAS_AMD_TRSM_POLL_LIMIT", 0);
    g_knobs = k;
}
}  // namespace

const DebugKnobs &knobs() {
    std::call_once(g_knobs_once, read_knobs);
    return g_knobs;
}

// Debugging only: must not run while another thread is inside a library call.
void reload_knobs() {
    std::call_once(g_knobs_once, read_knobs);
    read_knobs();
}

DispatchRecord &dispatch_record() {
    static thread_local DispatchRecord rec;
    return rec;
}

namespace {
void *hip_ws_alloc(int device, size_t bytes) {
    int cur = 0;
    if (hipGetDevice(&cur) != hipSuccess) return nullptr;
    if (cur != device && hipSetDevice(device) != hipSuccess) return nullptr;
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();  // the failed allocation is reported through the return value
        p = nullptr;
    }
    if (cur != device) (void)hipSetDevice(cur);
    return p;
}
void hip_ws_release(int device, void *ptr) {
    int cur = 0;
    (void)hipGetDevice(&cur);
    if (cur != device) (void)hipSetDevice(device);
    (void)hipFree(ptr);
    if (cur != device) (void)hipSetDevice(cur);
}
bool hip_ws_sync(int device) {
    int cur = 0;
    (void)hipGetDevice(&cur);
    if (cur != device) (void)hipSetDevice(device);
    // (fails, for one, while a stream of the device is being captured in global mode)
    const hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) (void)hipGetLastError();
    if (cur != device) (void)hipSetDevice(cur);
    return e == hipSuccess;
}
WorkspaceCache &ws_cache() {
    static WorkspaceCache cache(WorkspaceAllocator{hip_ws_alloc, hip_ws_release, hip_ws_sync});
    return cache;
}
std::mutex g_lds_mutex;
std::map<std::pair<int, const void *>, size_t> g_lds_limit;

thread_local DryRun *tl_dry_run = nullptr;
thread_local CallLease *tl_lease = nullptr;

bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cap != hipStreamCaptureStatusNone;
}
}  // namespace

DryRun *&dry_run_slot() { return tl_dry_run; }

CallLease::CallLease() : outer(tl_lease) { tl_lease = this; }
CallLease::~CallLease() {
    if (held) ws_cache().unlease(device, (const void *)stream);
    tl_lease = outer;
}

hipError_t workspace_get(hipStream_t stream, size_t bytes, int kind, void **out) {
    *out = nullptr;
    if (DryRun *dry = tl_dry_run) {  // only the size is wanted; the pointer is never used
        if (bytes > dry->need[kind]) dry->need[kind] = bytes;
        *out = reinterpret_cast<void *>(uintptr_t(256));
        return hipSuccess;
    }
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    // The first request of an API call takes the call's lease on the stream's entry (CallLease).
    CallLease *lease = tl_lease;
    const bool want_lease = lease && !lease->held;
    WorkspaceError why = WS_OK;
    bool pinned = false;
    // Fast path: the buffer exists.
    void *p = ws_cache().get(dev, (const void *)stream, kind, bytes, false, &why, want_lease, &pinned);
    if (p) {
        // A buffer handed out under capture ends up in a graph: the entry is pinned from then on.
        if (!pinned && stream_is_capturing(stream)) ws_cache().pin(dev, (const void *)stream);
    } else {
        // It has to be allocated: not on a stream that is being captured into a graph (hipMalloc
        // there would fail and invalidate the capture).
        if (stream_is_capturing(stream)) return hipErrorStreamCaptureUnsupported;
        p = ws_cache().get(dev, (const void *)stream, kind, bytes, true, &why, want_lease, &pinned);
        if (!p) return hipErrorOutOfMemory;
    }
    if (want_lease) {
        lease->held = true;
        lease->device = dev;
        lease->stream = stream;
    }
    *out = p;
    return hipSuccess;
}

bool workspace_release_all() { return ws_cache().release_all(); }
void ws_release_stream(int device, hipStream_t stream) { ws_cache().release_stream(device, (const void *)stream); }
void ws_stats(size_t *streams, size_t *bytes) {
    if (streams) *streams = ws_cache().stream_count();
    if (bytes) *bytes = ws_cache().bytes_held();
}

// Kernels that need more than 64 KiB of dynamic LDS have the limit raised once per (function,
// device).  Every launch of such a kernel asks, so the answer for the usual case - already raised -
// comes from a small open-addressed table of atomics without taking a lock; the mutex and the map
// behind it serve the first call per pair and anything the table has no room for.
namespace {
constexpr int kLdsSlots = 1024, kLdsDevices = 16;
struct LdsSlot {
    std::atomic<const void *> fn{nullptr};
    std::atomic<size_t> limit[kLdsDevices];
};
LdsSlot g_lds_slots[kLdsSlots];

std::atomic<size_t> *lds_slot_for(const void *fn, int dev) {
    if (dev < 0 || dev >= kLdsDevices) return nullptr;
    size_t h = (reinterpret_cast<uintptr_t>(fn) >> 4) * 0x9e3779b97f4a7c15ULL >> 40;
    for (int probe = 0; probe < 16; ++probe, ++h) {
        LdsSlot &s = g_lds_slots[h % kLdsSlots];
        const void *cur = s.fn.load(std::memory_order_acquire);
        if (cur == nullptr) {
            const void *expected = nullptr;
            if (s.fn.compare_exchange_strong(expected, fn, std::memory_order_acq_rel)) cur = fn;
            else cur = expected;
        }
        if (cur == fn) return &s.limit[dev];
    }
    return nullptr;
}
}  // namespace

hipError_t ensure_dynamic_lds(const void *fn, size_t bytes) {
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    std::atomic<size_t> *fast = lds_slot_for(fn, dev);
    if (fast && fast->load(std::memory_order_acquire) >= bytes) return hipSuccess;
    std::lock_guard<std::mutex> lock(g_lds_mutex);
    size_t &cur = g_lds_limit[std::make_pair(dev, fn)];
    if (cur < bytes) {
        err = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (err != hipSuccess) return err;
        cur = bytes;
    }
    if (fast) fast->store(cur, std::memory_order_release);
    return hipSuccess;
}

// ---- CLBLAS_AMD_CHECK_MEM: how much memory lies behind a device pointer ----
namespace {
size_t hip_mem_probe(const void *ptr) {
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr) != hipSuccess || !base) {
        (void)hipGetLastError();
        return 0;
    }
    const uintptr_t b = reinterpret_cast<uintptr_t>(base), p = reinterpret_cast<uintptr_t>(ptr);
    return (p >= b && p - b < size) ? size - (p - b) : 0;
}
std::atomic<MemProbe> g_mem_probe{hip_mem_probe};
}  // namespace

void set_mem_probe(MemProbe probe) { g_mem_probe.store(probe ? probe : hip_mem_probe); }
size_t mem_behind(const void *ptr) { return g_mem_probe.load()(ptr); }

}  // namespace cba

namespace {

enum MatId { MAT_A = 0, MAT_B = 1, MAT_C = 2 };

clblasStatus lead_dim_error(MatId m) {
    return m == MAT_A ? clblasInvalidLeadDimA : (m == MAT_B ? clblasInvalidLeadDimB : clblasInvalidLeadDimC);
}

clblasStatus mem_error(MatId m, bool insufficient) {
    if (insufficient)
        return m == MAT_A ? clblasInsufficientMemMatA : (m == MAT_B ? clblasInsufficientMemMatB : clblasInsufficientMemMatC);
    return m == MAT_A ? clblasInvalidMatA : (m == MAT_B ? clblasInvalidMatB : clblasInvalidMatC);
}

// Restates checkMatrixSizes (generic/common.c:585-688) for a rows x cols logical matrix:
// zero dimension -> InvalidDim; ld below the number of elements that are contiguous in
// memory -> InvalidLeadDim{A,B,C}.  The reference's third outcome, InsufficientMemMat*
// (common.c:644-684), compares offset + footprint against CL_MEM_SIZE of the cl_mem.  A raw
// device pointer carries no size, so by default that code cannot arise; with the debug switch
// CLBLAS_AMD_CHECK_MEM=1 the allocation behind `base` is looked up and the same rule applied:
// (off + (lines - 1) ld + run) sizeof(T) beyond the memory behind the pointer ->
// InsufficientMemMat{A,B,C}; a pointer that no allocation holds -> InvalidMat{A,B,C} (the
// reference's answer when clGetMemObjectInfo fails).
clblasStatus check_matrix_sizes(clblasOrder order, clblasTranspose trans, size_t rows, size_t cols, size_t ld,
                                MatId which, const void *base, size_t off, size_t tsize) {
    if (rows == 0 || cols == 0) return clblasInvalidDim;
    const bool rows_contiguous = (order == clblasRowMajor && trans != clblasNoTrans) ||
                                 (order == clblasColumnMajor && trans == clblasNoTrans);
    if (rows_contiguous ? (ld < rows) : (ld < cols)) return lead_dim_error(which);
    if (cba::knobs().check_mem) {
        const size_t mem = cba::mem_behind(base);
        if (mem == 0) return mem_error(which, false);
        const size_t run = rows_contiguous ? rows : cols, lines = rows_contiguous ? cols : rows;
        // ((lines - 1) ld + run + off) tsize, refusing anything that leaves 64 bits on the way
        unsigned __int128 used = (unsigned __int128)(lines - 1) * ld + run + off;
        used *= tsize;
        if (used > (unsigned __int128)mem) return mem_error(which, true);
    }
    return clblasSuccess;
}

bool valid_order(clblasOrder o) { return o == clblasRowMajor || o == clblasColumnMajor; }
bool valid_trans(clblasTranspose t) { return t == clblasNoTrans || t == clblasTrans || t == clblasConjTrans; }

clblasStatus map_hip_error(hipError_t e) {
    if (e == hipSuccess) return clblasSuccess;
    (void)hipGetLastError();
    if (e == hipErrorOutOfMemory) return clblasOutOfResources;
    if (e == hipErrorInvalidValue) return clblasInvalidValue;
    if (e == hipErrorNotSupported) return clblasNotImplemented;
    if (e == hipErrorStreamCaptureUnsupported) return clblasInvalidOperation;  // would have had to allocate under capture
    return clblasOutOfResources;
}

// Kernels index rows and columns with 32-bit ints (reference: cl_uint, xgemm.cc:362-372); the largest
// index they form is a dimension rounded up to a whole tile (edge 256) plus one vector, so dimensions
// stop one tile short of 2^31.
const size_t kMaxDim = 0x7fffffff - 512;

template <typename T, bool NOALLOC = false>
clblasStatus gemm_front(clblasOrder order, clblasTranspose transA, clblasTranspose transB, size_t M,
                        size_t N, size_t K, T alpha, const T *A, size_t offA, size_t lda, const T *B, size_t offB,
                        size_t ldb, T beta, T *C, size_t offC, size_t ldc, hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    // Order of checks follows xgemm.cc:685-706: objects A, B, C; then (K != 0) sizes of A,
    // sizes of B; then sizes of C.
    if (!A) return clblasInvalidMatA;
    if (!B) return clblasInvalidMatB;
    if (!C) return clblasInvalidMatC;
    if (!valid_order(order) || !valid_trans(transA) || !valid_trans(transB)) return clblasInvalidValue;
    clblasStatus st;
    if (K != 0) {
        if ((st = check_matrix_sizes(order, transA, M, K, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
        if ((st = check_matrix_sizes(order, transB, K, N, ldb, MAT_B, B, offB, sizeof(*B))) != clblasSuccess) return st;
    }
    if ((st = check_matrix_sizes(order, clblasNoTrans, M, N, ldc, MAT_C, C, offC, sizeof(*C))) != clblasSuccess) return st;
    if (M > kMaxDim || N > kMaxDim || K > kMaxDim) return clblasNotImplemented;

    // Real types: ConjTrans is Trans (xgemm.cc:330-335); the real launchers ignore cA / cB.
    bool tA = transA != clblasNoTrans, tB = transB != clblasNoTrans;
    bool cA = transA == clblasConjTrans, cB = transB == clblasConjTrans;
    const T *pa = A + offA, *pb = B + offB;
    // Row major is the column-major product C^T = op(B)^T op(A)^T (xgemm.cc:40-61):
    // swap the operands, their transposes, leading dimensions, and M with N.
    if (order == clblasRowMajor) {
        std::swap(tA, tB);
        std::swap(cA, cB);
        std::swap(M, N);
        std::swap(lda, ldb);
        std::swap(pa, pb);
    }
    if constexpr (NOALLOC)
        return map_hip_error(cba::sgemm_colmajor_noalloc(tA, tB, (int)M, (int)N, (int)K, alpha, pa, (int64_t)lda, pb,
                                                         (int64_t)ldb, beta, C + offC, (int64_t)ldc, stream));
    else
        // (a product may be made in two or three launches - see run_gemm_colmajor - so under capture every
        // scratch buffer is secured before the first of them)
        return map_hip_error(cba::with_workspaces_secured(stream, [&] {
            return cba::launch_gemm<T>(tA, tB, cA, cB, (int)M, (int)N, (int)K, alpha, pa, (int64_t)lda, pb, (int64_t)ldb, beta,
                                       C + offC, (int64_t)ldc, stream);
        }));
}

template <typename T> struct IsComplex { static const bool value = false; };
template <typename R> struct IsComplex<cba::Cx<R>> { static const bool value = true; };

// SYRK front end.  Checks as doSyrk (src/library/blas/xsyrk.c:56-72): objects A, C; ConjTrans
// is invalid for complex types; A is N x K, C is N x N.  Row major: the same memory read
// column-major holds A^T and C^T, so flip the transpose flag and the triangle.
template <typename T>
clblasStatus syrk_front(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K, T alpha,
                        const T *A, size_t offA, size_t lda, T beta, T *C, size_t offC, size_t ldc,
                        hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    if (!A) return clblasInvalidMatA;
    if (!C) return clblasInvalidMatC;
    if (!valid_order(order) || !valid_trans(transA) || (uplo != clblasUpper && uplo != clblasLower))
        return clblasInvalidValue;
    if (IsComplex<T>::value && transA == clblasConjTrans) return clblasInvalidValue;
    clblasStatus st;
    if ((st = check_matrix_sizes(order, transA, N, K, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, N, N, ldc, MAT_C, C, offC, sizeof(*C))) != clblasSuccess) return st;
    if (N > kMaxDim || K > kMaxDim) return clblasNotImplemented;
    bool lower = uplo == clblasLower, trans = transA != clblasNoTrans;
    if (order == clblasRowMajor) {
        lower = !lower;
        trans = !trans;
    }
    return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::syrk_colmajor<T>(lower, trans, (int)N, (int)K, alpha, A + offA, (int64_t)lda, beta,
                                               C + offC, (int64_t)ldc, stream); }));
}

// TRMM front end.  Checks as doTrmm (src/library/blas/xtrmm.c:47-64), the same as TRSM's;
// row-major folding as for TRSM.
template <typename T>
clblasStatus trmm_front(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA,
                        clblasDiag diag, size_t M, size_t N, T alpha, const T *A, size_t offA, size_t lda, T *B,
                        size_t offB, size_t ldb, hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    if (!A) return clblasInvalidMatA;
    if (!B) return clblasInvalidMatB;
    if (!valid_order(order) || !valid_trans(transA) || (side != clblasLeft && side != clblasRight) ||
        (uplo != clblasUpper && uplo != clblasLower) || (diag != clblasUnit && diag != clblasNonUnit))
        return clblasInvalidValue;
    const size_t msize = side == clblasLeft ? M : N;
    clblasStatus st;
    if ((st = check_matrix_sizes(order, transA, msize, msize, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, M, N, ldb, MAT_B, B, offB, sizeof(*B))) != clblasSuccess) return st;
    if (M > kMaxDim || N > kMaxDim) return clblasNotImplemented;
    bool right = side == clblasRight, lower = uplo == clblasLower;
    if (order == clblasRowMajor) {
        std::swap(M, N);
        right = !right;
        lower = !lower;
    }
    return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::trmm_colmajor<T>(right, lower, transA != clblasNoTrans,
                                               IsComplex<T>::value && transA == clblasConjTrans, diag == clblasUnit,
                                               (int)M, (int)N, alpha, A + offA, (int64_t)lda, B + offB, (int64_t)ldb,
                                               stream); }));
}

// SYMM front end.  Checks as doSymm (src/library/blas/xsymm.c:50-71): objects A, B, C; A is
// M x M (left) or N x N (right); B and C are M x N.  Row major swaps M and N and flips side
// and triangle (xsymm.c:104-124).
template <typename T, bool HERM = false>
clblasStatus symm_front(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, T alpha, const T *A,
                        size_t offA, size_t lda, const T *B, size_t offB, size_t ldb, T beta, T *C, size_t offC,
                        size_t ldc, hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    if (!A) return clblasInvalidMatA;
    if (!B) return clblasInvalidMatB;
    if (!C) return clblasInvalidMatC;
    if (!valid_order(order) || (side != clblasLeft && side != clblasRight) ||
        (uplo != clblasUpper && uplo != clblasLower))
        return clblasInvalidValue;
    const size_t msize = side == clblasLeft ? M : N;
    clblasStatus st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, msize, msize, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, M, N, ldb, MAT_B, B, offB, sizeof(*B))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, M, N, ldc, MAT_C, C, offC, sizeof(*C))) != clblasSuccess) return st;
    if (M > kMaxDim || N > kMaxDim) return clblasNotImplemented;
    bool right = side == clblasRight, lower = uplo == clblasLower;
    if (order == clblasRowMajor) {
        std::swap(M, N);
        right = !right;
        lower = !lower;
    }
    if constexpr (HERM)  // HEMM goes through doSymm as well (xhemm.c:69-73), same checks and folding
        return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::hemm_colmajor<T>(right, lower, (int)M, (int)N, alpha, A + offA, (int64_t)lda,
                                                   B + offB, (int64_t)ldb, beta, C + offC, (int64_t)ldc, stream); }));
    else
        return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::symm_colmajor<T>(right, lower, (int)M, (int)N, alpha, A + offA, (int64_t)lda,
                                                   B + offB, (int64_t)ldb, beta, C + offC, (int64_t)ldc, stream); }));
}

// SYR2K front end.  Checks as doSyr2k (src/library/blas/xsyr2k.c:58-76): objects A, B, C;
// ConjTrans is invalid for complex types; A and B are N x K, C is N x N.  Row-major folding as
// for SYRK.
template <typename T>
clblasStatus syr2k_front(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K, T alpha,
                         const T *A, size_t offA, size_t lda, const T *B, size_t offB, size_t ldb, T beta, T *C,
                         size_t offC, size_t ldc, hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    if (!A) return clblasInvalidMatA;
    if (!B) return clblasInvalidMatB;
    if (!C) return clblasInvalidMatC;
    if (!valid_order(order) || !valid_trans(transAB) || (uplo != clblasUpper && uplo != clblasLower))
        return clblasInvalidValue;
    if (IsComplex<T>::value && transAB == clblasConjTrans) return clblasInvalidValue;
    clblasStatus st;
    if ((st = check_matrix_sizes(order, transAB, N, K, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, transAB, N, K, ldb, MAT_B, B, offB, sizeof(*B))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, N, N, ldc, MAT_C, C, offC, sizeof(*C))) != clblasSuccess) return st;
    if (N > kMaxDim || K > kMaxDim) return clblasNotImplemented;
    bool lower = uplo == clblasLower, trans = transAB != clblasNoTrans;
    if (order == clblasRowMajor) {
        lower = !lower;
        trans = !trans;
    }
    return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::syr2k_colmajor<T>(lower, trans, (int)N, (int)K, alpha, A + offA, (int64_t)lda, B + offB,
                                                (int64_t)ldb, beta, C + offC, (int64_t)ldc, stream); }));
}

// HERK / HER2K front end (B == nullptr with `two` false: HERK).  Checks as doHerk / doHer2k
// (src/library/blas/xherk.c:64-84, xher2k.c:73-97): objects; plain Trans is invalid; A (and B)
// N x K, C N x N.  Row major (xherk.c:88-89, xher2k.c:99-100, 192-195): the same memory read
// column-major holds the transposes, so flip the triangle, swap NoTrans <-> ConjTrans and
// conjugate alpha.
template <typename R>
clblasStatus herk_front(bool two, clblasOrder order, clblasUplo uplo, clblasTranspose trans, size_t N, size_t K,
                        cba::Cx<R> alpha, const cba::Cx<R> *A, size_t offA, size_t lda, const cba::Cx<R> *B,
                        size_t offB, size_t ldb, R beta, cba::Cx<R> *C, size_t offC, size_t ldc, hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    if (!A) return clblasInvalidMatA;
    if (two && !B) return clblasInvalidMatB;
    if (!C) return clblasInvalidMatC;
    if (!valid_order(order) || !valid_trans(trans) || (uplo != clblasUpper && uplo != clblasLower))
        return clblasInvalidValue;
    if (trans == clblasTrans) return clblasInvalidValue;
    clblasStatus st;
    if ((st = check_matrix_sizes(order, trans, N, K, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
    if (two && (st = check_matrix_sizes(order, trans, N, K, ldb, MAT_B, B, offB, sizeof(*B))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, N, N, ldc, MAT_C, C, offC, sizeof(*C))) != clblasSuccess) return st;
    if (N > kMaxDim || K > kMaxDim) return clblasNotImplemented;
    bool lower = uplo == clblasLower, ctrans = trans != clblasNoTrans;
    if (order == clblasRowMajor) {
        lower = !lower;
        ctrans = !ctrans;
        alpha.im = -alpha.im;
    }
    if (!two)
        return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::herk_colmajor<R>(lower, ctrans, (int)N, (int)K, alpha.re, A + offA, (int64_t)lda,
                                                   beta, C + offC, (int64_t)ldc, stream); }));
    return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::her2k_colmajor<R>(lower, ctrans, (int)N, (int)K, alpha, A + offA, (int64_t)lda,
                                                B + offB, (int64_t)ldb, beta, C + offC, (int64_t)ldc, stream); }));
}

static_assert(sizeof(FloatComplex) == sizeof(cba::Cx<float>) && sizeof(DoubleComplex) == sizeof(cba::Cx<double>),
              "complex layouts must agree");
inline cba::Cx<float> cx(FloatComplex z) { return cba::Cx<float>{z.s[0], z.s[1]}; }
inline cba::Cx<double> cx(DoubleComplex z) { return cba::Cx<double>{z.s[0], z.s[1]}; }
// Interleaved (re, im) arrays: the same memory seen through the kernels' element type.
inline const cba::Cx<float> *cx(const FloatComplex *p) { return reinterpret_cast<const cba::Cx<float> *>(p); }
inline cba::Cx<float> *cx(FloatComplex *p) { return reinterpret_cast<cba::Cx<float> *>(p); }
inline const cba::Cx<double> *cx(const DoubleComplex *p) { return reinterpret_cast<const cba::Cx<double> *>(p); }
inline cba::Cx<double> *cx(DoubleComplex *p) { return reinterpret_cast<cba::Cx<double> *>(p); }

template <typename T>
clblasStatus trsm_front(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA,
                        clblasDiag diag, size_t M, size_t N, T alpha, const T *A, size_t offA, size_t lda, T *B,
                        size_t offB, size_t ldb, hipStream_t stream) {
    cba::CallLease lease;  // scratch handed out during this call stays ours until it returns
    // Order of checks follows doTrsm (functor_xtrsm.cc:57-75): objects, A (msize^2), B (M x N).
    if (!A) return clblasInvalidMatA;
    if (!B) return clblasInvalidMatB;
    if (!valid_order(order) || !valid_trans(transA) || (side != clblasLeft && side != clblasRight) ||
        (uplo != clblasUpper && uplo != clblasLower) || (diag != clblasUnit && diag != clblasNonUnit))
        return clblasInvalidValue;
    const size_t msize = side == clblasLeft ? M : N;
    clblasStatus st;
    if ((st = check_matrix_sizes(order, transA, msize, msize, lda, MAT_A, A, offA, sizeof(*A))) != clblasSuccess) return st;
    if ((st = check_matrix_sizes(order, clblasNoTrans, M, N, ldb, MAT_B, B, offB, sizeof(*B))) != clblasSuccess) return st;
    if (M > kMaxDim || N > kMaxDim) return clblasNotImplemented;

    bool right = side == clblasRight, lower = uplo == clblasLower;
    // Row major: the same memory read column-major holds A^T and B^T, so solve the
    // transposed system: swap M and N, flip side and uplo; trans and diag stay
    // (xtrsm.cc:54-64).
    if (order == clblasRowMajor) {
        std::swap(M, N);
        right = !right;
        lower = !lower;
    }
    return map_hip_error(cba::with_workspaces_secured(stream, [&] { return cba::trsm_colmajor<T>(right, lower, transA != clblasNoTrans, transA == clblasConjTrans,
                                               diag == clblasUnit, (int)M, (int)N, alpha, A + offA, (int64_t)lda,
                                               B + offB, (int64_t)ldb, stream); }));
}

}  // namespace

extern "C" {

clblasStatus clblasGetVersion(unsigned int *major, unsigned int *minor, unsigned int *patch) {
    if (major) *major = 0;
    if (minor) *minor = 1;
    if (patch) *patch = 0;
    return clblasSuccess;
}

clblasStatus clblasSetup(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return clblasInvalidDevice;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return clblasInvalidDevice;
    }
    // The code object holds gfx950 ISA only.
    const char *arch = prop.gcnArchName;
    const char want[] = "gfx950";
    for (int i = 0; i < 6; ++i)
        if (arch[i] != want[i]) return clblasInvalidDevice;
    // Address of this GPU's fixed scratch array, for clblasSgemmNoAlloc (which also looks it up
    // itself on its first call per device if Setup was not called).
    void *scratch = nullptr;
    if (cba::noalloc_scratch(&scratch) != hipSuccess) {
        (void)hipGetLastError();
        return clblasOutOfResources;
    }
    return clblasSuccess;
}

// Synchronises every device that holds scratch buffers, then frees them (buffers of a device that
// cannot be synchronised - one of its streams is being captured - stay until the next call).
void clblasTeardown(void) { (void)cba::workspace_release_all(); }

void clblasAmdReloadDebugEnv(void) { cba::reload_knobs(); }

size_t clblasAmdLastDispatch(char *text, size_t size) {
    const cba::DispatchRecord &r = cba::dispatch_record();
    if (text && size) {
        if (r.launches == 0)
            std::snprintf(text, size, "none");
        else
            std::snprintf(text, size, "%s<%c,%dx%dx%d,%d threads> %c%c M=%d N=%d K=%d grid=(%u,%u) splits=%d tail_slices=%d%s",
                          r.kernel, r.type, r.bm, r.bn, r.bk, r.threads, r.trans_a ? 'T' : 'N', r.trans_b ? 'T' : 'N',
                          r.M, r.N, r.K, r.grid_x, r.grid_y, r.splits, r.tail_slices, r.tri ? " tri" : "");
    }
    return (size_t)r.launches;
}

clblasStatus clblasAmdReleaseStream(hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return clblasInvalidDevice;
    }
    // The buffers go back to the device at once, so everything the stream was given has to be through
    // with them: wait for the stream first.  A stream under capture cannot be waited for (and the
    // graph would keep pointers into the buffers): refuse.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) return clblasInvalidOperation;
    (void)hipGetLastError();
    if (hipStreamSynchronize(stream) != hipSuccess) {
        (void)hipGetLastError();
        return clblasInvalidCommandQueue;
    }
    cba::ws_release_stream(dev, stream);
    return clblasSuccess;
}

clblasStatus clblasAmdReserveWorkspace(hipStream_t stream, size_t gemm_bytes, size_t trmm_bytes, size_t trsm_bytes) {
    const size_t want[3] = {gemm_bytes, trmm_bytes, trsm_bytes};
    for (int kind = 0; kind < 3; ++kind) {
        if (!want[kind]) continue;
        void *p = nullptr;
        hipError_t e = cba::workspace_get(stream, want[kind], kind, &p);
        if (e != hipSuccess) return map_hip_error(e);
    }
    return clblasSuccess;
}

void clblasAmdWorkspaceStats(size_t *streams, size_t *bytes) { cba::ws_stats(streams, bytes); }

int clblasAmdTileModelQuery(char type, size_t M, size_t N, size_t K, int *tile, int *splits, int *tail_slices,
                            double *costs, int *dims, int max_tiles) {
    if (!tile || !splits || !tail_slices || !costs || !dims || max_tiles < 1) return -1;
    if (M == 0 || N == 0 || K == 0 || M > kMaxDim || N > kMaxDim || K > kMaxDim) return -1;
    if (type == 's') return cba::sgemm_model_query((int)M, (int)N, (int)K, tile, splits, tail_slices, costs, max_tiles, dims);
    if (type == 'd') return cba::dgemm_model_query((int)M, (int)N, (int)K, tile, splits, tail_slices, costs, max_tiles, dims);
    if (type == 'c') return cba::cgemm_model_query((int)M, (int)N, (int)K, tile, splits, tail_slices, costs, max_tiles, dims);
    if (type == 'z') return cba::zgemm_model_query((int)M, (int)N, (int)K, tile, splits, tail_slices, costs, max_tiles, dims);
    return -1;
}

int clblasAmdTileModelParam(char type, int tile, int which, double *value, int set) {
    double *p = type == 's' ? cba::sgemm_model_param(tile, which) : type == 'd' ? cba::dgemm_model_param(tile, which)
                : type == 'c' ? cba::cgemm_model_param(tile, which) : type == 'z' ? cba::zgemm_model_param(tile, which) : nullptr;
    if (!p || !value) return -1;
    if (set) *p = *value;
    else *value = *p;
    return 0;
}

clblasStatus clblasAmdTrsmPollTimeouts(unsigned int *count, int reset) {
    return map_hip_error(cba::trsm_poll_timeouts_read(count, reset != 0));
}

clblasStatus clblasSgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB, size_t M, size_t N,
                         size_t K, float alpha, const float *A, size_t offA, size_t lda, const float *B, size_t offB,
                         size_t ldb, float beta, float *C, size_t offC, size_t ldc, hipStream_t stream) {
    return gemm_front<float>(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc,
                             stream);
}

clblasStatus clblasSgemmNoAlloc(clblasOrder order, clblasTranspose transA, clblasTranspose transB, size_t M, size_t N,
                                size_t K, float alpha, const float *A, size_t offA, size_t lda, const float *B,
                                size_t offB, size_t ldb, float beta, float *C, size_t offC, size_t ldc,
                                hipStream_t stream) {
    return gemm_front<float, true>(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC,
                                   ldc, stream);
}

clblasStatus clblasDgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB, size_t M, size_t N,
                         size_t K, double alpha, const double *A, size_t offA, size_t lda, const double *B,
                         size_t offB, size_t ldb, double beta, double *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return gemm_front<double>(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc,
                              stream);
}

clblasStatus clblasCgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB, size_t M, size_t N,
                         size_t K, FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                         const FloatComplex *B, size_t offB, size_t ldb, FloatComplex beta, FloatComplex *C,
                         size_t offC, size_t ldc, hipStream_t stream) {
    return gemm_front<cba::Cx<float>>(order, transA, transB, M, N, K, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                      cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasZgemm(clblasOrder order, clblasTranspose transA, clblasTranspose transB, size_t M, size_t N,
                         size_t K, DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                         const DoubleComplex *B, size_t offB, size_t ldb, DoubleComplex beta, DoubleComplex *C,
                         size_t offC, size_t ldc, hipStream_t stream) {
    return gemm_front<cba::Cx<double>>(order, transA, transB, M, N, K, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                       cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasStrsm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, float alpha, const float *A, size_t offA, size_t lda, float *B,
                         size_t offB, size_t ldb, hipStream_t stream) {
    return trsm_front<float>(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream);
}

clblasStatus clblasDtrsm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, double alpha, const double *A, size_t offA, size_t lda, double *B,
                         size_t offB, size_t ldb, hipStream_t stream) {
    return trsm_front<double>(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream);
}

clblasStatus clblasCtrsm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                         FloatComplex *B, size_t offB, size_t ldb, hipStream_t stream) {
    return trsm_front<cba::Cx<float>>(order, side, uplo, transA, diag, M, N, cx(alpha), cx(A), offA, lda, cx(B), offB,
                                      ldb, stream);
}

clblasStatus clblasZtrsm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                         DoubleComplex *B, size_t offB, size_t ldb, hipStream_t stream) {
    return trsm_front<cba::Cx<double>>(order, side, uplo, transA, diag, M, N, cx(alpha), cx(A), offA, lda, cx(B),
                                       offB, ldb, stream);
}

clblasStatus clblasSsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K, float alpha,
                         const float *A, size_t offA, size_t lda, float beta, float *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return syrk_front<float>(order, uplo, transA, N, K, alpha, A, offA, lda, beta, C, offC, ldc, stream);
}

clblasStatus clblasStrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, float alpha, const float *A, size_t offA, size_t lda, float *B,
                         size_t offB, size_t ldb, hipStream_t stream) {
    return trmm_front<float>(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream);
}

clblasStatus clblasSsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, float alpha,
                         const float *A, size_t offA, size_t lda, const float *B, size_t offB, size_t ldb, float beta,
                         float *C, size_t offC, size_t ldc, hipStream_t stream) {
    return symm_front<float>(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream);
}

clblasStatus clblasDsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K, double alpha,
                         const double *A, size_t offA, size_t lda, double beta, double *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return syrk_front<double>(order, uplo, transA, N, K, alpha, A, offA, lda, beta, C, offC, ldc, stream);
}

clblasStatus clblasDtrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, double alpha, const double *A, size_t offA, size_t lda, double *B,
                         size_t offB, size_t ldb, hipStream_t stream) {
    return trmm_front<double>(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream);
}

clblasStatus clblasDsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, double alpha,
                         const double *A, size_t offA, size_t lda, const double *B, size_t offB, size_t ldb,
                         double beta, double *C, size_t offC, size_t ldc, hipStream_t stream) {
    return symm_front<double>(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream);
}

clblasStatus clblasCsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda, FloatComplex beta,
                         FloatComplex *C, size_t offC, size_t ldc, hipStream_t stream) {
    return syrk_front<cba::Cx<float>>(order, uplo, transA, N, K, cx(alpha), cx(A), offA, lda, cx(beta), cx(C), offC,
                                      ldc, stream);
}

clblasStatus clblasCtrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda,
                         FloatComplex *B, size_t offB, size_t ldb, hipStream_t stream) {
    return trmm_front<cba::Cx<float>>(order, side, uplo, transA, diag, M, N, cx(alpha), cx(A), offA, lda, cx(B), offB,
                                      ldb, stream);
}

clblasStatus clblasCsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, FloatComplex alpha,
                         const FloatComplex *A, size_t offA, size_t lda, const FloatComplex *B, size_t offB,
                         size_t ldb, FloatComplex beta, FloatComplex *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return symm_front<cba::Cx<float>>(order, side, uplo, M, N, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                      cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasZsyrk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K,
                         DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda, DoubleComplex beta,
                         DoubleComplex *C, size_t offC, size_t ldc, hipStream_t stream) {
    return syrk_front<cba::Cx<double>>(order, uplo, transA, N, K, cx(alpha), cx(A), offA, lda, cx(beta), cx(C), offC,
                                       ldc, stream);
}

clblasStatus clblasZtrmm(clblasOrder order, clblasSide side, clblasUplo uplo, clblasTranspose transA, clblasDiag diag,
                         size_t M, size_t N, DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                         DoubleComplex *B, size_t offB, size_t ldb, hipStream_t stream) {
    return trmm_front<cba::Cx<double>>(order, side, uplo, transA, diag, M, N, cx(alpha), cx(A), offA, lda, cx(B),
                                       offB, ldb, stream);
}

clblasStatus clblasZsymm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, DoubleComplex alpha,
                         const DoubleComplex *A, size_t offA, size_t lda, const DoubleComplex *B, size_t offB,
                         size_t ldb, DoubleComplex beta, DoubleComplex *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return symm_front<cba::Cx<double>>(order, side, uplo, M, N, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                       cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasSsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          float alpha, const float *A, size_t offA, size_t lda, const float *B, size_t offB,
                          size_t ldb, float beta, float *C, size_t offC, size_t ldc, hipStream_t stream) {
    return syr2k_front<float>(order, uplo, transAB, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc,
                              stream);
}

clblasStatus clblasDsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          double alpha, const double *A, size_t offA, size_t lda, const double *B, size_t offB,
                          size_t ldb, double beta, double *C, size_t offC, size_t ldc, hipStream_t stream) {
    return syr2k_front<double>(order, uplo, transAB, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc,
                               stream);
}

clblasStatus clblasCsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda, const FloatComplex *B,
                          size_t offB, size_t ldb, FloatComplex beta, FloatComplex *C, size_t offC, size_t ldc,
                          hipStream_t stream) {
    return syr2k_front<cba::Cx<float>>(order, uplo, transAB, N, K, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                       cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasZsyr2k(clblasOrder order, clblasUplo uplo, clblasTranspose transAB, size_t N, size_t K,
                          DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                          const DoubleComplex *B, size_t offB, size_t ldb, DoubleComplex beta, DoubleComplex *C,
                          size_t offC, size_t ldc, hipStream_t stream) {
    return syr2k_front<cba::Cx<double>>(order, uplo, transAB, N, K, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                        cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasCherk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K, float alpha,
                         const FloatComplex *A, size_t offA, size_t lda, float beta, FloatComplex *C, size_t offC,
                         size_t ldc, hipStream_t stream) {
    return herk_front<float>(false, order, uplo, transA, N, K, cba::Cx<float>{alpha, 0}, cx(A), offA, lda, nullptr, 0,
                             0, beta, cx(C), offC, ldc, stream);
}

clblasStatus clblasCher2k(clblasOrder order, clblasUplo uplo, clblasTranspose trans, size_t N, size_t K,
                          FloatComplex alpha, const FloatComplex *A, size_t offA, size_t lda, const FloatComplex *B,
                          size_t offB, size_t ldb, float beta, FloatComplex *C, size_t offC, size_t ldc,
                          hipStream_t stream) {
    return herk_front<float>(true, order, uplo, trans, N, K, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb, beta,
                             cx(C), offC, ldc, stream);
}

clblasStatus clblasChemm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, FloatComplex alpha,
                         const FloatComplex *A, size_t offA, size_t lda, const FloatComplex *B, size_t offB,
                         size_t ldb, FloatComplex beta, FloatComplex *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return symm_front<cba::Cx<float>, true>(order, side, uplo, M, N, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                            cx(beta), cx(C), offC, ldc, stream);
}

clblasStatus clblasZherk(clblasOrder order, clblasUplo uplo, clblasTranspose transA, size_t N, size_t K, double alpha,
                         const DoubleComplex *A, size_t offA, size_t lda, double beta, DoubleComplex *C, size_t offC,
                         size_t ldc, hipStream_t stream) {
    return herk_front<double>(false, order, uplo, transA, N, K, cba::Cx<double>{alpha, 0}, cx(A), offA, lda, nullptr,
                              0, 0, beta, cx(C), offC, ldc, stream);
}

clblasStatus clblasZher2k(clblasOrder order, clblasUplo uplo, clblasTranspose trans, size_t N, size_t K,
                          DoubleComplex alpha, const DoubleComplex *A, size_t offA, size_t lda,
                          const DoubleComplex *B, size_t offB, size_t ldb, double beta, DoubleComplex *C, size_t offC,
                          size_t ldc, hipStream_t stream) {
    return herk_front<double>(true, order, uplo, trans, N, K, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb, beta,
                              cx(C), offC, ldc, stream);
}

clblasStatus clblasZhemm(clblasOrder order, clblasSide side, clblasUplo uplo, size_t M, size_t N, DoubleComplex alpha,
                         const DoubleComplex *A, size_t offA, size_t lda, const DoubleComplex *B, size_t offB,
                         size_t ldb, DoubleComplex beta, DoubleComplex *C, size_t offC, size_t ldc,
                         hipStream_t stream) {
    return symm_front<cba::Cx<double>, true>(order, side, uplo, M, N, cx(alpha), cx(A), offA, lda, cx(B), offB, ldb,
                                             cx(beta), cx(C), offC, ldc, stream);
}

}  // extern "C"
