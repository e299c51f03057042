// Declarations shared between the translation units of libclblas_amd.so.
// Nothing here is part of the exported C ABI.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

#include <tuple>
#include <utility>

namespace cba {

// Dry run of a call's launch sequence on the calling thread: while one is active, launch_kernel
// launches nothing and workspace_get only records how much scratch of each kind was asked for.
// Routines made of several launches use it on a stream under graph capture to secure every buffer
// before the first kernel is enqueued (see with_workspaces_secured).
struct DryRun {
    size_t need[3] = {0, 0, 0};
};
DryRun *&dry_run_slot();  // thread-local; nullptr: launches are real

// Launches `fn` and returns the status of THIS launch.  (The <<<>>> form reports through the
// thread's sticky error, which would also pick up - and clear - an error that unrelated code of
// the caller left there.)
template <typename... KArgs, size_t... I>
inline hipError_t launch_kernel_impl(void (*fn)(KArgs...), dim3 grid, dim3 block, size_t smem, hipStream_t stream,
                                     std::tuple<KArgs...> &args, std::index_sequence<I...>) {
    void *ptrs[] = {(void *)&std::get<I>(args)..., nullptr};
    return hipLaunchKernel((const void *)fn, grid, block, ptrs, smem, stream);
}
template <typename... KArgs, typename... Args>
inline hipError_t launch_kernel(void (*fn)(KArgs...), dim3 grid, dim3 block, size_t smem, hipStream_t stream,
                                Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "argument count");
    if (dry_run_slot()) return hipSuccess;
    std::tuple<KArgs...> t(static_cast<KArgs>(args)...);
    return launch_kernel_impl(fn, grid, block, smem, stream, t, std::index_sequence_for<KArgs...>());
}

// Complex element, laid out as the reference's FloatComplex / DoubleComplex (cl_float2 /
// cl_double2, src/clBLAS-complex.h:25-26: real part first).
template <typename R> struct Cx { R re, im; };

// Debug switches, read from the environment once (first use) and again only when
// clblasAmdReloadDebugEnv() is called: the launch path itself never calls getenv.
//   CLBLAS_AMD_GEMM_TILE (index into the per-type tile table, -1: model's choice), _SPLIT_MODEL,
//   _SPLITS, _TAIL, _GROUP_M (0: default), _XCD, _STAGGER: see the tile choice in gemm_launch.hpp;
//   CLBLAS_AMD_LOG=1: one line per kernel launch on stderr.
//   CLBLAS_AMD_CHECK_MEM=1: every operand is looked up among the device allocations and a matrix that
//   does not fit behind its pointer is refused with clblasInsufficientMemMat{A,B,C}.
struct DebugKnobs {
    int gemm_tile = -1, split_model = 1, splits = 0, tail = 1, group_m = 0, xcd = 1, stagger = 1, log = 0;
    int check_mem = 0;
    int trsm_poll_limit = 0;  // CLBLAS_AMD_TRSM_POLL_LIMIT: polls after which a flag wait of the substitution leaf gives up (0: 2^22); tests
    int peel = 1;          // CLBLAS_AMD_GEMM_PEEL: 0 never splits a strip of rows / columns off a product, 2 always where one exists (tests)
    int trsm_wide = -1;    // CLBLAS_AMD_TRSM_WIDE (real types, substitution leaf): 0 / 1 forces 16 / 32 right-hand sides per workgroup
    int trsm_leaf = 0;     // CLBLAS_AMD_TRSM_LEAF (real types): 0 substitution over 16-row sub-blocks, 1 inverted 64 x 64 triangles
    int wide_ld = 0;       // CLBLAS_AMD_GEMM_WIDE_LD=1: the wide-ld kernels whatever the leading dimensions (tests)
    int deep_panels = 1;   // CLBLAS_AMD_GEMM_DEEP: 0 never the deep-panel variant of a tile, 1 by the rule, 2 wherever built, more: from that depth of a K range
};
const DebugKnobs &knobs();
void reload_knobs();

// What the last GEMM launch of the calling thread was (diagnostics: clblasAmdLastDispatch).
struct DispatchRecord {
    char type = '?';           // s, d, c, z
    int bm = 0, bn = 0, bk = 0, threads = 0;
    int trans_a = 0, trans_b = 0;
    int M = 0, N = 0, K = 0;
    int splits = 1, tail_slices = 1, tri = 0;
    unsigned grid_x = 0, grid_y = 0;
    unsigned long long launches = 0;  // kernel launches by this thread since the library was loaded
    const char *kernel = "";          // kernel family ("gemm_mfma_kernel", "gemm_mfma_kernel(wide ld)", "scale_c_kernel")
};
DispatchRecord &dispatch_record();  // thread-local

// Library-owned device scratch for `stream` on the current device, at least `bytes` long
// (kinds: workspace.hpp).  Grown on demand; see workspace.hpp for the lifetime rules.
// hipErrorOutOfMemory if the allocation fails; hipErrorStreamCaptureUnsupported if `stream`
// is being captured into a graph and the buffer would have to be allocated now.
hipError_t workspace_get(hipStream_t stream, size_t bytes, int kind, void **out);
bool workspace_release_all();  // false: some device could not be synchronised and keeps its buffers
void ws_release_stream(int device, hipStream_t stream);
void ws_stats(size_t *streams, size_t *bytes);

// Holds the calling thread's claim on the scratch buffers it is handed between the first
// workspace_get of an API call and the end of that call: while the claim stands the buffers of
// that (device, stream) are not given up to make room for another stream (a thread that has its
// pointer but has not enqueued its kernels yet would otherwise launch on freed memory).  One per
// extern "C" entry point, on the stack.
struct CallLease {
    CallLease();
    ~CallLease();
    CallLease(const CallLease &) = delete;
    CallLease &operator=(const CallLease &) = delete;
    bool held = false;
    int device = 0;
    hipStream_t stream = nullptr;
    CallLease *outer = nullptr;
};

// Runs `body` (a sequence of launches on `stream`).  On a stream that is being captured into a graph
// the sequence is first walked dry, and every scratch buffer it will ask for is secured before the
// first kernel is enqueued: a call that would have to allocate fails with
// hipErrorStreamCaptureUnsupported and leaves its operands untouched, instead of failing half-way.
template <typename F> hipError_t with_workspaces_secured(hipStream_t stream, F &&body);

// Bytes from `ptr` to the end of the device allocation that holds it; 0 if no allocation is known
// to hold it.  The default asks the HIP runtime; tests put their own table in its place.
typedef size_t (*MemProbe)(const void *ptr);
void set_mem_probe(MemProbe probe);  // nullptr: back to the HIP lookup
size_t mem_behind(const void *ptr);

// Caller-supplied scratch that replaces workspace_get for one call (the entry point that
// must not allocate): requests beyond `bytes` fail with hipErrorOutOfMemory.
struct FixedScratch {
    void *ptr;
    size_t bytes;
};

// Raises a kernel's dynamic LDS limit (needed above 64 KiB); cached per function.
hipError_t ensure_dynamic_lds(const void *fn, size_t bytes);

// Triangular structure of a GEMM-shaped call (SYRK, TRMM).
//   tri_c: only the lower (1) / upper (2) triangle of C is computed and stored.
//   tri_a / tri_b: op(A)(m,k) / op(B)(k,n) is triangular: entries with k > x (1) or k < x (2),
//   x = m resp. n, count as zero whatever memory holds; unit_* = 1: the diagonal counts as
//   one, 2: as zero (strict triangle), 3: as its real part (diagonal of a Hermitian matrix).
//   herm_c (with tri_c, complex types): C is Hermitian, its diagonal is stored with zero
//   imaginary parts.
struct GemmTri {
    int tri_c = 0, tri_a = 0, tri_b = 0, unit_a = 0, unit_b = 0, herm_c = 0;
    bool any() const { return tri_c || tri_a || tri_b; }
};

// Column-major GEMM launchers.  Arguments are already validated and folded to column
// major; pointers already include their element offsets.
hipError_t sgemm_colmajor(bool transA, bool transB, int M, int N, int K, float alpha, const float *A, int64_t lda,
                          const float *B, int64_t ldb, float beta, float *C, int64_t ldc, hipStream_t stream,
                          const GemmTri *tri = nullptr, const FixedScratch *fixed = nullptr);
// SGEMM with the fixed per-GPU scratch array instead of the per-stream buffers (noalloc.hip):
// allocates nothing; hipErrorOutOfMemory when the call needs more scratch than the array holds.
hipError_t sgemm_colmajor_noalloc(bool transA, bool transB, int M, int N, int K, float alpha, const float *A,
                                  int64_t lda, const float *B, int64_t ldb, float beta, float *C, int64_t ldc,
                                  hipStream_t stream);
// Device address of the current GPU's fixed scratch array (looked up once per device).
hipError_t noalloc_scratch(void **ptr);
hipError_t dgemm_colmajor(bool transA, bool transB, int M, int N, int K, double alpha, const double *A,
                          int64_t lda, const double *B, int64_t ldb, double beta, double *C, int64_t ldc,
                          hipStream_t stream, const GemmTri *tri = nullptr);

// The tile choice model of SGEMM / DGEMM from outside (diagnostics, clblasAmdTileModelQuery / ...Param):
// the choice for a plain M x N x K product, the model's cost of every tile of the table in one K range
// (negative: not offered), the tiles' dimensions (bm, bn, bk per tile); returns the number of tiles.
int sgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims);
int dgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims);
double *sgemm_model_param(int tile, int which);  // nullptr: no such tile / parameter
double *dgemm_model_param(int tile, int which);
int zgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims);
double *zgemm_model_param(int tile, int which);
int cgemm_model_query(int M, int N, int K, int *tile, int *splits, int *tail_slices, double *costs, int max_costs, int *dims);
double *cgemm_model_param(int tile, int which);

// Complex variants: conjA / conjB conjugate the elements of op(A) / op(B) (clblasConjTrans).
hipError_t cgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<float> alpha,
                          const Cx<float> *A, int64_t lda, const Cx<float> *B, int64_t ldb, Cx<float> beta,
                          Cx<float> *C, int64_t ldc, hipStream_t stream, const GemmTri *tri = nullptr);
hipError_t zgemm_colmajor(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, Cx<double> alpha,
                          const Cx<double> *A, int64_t lda, const Cx<double> *B, int64_t ldb, Cx<double> beta,
                          Cx<double> *C, int64_t ldc, hipStream_t stream, const GemmTri *tri = nullptr);

// The four launchers above behind one name (conjA / conjB are ignored by the real types).
template <typename T>
hipError_t launch_gemm(bool transA, bool transB, bool conjA, bool conjB, int M, int N, int K, T alpha, const T *A,
                       int64_t lda, const T *B, int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream,
                       const GemmTri *tri = nullptr);

// Column-major SYRK / TRMM / SYMM drivers built on the GEMM launchers (level3.hip).
//   syrk: C <- alpha op(A) op(A)^T + beta C on the `lower` / upper triangle of C (N x N).
//   trmm: B <- alpha op(A) B (left) or alpha B op(A) (right), A triangular, in place.
//   symm: C <- alpha A B + beta C (left) or alpha B A + beta C (right), A symmetric with only
//         its `lower` / upper triangle stored.
template <typename T>
hipError_t syrk_colmajor(bool lower, bool trans, int N, int K, T alpha, const T *A, int64_t lda, T beta, T *C,
                         int64_t ldc, hipStream_t stream);
template <typename T>
hipError_t trmm_colmajor(bool right, bool lower, bool trans, bool conj, bool unit, int M, int N, T alpha, const T *A,
                         int64_t lda, T *B, int64_t ldb, hipStream_t stream);
template <typename T>
hipError_t symm_colmajor(bool right, bool lower, int M, int N, T alpha, const T *A, int64_t lda, const T *B,
                         int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream);
// syr2k: C <- alpha (op(A) op(B)^T + op(B) op(A)^T) + beta C on one triangle of C.
template <typename T>
hipError_t syr2k_colmajor(bool lower, bool trans, int N, int K, T alpha, const T *A, int64_t lda, const T *B,
                          int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream);
// herk: C <- alpha op(A) op(A)^H + beta C; her2k: C <- alpha op(A) op(B)^H + conj(alpha) op(B) op(A)^H
// + beta C; op = identity or conjugate transpose (`ctrans`), real beta (and alpha for herk), C Hermitian.
template <typename R>
hipError_t herk_colmajor(bool lower, bool ctrans, int N, int K, R alpha, const Cx<R> *A, int64_t lda, R beta,
                         Cx<R> *C, int64_t ldc, hipStream_t stream);
template <typename R>
hipError_t her2k_colmajor(bool lower, bool ctrans, int N, int K, Cx<R> alpha, const Cx<R> *A, int64_t lda,
                          const Cx<R> *B, int64_t ldb, R beta, Cx<R> *C, int64_t ldc, hipStream_t stream);
// hemm: as symm with A Hermitian (complex types).
template <typename T>
hipError_t hemm_colmajor(bool right, bool lower, int M, int N, T alpha, const T *A, int64_t lda, const T *B,
                         int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t stream);


// Column-major TRSM driver (trsm.hip), all four types: solves op(A) X = alpha B (left) or
// X op(A) = alpha B (right) in place; `conj` conjugates op(A) (complex, clblasConjTrans).
template <typename T>
hipError_t trsm_colmajor(bool right, bool lower, bool trans, bool conj, bool unit, int M, int N, T alpha, const T *A,
                         int64_t lda, T *B, int64_t ldb, hipStream_t stream);

// Flag waits of the TRSM leaf that ran into their poll limit on the current GPU (trsm.hip); waits for
// the device's copy queue, so not for use between enqueues of a benchmark.
hipError_t trsm_poll_timeouts_read(unsigned int *count, bool reset);

template <typename F> hipError_t with_workspaces_secured(hipStream_t stream, F &&body) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (dry_run_slot() || hipStreamIsCapturing(stream, &cap) != hipSuccess || cap == hipStreamCaptureStatusNone)
        return body();
    DryRun dry;
    const DispatchRecord kept = dispatch_record();
    dry_run_slot() = &dry;
    hipError_t e = body();
    dry_run_slot() = nullptr;
    dispatch_record() = kept;
    if (e != hipSuccess) return e;
    for (int kind = 0; kind < 3; ++kind) {
        if (!dry.need[kind]) continue;
        void *p = nullptr;
        if ((e = workspace_get(stream, dry.need[kind], kind, &p)) != hipSuccess) return e;
    }
    return body();
}

}  // namespace cba
