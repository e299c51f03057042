// clblasSgemmNoAlloc: clblasSgemm for callers that cannot allocate device memory (code under HIP
// graph capture, serving loops, harnesses that forbid hipMalloc).
//
// clblasSgemm cuts K into ranges when C has few tiles, and slices the tiles of a partly filled
// last round; both keep partial sums in a scratch buffer that the library otherwise allocates per
// stream on first use.  Here that buffer is a file-scope device array of fixed size, so the call
// only enqueues kernels.  Every GPU holds its own copy of the array; its address is looked up once
// per device and kept.  All calls on one GPU share the array: calls that overlap in time on one GPU
// (different streams) race on it, calls in stream order on one stream do not.  Nothing in it has to
// start at zero: every kernel writes the partial sums it later reads.
#include <hip/hip_runtime.h>

#include <mutex>

#include "../../include/clblas_amd.h"
#include "internal.h"

namespace cba {

namespace {

constexpr size_t kScratchBytes = CLBLAS_AMD_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;  // device ordinals beyond this are refused (hipErrorInvalidDevice)
std::mutex g_mutex;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, once looked up

}  // namespace

// Device address of this GPU's scratch array (looked up on the first call per device, with
// that device current).  The array's name itself is only a host-side handle.
hipError_t noalloc_scratch(void **ptr) {
    *ptr = nullptr;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return hipSuccess;
}

hipError_t sgemm_colmajor_noalloc(bool transA, bool transB, int M, int N, int K, float alpha, const float *A,
                                  int64_t lda, const float *B, int64_t ldb, float beta, float *C, int64_t ldc,
                                  hipStream_t stream) {
    FixedScratch fixed;
    fixed.ptr = nullptr;
    {
        // The address is looked up once per device.  That lookup may load the code object, which is
        // not something to do in the middle of a stream capture: a first call per device that finds
        // its stream being captured is refused (clblasSetup, or one call outside a capture, comes first).
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        bool known = false;
        if (dev >= 0 && dev < kMaxDevices) {
            std::lock_guard<std::mutex> lock(g_mutex);
            known = g_scratch_ptr[dev] != nullptr;
        }
        if (!known) {
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
                return hipErrorStreamCaptureUnsupported;
        }
    }
    hipError_t e = noalloc_scratch(&fixed.ptr);
    if (e != hipSuccess) return e;
    fixed.bytes = kScratchBytes;
    // A product may take two or three launches (a strip of rows or columns as a product of its own): walk the
    // sequence dry first, so that a part that needs more scratch than the array holds is found before the
    // first kernel is enqueued.
    if (!dry_run_slot()) {
        DryRun dry;
        const DispatchRecord kept = dispatch_record();
        dry_run_slot() = &dry;
        e = sgemm_colmajor(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, nullptr, &fixed);
        dry_run_slot() = nullptr;
        dispatch_record() = kept;
        if (e != hipSuccess) return e;
    }
    return sgemm_colmajor(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, nullptr, &fixed);
}

}  // namespace cba
