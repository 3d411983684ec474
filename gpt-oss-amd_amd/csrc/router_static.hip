// moe_gemm_router_static: the router GEMM with the reference's own eight-argument list
// (src/hip/gemms/gemm_router.hip:184-185) for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The fp64 partial
// sums that moe_gemm_router takes from a caller-provided scratch buffer live here in a file-scope
// device array instead.  Same kernels, same arithmetic, same bits as moe_gemm_router.
//
// Each GPU the library runs on holds its own copy of the array until the process ends.  Every call
// on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two host threads)
// race on it.  Nothing in the array has to start at zero: the partial kernels write every element
// the finalise kernel reads.
#include <atomic>
#include <mutex>

#include "common.h"
#include "kernels.h"

namespace {

constexpr size_t kStaticScratchBytes = MOE_ROUTER_STATIC_SCRATCH_BYTES;

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// In host code `scratch` is only a handle for the symbol, not a device address.  The address of
// each GPU's copy is looked up once per device, with that device current, and kept here.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

int scratch_for_current_device(void** out) {
    int dev = -1;
    MOE_RETURN_IF_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return MOE_ERR_LIMIT;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            MOE_RETURN_IF_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            if (!p) return MOE_ERR_WORKSPACE;
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return MOE_OK;
}

}  // namespace

extern "C" {

size_t moe_gemm_router_static_max_bytes(void) { return kStaticScratchBytes; }

int moe_gemm_router_static(float* xout, const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias, int N,
                           int K, int M, moe_stream_t stream) {
    using namespace moe;
    if (!xout || !x_batch || !w || !bias) return MOE_ERR_NULL;
    if (N <= 0 || K <= 0 || M <= 0 || K % 8 != 0) return MOE_ERR_SHAPE;
    if (M > 1024) return MOE_ERR_LIMIT;
    if (((uintptr_t)x_batch | (uintptr_t)w) & 15u) return MOE_ERR_ALIGN;
    const int S = router_segments(N, M, K, false);
    // beyond the fixed array: the caller has to use moe_gemm_router with its own scratch
    if ((size_t)S * (size_t)N * (size_t)M * sizeof(double) > kStaticScratchBytes) return MOE_ERR_LIMIT;
    void* ptr = nullptr;
    int rc = scratch_for_current_device(&ptr);
    if (rc) return rc;
    double* partial = static_cast<double*>(ptr);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    rc = launch_router_partial(x_batch, w, partial, nullptr, N, K, M, S, s);
    if (rc) return rc;
    return launch_router_finalize(partial, S, nullptr, bias, xout, nullptr, nullptr, N, M, 0, 0, 0, s);
}

}  // extern "C"
