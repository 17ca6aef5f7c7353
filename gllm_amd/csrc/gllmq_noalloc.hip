// gllmq_quantized_matmul_noalloc: the quantized matmul for callers that cannot allocate device
// memory (code under stream capture, tight serving loops, harnesses that forbid hipMalloc).
// The scratch that gllmq_quantized_matmul keeps per stream and grows on demand (arrival
// counters and slice sums of the K split, activation images and partial sums of the GEMM) is
// here one array in device memory whose address gllmq_init looks up (which is also what places it
// on the device); the entry point itself makes no call that can allocate.
#include <hip/hip_runtime.h>

#include <mutex>

#include "gq_host_internal.h"

namespace {

constexpr size_t kNoAllocScratchBytes = GLLMQ_NOALLOC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;

// Every GPU the library runs on holds its own copy of this array, at its own address, until the
// process ends.  Zero at load; the arrival counters at its head are left zero by every launch
// that uses them, and nothing else in it needs a defined value.
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[kNoAllocScratchBytes];

std::mutex g_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// The array's address on `device`, looked up with that device current.  In host code the array's
// name is only a handle for this lookup, never a device address.  The lookup is what makes the
// runtime load this file's device code on that GPU and place the array, so it belongs to set-up
// (gllmq_init), where allocating is allowed; the entry point below only reads the table.
int resolve_scratch(gllmq_ctx *ctx, int device)
{
    if (device < 0 || device >= kMaxDevices)
        return gq_ctx_set_error(ctx, GLLMQ_ERR_INVALID, "quantized_matmul_noalloc: device index out of range");
    std::lock_guard<std::mutex> g(g_mutex);
    if (g_scratch_ptr[device]) return GLLMQ_OK;
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    if (e == hipSuccess && current != device)
        return gq_ctx_set_error(ctx, GLLMQ_ERR_INVALID, "quantized_matmul_noalloc: the context's device is not the current device");
    void *ptr = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return gq_ctx_set_error(ctx, GLLMQ_ERR_HIP, e != hipSuccess ? hipGetErrorString(e) : "hipGetSymbolAddress returned no address");
    }
    g_scratch_ptr[device] = ptr;
    return GLLMQ_OK;
}

} // namespace

extern "C" int gq_noalloc_init(gllmq_ctx *ctx, int device) { return resolve_scratch(ctx, device); }

extern "C" int gllmq_quantized_matmul_noalloc(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes, const float *x_dev,
                                              float *y_dev, uint32_t ggml_dtype, size_t m, size_t n, size_t k, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    const int device = gq_ctx_device(ctx);
    // every call: launches go to the calling thread's current device, the array's address is the context's device's
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != device) {
        (void)hipGetLastError();
        return gq_ctx_set_error(ctx, GLLMQ_ERR_INVALID,
                                "quantized_matmul_noalloc: the context's device must be the calling thread's current device");
    }
    void *ptr = nullptr;
    if (device >= 0 && device < kMaxDevices) {
        std::lock_guard<std::mutex> g(g_mutex);
        ptr = g_scratch_ptr[device];
    }
    if (!ptr) // gllmq_init resolves it or fails; nothing is looked up (or placed on the device) here
        return gq_ctx_set_error(ctx, GLLMQ_ERR_INVALID, "quantized_matmul_noalloc: no scratch array was set up for the context's device");
    return gq_quantized_matmul_on_block(ctx, w_dev, w_bytes, x_dev, y_dev, ggml_dtype, m, n, k, ptr, kNoAllocScratchBytes,
                                        stream);
}
