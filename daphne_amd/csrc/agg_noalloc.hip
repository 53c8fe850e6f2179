// Column aggregation for callers that may not allocate: the per-block partials of the two-stage kernels go to
// a fixed array in device memory instead of the context's workspace, so the call reaches no hipMalloc, hipFree
// or other allocating routine (code under stream capture, serving loops, harnesses that forbid allocation).
//
// The array exists once per device (every GPU that loads this library holds its own copy at its own address
// until the process ends). In host code its name stands for the symbol, not for device memory: the address that
// kernels, copies and fills may use comes from hipGetSymbolAddress, taken once per device with that device
// current, and only that address is ever handed on.
#include "agg_impl.h"

namespace {

constexpr size_t NOALLOC_SCRATCH_BYTES = size_t(8) << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_bind_lock;
void *g_scratch_ptr[MAX_DEVICES]; // device address of `scratch` on each device, null until bound

} // namespace

// Looks up the address of this device's copy of the scratch array. The device must be current. Called by
// dh_ctx_create for the context's device; the entry point below repeats it if it finds no address yet.
dh_status dh_noalloc_bind_device(int device) {
    if (device < 0 || device >= MAX_DEVICES)
        return dh_fail(DH_ERR_RUNTIME, "dh_agg_col_noalloc: device %d is beyond the %d devices this library keeps scratch for",
                       device, MAX_DEVICES);
    std::lock_guard<std::mutex> g(g_bind_lock);
    if (g_scratch_ptr[device] != nullptr)
        return DH_OK;
    void *ptr = nullptr;
    DH_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr)
        return dh_fail(DH_ERR_HIP, "hipGetSymbolAddress returned a null address for the scratch array on device %d", device);
    g_scratch_ptr[device] = ptr;
    return DH_OK;
}

extern "C" size_t dh_agg_col_noalloc_scratch_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

extern "C" dh_status dh_agg_col_noalloc_f32(dh_ctx *ctx, int op, float *res, const float *arg, size_t rows, size_t cols,
                                           size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ctx->device < 0 || ctx->device >= MAX_DEVICES)
        return dh_fail(DH_ERR_RUNTIME, "dh_agg_col_noalloc: device %d is beyond the %d devices this library keeps scratch for",
                       ctx->device, MAX_DEVICES);
    void *ptr;
    {
        std::lock_guard<std::mutex> g(g_bind_lock);
        ptr = g_scratch_ptr[ctx->device];
    }
    if (ptr == nullptr) {
        dh_status st = dh_noalloc_bind_device(ctx->device); // DH_REQUIRE_CTX made the device current
        if (st != DH_OK)
            return st;
        std::lock_guard<std::mutex> g(g_bind_lock);
        ptr = g_scratch_ptr[ctx->device];
    }
    // The first stage writes every partial the second stage reads, so nothing of the previous call's contents
    // has to be cleared. Two calls on one device share the array: they must not overlap.
    dh_agg::ColScratch sc;
    sc.buf = ptr;
    sc.bytes = NOALLOC_SCRATCH_BYTES;
    return dh_agg::agg_col<float>(ctx, op, res, arg, rows, cols, ld, sc);
}
