// Device context and allocator of libdaphne_hip.so.
//
// Stands in for the reference's CUDAContext (runtime/local/context/CUDAContext.cpp:41-135):
// device selection, property query, a memory budget of 90 % of the device total, and a
// registry of allocations that are released when the context is destroyed. There are no
// library handles: every kernel in this library is hand-written.
#include "common.h"

#include <cstring>

namespace {
thread_local std::string g_last_error;
}

void dh_set_error(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

dh_status dh_fail(dh_status st, const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return st;
}

extern "C" const char *dh_last_error(void) { return g_last_error.c_str(); }

extern "C" dh_status dh_ctx_create(int device, dh_ctx **out) {
    if (out == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "dh_ctx_create: out is null");
    *out = nullptr;
    int count = 0;
    DH_CHECK_HIP(hipGetDeviceCount(&count));
    if (device < 0 || device >= count)
        return dh_fail(DH_ERR_RUNTIME, "dh_ctx_create: requested device %d but only %d device(s) are visible",
                       device, count);
    DH_CHECK_HIP(hipSetDevice(device));
    auto *ctx = new dh_ctx();
    ctx->device = device;
    hipError_t e = hipGetDeviceProperties(&ctx->props, device);
    if (e != hipSuccess) {
        delete ctx;
        return dh_fail(DH_ERR_HIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    }
    if (strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
        std::string arch = ctx->props.gcnArchName;
        delete ctx;
        return dh_fail(DH_ERR_RUNTIME, "dh_ctx_create: this library holds gfx950 code only, device %d is %s", device,
                       arch.c_str());
    }
    size_t free_b = 0, total_b = 0;
    e = hipMemGetInfo(&free_b, &total_b);
    if (e != hipSuccess) {
        delete ctx;
        return dh_fail(DH_ERR_HIP, "hipMemGetInfo: %s", hipGetErrorString(e));
    }
    // 90 % of the device total, like CUDAContext.cpp:49-50.
    ctx->mem_budget = static_cast<size_t>(static_cast<double>(total_b) * 0.9);
    ctx->num_cus = ctx->props.multiProcessorCount;
    bool ok = hipMalloc(reinterpret_cast<void **>(&ctx->flag_dev), 256) == hipSuccess &&
              hipHostMalloc(reinterpret_cast<void **>(&ctx->flag_host), 256, hipHostMallocMapped) == hipSuccess &&
              hipHostGetDevicePointer(reinterpret_cast<void **>(&ctx->flag_host_dev), ctx->flag_host, 0) == hipSuccess &&
              hipEventCreate(&ctx->ev_start) == hipSuccess && hipEventCreate(&ctx->ev_stop) == hipSuccess;
    ok = ok && hipMemset(ctx->flag_dev, 0, 256) == hipSuccess; // no deferred verdict pending
    if (!ok) {
        dh_ctx_destroy(ctx);
        return dh_fail(DH_ERR_HIP, "dh_ctx_create: could not allocate the context's flag words / events");
    }
    // the fixed scratch array of the entry point that allocates nothing: bound here, with the device current
    if (dh_status st = dh_noalloc_bind_device(device); st != DH_OK) {
        dh_ctx_destroy(ctx);
        return st;
    }
    *out = ctx;
    return DH_OK;
}

extern "C" dh_status dh_ctx_destroy(dh_ctx *ctx) {
    if (ctx == nullptr)
        return DH_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipDeviceSynchronize();
    for (auto &kv : ctx->allocations)
        (void)hipFree(kv.first);
    ctx->allocations.clear();
    for (auto &kv : ctx->cached)
        (void)hipFree(kv.second);
    ctx->cached.clear();
    if (ctx->ws)
        (void)hipFree(ctx->ws);
    if (ctx->flag_dev)
        (void)hipFree(ctx->flag_dev);
    if (ctx->flag_host)
        (void)hipHostFree(ctx->flag_host);
    if (ctx->ev_start)
        (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop)
        (void)hipEventDestroy(ctx->ev_stop);
    for (auto &pair : ctx->kernel_events) {
        (void)hipEventDestroy(pair.first);
        (void)hipEventDestroy(pair.second);
    }
    delete ctx;
    return DH_OK;
}

extern "C" size_t dh_ctx_mem_budget(const dh_ctx *ctx) { return ctx ? ctx->mem_budget : 0; }
extern "C" size_t dh_ctx_mem_in_use(const dh_ctx *ctx) { return ctx ? ctx->mem_in_use : 0; }
extern "C" int dh_ctx_device(const dh_ctx *ctx) { return ctx ? ctx->device : -1; }

extern "C" dh_status dh_ctx_props(const dh_ctx *ctx, int *compute_units, int *clock_khz, size_t *total_mem,
                                  char *name, size_t name_cap) {
    if (ctx == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "dh_ctx_props: context is null");
    if (compute_units)
        *compute_units = ctx->props.multiProcessorCount;
    if (clock_khz)
        *clock_khz = ctx->props.clockRate;
    if (total_mem)
        *total_mem = ctx->props.totalGlobalMem;
    if (name && name_cap) {
        snprintf(name, name_cap, "%s (%s)", ctx->props.name, ctx->props.gcnArchName);
    }
    return DH_OK;
}

extern "C" dh_status dh_ctx_set_stream(dh_ctx *ctx, void *hip_stream) {
    DH_REQUIRE_CTX(ctx);
    if (ctx->stream != static_cast<hipStream_t>(hip_stream)) {
        // cached blocks may still be in use by work queued on the old stream
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    }
    ctx->stream = static_cast<hipStream_t>(hip_stream);
    return DH_OK;
}

extern "C" void *dh_ctx_get_stream(const dh_ctx *ctx) { return ctx ? static_cast<void *>(ctx->stream) : nullptr; }

extern "C" dh_status dh_sync(dh_ctx *ctx) {
    DH_REQUIRE_CTX(ctx);
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// deferred verdicts
// ---------------------------------------------------------------------------------------
dh_status dh_fail_int_divmod(int op) {
    return dh_fail(DH_ERR_DOMAIN, "integer %s: a divisor is zero%s", op == DH_BIN_DIV ? "division" : "remainder",
                   op == DH_BIN_DIV ? " or the quotient does not fit the value type" : "");
}

dh_status dh_fail_unary_domain(int op) {
    const char *dom = op == DH_UN_SQRT   ? "SQRT with domain [-0, inf]"
                      : op == DH_UN_LN   ? "LN with domain [-0, inf]"
                      : op == DH_UN_ASIN ? "ASIN with domain [-1, 1]"
                                         : "ACOS with domain [-1, 1]";
    return dh_fail(DH_ERR_DOMAIN, "invalid argument passed to unary func %s", dom);
}

dh_status dh_fail_extract_col(long long position, size_t cols) {
    return dh_fail(DH_ERR_OUT_OF_RANGE,
                   "invalid argument '%lld' passed to ExtractCol: out of bounds for dense matrix with column "
                   "boundaries '[0, %zu)'",
                   position, cols);
}

dh_status dh_fail_pipeline_domain() {
    return dh_fail(DH_ERR_DOMAIN, "invalid argument passed to a unary function inside the pipeline");
}

dh_status dh_fail_solve_singular() {
    // Solve.h:113-115
    return dh_fail(DH_ERR_RUNTIME, "A factor Ui is exactly singular, so the solution could not be computed");
}

// One thread: the record keeps the first failure of the stream's order.
static __global__ void latch_deferred_kernel(const int *flag, int ok_value, int *rec, int kind, int op, const long long *sel,
                                             size_t ld_sel, long long bound) {
    const int f = *flag;
    if (f == ok_value || rec[0] != DH_DEFERRED_NONE)
        return;
    const long long v = sel ? sel[static_cast<size_t>(f - 1) * ld_sel] : 0;
    rec[1] = op;
    rec[2] = static_cast<int>(static_cast<unsigned long long>(v) & 0xffffffffull);
    rec[3] = static_cast<int>(static_cast<unsigned long long>(v) >> 32);
    rec[4] = static_cast<int>(static_cast<unsigned long long>(bound) & 0xffffffffull);
    rec[5] = static_cast<int>(static_cast<unsigned long long>(bound) >> 32);
    rec[0] = kind;
}

static __global__ void clear_deferred_kernel(int *rec) {
    if (threadIdx.x < DH_DEFERRED_INTS)
        rec[threadIdx.x] = 0;
}

dh_status dh_latch_deferred(dh_ctx *ctx, int ok_value, int kind, int op, const long long *sel, size_t ld_sel, long long bound) {
    hipLaunchKernelGGL(latch_deferred_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev, ok_value,
                       ctx->flag_dev + DH_DEFERRED_AT, kind, op, sel, ld_sel, bound);
    DH_CHECK_LAUNCH();
    ctx->deferred_enqueued++;
    return DH_OK;
}

extern "C" dh_status dh_defer_checks(dh_ctx *ctx, int on) {
    DH_REQUIRE_CTX(ctx);
    if (on)
        ctx->deferred_depth++;
    else if (ctx->deferred_depth > 0)
        ctx->deferred_depth--;
    else
        return dh_fail(DH_ERR_RUNTIME, "dh_defer_checks: left more often than entered");
    return DH_OK;
}

extern "C" dh_status dh_check_deferred(dh_ctx *ctx) {
    DH_REQUIRE_CTX(ctx);
    if (ctx->deferred_enqueued == 0)
        return DH_OK; // no checked call since the last verdict: nothing can be pending
    ctx->deferred_enqueued = 0;
    int *rec = ctx->flag_host + DH_DEFERRED_AT;
    DH_CHECK_HIP(hipMemcpyAsync(rec, ctx->flag_dev + DH_DEFERRED_AT, DH_DEFERRED_INTS * sizeof(int), hipMemcpyDeviceToHost,
                                ctx->stream));
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (rec[0] == DH_DEFERRED_NONE)
        return DH_OK;
    // a small kernel, not a memset, so that a caller may capture this stream (memset nodes replay badly)
    hipLaunchKernelGGL(clear_deferred_kernel, dim3(1), dim3(64), 0, ctx->stream, ctx->flag_dev + DH_DEFERRED_AT);
    DH_CHECK_LAUNCH();
    const long long value = static_cast<long long>((static_cast<unsigned long long>(static_cast<unsigned>(rec[3])) << 32) |
                                                   static_cast<unsigned>(rec[2]));
    const unsigned long long bound = (static_cast<unsigned long long>(static_cast<unsigned>(rec[5])) << 32) | static_cast<unsigned>(rec[4]);
    switch (rec[0]) {
    case DH_DEFERRED_INT_DIVMOD:
        return dh_fail_int_divmod(rec[1]);
    case DH_DEFERRED_UNARY_DOMAIN:
        return dh_fail_unary_domain(rec[1]);
    case DH_DEFERRED_EXTRACT_COL:
        return dh_fail_extract_col(value, static_cast<size_t>(bound));
    case DH_DEFERRED_PIPELINE_DOMAIN:
        return dh_fail_pipeline_domain();
    case DH_DEFERRED_SOLVE_SINGULAR:
        return dh_fail_solve_singular();
    default:
        return dh_fail(DH_ERR_RUNTIME, "dh_check_deferred: unknown record kind %d", rec[0]);
    }
}

// Capacity class of a request: multiples of 512 B below 64 KiB, above that 1/16 of the largest
// power of two not above the request (at most 6.25 % slack), so that repeated requests of similar
// size share cached blocks.
static size_t block_capacity(size_t bytes) {
    if (bytes == 0)
        bytes = 1; // a zero-size request still gets a distinct pointer as its registry key
    size_t gran = 512;
    if (bytes >= (size_t(64) << 10)) {
        size_t p2 = size_t(1) << 16;
        while ((p2 << 1) != 0 && (p2 << 1) <= bytes)
            p2 <<= 1;
        gran = p2 / 16;
    }
    return (bytes + gran - 1) / gran * gran;
}

// Returns every cached block to the driver. Caller holds ctx->lock.
static void release_cached_locked(dh_ctx *ctx) {
    if (ctx->cached.empty())
        return;
    (void)hipStreamSynchronize(ctx->stream);
    for (auto &kv : ctx->cached)
        (void)hipFree(kv.second);
    ctx->reserved_bytes -= ctx->cached_bytes;
    ctx->cached_bytes = 0;
    ctx->cached.clear();
}

extern "C" dh_status dh_malloc(dh_ctx *ctx, size_t bytes, int zero, void **out) {
    DH_REQUIRE_CTX(ctx);
    if (out == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "dh_malloc: out is null");
    *out = nullptr;
    std::lock_guard<std::mutex> g(ctx->lock);
    if (ctx->mem_in_use + bytes > ctx->mem_budget)
        return dh_fail(DH_ERR_OOM, "dh_malloc: %zu bytes requested, %zu in use, budget %zu", bytes, ctx->mem_in_use,
                       ctx->mem_budget);
    const size_t cap = block_capacity(bytes);
    void *p = nullptr;
    auto it = ctx->cached.lower_bound(cap);
    if (it != ctx->cached.end() && it->first == cap) {
        p = it->second;
        ctx->cached.erase(it);
        ctx->cached_bytes -= cap;
    } else {
        if (ctx->reserved_bytes + cap > ctx->mem_budget)
            release_cached_locked(ctx);
        hipError_t e = hipMalloc(&p, cap);
        if (e == hipErrorOutOfMemory && !ctx->cached.empty()) {
            (void)hipGetLastError();
            release_cached_locked(ctx);
            e = hipMalloc(&p, cap);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return dh_fail(e == hipErrorOutOfMemory ? DH_ERR_OOM : DH_ERR_HIP, "hipMalloc(%zu): %s", cap,
                           hipGetErrorString(e));
        }
        ctx->reserved_bytes += cap;
    }
    if (zero && bytes) {
        hipError_t e = hipMemsetAsync(p, 0, bytes, ctx->stream);
        if (e != hipSuccess) {
            (void)hipFree(p);
            ctx->reserved_bytes -= cap;
            return dh_fail(DH_ERR_HIP, "hipMemsetAsync: %s", hipGetErrorString(e));
        }
    }
    ctx->allocations[p] = dh_ctx::Block{bytes, cap};
    ctx->mem_in_use += bytes;
    *out = p;
    return DH_OK;
}

extern "C" dh_status dh_free(dh_ctx *ctx, void *ptr) {
    DH_REQUIRE_CTX(ctx);
    if (ptr == nullptr)
        return DH_OK;
    std::lock_guard<std::mutex> g(ctx->lock);
    auto it = ctx->allocations.find(ptr);
    if (it == ctx->allocations.end())
        return dh_fail(DH_ERR_RUNTIME, "dh_free: pointer %p was not allocated by this context", ptr);
    // The block goes back to the cache without waiting: whatever still uses it was queued on the
    // context's stream, and so is whatever will use it next.
    ctx->mem_in_use -= it->second.requested;
    ctx->cached.emplace(it->second.capacity, ptr);
    ctx->cached_bytes += it->second.capacity;
    ctx->allocations.erase(it);
    return DH_OK;
}

extern "C" size_t dh_ctx_mem_cached(const dh_ctx *ctx) { return ctx ? ctx->cached_bytes : 0; }

extern "C" dh_status dh_ctx_release_cached(dh_ctx *ctx) {
    DH_REQUIRE_CTX(ctx);
    std::lock_guard<std::mutex> g(ctx->lock);
    release_cached_locked(ctx);
    return DH_OK;
}

extern "C" dh_status dh_h2d(dh_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    DH_REQUIRE_CTX(ctx);
    if (bytes == 0)
        return DH_OK;
    DH_CHECK_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return DH_OK;
}

extern "C" dh_status dh_d2h(dh_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    DH_REQUIRE_CTX(ctx);
    if (bytes == 0)
        return DH_OK;
    DH_CHECK_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return DH_OK;
}

extern "C" dh_status dh_d2d(dh_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes) {
    DH_REQUIRE_CTX(ctx);
    if (bytes == 0)
        return DH_OK;
    DH_CHECK_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return DH_OK;
}

extern "C" dh_status dh_device_memory(int device, size_t *free_bytes, size_t *total_bytes) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count)
        return dh_fail(DH_ERR_HIP, "dh_device_memory: no HIP device %d (%d visible)", device, count);
    int prev = 0;
    DH_CHECK_HIP(hipGetDevice(&prev));
    DH_CHECK_HIP(hipSetDevice(device));
    size_t f = 0, tot = 0;
    const hipError_t e = hipMemGetInfo(&f, &tot);
    (void)hipSetDevice(prev);
    if (e != hipSuccess)
        return dh_fail(DH_ERR_HIP, "dh_device_memory: hipMemGetInfo failed: %s", hipGetErrorString(e));
    if (free_bytes)
        *free_bytes = f;
    if (total_bytes)
        *total_bytes = tot;
    return DH_OK;
}

extern "C" dh_status dh_d2d_2d(dh_ctx *ctx, void *dst_dev, size_t dst_pitch, const void *src_dev, size_t src_pitch,
                               size_t width_bytes, size_t rows) {
    DH_REQUIRE_CTX(ctx);
    if (width_bytes == 0 || rows == 0)
        return DH_OK;
    if (dst_pitch < width_bytes || src_pitch < width_bytes)
        return dh_fail(DH_ERR_INVALID_ARG, "dh_d2d_2d: a pitch (%zu, %zu) is smaller than the row width %zu", dst_pitch,
                       src_pitch, width_bytes);
    if (dst_pitch == width_bytes && src_pitch == width_bytes) {
        DH_CHECK_HIP(hipMemcpyAsync(dst_dev, src_dev, width_bytes * rows, hipMemcpyDeviceToDevice, ctx->stream));
        return DH_OK;
    }
    DH_CHECK_HIP(hipMemcpy2DAsync(dst_dev, dst_pitch, src_dev, src_pitch, width_bytes, rows, hipMemcpyDeviceToDevice,
                                  ctx->stream));
    return DH_OK;
}

extern "C" dh_status dh_d2h_2d(dh_ctx *ctx, void *dst_host, size_t dst_pitch, const void *src_dev, size_t src_pitch,
                               size_t width_bytes, size_t rows) {
    DH_REQUIRE_CTX(ctx);
    if (width_bytes == 0 || rows == 0)
        return DH_OK;
    if (dst_pitch < width_bytes || src_pitch < width_bytes)
        return dh_fail(DH_ERR_INVALID_ARG, "dh_d2h_2d: a pitch (%zu, %zu) is smaller than the row width %zu", dst_pitch,
                       src_pitch, width_bytes);
    if (dst_pitch == width_bytes && src_pitch == width_bytes)
        DH_CHECK_HIP(hipMemcpyAsync(dst_host, src_dev, width_bytes * rows, hipMemcpyDeviceToHost, ctx->stream));
    else
        DH_CHECK_HIP(hipMemcpy2DAsync(dst_host, dst_pitch, src_dev, src_pitch, width_bytes, rows, hipMemcpyDeviceToHost,
                                      ctx->stream));
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return DH_OK;
}

extern "C" dh_status dh_timer_start(dh_ctx *ctx) {
    DH_REQUIRE_CTX(ctx);
    DH_CHECK_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
    return DH_OK;
}

extern "C" dh_status dh_timer_stop_ms(dh_ctx *ctx, float *ms) {
    DH_REQUIRE_CTX(ctx);
    DH_CHECK_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
    DH_CHECK_HIP(hipEventSynchronize(ctx->ev_stop));
    float t = 0.f;
    DH_CHECK_HIP(hipEventElapsedTime(&t, ctx->ev_start, ctx->ev_stop));
    if (ms)
        *ms = t;
    return DH_OK;
}

extern "C" dh_status dh_kernel_timing(dh_ctx *ctx, int on) {
    DH_REQUIRE_CTX(ctx);
    ctx->kernel_timing = on != 0;
    ctx->kernel_events_used = 0;
    return DH_OK;
}

extern "C" dh_status dh_kernel_timing_read(dh_ctx *ctx, double *total_ms, size_t *launches) {
    DH_REQUIRE_CTX(ctx);
    double total = 0.0;
    const size_t n = ctx->kernel_events_used;
    if (n > 0)
        DH_CHECK_HIP(hipEventSynchronize(ctx->kernel_events[n - 1].second));
    for (size_t i = 0; i < n; i++) {
        float t = 0.f;
        DH_CHECK_HIP(hipEventElapsedTime(&t, ctx->kernel_events[i].first, ctx->kernel_events[i].second));
        total += t;
    }
    ctx->kernel_events_used = 0;
    if (total_ms)
        *total_ms = total;
    if (launches)
        *launches = n;
    return DH_OK;
}

dh_status dh_workspace(dh_ctx *ctx, size_t bytes, void **out) {
    std::lock_guard<std::mutex> g(ctx->ws_lock);
    if (bytes > ctx->ws_bytes) {
        size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes;
        if (ctx->ws) {
            DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
            DH_CHECK_HIP(hipFree(ctx->ws));
            ctx->ws = nullptr;
            ctx->ws_bytes = 0;
        }
        hipError_t e = hipMalloc(&ctx->ws, want);
        if (e != hipSuccess)
            return dh_fail(e == hipErrorOutOfMemory ? DH_ERR_OOM : DH_ERR_HIP, "workspace hipMalloc(%zu): %s", want,
                           hipGetErrorString(e));
        ctx->ws_bytes = want;
    }
    *out = ctx->ws;
    return DH_OK;
}
