// Shared internals of libdaphne_hip.so: the context object, error plumbing and small device
// helpers for 64-lane wavefront reductions. Not part of the public C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "../../include/daphne_hip.h"

// ---------------------------------------------------------------------------------------
// context
// ---------------------------------------------------------------------------------------
struct dh_ctx {
    int device = 0;
    hipStream_t stream = nullptr; // not owned; nullptr = default stream
    hipDeviceProp_t props{};
    size_t mem_budget = 0;
    size_t mem_in_use = 0;
    std::mutex lock;                  // guards allocations / mem_in_use / the block cache
    // Held by every entry point from its first line to its return (DH_REQUIRE_CTX). The workspace, the domain
    // flag and the AggAll result slot below exist once per context, and a call that reads one of them back
    // synchronises the stream before it returns: with the whole call under this lock, host threads that share
    // a context take turns, their kernels run in the order of the context's stream, and none sees another's
    // flag, scalar or partials. Recursive because entry points call each other (Affine -> MatMul, ...).
    std::recursive_mutex call_lock;
    struct Block {
        size_t requested, capacity;
    };
    std::map<void *, Block> allocations;
    // Blocks returned by dh_free, kept for reuse (hipMalloc/hipFree cost hundreds of microseconds
    // and synchronise the device). Reuse is ordered by the context's stream.
    std::multimap<size_t, void *> cached;
    size_t cached_bytes = 0;   // sum of the capacities in `cached`
    size_t reserved_bytes = 0; // capacities of live + cached blocks

    // Reduction workspace (partials of the two-stage aggregations, split-K slabs). Grown on
    // demand under ws_lock (after a stream synchronise); its users are ordered by call_lock and
    // the context's stream.
    std::mutex ws_lock;
    void *ws = nullptr;
    size_t ws_bytes = 0;

    // One int on the device + its pinned host mirror, for domain-error flags.
    int *flag_dev = nullptr;
    int *flag_host = nullptr;
    // The host mirror as the device sees it: a kernel that reports through it spares the copy back (the caller still
    // waits for the stream before it reads flag_host). Plain stores only - no atomics on host memory.
    int *flag_host_dev = nullptr;
    // Deferred verdicts (dh_defer_checks): while deferred_depth > 0 a checked call does not read its flag back; a
    // one-thread kernel copies a raised flag into the record at flag_dev + DH_DEFERRED_AT (the first one stays) and
    // dh_check_deferred reads that record. The record's host mirror is flag_host + DH_DEFERRED_AT.
    int deferred_depth = 0;
    size_t deferred_enqueued = 0; // checked calls since the last dh_check_deferred (none: nothing to wait for)

    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    // dh_kernel_timing: pairs of events around the dominant kernel of each timed call since the last reading
    bool kernel_timing = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> kernel_events; // created on demand, reused after a reading
    size_t kernel_events_used = 0;
    int num_cus = 0;
    // How fused pipeline bodies run on this context: -1 as the environment says (DH_PIPELINE_JIT, default:
    // specialised at run time), 0 interpreted, 1 specialised.
    int pipeline_mode = -1;
};

// ---------------------------------------------------------------------------------------
// error plumbing
// ---------------------------------------------------------------------------------------
void dh_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
dh_status dh_fail(dh_status st, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define DH_CHECK_HIP(expr)                                                                         \
    do {                                                                                           \
        hipError_t e__ = (expr);                                                                   \
        if (e__ != hipSuccess)                                                                     \
            return dh_fail(DH_ERR_HIP, "%s:%d: %s failed: %s", __FILE__, __LINE__, #expr,          \
                           hipGetErrorString(e__));                                                \
    } while (0)

#define DH_CHECK_LAUNCH()                                                                          \
    do {                                                                                           \
        hipError_t e__ = hipGetLastError();                                                        \
        if (e__ != hipSuccess)                                                                     \
            return dh_fail(DH_ERR_HIP, "%s:%d: kernel launch failed: %s", __FILE__, __LINE__,      \
                           hipGetErrorString(e__));                                                \
    } while (0)

// First statement of every entry point: rejects a null context, takes the context's call lock until the
// enclosing function returns, and makes the context's device current for the calling thread.
#define DH_CAT2(a, b) a##b
#define DH_CAT(a, b) DH_CAT2(a, b)
#define DH_REQUIRE_CTX(ctx)                                                                        \
    if ((ctx) == nullptr)                                                                          \
        return dh_fail(DH_ERR_RUNTIME, "%s: context is null", __func__);                           \
    std::lock_guard<std::recursive_mutex> DH_CAT(dh_call_guard_, __LINE__)((ctx)->call_lock);      \
    do {                                                                                           \
        hipError_t e__ = hipSetDevice((ctx)->device);                                              \
        if (e__ != hipSuccess)                                                                     \
            return dh_fail(DH_ERR_HIP, "hipSetDevice(%d): %s", (ctx)->device,                      \
                           hipGetErrorString(e__));                                                \
    } while (0)

// The deferred-verdict record, in ints from flag_dev / flag_host (both are 256 bytes; int 0 is the flag of a checked
// call and the 8 bytes at byte 64 are the result slot of AggAll):
//   [0] kind (0: nothing pending)  [1] operator code  [2..3] a 64-bit value  [4..5] a 64-bit bound
constexpr int DH_DEFERRED_AT = 32, DH_DEFERRED_INTS = 6;
enum { DH_DEFERRED_NONE = 0, DH_DEFERRED_INT_DIVMOD = 1, DH_DEFERRED_UNARY_DOMAIN = 2, DH_DEFERRED_EXTRACT_COL = 3, DH_DEFERRED_PIPELINE_DOMAIN = 4, DH_DEFERRED_SOLVE_SINGULAR = 5 };
// The failures a checked call reports, immediately or from dh_check_deferred (context.hip).
dh_status dh_fail_int_divmod(int op);
dh_status dh_fail_unary_domain(int op);
dh_status dh_fail_extract_col(long long position, size_t cols);
dh_status dh_fail_pipeline_domain();
dh_status dh_fail_solve_singular();
// After the kernels of a checked call on a context that defers its verdicts: enqueues the kernel that keeps the
// call's flag (at ctx->flag_dev, raised if != ok_value) in the deferred record. sel != nullptr: the flag is the
// index + 1 of the offending entry of sel (stride ld_sel), whose value is kept along with `bound`.
dh_status dh_latch_deferred(dh_ctx *ctx, int ok_value, int kind, int op, const long long *sel, size_t ld_sel, long long bound);

// Returns a workspace of at least `bytes` bytes (256-byte aligned). Growing frees the old
// buffer after a stream synchronise.
dh_status dh_workspace(dh_ctx *ctx, size_t bytes, void **out);

// agg_noalloc.hip: looks up the address of the current device's fixed scratch array (once per device).
dh_status dh_noalloc_bind_device(int device);

static inline size_t dh_ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
static inline bool dh_aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Lane mapping of a fused pipeline for rows of a given width (pipeline_jit.hip): vec values per load,
// G lanes per row, KV vectors per lane, U = 4 / KV rows in flight per lane group, S steps per run.
namespace dh_pipe {
struct PipeShape {
    int vec, G, KV, U, S;
};
bool pipe_shape(size_t cols, int vec, PipeShape *sh);
} // namespace dh_pipe

// Brackets one kernel launch with a pair of events while dh_kernel_timing is on (nothing otherwise): construct right
// before the launch, let it go out of scope right after.
struct DhKernelStopwatch {
    dh_ctx *ctx;
    hipEvent_t stop = nullptr;
    explicit DhKernelStopwatch(dh_ctx *c) : ctx(c) {
        if (!c->kernel_timing || c->kernel_events_used >= 4096)
            return;
        if (c->kernel_events_used == c->kernel_events.size()) {
            hipEvent_t a = nullptr, b = nullptr;
            if (hipEventCreate(&a) != hipSuccess)
                return;
            if (hipEventCreate(&b) != hipSuccess) {
                (void)hipEventDestroy(a);
                return;
            }
            c->kernel_events.emplace_back(a, b);
        }
        auto &pair = c->kernel_events[c->kernel_events_used];
        if (hipEventRecord(pair.first, c->stream) != hipSuccess)
            return;
        c->kernel_events_used++;
        stop = pair.second;
    }
    ~DhKernelStopwatch() {
        if (stop)
            (void)hipEventRecord(stop, ctx->stream);
    }
    DhKernelStopwatch(const DhKernelStopwatch &) = delete;
    DhKernelStopwatch &operator=(const DhKernelStopwatch &) = delete;
};

#include "dev_common.h"
