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
    // demand under ws_lock; kernels using it are serialised by that lock only for the
    // duration of the enqueue, so concurrent host threads must not share one context for
    // overlapping workspace kernels on different streams.
    std::mutex ws_lock;
    void *ws = nullptr;
    size_t ws_bytes = 0;

    // One int on the device + its pinned host mirror, for domain-error flags.
    int *flag_dev = nullptr;
    int *flag_host = nullptr;

    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int num_cus = 0;
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

#define DH_REQUIRE_CTX(ctx)                                                                        \
    do {                                                                                           \
        if ((ctx) == nullptr)                                                                      \
            return dh_fail(DH_ERR_RUNTIME, "%s: context is null", __func__);                       \
        hipError_t e__ = hipSetDevice((ctx)->device);                                              \
        if (e__ != hipSuccess)                                                                     \
            return dh_fail(DH_ERR_HIP, "hipSetDevice(%d): %s", (ctx)->device,                      \
                           hipGetErrorString(e__));                                                \
    } while (0)

// Returns a workspace of at least `bytes` bytes (256-byte aligned). Growing frees the old
// buffer after a stream synchronise.
dh_status dh_workspace(dh_ctx *ctx, size_t bytes, void **out);

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

#include "dev_common.h"
