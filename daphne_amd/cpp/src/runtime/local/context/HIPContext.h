// HIPContext: the device context the DAPHNE run-time keeps per GPU, on top of the C ABI of libdaphne_hip.so.
//
// Takes the place of CUDAContext (src/runtime/local/context/CUDAContext.h:29-114, CUDAContext.cpp:41-135) in
// DaphneContext::hip_contexts: device selection and properties, the 90 % memory budget, and the allocation
// registry `malloc(size, zero, id) -> shared_ptr<byte>` / `free(id)` that AllocationDescriptorHIP uses. There are
// no library handles to keep (no BLAS / DNN / solver library is involved) and therefore no shared mutable
// descriptors either. Unlike the reference's registry this one is mutex-guarded: kernels are called from the
// compiled program's thread, the CPU workers and the device worker (src/runtime/local/vectorized/MTWrapper.h:94-98).
//
// In DAPHNE this file is src/runtime/local/context/HIPContext.h; it needs a host compiler only.
#pragma once

#include <runtime/local/context/DaphneContext.h>

#include <cstddef>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>

#include <daphne_hip.h>

namespace HIP {
// Re-throws a failed C-ABI status as the exception type the reference's kernels throw for that condition
// (std::runtime_error for shapes / op codes / device errors, std::invalid_argument, std::domain_error,
// std::out_of_range).
inline void check(dh_status st) {
    if (st == DH_OK)
        return;
    const std::string msg = dh_last_error();
    switch (st) {
    case DH_ERR_INVALID_ARG:
        throw std::invalid_argument(msg);
    case DH_ERR_DOMAIN:
        throw std::domain_error(msg);
    case DH_ERR_OUT_OF_RANGE:
        throw std::out_of_range(msg);
    default:
        throw std::runtime_error(msg);
    }
}

// While one of these lives, kernels that validate their arguments on the device (integer DIV / MOD, SQRT / LN /
// ASIN / ACOS, ExtractCol positions) do not wait for their verdict after every call (dh_defer_checks). finish()
// leaves that mode and throws what the first failing call would have thrown; a scope left without finish() - an
// exception on its way out - leaves the mode too and drops a pending verdict, so that none outlives its scope.
class DeferredChecks {
    dh_ctx *ctx;
    bool open = false;

  public:
    explicit DeferredChecks(dh_ctx *c) : ctx(c) {
        check(dh_defer_checks(ctx, 1));
        open = true;
    }
    DeferredChecks(const DeferredChecks &) = delete;
    DeferredChecks &operator=(const DeferredChecks &) = delete;
    void finish() {
        if (!open)
            return;
        open = false;
        check(dh_defer_checks(ctx, 0));
        check(dh_check_deferred(ctx));
    }
    ~DeferredChecks() {
        if (open) {
            (void)dh_defer_checks(ctx, 0);
            (void)dh_check_deferred(ctx);
        }
    }
};
} // namespace HIP

class HIPContext final : public IContext {
    // The C-ABI handle, shared with the deleters of the buffers handed out: a buffer that outlives the context
    // (a matrix destroyed after its DaphneContext) finds the handle gone and frees nothing a second time.
    struct Handle {
        std::mutex m;
        dh_ctx *ctx = nullptr;
    };
    std::shared_ptr<Handle> handle = std::make_shared<Handle>();
    int device_id = -1;
    std::mutex registry_lock;
    std::map<size_t, std::shared_ptr<std::byte>> allocations;
    size_t alloc_count = 0;

    explicit HIPContext(int id) : device_id(id) { HIP::check(dh_ctx_create(id, &handle->ctx)); }

  public:
    HIPContext() = delete;
    HIPContext(const HIPContext &) = delete;
    HIPContext &operator=(const HIPContext &) = delete;
    ~HIPContext() override { destroy(); }

    void destroy() override {
        {
            std::lock_guard<std::mutex> g(registry_lock);
            allocations.clear();
        }
        std::lock_guard<std::mutex> g(handle->m);
        if (handle->ctx) {
            dh_ctx_destroy(handle->ctx); // frees whatever is still registered on the device
            handle->ctx = nullptr;
        }
    }
    static std::unique_ptr<IContext> createHipContext(int id) { return std::unique_ptr<IContext>(new HIPContext(id)); }
    static HIPContext *get(DaphneContext *ctx, size_t id) {
        if (ctx == nullptr)
            throw std::runtime_error("HIPContext::get: the DaphneContext is null");
        auto *hc = dynamic_cast<HIPContext *>(ctx->getHIPContext(id));
        if (hc == nullptr)
            throw std::runtime_error("HIPContext::get: no HIP context with id " + std::to_string(id));
        return hc;
    }

    [[nodiscard]] size_t getMemBudget() const { return dh_ctx_mem_budget(handle->ctx); }
    [[nodiscard]] size_t getMemInUse() const { return dh_ctx_mem_in_use(handle->ctx); }
    [[nodiscard]] int getDeviceId() const { return device_id; }
    [[nodiscard]] dh_ctx *raw() const { return handle->ctx; }
    [[nodiscard]] size_t numAllocations() {
        std::lock_guard<std::mutex> g(registry_lock);
        return allocations.size();
    }

    // CUDAContext::malloc (CUDAContext.cpp:120-129): registers the buffer under a fresh id and shares it out.
    std::shared_ptr<std::byte> malloc(size_t size, bool zero, size_t &id) {
        void *p = nullptr;
        HIP::check(dh_malloc(handle->ctx, size, zero ? 1 : 0, &p));
        std::shared_ptr<Handle> h = handle;
        std::shared_ptr<std::byte> sp(static_cast<std::byte *>(p), [h](std::byte *q) {
            std::lock_guard<std::mutex> g(h->m);
            if (h->ctx)
                dh_free(h->ctx, q);
        });
        std::lock_guard<std::mutex> g(registry_lock);
        id = alloc_count++;
        allocations.emplace(id, sp);
        return sp;
    }
    // CUDAContext::free (CUDAContext.cpp:131-135): drops the registry's reference; the device block goes back to
    // the allocator when the last holder lets go. An id that is no longer registered (context destroyed first)
    // is ignored, because descriptors call this from their destructors.
    void free(size_t id) {
        std::lock_guard<std::mutex> g(registry_lock);
        allocations.erase(id);
    }
};
