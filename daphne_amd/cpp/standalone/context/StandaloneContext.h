// Stand-ins for the context side of DAPHNE's run-time, as far as the HIP kernel layer touches it, so that this layer
// builds and is tested without the DAPHNE source tree (plain host compiler, no MLIR, no spdlog). Names, members and
// behaviour follow the reference:
//   IContext / DaphneContext            src/runtime/local/context/DaphneContext.h:40-114 (+ hip_contexts)
//   DaphneUserConfig                    src/api/cli/DaphneUserConfig.h (the fields the kernel layer reads)
//   KernelDispatchMapping, ErrorHandler src/util/KernelDispatchMapping.h, src/util/ErrorHandler.cpp:80-90
//   pre/postKernelInstrumentation       src/runtime/local/instrumentation/KernelInstrumentation.cpp:19-27
// The reference's own DaphneContext.h pulls in MLIR through KernelDispatchMapping.h, so this header also serves the
// context when the kernel layer is compiled against the reference's real data structures.
#pragma once

#include <chrono>
#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

// ------------------------------------------------------------------------------------------
// contexts
// ------------------------------------------------------------------------------------------
struct IContext {
    virtual ~IContext() = default;
    virtual void destroy() = 0;
};

struct DaphneUserConfig {
    bool use_hip = false;           // counterpart of use_cuda
    bool enable_statistics = false; // --statistics: kernels are timed by their dispatch id
    bool hip_fuse_any = false;      // counterpart of cuda_fuse_any (MarkCUDAOpsPass.cpp:55-72)
    bool force_hip = false;
    // HIP::vectorizedPipeline: into how many tasks the rows are cut, and how many rows a task runs per launch
    // (0: all of its rows at once)
    uint64_t hip_vect_shares = 1;
    uint64_t hip_vect_batch_rows = 0;
    // the share of a pipeline's rows that the device takes; below 1 the CPU workers take the other rows
    double hip_vect_device_share = 1.0;
    int numberOfThreads = -1;         // CPU workers of a vectorized pipeline (-1: one per hardware thread)
    size_t phyBatchSize = 96 * 1024;  // bytes of input and output rows that a CPU worker handles per call of the body
};

struct KernelDispatchInfo {
    std::string kernelName, fileName;
    int line = 0, column = 0;
};
// Maps the id the compiler gives every kernel call site to its name and source position.
class KernelDispatchMapping {
    std::mutex m;
    std::vector<KernelDispatchInfo> infos;

  public:
    int registerKernel(std::string name, std::string file = "", int line = 0, int column = 0) {
        std::lock_guard<std::mutex> g(m);
        infos.push_back({std::move(name), std::move(file), line, column});
        return static_cast<int>(infos.size()) - 1;
    }
    KernelDispatchInfo getKernelDispatchInfo(int kId) {
        std::lock_guard<std::mutex> g(m);
        return infos.at(static_cast<size_t>(kId));
    }
};

struct DaphneContext {
    std::vector<std::unique_ptr<IContext>> hip_contexts; // counterpart of cuda_contexts
    DaphneUserConfig config;
    KernelDispatchMapping dispatchMapping;
    // --statistics: accumulated time and call count per dispatch id
    std::mutex stats_lock;
    std::map<int, std::chrono::steady_clock::time_point> kernel_started;
    std::map<int, std::pair<uint64_t, double>> kernel_stats; // id -> (calls, seconds)

    DaphneContext() = default;
    DaphneContext(const DaphneContext &) = delete;
    ~DaphneContext() {
        for (auto &c : hip_contexts)
            c->destroy();
        hip_contexts.clear();
    }
    [[nodiscard]] const DaphneUserConfig &getUserConfig() const { return config; }
    [[nodiscard]] bool useHIP() const { return !hip_contexts.empty(); }
    [[nodiscard]] IContext *getHIPContext(size_t dev_id) const {
        if (dev_id >= hip_contexts.size())
            throw std::runtime_error("DaphneContext: no HIP context for device " + std::to_string(dev_id) +
                                     " (createHIPContext not called?)");
        return hip_contexts[dev_id].get();
    }
    void startKernelTimer(int kId) {
        std::lock_guard<std::mutex> g(stats_lock);
        kernel_started[kId] = std::chrono::steady_clock::now();
    }
    void stopKernelTimer(int kId) {
        std::lock_guard<std::mutex> g(stats_lock);
        auto &s = kernel_stats[kId];
        s.first++;
        s.second += std::chrono::duration<double>(std::chrono::steady_clock::now() - kernel_started[kId]).count();
    }
};
#define DCTX(varname) DaphneContext *varname

inline void preKernelInstrumentation(int kId, DaphneContext *ctx) {
    if (ctx->getUserConfig().enable_statistics)
        ctx->startKernelTimer(kId);
}
inline void postKernelInstrumentation(int kId, DaphneContext *ctx) {
    if (ctx->getUserConfig().enable_statistics)
        ctx->stopKernelTimer(kId);
}

struct ErrorHandler {
    static constexpr int UNREGISTERED = -1;
    // The exception a generated kernel wrapper throws: the kernel's message, prefixed with the name and the
    // source position of the call site that the dispatch id stands for.
    static std::runtime_error runtimeError(int kId, const std::string &msg, KernelDispatchMapping *kdm) {
        if (kId == UNREGISTERED)
            return std::runtime_error(msg);
        const KernelDispatchInfo kdi = kdm->getKernelDispatchInfo(kId);
        return std::runtime_error("The kernel-function " + kdi.kernelName + " failed during runtime with the following message [ " +
                                  msg + " ]\n" + kdi.fileName + ":" + std::to_string(kdi.line) + ":" + std::to_string(kdi.column));
    }
};
