// MTWrapperHIP: one vectorized pipeline shared between the HIP device and the CPU workers.
//
// The counterpart of MTWrapper<DenseMatrix<VT>>::executeQueuePerDeviceType and combineOutputs
// (src/runtime/local/vectorized/MTWrapper_dense.cpp:203-336, 339-373) with initCUDAWorkers / cudaPrefetchInputs
// (MTWrapper.h:94-114): the first `deviceShare` of the rows (the reference: a fixed quarter) go to a queue of device
// tasks served by one WorkerHIP, the other rows to a queue of CPU tasks served by WorkerCPU threads that run the
// pipeline's host body (fun[0]); when both queues have run empty the device's part of every result is put into the
// result in host memory. What differs from the reference:
//   - the device works on a result of its own in device memory, of its share's size, and one pitched copy per result
//     brings it home; the reference lets the device task write through views of the host result and copies whole
//     buffers back;
//   - only the device's rows of the row-split inputs cross the bus (a view of them is uploaded once, before any task
//     runs; the tasks cut their batches out of that view without further copies);
//   - aggregating results (ADD / MIN / MAX) are folded on the device over the device's rows and on the host over the
//     CPU's rows, and the two partial results meet on the host at the end. The reference hands both kinds of task the
//     same result object;
//   - an exception in a device task reaches the caller (WorkerHIP keeps it) after every worker has finished.
// Everything the two sides share is made current in both memory spaces before the first worker starts, so that no
// worker changes the placement records of an object that another one reads.
//
// HIP::VectorizedPipeline runs all rows on the device unless the user configuration's hip_vect_device_share is below
// 1; then it calls this. In DAPHNE this file is src/runtime/local/vectorized/MTWrapperHIP.h (header only).
#pragma once

#include <runtime/local/datastructures/AllocationDescriptorHIP.h>
#include <runtime/local/vectorized/TasksHIP.h>
#include <runtime/local/vectorized/WorkerCPU.h>
#include <runtime/local/vectorized/WorkerHIP.h>

#include <algorithm>
#include <cmath>
#include <functional>
#include <limits>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace HIP {

template <class DT> struct MTWrapperHIP {};

template <typename VT> struct MTWrapperHIP<DenseMatrix<VT>> {
    using DT = DenseMatrix<VT>;
    using PipelineFunc = void(DT ***, Structure **, DCTX(ctx));

  private:
    static bool isAggregating(VectorCombine c) { return c == VectorCombine::ADD || c == VectorCombine::MIN || c == VectorCombine::MAX; }

    // the neutral element that an aggregating result starts from (MTWrapperBase::allocateOutput, MTWrapper.h:116-140)
    static VT identity(VectorCombine c) {
        if (c == VectorCombine::MIN)
            return std::numeric_limits<VT>::has_infinity ? std::numeric_limits<VT>::infinity() : std::numeric_limits<VT>::max();
        if (c == VectorCombine::MAX)
            return std::numeric_limits<VT>::has_infinity ? -std::numeric_limits<VT>::infinity() : std::numeric_limits<VT>::lowest();
        return VT(0);
    }

    // result (host) = result combined with the device's partial result
    static void foldOnHost(VectorCombine c, DT *result, const DT *partial) {
        if (result->getNumRows() != partial->getNumRows() || result->getNumCols() != partial->getNumCols())
            throw std::runtime_error("HIP::MTWrapperHIP: the device's partial result is " + std::to_string(partial->getNumRows()) + "x" +
                                     std::to_string(partial->getNumCols()) + ", the result " + std::to_string(result->getNumRows()) +
                                     "x" + std::to_string(result->getNumCols()));
        const VT *p = partial->getValues(); // brings the partial result to the host
        VT *r = result->getValues();
        for (size_t i = 0; i < result->getNumRows(); i++)
            for (size_t j = 0; j < result->getNumCols(); j++) {
                VT &x = r[i * result->getRowSkip() + j];
                const VT y = p[i * partial->getRowSkip() + j];
                x = c == VectorCombine::ADD ? x + y : (c == VectorCombine::MIN ? std::min(x, y) : std::max(x, y));
            }
    }

  public:
    // `outputs` are the pipeline's results (allocated here in host memory where the caller brought none); `funcs` the
    // outlined bodies: the first one for the CPU, the last one for the device.
    static void executeQueuePerDeviceType(std::vector<std::function<PipelineFunc>> funcs, DT **outputs, size_t numOutputs,
                                          const bool *isScalar, Structure **inputs, size_t numInputs, const int64_t *outRows,
                                          const int64_t *outCols, const VectorSplit *splits, const VectorCombine *combines,
                                          double deviceShare, DCTX(ctx)) {
        if (funcs.size() < 2)
            throw std::runtime_error("HIP::MTWrapperHIP: sharing a pipeline with the CPU needs a host body and a device body");
        if (!(deviceShare >= 0.0 && deviceShare <= 1.0))
            throw std::runtime_error("HIP::MTWrapperHIP: the device's share of the rows must lie in [0, 1]");
        const size_t deviceID = 0; // ToDo: multi device support
        AllocationDescriptorHIP alloc_desc(ctx, deviceID);
        dh_ctx *raw = HIPContext::get(ctx, deviceID)->raw();
        const auto &cfg = ctx->getUserConfig();
        auto rowSplit = [&](size_t i) { return splits[i] == VectorSplit::ROWS && !isScalar[i] && inputs[i]->getNumRows() > 1; };

        // rows to split, and the bytes of input and output that one row stands for
        uint64_t len = 0;
        size_t mem_required = 0;
        for (size_t i = 0; i < numInputs; i++)
            if (splits[i] == VectorSplit::ROWS && !isScalar[i]) {
                len = std::max<uint64_t>(len, inputs[i]->getNumRows());
                mem_required += inputs[i]->getNumItems() * sizeof(VT);
            }
        for (size_t o = 0; o < numOutputs; o++) {
            if (outputs[o] == nullptr && outRows[o] != -1 && outCols[o] != -1) {
                outputs[o] = DataObjectFactory::create<DT>(outRows[o], outCols[o], combines[o] == VectorCombine::ADD);
                if (combines[o] == VectorCombine::MIN || combines[o] == VectorCombine::MAX)
                    std::fill(outputs[o]->getValues(), outputs[o]->getValues() + outputs[o]->getNumRows() * outputs[o]->getRowSkip(),
                              identity(combines[o]));
            }
            if (outputs[o] != nullptr)
                mem_required += outputs[o]->getNumItems() * sizeof(VT);
        }
        if (len == 0)
            return;
        const uint64_t device_len = std::min<uint64_t>(len, static_cast<uint64_t>(std::ceil(static_cast<double>(len) * deviceShare)));
        const uint64_t cpu_len = len - device_len;
        if (cpu_len > 0 && !funcs.front())
            throw std::runtime_error("HIP::MTWrapperHIP: the pipeline has no host body for the CPU's share of the rows");
        const size_t row_mem = std::max<size_t>(mem_required / len, 1);
        const uint32_t cpuBatch = static_cast<uint32_t>(std::min<size_t>(std::max<size_t>(1, cfg.phyBatchSize / row_mem), 1u << 30));

        // both memory spaces current before any worker runs (see the head of this file)
        for (size_t i = 0; i < numInputs; i++) {
            if (isScalar[i])
                continue;
            auto *in = static_cast<const DT *>(inputs[i]);
            if (cpu_len > 0)
                (void)in->getValues();
            if (device_len > 0 && !rowSplit(i))
                (void)in->getValues(&alloc_desc);
        }
        for (size_t o = 0; o < numOutputs; o++)
            if (outputs[o] != nullptr)
                (void)outputs[o]->getValues(); // written in host memory from here on

        // the device's side: views of its rows of the row-split inputs, results of its own
        std::vector<Structure *> inputsDev(inputs, inputs + numInputs);
        std::vector<DT *> viewsDev, resDev(numOutputs, nullptr), resCpu(numOutputs, nullptr);
        std::vector<DT **> resDevPtr(numOutputs), resCpuPtr(numOutputs);
        auto cleanup = [&] {
            for (DT *v : viewsDev)
                DataObjectFactory::destroy(v);
            for (size_t o = 0; o < numOutputs; o++) {
                if (resDev[o] != nullptr)
                    DataObjectFactory::destroy(resDev[o]);
                if (resCpu[o] != nullptr)
                    DataObjectFactory::destroy(resCpu[o]);
            }
            viewsDev.clear();
            std::fill(resDev.begin(), resDev.end(), nullptr);
            std::fill(resCpu.begin(), resCpu.end(), nullptr);
        };
        try {
            for (size_t i = 0; i < numInputs && device_len > 0; i++)
                if (rowSplit(i)) {
                    DT *view = static_cast<const DT *>(inputs[i])->sliceRow(0, device_len);
                    viewsDev.push_back(view);
                    (void)static_cast<const DT *>(view)->getValues(&alloc_desc); // the one upload of these rows
                    inputsDev[i] = view;
                }
            for (size_t o = 0; o < numOutputs; o++) {
                resDevPtr[o] = &resDev[o];
                resCpuPtr[o] = &resCpu[o];
                if (outputs[o] == nullptr && !isAggregating(combines[o]))
                    throw std::runtime_error("HIP::MTWrapperHIP: output " + std::to_string(o) +
                                             " has no known shape; its rows cannot be shared out");
                if (combines[o] == VectorCombine::ROWS) {
                    if (device_len > 0)
                        resDev[o] = DataObjectFactory::create<DT>(device_len, outputs[o]->getNumCols(), false, &alloc_desc);
                    if (cpu_len > 0)
                        resCpu[o] = outputs[o]->sliceRow(device_len, len);
                } else if (combines[o] == VectorCombine::COLS) {
                    if (device_len > 0)
                        resDev[o] = DataObjectFactory::create<DT>(outputs[o]->getNumRows(), device_len, false, &alloc_desc);
                    if (cpu_len > 0)
                        resCpu[o] = outputs[o]->sliceCol(device_len, len);
                } else if (isAggregating(combines[o]))
                    resCpuPtr[o] = outputs + o; // CPU tasks fold into the result itself; the device's partial starts empty
                else
                    throw std::runtime_error("VectorCombine case `" + std::to_string(static_cast<int64_t>(combines[o])) + "` not supported");
            }

            std::mutex lockDev, lockCpu;
            {
                // the device's queue and its worker
                const uint64_t shares = std::max<uint64_t>(1, std::min<uint64_t>(cfg.hip_vect_shares, std::max<uint64_t>(device_len, 1)));
                const uint64_t share_len = (device_len + shares - 1) / shares;
                const uint64_t batchDev = cfg.hip_vect_batch_rows ? cfg.hip_vect_batch_rows : std::max<uint64_t>(share_len, 1);
                if (batchDev > std::numeric_limits<uint32_t>::max())
                    throw std::runtime_error("HIP::MTWrapperHIP: a batch of " + std::to_string(batchDev) +
                                             " rows exceeds the task interface (set hip_vect_batch_rows)");
                BlockingTaskQueue qDev(shares), qCpu(std::max<uint64_t>(cpu_len, 1));
                std::unique_ptr<WorkerHIP> workerDev;
                std::vector<std::unique_ptr<WorkerCPU>> workersCpu;
                // Workers join in their destructors and would wait for ever on a queue that nobody closes: should an
                // exception pass by here, this closes both queues before the workers (declared earlier) go away.
                struct CloseQueues {
                    BlockingTaskQueue &a, &b;
                    ~CloseQueues() {
                        a.closeInput();
                        b.closeInput();
                    }
                } closeQueues{qDev, qCpu};
                if (device_len > 0)
                    workerDev = std::make_unique<WorkerHIP>(&qDev, ctx, static_cast<uint32_t>(funcs.size() - 1),
                                                            static_cast<uint32_t>(batchDev));
                const unsigned hw = std::max(1u, std::thread::hardware_concurrency());
                const uint64_t numCpu = cpu_len == 0 ? 0 : std::min<uint64_t>(cfg.numberOfThreads > 0 ? cfg.numberOfThreads : hw, cpu_len);
                for (uint64_t w = 0; w < numCpu; w++)
                    workersCpu.push_back(std::make_unique<WorkerCPU>(std::vector<TaskQueue *>{&qCpu}, std::vector<int>(numCpu, 0),
                                                                     std::vector<int>(numCpu, 0), ctx, false, 0, cpuBatch,
                                                                     static_cast<int>(w), 1, QueueTypeOption::CENTRALIZED,
                                                                     VictimSelectionLogic::SEQ, false));
                for (uint64_t k = 0; k < device_len; k += share_len)
                    qDev.enqueueTask(new CompiledPipelineTaskHIP<DT>(
                        CompiledPipelineTaskData<DT>{funcs, isScalar, inputsDev.data(), numInputs, numOutputs, outRows, outCols, splits,
                                                     combines, k, std::min(k + share_len, device_len), outRows, outCols, 0, ctx},
                        lockDev, resDevPtr.data()));
                qDev.closeInput();
                // the CPU's rows in equal chunks, one per worker (the reference's default partitioning, STATIC)
                const uint64_t chunk = numCpu ? (cpu_len + numCpu - 1) / numCpu : 1;
                for (uint64_t k = device_len; k < len; k += chunk)
                    qCpu.enqueueTask(new CompiledPipelineTask<DT>(
                        CompiledPipelineTaskData<DT>{funcs, isScalar, inputs, numInputs, numOutputs, outRows, outCols, splits, combines, k,
                                                     std::min(k + chunk, len), outRows, outCols, device_len, ctx},
                        lockCpu, resCpuPtr.data()));
                qCpu.closeInput();
                for (auto &w : workersCpu)
                    w->join();
                if (workerDev) {
                    workerDev->join();
                    workerDev->rethrowIfFailed();
                }
            }

            // the device's part of every result comes home
            for (size_t o = 0; o < numOutputs && device_len > 0; o++) {
                if (resDev[o] == nullptr)
                    throw std::runtime_error("HIP::MTWrapperHIP: the device tasks left output " + std::to_string(o) + " empty");
                if (isAggregating(combines[o])) {
                    if (outputs[o] == nullptr) { // a result of unknown shape, and no CPU task to bring one
                        outputs[o] = resDev[o];
                        resDev[o] = nullptr;
                    } else
                        foldOnHost(combines[o], outputs[o], resDev[o]);
                    continue;
                }
                const VT *src = static_cast<const DT *>(resDev[o])->getValues(&alloc_desc);
                HIP::check(dh_d2h_2d(raw, outputs[o]->getValues(), outputs[o]->getRowSkip() * sizeof(VT), src,
                                     resDev[o]->getRowSkip() * sizeof(VT), resDev[o]->getNumCols() * sizeof(VT), resDev[o]->getNumRows()));
            }
        } catch (...) {
            cleanup();
            throw;
        }
        cleanup();
    }
};

} // namespace HIP
