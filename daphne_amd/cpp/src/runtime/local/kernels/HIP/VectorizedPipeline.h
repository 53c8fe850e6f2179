// HIP::VectorizedPipeline: runs a vectorized pipeline on the HIP device - all of its rows, or a share of them beside
// the CPU workers.
//
// Same parameters as the reference's kernel (src/runtime/local/kernels/VectorizedPipeline.h:35-69), which hands
// the pipeline to MTWrapper<DenseMatrix<VT>>::executeQueuePerDeviceType (src/runtime/local/vectorized/
// MTWrapper_dense.cpp:203-336). That one gives a quarter of the rows to the device in batches of a few MiB and
// the rest to the CPU workers. With 288 GB of device memory and a body that runs as one kernel, the device takes
// all rows here and takes them in as few launches as possible: the row range is cut into `hip_vect_shares` tasks
// (default 1) and each task runs in batches of `hip_vect_batch_rows` rows (default 0: the whole task at once).
// More shares and smaller batches give the same result (that is what the tests check) and are there for results
// too large for one pass. A caller that wants the reference's hybrid execution sets `hip_vect_device_share` below 1:
// then MTWrapperHIP (runtime/local/vectorized/MTWrapperHIP.h) gives that share of the rows to a device worker and
// the rest to CPU workers that run the host body, and the results end up in host memory.
//
// Outputs are allocated on the device as MTWrapperBase::allocateOutput does on the host
// (src/runtime/local/vectorized/MTWrapper.h:116-140): ROWS / COLS results uninitialised, aggregating results
// filled with the identity of their combine (0, +inf, -inf) so that every share folds into them the same way.
// The tasks run one after the other on the calling thread: they share one device stream, so there is nothing to
// win by threads. `fun` holds the outlined bodies; the last one is the device body (the reference passes
// {cpu body, device body}).
#pragma once

#include <runtime/local/kernels/HIP/Fill.h>
#include <runtime/local/kernels/HIP/HostUtils.h>
#include <runtime/local/vectorized/MTWrapperHIP.h>
#include <runtime/local/vectorized/TasksHIP.h>

#include <functional>
#include <limits>
#include <mutex>
#include <vector>

namespace HIP {

template <class DTRes> struct VectorizedPipeline {
    static void apply(DTRes **outputs, size_t numOutputs, bool *isScalar, Structure **inputs, size_t numInputs, int64_t *outRows,
                      int64_t *outCols, int64_t *splits, int64_t *combines, size_t numFuncs, void **fun, DCTX(ctx)) = delete;
};

template <typename VT> struct VectorizedPipeline<DenseMatrix<VT>> {
    using DT = DenseMatrix<VT>;
    using PipelineFunc = void(DT ***, Structure **, DCTX(ctx));

    static void apply(DT **outputs, size_t numOutputs, bool *isScalar, Structure **inputs, size_t numInputs, int64_t *outRows,
                      int64_t *outCols, int64_t *splits, int64_t *combines, size_t numFuncs, void **fun, DCTX(ctx)) {
        if (numFuncs == 0)
            throw std::runtime_error("HIP::vectorizedPipeline: no pipeline body given");
        std::vector<std::function<PipelineFunc>> funcs;
        for (size_t i = 0; i < numFuncs; ++i) {
            if (fun[i] != nullptr)
                funcs.emplace_back(reinterpret_cast<PipelineFunc *>(fun[i]));
            else
                funcs.emplace_back(); // no such body: only an error if somebody has to run it
        }
        apply(outputs, numOutputs, isScalar, inputs, numInputs, outRows, outCols, reinterpret_cast<VectorSplit *>(splits),
              reinterpret_cast<VectorCombine *>(combines), funcs, ctx);
    }

    // the same with the bodies as function objects (how MTWrapper takes them)
    static void apply(DT **outputs, size_t numOutputs, const bool *isScalar, Structure **inputs, size_t numInputs,
                      const int64_t *outRows, const int64_t *outCols, const VectorSplit *splits, const VectorCombine *combines,
                      std::vector<std::function<PipelineFunc>> funcs, DCTX(ctx)) {
        // The reference's division of labour, on request: the device takes hip_vect_device_share of the rows and the
        // CPU workers run the host body on the others; the results then live in host memory.
        if (ctx->getUserConfig().hip_vect_device_share < 1.0 && funcs.size() > 1) {
            MTWrapperHIP<DT>::executeQueuePerDeviceType(std::move(funcs), outputs, numOutputs, isScalar, inputs, numInputs, outRows,
                                                        outCols, splits, combines, ctx->getUserConfig().hip_vect_device_share, ctx);
            return;
        }
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        // the number of rows to split: the tallest row-split input (others are broadcast)
        uint64_t len = 0;
        for (size_t i = 0; i < numInputs; ++i)
            if (splits[i] == VectorSplit::ROWS && !isScalar[i])
                len = std::max<uint64_t>(len, inputs[i]->getNumRows());

        for (size_t o = 0; o < numOutputs; ++o) {
            if (outputs[o] != nullptr || outRows[o] == -1 || outCols[o] == -1)
                continue;
            switch (combines[o]) {
            case VectorCombine::ADD:
                HIP::fill(outputs[o], VT(0), outRows[o], outCols[o], ctx);
                break;
            case VectorCombine::MIN:
                HIP::fill(outputs[o], std::numeric_limits<VT>::infinity(), outRows[o], outCols[o], ctx);
                break;
            case VectorCombine::MAX:
                HIP::fill(outputs[o], -std::numeric_limits<VT>::infinity(), outRows[o], outCols[o], ctx);
                break;
            default:
                outputs[o] = DataObjectFactory::create<DT>(outRows[o], outCols[o], false, &alloc_desc);
            }
        }
        std::vector<DT **> res(numOutputs);
        for (size_t o = 0; o < numOutputs; ++o)
            res[o] = outputs + o;
        // A view takes over its parent's placements as they are when it is cut (Structure.cpp:24-36), so the device
        // copies are made current in the whole objects before any task slices them: the row-split inputs are
        // uploaded once (what cudaPrefetchInputs does, MTWrapper.h:94-114) instead of batch by batch, and a result
        // the caller brought along is marked as written on the device.
        for (size_t i = 0; i < numInputs; ++i)
            if (splits[i] == VectorSplit::ROWS && !isScalar[i] && inputs[i]->getNumRows() > 1)
                (void)static_cast<const DT *>(inputs[i])->getValues(&alloc_desc);
        for (size_t o = 0; o < numOutputs; ++o)
            if (outputs[o] != nullptr && (combines[o] == VectorCombine::ROWS || combines[o] == VectorCombine::COLS))
                (void)outputs[o]->getValues(&alloc_desc);

        const auto &cfg = ctx->getUserConfig();
        const uint64_t shares = std::max<uint64_t>(1, std::min<uint64_t>(cfg.hip_vect_shares, std::max<uint64_t>(len, 1)));
        const uint64_t share_len = (len + shares - 1) / shares;
        const uint64_t batch = cfg.hip_vect_batch_rows ? cfg.hip_vect_batch_rows : std::max<uint64_t>(share_len, 1);
        if (batch > std::numeric_limits<uint32_t>::max())
            throw std::runtime_error("HIP::vectorizedPipeline: a batch of " + std::to_string(batch) +
                                     " rows exceeds the task interface (set hip_vect_batch_rows)");
        std::mutex resLock;
        const uint32_t fid = static_cast<uint32_t>(funcs.size() - 1);
        for (uint64_t k = 0; k < len; k += share_len) {
            CompiledPipelineTaskHIP<DT> task(
                CompiledPipelineTaskData<DT>{funcs, isScalar, inputs, numInputs, numOutputs, outRows, outCols, splits, combines, k,
                                             std::min(k + share_len, len), outRows, outCols, 0, ctx},
                resLock, res.data());
            task.execute(fid, static_cast<uint32_t>(batch));
        }
    }
};

template <class DTRes>
void vectorizedPipeline(DTRes **outputs, size_t numOutputs, bool *isScalar, Structure **inputs, size_t numInputs, int64_t *outRows,
                        int64_t *outCols, int64_t *splits, int64_t *combines, size_t numFuncs, void **fun, DCTX(ctx)) {
    VectorizedPipeline<DTRes>::apply(outputs, numOutputs, isScalar, inputs, numInputs, outRows, outCols, splits, combines, numFuncs,
                                     fun, ctx);
}

} // namespace HIP
