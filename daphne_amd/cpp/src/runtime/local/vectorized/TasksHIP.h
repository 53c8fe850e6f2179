// CompiledPipelineTaskHIP: one row range of a vectorized pipeline, run on the HIP device.
//
// The counterpart of CompiledPipelineTaskCUDA (src/runtime/local/vectorized/TasksCUDA.h:24-42,
// TasksCUDA.cpp:21-119). execute() walks the task's rows [_rl, _ru) in batches: it cuts the batch out of the
// row-split inputs (views, no copies), runs the pipeline body on them, and puts the body's results into the
// pipeline's results by their combine kind:
//   ROWS  the batch's rows of the result. The body is offered a view of exactly those rows as its output; a body
//         that writes there (every HIP kernel does when `res` is not null) needs no copy at all. A body that
//         returns a matrix of its own instead (the reference's compiled bodies replace the pointer) is copied in
//         with one pitched device-to-device copy.
//   COLS  the batch's columns of the result, same two ways.
//   ADD / MIN / MAX
//         folded into a task-local partial with the elementwise kernel in place (res == lhs), and the partial into
//         the shared result under the result lock when the task ends. The reference's device task knows ADD only;
//         MIN and MAX follow its CPU task (Tasks.cpp:51-84).
// Everything stays in device memory, and no batch waits for the host: kernels of the body that validate their
// arguments on the device (integer DIV / MOD, SQRT / LN / ASIN / ACOS, ExtractCol) run with deferred verdicts
// (HIP::DeferredChecks), and execute() throws the first failure of any batch when the task's batches are enqueued -
// the same exception, from the same call, as a body that checked after every kernel. A task whose body has no such
// kernel never waits at all.
//
// In DAPHNE this file is src/runtime/local/vectorized/TasksHIP.h (header only: no device compiler needed).
#pragma once

#include <runtime/local/datastructures/AllocationDescriptorHIP.h>
#include <runtime/local/kernels/HIP/EwBinaryMat.h>
#include <runtime/local/vectorized/Tasks.h>

#include <algorithm>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

// Batches are handed to the pipeline body as views, and the body's kernels take their device pointers from
// getValues(&alloc_desc) on those views. In an unpatched DAPHNE that call returns the base of the parent's device
// buffer for every view (DenseMatrix.cpp:99-114, 176-182: the cloned placement yields allocation->getData().get()),
// so every batch after the first would read and write row 0. patches/0011-dense-matrix-device-views.patch makes
// views address their parent's device buffer at their own offset and announces it with this macro.
#ifndef DAPHNE_DENSE_MATRIX_DEVICE_VIEWS
#error "TasksHIP.h needs DenseMatrix views that address device placements at their offset: apply patches/0011-dense-matrix-device-views.patch"
#endif

template <class DT> class CompiledPipelineTaskHIP : public CompiledPipelineTaskBase<DT> {};

template <typename VT> class CompiledPipelineTaskHIP<DenseMatrix<VT>> : public CompiledPipelineTaskBase<DenseMatrix<VT>> {
    using DT = DenseMatrix<VT>;
    std::mutex &_resLock;
    DT ***_res;
    using CompiledPipelineTaskBase<DT>::_data;

    static BinaryOpCode combineOp(VectorCombine c) {
        switch (c) {
        case VectorCombine::ADD:
            return BinaryOpCode::ADD;
        case VectorCombine::MIN:
            return BinaryOpCode::MIN;
        case VectorCombine::MAX:
            return BinaryOpCode::MAX;
        default:
            throw std::runtime_error("VectorCombine case `" + std::to_string(static_cast<int64_t>(c)) + "` not supported");
        }
    }
    static bool isAggregating(VectorCombine c) {
        return c == VectorCombine::ADD || c == VectorCombine::MIN || c == VectorCombine::MAX;
    }

    // the part of result `o` that the batch [rowStart, rowEnd) fills, as a view (nullptr for aggregating combines)
    DT *targetView(size_t o, uint64_t rowStart, uint64_t rowEnd) const {
        DT *result = *_res[o];
        const uint64_t lo = rowStart - _data._offset, hi = rowEnd - _data._offset;
        switch (_data._combines[o]) {
        case VectorCombine::ROWS:
            return result->sliceRow(lo, hi);
        case VectorCombine::COLS:
            return result->sliceCol(lo, hi);
        default:
            return nullptr;
        }
    }

    void accumulateOutputs(std::vector<DT *> &localResults, std::vector<DT *> &localAggRes, std::vector<DT *> &targets) {
        const size_t deviceID = 0; // ToDo: multi device support
        AllocationDescriptorHIP alloc_desc(_data._ctx, deviceID);
        dh_ctx *raw = HIPContext::get(_data._ctx, deviceID)->raw();
        for (size_t o = 0; o < _data._numOutputs; ++o) {
            const VectorCombine c = _data._combines[o];
            if (c == VectorCombine::ROWS || c == VectorCombine::COLS) {
                DT *target = targets[o];
                const DT *local = localResults[o];
                if (local == nullptr)
                    throw std::runtime_error("CompiledPipelineTaskHIP: the pipeline body left output " + std::to_string(o) + " empty");
                if (local != target) {
                    if (local->getNumRows() != target->getNumRows() || local->getNumCols() != target->getNumCols())
                        throw std::runtime_error("CompiledPipelineTaskHIP: output " + std::to_string(o) + " of the pipeline body is " +
                                                 std::to_string(local->getNumRows()) + "x" + std::to_string(local->getNumCols()) +
                                                 ", its place in the result is " + std::to_string(target->getNumRows()) + "x" +
                                                 std::to_string(target->getNumCols()));
                    const VT *src = local->getValues(&alloc_desc);
                    VT *dst = target->getValues(&alloc_desc);
                    if (src != dst)
                        HIP::check(dh_d2d_2d(raw, dst, target->getRowSkip() * sizeof(VT), src, local->getRowSkip() * sizeof(VT),
                                             target->getNumCols() * sizeof(VT), target->getNumRows()));
                }
            } else if (isAggregating(c)) {
                if (localResults[o] == nullptr)
                    throw std::runtime_error("CompiledPipelineTaskHIP: the pipeline body left output " + std::to_string(o) + " empty");
                if (localAggRes[o] == nullptr) {
                    localAggRes[o] = localResults[o]; // the first partial is taken over as it is
                    localResults[o] = nullptr;
                } else
                    HIP::ewBinaryMat(combineOp(c), localAggRes[o], localAggRes[o], localResults[o], _data._ctx);
            } else
                throw std::runtime_error("VectorCombine case `" + std::to_string(static_cast<int64_t>(c)) + "` not supported");
        }
    }

  public:
    CompiledPipelineTaskHIP(CompiledPipelineTaskData<DT> data, std::mutex &resLock, DT ***res)
        : CompiledPipelineTaskBase<DT>(data), _resLock(resLock), _res(res) {}

    void execute(uint32_t fid, uint32_t batchSize) override {
        if (batchSize == 0)
            throw std::runtime_error("CompiledPipelineTaskHIP: the batch size must not be 0");
        const size_t n = _data._numOutputs;
        std::vector<DT *> localAggRes(n, nullptr), localResults(n, nullptr), targets(n, nullptr);
        std::vector<DT **> outputs(n);
        HIP::DeferredChecks verdicts(HIPContext::get(_data._ctx, 0)->raw());
        auto dropBatch = [&] { // the views into the results and what the body returned for the current batch
            for (size_t o = 0; o < n; ++o) {
                if (localResults[o] != nullptr && localResults[o] != targets[o])
                    DataObjectFactory::destroy(localResults[o]);
                if (targets[o] != nullptr)
                    DataObjectFactory::destroy(targets[o]);
                localResults[o] = targets[o] = nullptr;
            }
        };
        try {
            for (uint64_t r = _data._rl; r < _data._ru; r += batchSize) {
                const uint64_t r2 = std::min<uint64_t>(r + batchSize, _data._ru);
                auto linputs = this->createFuncInputs(r, r2);
                for (size_t o = 0; o < n; ++o) {
                    targets[o] = targetView(o, r, r2);
                    localResults[o] = targets[o]; // the body may write straight into the result
                    outputs[o] = &localResults[o];
                }
                _data._funcs[fid](outputs.data(), linputs.data(), _data._ctx);
                accumulateOutputs(localResults, localAggRes, targets);
                dropBatch();
                // The body owns the references to its inputs (views included) and gives them back itself.
            }
            verdicts.finish(); // before the task's partial aggregates are folded into the shared results
        } catch (...) {
            // a view holds on to the device buffer it looks into: none may outlive the failure
            dropBatch();
            for (DT *partial : localAggRes)
                if (partial != nullptr)
                    DataObjectFactory::destroy(partial);
            throw;
        }
        for (size_t o = 0; o < n; ++o) {
            if (!isAggregating(_data._combines[o]) || localAggRes[o] == nullptr)
                continue;
            DT *&result = *_res[o];
            std::lock_guard<std::mutex> g(_resLock);
            if (result == nullptr)
                result = localAggRes[o];
            else {
                HIP::ewBinaryMat(combineOp(_data._combines[o]), result, result, localAggRes[o], _data._ctx);
                DataObjectFactory::destroy(localAggRes[o]);
            }
        }
    }

    uint64_t getTaskSize() override { return _data._ru - _data._rl; }
};
