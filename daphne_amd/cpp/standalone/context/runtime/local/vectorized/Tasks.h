// Stand-in for DAPHNE's src/runtime/local/vectorized/Tasks.h:30-112 and the split / combine kinds of
// src/ir/daphneir/DaphneVectorizableOpInterface.td:23-34, as far as the device side needs them: what a task is,
// the data every task of one pipeline call shares, how a task cuts its row range out of the inputs, the end marker
// of a task queue, and the CPU task (Tasks.cpp:22-150) that the CPU workers of a pipeline shared between the device
// and the CPU run.
#pragma once

#include <runtime/local/context/DaphneContext.h>
#include <runtime/local/datastructures/DataObjectFactory.h>
#include <runtime/local/datastructures/DenseMatrix.h>
#include <runtime/local/datastructures/Structure.h>

#include <algorithm>
#include <cstdint>
#include <functional>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

namespace mlir::daphne {
enum class VectorSplit : int64_t { NONE = 0, ROWS = 1 };
enum class VectorCombine : int64_t { ROWS = 1, COLS = 2, ADD = 3, MIN = 4, MAX = 5 };
} // namespace mlir::daphne
using mlir::daphne::VectorCombine;
using mlir::daphne::VectorSplit;

class Task {
  public:
    virtual ~Task() = default;
    virtual void execute(uint32_t fid, uint32_t batchSize) = 0;
    virtual uint64_t getTaskSize() = 0;
};

// what a closed, empty queue hands out (Tasks.h:37-43)
class EOFTask : public Task {
  public:
    void execute(uint32_t, uint32_t) override {}
    uint64_t getTaskSize() override { return 0; }
};

template <class DT> struct CompiledPipelineTaskData {
    std::vector<std::function<void(DT ***, Structure **, DCTX(ctx))>> _funcs;
    const bool *_isScalar;
    Structure **_inputs;
    const size_t _numInputs;
    const size_t _numOutputs;
    const int64_t *_outRows;
    const int64_t *_outCols;
    const VectorSplit *_splits;
    const VectorCombine *_combines;
    const uint64_t _rl; // first row of the task
    const uint64_t _ru; // one past its last row
    const int64_t *_wholeResultRows;
    const int64_t *_wholeResultCols;
    const uint64_t _offset; // row of the whole result at which this worker group's result starts
    DCTX(_ctx);
};

template <class DT> class CompiledPipelineTaskBase : public Task {
  protected:
    CompiledPipelineTaskData<DT> _data;

    bool isBroadcast(VectorSplit splitMethod, Structure *input) {
        return splitMethod == VectorSplit::NONE || (splitMethod == VectorSplit::ROWS && input->getNumRows() == 1);
    }
    // The inputs of one batch: row-split inputs as views of rows [rowStart, rowEnd), everything else as it is
    // (with one more reference, which the pipeline body gives back).
    std::vector<Structure *> createFuncInputs(uint64_t rowStart, uint64_t rowEnd) {
        std::vector<Structure *> linputs;
        for (size_t i = 0; i < _data._numInputs; i++) {
            Structure *in = _data._inputs[i];
            if (isBroadcast(_data._splits[i], in)) {
                if (!_data._isScalar[i])
                    in->increaseRefCounter();
                linputs.push_back(in);
            } else
                linputs.push_back(in->sliceRow(rowStart, rowEnd));
        }
        return linputs;
    }

  public:
    explicit CompiledPipelineTaskBase(CompiledPipelineTaskData<DT> data) : _data(data) {}
};

// The CPU task: runs body `fid` on its rows batch by batch in host memory. ROWS / COLS results are copied into their
// place in the (worker group's part of the) result; aggregating results are folded into a task-local partial first
// and into the shared result under the lock at the end.
template <class DT> class CompiledPipelineTask : public CompiledPipelineTaskBase<DT> {};

template <typename VT> class CompiledPipelineTask<DenseMatrix<VT>> : public CompiledPipelineTaskBase<DenseMatrix<VT>> {
    using DT = DenseMatrix<VT>;
    std::mutex &_resLock;
    DT ***_res;
    using CompiledPipelineTaskBase<DT>::_data;

    static void fold(VectorCombine c, DT *into, const DT *from) {
        if (into->getNumRows() != from->getNumRows() || into->getNumCols() != from->getNumCols())
            throw std::runtime_error("CompiledPipelineTask: partial results of different shapes");
        VT *a = into->getValues();
        const VT *b = from->getValues();
        for (size_t r = 0; r < into->getNumRows(); r++)
            for (size_t k = 0; k < into->getNumCols(); k++) {
                VT &x = a[r * into->getRowSkip() + k];
                const VT y = b[r * from->getRowSkip() + k];
                switch (c) {
                case VectorCombine::ADD:
                    x = x + y;
                    break;
                case VectorCombine::MIN:
                    x = std::min(x, y);
                    break;
                case VectorCombine::MAX:
                    x = std::max(x, y);
                    break;
                default:
                    throw std::runtime_error("VectorCombine case `" + std::to_string(static_cast<int64_t>(c)) + "` not supported");
                }
            }
    }

  public:
    CompiledPipelineTask(CompiledPipelineTaskData<DT> data, std::mutex &resLock, DT ***res)
        : CompiledPipelineTaskBase<DT>(data), _resLock(resLock), _res(res) {}

    void execute(uint32_t fid, uint32_t batchSize) override {
        const size_t n = _data._numOutputs;
        std::vector<DT *> partial(n, nullptr), local(n, nullptr);
        std::vector<DT **> outputs(n);
        for (size_t o = 0; o < n; o++)
            outputs[o] = &local[o];
        for (uint64_t r = _data._rl; r < _data._ru; r += batchSize) {
            const uint64_t r2 = std::min<uint64_t>(r + batchSize, _data._ru);
            auto linputs = this->createFuncInputs(r, r2);
            _data._funcs[fid](outputs.data(), linputs.data(), _data._ctx);
            for (size_t o = 0; o < n; o++) {
                const VectorCombine c = _data._combines[o];
                if (c == VectorCombine::ROWS || c == VectorCombine::COLS) {
                    DT *whole = *_res[o];
                    DT *place = c == VectorCombine::ROWS ? whole->sliceRow(r - _data._offset, r2 - _data._offset)
                                                         : whole->sliceCol(r - _data._offset, r2 - _data._offset);
                    const VT *src = static_cast<const DT *>(local[o])->getValues();
                    VT *dst = place->getValues();
                    for (size_t i = 0; i < place->getNumRows(); i++)
                        std::copy(src + i * local[o]->getRowSkip(), src + i * local[o]->getRowSkip() + place->getNumCols(),
                                  dst + i * place->getRowSkip());
                    DataObjectFactory::destroy(place);
                } else if (partial[o] == nullptr) {
                    partial[o] = local[o];
                    local[o] = nullptr;
                } else
                    fold(c, partial[o], local[o]);
                if (local[o] != nullptr) {
                    DataObjectFactory::destroy(local[o]);
                    local[o] = nullptr;
                }
            }
        }
        for (size_t o = 0; o < n; o++) {
            const VectorCombine c = _data._combines[o];
            if (c == VectorCombine::ROWS || c == VectorCombine::COLS || partial[o] == nullptr)
                continue;
            std::lock_guard<std::mutex> g(_resLock);
            DT *&result = *_res[o];
            if (result == nullptr)
                result = partial[o];
            else {
                fold(c, result, partial[o]);
                DataObjectFactory::destroy(partial[o]);
            }
        }
    }
    uint64_t getTaskSize() override { return _data._ru - _data._rl; }
};
