// Stand-in for DAPHNE's src/runtime/local/vectorized/Tasks.h:30-112 and the split / combine kinds of
// src/ir/daphneir/DaphneVectorizableOpInterface.td:23-34, as far as a device task needs them: what a task is,
// the data every task of one pipeline call shares, and how a task cuts its row range out of the inputs.
#pragma once

#include <runtime/local/context/DaphneContext.h>
#include <runtime/local/datastructures/Structure.h>

#include <cstdint>
#include <functional>
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
