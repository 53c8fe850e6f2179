// FusedPipelineBody: a vectorized-pipeline body that runs as ONE device kernel per batch.
//
// The reference's compiler outlines the body of a VectorizedPipelineOp into a function
// `void body(DT ***outputs, Structure **inputs, DaphneContext *)` that calls one device kernel per operator
// (src/compiler/lowering/LowerToLLVMPass.cpp:654-726; run per batch by TasksCUDA.cpp:36). For bodies made of
// elementwise operators, row aggregations and full aggregations, the HIP library instead takes the body as a short
// instruction list and runs it in a single pass over the rows (dh_vectorized_pipeline_*). This struct is the glue
// between the two: it has the call signature of an outlined body, so it goes wherever such a function goes
// (CompiledPipelineTaskData::_funcs), and it says how the pipeline's inputs and outputs bind to the kernel's
// operand slots.
//
// Output kinds and the combine they are meant for:
//   TILE  rows x cols, one row per input row           -> VectorCombine::ROWS
//   ROW   rows x 1, the row scalar r                   -> VectorCombine::ROWS
//   ALL   1 x 1, a reduction over all rows of the batch -> VectorCombine::ADD / MIN / MAX (as the REDUCE_ALL op)
// An output that is not null on entry is written in place (a view of the result's rows); otherwise it is created
// on the device. Like a compiled body, the call gives back the references to its inputs when it is done.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

#include <vector>

namespace HIP {

enum class PipeInput { PRIMARY, MATRIX, ROWVEC, COLVEC };
enum class PipeOutput { TILE, ROW, ALL };

template <typename VT> struct FusedPipelineBody {
    static_assert(std::is_same<VT, float>::value || std::is_same<VT, double>::value,
                  "the fused pipeline kernel exists for float and double");
    using DT = DenseMatrix<VT>;
    using IO = typename std::conditional<std::is_same<VT, float>::value, dh_pipe_io_f32, dh_pipe_io_f64>::type;
    struct In {
        PipeInput role;
        int slot; // index into the kernel's matrix / rowvec / colvec operands (ignored for PRIMARY)
    };
    struct Out {
        PipeOutput role;
        int slot; // index into the kernel's out_tile / out_row / out_all
    };
    std::vector<dh_pipe_instr> program;
    std::vector<In> inputs;   // one per pipeline input, in the pipeline's order
    std::vector<Out> outputs; // one per pipeline output

    void operator()(DT ***outs, Structure **ins, DCTX(ctx)) const {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        IO io{};
        const DT *x = nullptr;
        for (size_t i = 0; i < inputs.size(); i++) {
            const DT *m = static_cast<const DT *>(ins[i]);
            const In &b = inputs[i];
            if (b.role != PipeInput::PRIMARY && (b.slot < 0 || b.slot >= DH_PIPE_MAX_OPERANDS))
                throw std::runtime_error("FusedPipelineBody: operand slot " + std::to_string(b.slot) + " out of range");
            switch (b.role) {
            case PipeInput::PRIMARY:
                x = m;
                io.x = m->getValues(&alloc_desc);
                io.ld_x = m->getRowSkip();
                break;
            case PipeInput::MATRIX:
                io.matrix[b.slot] = m->getValues(&alloc_desc);
                io.ld_matrix[b.slot] = m->getRowSkip();
                break;
            case PipeInput::ROWVEC:
                io.rowvec[b.slot] = m->getValues(&alloc_desc);
                break;
            case PipeInput::COLVEC:
                io.colvec[b.slot] = m->getValues(&alloc_desc);
                io.ld_colvec[b.slot] = m->getRowSkip();
                break;
            }
        }
        if (x == nullptr)
            throw std::runtime_error("FusedPipelineBody: no primary input bound");
        const size_t rows = x->getNumRows(), cols = x->getNumCols();
        for (size_t o = 0; o < outputs.size(); o++) {
            const Out &b = outputs[o];
            const int limit = b.role == PipeOutput::ALL ? 2 : DH_PIPE_MAX_OPERANDS;
            if (b.slot < 0 || b.slot >= limit)
                throw std::runtime_error("FusedPipelineBody: output slot " + std::to_string(b.slot) + " out of range");
            DT *&res = *outs[o];
            const size_t r = b.role == PipeOutput::ALL ? 1 : rows, c = b.role == PipeOutput::TILE ? cols : 1;
            if (res == nullptr)
                res = DataObjectFactory::create<DT>(r, c, false, &alloc_desc);
            else if (res->getNumRows() != r || res->getNumCols() != c)
                throw std::runtime_error("FusedPipelineBody: output " + std::to_string(o) + " is " + std::to_string(res->getNumRows()) +
                                         "x" + std::to_string(res->getNumCols()) + ", the body produces " + std::to_string(r) + "x" +
                                         std::to_string(c));
            switch (b.role) {
            case PipeOutput::TILE:
                io.out_tile[b.slot] = res->getValues(&alloc_desc);
                io.ld_out_tile[b.slot] = res->getRowSkip();
                break;
            case PipeOutput::ROW:
                io.out_row[b.slot] = res->getValues(&alloc_desc);
                io.ld_out_row[b.slot] = res->getRowSkip();
                break;
            case PipeOutput::ALL:
                io.out_all[b.slot] = res->getValues(&alloc_desc);
                break;
            }
        }
        dh_status st;
        if constexpr (std::is_same<VT, float>::value)
            st = dh_vectorized_pipeline_f32(detail::raw(ctx), program.data(), static_cast<int>(program.size()), &io, rows, cols);
        else
            st = dh_vectorized_pipeline_f64(detail::raw(ctx), program.data(), static_cast<int>(program.size()), &io, rows, cols);
        for (size_t i = 0; i < inputs.size(); i++)
            DataObjectFactory::destroy(static_cast<const DT *>(ins[i]));
        check(st);
    }
};

} // namespace HIP
