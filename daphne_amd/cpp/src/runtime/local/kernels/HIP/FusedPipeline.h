// FusedPipelineBody: a vectorized-pipeline body that runs as ONE device kernel per batch, and HIP::fusedPipeline, the
// kernel that the compiler calls for a pipeline whose device body it could describe.
//
// The reference's compiler outlines the body of a VectorizedPipelineOp into a function
// `void body(DT ***outputs, Structure **inputs, DaphneContext *)` that calls one device kernel per operator
// (src/compiler/lowering/LowerToLLVMPass.cpp:654-726; run per batch by TasksCUDA.cpp:36). For bodies made of
// elementwise operators, row aggregations and full aggregations, the HIP library instead takes the body as a short
// instruction list and runs it in a single pass over the rows (dh_vectorized_pipeline_*). FusedPipelineBody is the
// glue between the two: it has the call signature of an outlined body, so it goes wherever such a function goes
// (CompiledPipelineTaskData::_funcs), and it says how the pipeline's inputs and outputs bind to the kernel's
// operand slots.
//
// Output kinds and the combine they are meant for:
//   TILE  rows x cols, one row per input row           -> VectorCombine::ROWS
//   ROW   rows x 1, the row scalar r                   -> VectorCombine::ROWS
//   ALL   1 x 1, a reduction over all rows of the batch -> VectorCombine::ADD / MIN / MAX (as the REDUCE_ALL op)
// An output that is not null on entry is written in place (a view of the result's rows); otherwise it is created
// on the device. Like a compiled body, the call gives back the references to its inputs when it is done.
//
// HIP::fusedPipeline has the parameters of vectorizedPipeline (src/runtime/local/kernels/VectorizedPipeline.h:35-69)
// plus the body's operator list as text (PipelineProgramBuilder.h). On the first call with inputs of a given shape
// it builds the instruction list; if the body fits, every batch is one launch, otherwise the outlined device body
// (the last entry of `fun`) runs operator by operator as before. Either way the rows go through
// HIP::VectorizedPipeline: shares, batches and combines are the same.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>
#include <runtime/local/kernels/HIP/PipelineProgramBuilder.h>
#include <runtime/local/kernels/HIP/VectorizedPipeline.h>

#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

namespace HIP {

template <typename VT> struct FusedPipelineBody {
    static_assert(std::is_same<VT, float>::value || std::is_same<VT, double>::value,
                  "the fused pipeline kernel exists for float and double");
    using DT = DenseMatrix<VT>;
    using IO = typename std::conditional<std::is_same<VT, float>::value, dh_pipe_io_f32, dh_pipe_io_f64>::type;
    using In = PipeInputBinding;
    using Out = PipeOutputBinding;
    std::vector<dh_pipe_instr> program;
    std::vector<In> inputs;   // one per pipeline input, in the pipeline's order
    std::vector<Out> outputs; // one per pipeline output

    FusedPipelineBody() = default;
    explicit FusedPipelineBody(const PipeProgram &p) : program(p.program), inputs(p.inputs), outputs(p.outputs) {}

    // A scalar input of a pipeline travels in the place of a pointer: the bits of the value as a double
    // (StoreVariadicPackOpLowering, src/compiler/lowering/LowerToLLVMPass.cpp:489-501, extends every floating-point
    // scalar to f64 first).
    static VT scalarOf(const Structure *disguised) {
        double d;
        std::memcpy(&d, &disguised, sizeof(d));
        return static_cast<VT>(d);
    }

    void operator()(DT ***outs, Structure **ins, DCTX(ctx)) const {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        IO io{};
        const DT *x = nullptr;
        std::vector<dh_pipe_instr> prog = program; // the immediates of scalar inputs are filled in per call
        for (size_t i = 0; i < inputs.size(); i++) {
            const In &b = inputs[i];
            if (b.role == PipeInput::SCALAR) {
                for (int at : b.instrs) {
                    if (at < 0 || size_t(at) >= prog.size())
                        throw std::runtime_error("FusedPipelineBody: scalar input " + std::to_string(i) + " names instruction " +
                                                 std::to_string(at) + " of " + std::to_string(prog.size()));
                    prog[size_t(at)].scalar = static_cast<double>(scalarOf(ins[i]));
                }
                continue;
            }
            const DT *m = static_cast<const DT *>(ins[i]);
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
            case PipeInput::SCALAR:
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
            st = dh_vectorized_pipeline_f32(detail::raw(ctx), prog.data(), static_cast<int>(prog.size()), &io, rows, cols);
        else
            st = dh_vectorized_pipeline_f64(detail::raw(ctx), prog.data(), static_cast<int>(prog.size()), &io, rows, cols);
        for (size_t i = 0; i < inputs.size(); i++)
            if (inputs[i].role != PipeInput::SCALAR)
                DataObjectFactory::destroy(static_cast<const DT *>(ins[i]));
        check(st);
    }
};

// ------------------------------------------------------------------------------------------------------------------
// fusedPipeline: vectorizedPipeline with the device body's operator list alongside
// ------------------------------------------------------------------------------------------------------------------
template <class DTRes> struct FusedPipeline {
    static void apply(DTRes **outputs, size_t numOutputs, bool *isScalar, Structure **inputs, size_t numInputs, int64_t *outRows,
                      int64_t *outCols, int64_t *splits, int64_t *combines, size_t numFuncs, void **fun, const char *body,
                      DCTX(ctx)) = delete;
};

// How the calling thread's last fusedPipeline ran: 1 as one kernel per batch, 0 operator by operator; the reason for
// the latter is kept beside it. (For tests and for --explain style diagnostics; nothing depends on it.)
inline int &fusedPipelineLastMode() {
    thread_local int mode = -1;
    return mode;
}
inline std::string &fusedPipelineLastReason() {
    thread_local std::string reason;
    return reason;
}

template <typename VT> struct FusedPipeline<DenseMatrix<VT>> {
    using DT = DenseMatrix<VT>;
    using PipelineFunc = void(DT ***, Structure **, DCTX(ctx));

    // one entry per (body text, shapes of the inputs, combines): the instruction list, or why there is none
    struct Built {
        bool fits = false;
        std::string why;
        PipeProgram program;
    };
    using Key = std::tuple<std::string, std::vector<std::tuple<bool, int64_t, size_t, size_t>>, std::vector<int64_t>>;
    static std::shared_ptr<const Built> lookup(const char *body, const std::vector<PipeInputShape> &shapes,
                                               const std::vector<VectorCombine> &combines) {
        static std::mutex lock;
        static std::map<Key, std::shared_ptr<const Built>> cache;
        Key key;
        std::get<0>(key) = body;
        for (const PipeInputShape &s : shapes)
            // the row count of a row-split input changes from call to call without changing its role
            std::get<1>(key).emplace_back(s.isScalar, static_cast<int64_t>(s.split), s.rows > 1 ? size_t(2) : s.rows, s.cols);
        for (VectorCombine c : combines)
            std::get<2>(key).push_back(static_cast<int64_t>(c));
        std::lock_guard<std::mutex> g(lock);
        auto it = cache.find(key);
        if (it != cache.end())
            return it->second;
        auto built = std::make_shared<Built>();
        PipeBodyDesc desc;
        built->fits = PipelineProgramBuilder::parse(body, desc, &built->why) &&
                      PipelineProgramBuilder::build(desc, shapes, combines, built->program, &built->why);
        if (cache.size() >= 256) // bodies are few; a program that keeps making new ones should not grow this for ever
            cache.clear();
        cache.emplace(std::move(key), built);
        return built;
    }

    static void apply(DT **outputs, size_t numOutputs, bool *isScalar, Structure **inputs, size_t numInputs, int64_t *outRows,
                      int64_t *outCols, int64_t *splits, int64_t *combines, size_t numFuncs, void **fun, const char *body, DCTX(ctx)) {
        std::shared_ptr<const Built> built;
        if (body != nullptr && body[0] != '\0') {
            std::vector<PipeInputShape> shapes(numInputs);
            for (size_t i = 0; i < numInputs; i++) {
                const VectorSplit split = static_cast<VectorSplit>(splits[i]);
                if (isScalar[i])
                    shapes[i] = {true, split, 1, 1};
                else
                    shapes[i] = {false, split, inputs[i]->getNumRows(), inputs[i]->getNumCols()};
            }
            std::vector<VectorCombine> comb(numOutputs);
            for (size_t o = 0; o < numOutputs; o++)
                comb[o] = static_cast<VectorCombine>(combines[o]);
            built = lookup(body, shapes, comb);
        }
        if (built && built->fits) {
            fusedPipelineLastMode() = 1;
            fusedPipelineLastReason().clear();
            // {host body, device body} as the caller has them, with the one kernel in the place of the device body
            std::vector<std::function<PipelineFunc>> funcs;
            if (numFuncs > 1 && fun[0] != nullptr)
                funcs.emplace_back(reinterpret_cast<PipelineFunc *>(fun[0]));
            funcs.emplace_back(FusedPipelineBody<VT>(built->program));
            VectorizedPipeline<DT>::apply(outputs, numOutputs, isScalar, inputs, numInputs, outRows, outCols,
                                          reinterpret_cast<const VectorSplit *>(splits), reinterpret_cast<const VectorCombine *>(combines),
                                          funcs, ctx);
            return;
        }
        fusedPipelineLastMode() = 0;
        fusedPipelineLastReason() = built ? built->why : "no description of the device body";
        VectorizedPipeline<DT>::apply(outputs, numOutputs, isScalar, inputs, numInputs, outRows, outCols, splits, combines, numFuncs, fun,
                                      ctx);
    }
};

template <class DTRes>
void fusedPipeline(DTRes **outputs, size_t numOutputs, bool *isScalar, Structure **inputs, size_t numInputs, int64_t *outRows,
                   int64_t *outCols, int64_t *splits, int64_t *combines, size_t numFuncs, void **fun, const char *body, DCTX(ctx)) {
    FusedPipeline<DTRes>::apply(outputs, numOutputs, isScalar, inputs, numInputs, outRows, outCols, splits, combines, numFuncs, fun,
                                body, ctx);
}

} // namespace HIP
