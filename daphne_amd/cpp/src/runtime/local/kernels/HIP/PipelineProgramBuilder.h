// PipelineProgramBuilder: from the operator list of a vectorized pipeline's device body to the instruction list of
// the fused pipeline kernel.
//
// The reference outlines the device region of a VectorizedPipelineOp as a function that calls one kernel per
// operator (src/compiler/lowering/LowerToLLVMPass.cpp:654-726; run per batch by TasksCUDA.cpp:36), every
// intermediate in memory. The HIP library runs such a body as ONE kernel if it is given as a short instruction list
// (dh_pipe_instr, include/daphne_hip.h). This file is the lowering between the two, at the level of DaphneIR
// mnemonics (ewSub, sumRow, sumAll, ...: the part of a kernel's name between "HIP_" and "__"), in plain C++17 with
// no MLIR in it, so that it can run where the shapes are known: at run time, on the first call of the pipeline.
//
// The body travels as text, one operator per line, which is what the compiler-side patch
// (patches/0012-describe-device-body.patch) emits next to the outlined `_vect_hip` function:
//     %0 = ewSub in0, in1          in<k>: input k of the pipeline     %<n>: result of line n
//     %1 = ewDiv %0, in2           #<v>:  a constant
//     %2 = ewMul %1, %1
//     %3 = sumRow %2
//     %4 = ewGt %3, #64
//     %5 = sumAll %4
//     return %3, %5
// `cast` lines (the scalar of a full aggregation turned into the 1 x 1 matrix that a pipeline returns) stand for
// their operand.
//
// The kernel is an accumulator machine: per row one tile t (the row's values) and one scalar r. A body fits if it
// is a chain through these two: every operator takes the value that is in t (or r) right now, plus at most one more
// operand that is a constant, a scalar input, a broadcast row vector, a row-split column vector or matrix, the value
// itself (x * x), or r while working on t. A value that is overwritten can only be returned (it is stored when it is
// made), not used again. Anything else - two live tiles, a matrix product, a result combined by COLS - does not
// fit; build() then says why and the caller runs the body operator by operator.
#pragma once

#include <runtime/local/kernels/AggOpCode.h>
#include <runtime/local/kernels/BinaryOpCode.h>
#include <runtime/local/kernels/UnaryOpCode.h>
#include <runtime/local/vectorized/Tasks.h>

#include <cstdint>
#include <cstdlib>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include <daphne_hip.h>

namespace HIP {

enum class PipeInput { PRIMARY, MATRIX, ROWVEC, COLVEC, SCALAR };
enum class PipeOutput { TILE, ROW, ALL };

// How the pipeline's inputs and outputs bind to the kernel's operand slots (used by FusedPipelineBody).
struct PipeInputBinding {
    PipeInput role;
    // index into the kernel's matrix / rowvec / colvec operands (ignored for PRIMARY and SCALAR)
    int slot;
    // SCALAR: the instructions whose immediate is this input's value (it is known only when the body is called)
    std::vector<int> instrs = {};
};
struct PipeOutputBinding {
    PipeOutput role;
    int slot; // index into the kernel's out_tile / out_row / out_all
};

struct PipeOperandRef {
    enum Kind { INPUT, RESULT, CONSTANT } kind;
    size_t index;    // INPUT: input number; RESULT: operator (line) number
    double constant; // CONSTANT
};
struct PipeOpDesc {
    std::string mnemonic;
    std::vector<PipeOperandRef> operands;
};
struct PipeBodyDesc {
    std::vector<PipeOpDesc> ops;
    std::vector<PipeOperandRef> results;
};
// What is known of an input when the pipeline is called.
struct PipeInputShape {
    bool isScalar;
    VectorSplit split;
    size_t rows, cols;
};

struct PipeProgram {
    std::vector<dh_pipe_instr> program;
    std::vector<PipeInputBinding> inputs;   // one per pipeline input
    std::vector<PipeOutputBinding> outputs; // one per pipeline output
};

class PipelineProgramBuilder {
    static bool lookup(const std::map<std::string, int> &table, const std::string &key, int &out) {
        auto it = table.find(key);
        if (it == table.end())
            return false;
        out = it->second;
        return true;
    }
    static const std::map<std::string, int> &binaryOps() {
        static const std::map<std::string, int> t = {
            {"ewAdd", int(BinaryOpCode::ADD)}, {"ewSub", int(BinaryOpCode::SUB)}, {"ewMul", int(BinaryOpCode::MUL)},
            {"ewDiv", int(BinaryOpCode::DIV)}, {"ewPow", int(BinaryOpCode::POW)}, {"ewMod", int(BinaryOpCode::MOD)},
            {"ewLog", int(BinaryOpCode::LOG)}, {"ewEq", int(BinaryOpCode::EQ)},   {"ewNeq", int(BinaryOpCode::NEQ)},
            {"ewLt", int(BinaryOpCode::LT)},   {"ewLe", int(BinaryOpCode::LE)},   {"ewGt", int(BinaryOpCode::GT)},
            {"ewGe", int(BinaryOpCode::GE)},   {"ewMin", int(BinaryOpCode::MIN)}, {"ewMax", int(BinaryOpCode::MAX)},
            {"ewAnd", int(BinaryOpCode::AND)}, {"ewOr", int(BinaryOpCode::OR)}};
        return t;
    }
    static const std::map<std::string, int> &unaryOps() {
        static const std::map<std::string, int> t = {
            {"ewMinus", int(UnaryOpCode::MINUS)}, {"ewAbs", int(UnaryOpCode::ABS)},     {"ewSign", int(UnaryOpCode::SIGN)},
            {"ewSqrt", int(UnaryOpCode::SQRT)},   {"ewExp", int(UnaryOpCode::EXP)},     {"ewLn", int(UnaryOpCode::LN)},
            {"ewSin", int(UnaryOpCode::SIN)},     {"ewCos", int(UnaryOpCode::COS)},     {"ewTan", int(UnaryOpCode::TAN)},
            {"ewAsin", int(UnaryOpCode::ASIN)},   {"ewAcos", int(UnaryOpCode::ACOS)},   {"ewAtan", int(UnaryOpCode::ATAN)},
            {"ewSinh", int(UnaryOpCode::SINH)},   {"ewCosh", int(UnaryOpCode::COSH)},   {"ewTanh", int(UnaryOpCode::TANH)},
            {"ewFloor", int(UnaryOpCode::FLOOR)}, {"ewCeil", int(UnaryOpCode::CEIL)},   {"ewRound", int(UnaryOpCode::ROUND)},
            {"ewIsnan", int(UnaryOpCode::ISNAN)}};
        return t;
    }
    static const std::map<std::string, int> &rowAggs() {
        static const std::map<std::string, int> t = {
            {"sumRow", int(AggOpCode::SUM)},       {"minRow", int(AggOpCode::MIN)},       {"maxRow", int(AggOpCode::MAX)},
            {"meanRow", int(AggOpCode::MEAN)},     {"varRow", int(AggOpCode::VAR)},       {"stddevRow", int(AggOpCode::STDDEV)},
            {"idxminRow", int(AggOpCode::IDXMIN)}, {"idxmaxRow", int(AggOpCode::IDXMAX)}};
        return t;
    }
    // full aggregations the kernel can fold over rows, with the combine that folds them over batches
    struct FullAgg {
        int op;
        VectorCombine combine;
    };
    static bool fullAgg(const std::string &m, FullAgg &out) {
        if (m == "sumAll")
            out = {int(AggOpCode::SUM), VectorCombine::ADD};
        else if (m == "minAll")
            out = {int(AggOpCode::MIN), VectorCombine::MIN};
        else if (m == "maxAll")
            out = {int(AggOpCode::MAX), VectorCombine::MAX};
        else
            return false;
        return true;
    }

    static bool fail(std::string *why, const std::string &msg) {
        if (why)
            *why = msg;
        return false;
    }
    static std::string trim(const std::string &s) {
        const size_t a = s.find_first_not_of(" \t\r");
        if (a == std::string::npos)
            return "";
        return s.substr(a, s.find_last_not_of(" \t\r") - a + 1);
    }
    static bool parseOperand(const std::string &tok, PipeOperandRef &out) {
        if (tok.size() < 2)
            return false;
        char *end = nullptr;
        if (tok.compare(0, 2, "in") == 0) {
            out = {PipeOperandRef::INPUT, size_t(std::strtoull(tok.c_str() + 2, &end, 10)), 0.0};
            return end != tok.c_str() + 2 && *end == '\0';
        }
        if (tok[0] == '%') {
            out = {PipeOperandRef::RESULT, size_t(std::strtoull(tok.c_str() + 1, &end, 10)), 0.0};
            return end != tok.c_str() + 1 && *end == '\0';
        }
        if (tok[0] == '#') {
            out = {PipeOperandRef::CONSTANT, 0, std::strtod(tok.c_str() + 1, &end)};
            return end != tok.c_str() + 1 && *end == '\0';
        }
        return false;
    }
    static bool parseOperandList(const std::string &list, std::vector<PipeOperandRef> &out) {
        std::stringstream ss(list);
        std::string tok;
        while (std::getline(ss, tok, ',')) {
            PipeOperandRef ref{};
            if (!parseOperand(trim(tok), ref))
                return false;
            out.push_back(ref);
        }
        return !out.empty();
    }

  public:
    // The text form of a body (see the head of this file) as an operator list. False if a line does not parse.
    static bool parse(const std::string &text, PipeBodyDesc &body, std::string *why = nullptr) {
        body = PipeBodyDesc{};
        std::stringstream ss(text);
        std::string line;
        bool returned = false;
        while (std::getline(ss, line)) {
            line = trim(line);
            if (line.empty())
                continue;
            if (returned)
                return fail(why, "text after the return line");
            if (line.compare(0, 7, "return ") == 0) {
                if (!parseOperandList(line.substr(7), body.results))
                    return fail(why, "cannot parse `" + line + "`");
                returned = true;
                continue;
            }
            const size_t eq = line.find('=');
            if (line[0] != '%' || eq == std::string::npos)
                return fail(why, "cannot parse `" + line + "`");
            char *end = nullptr;
            const size_t number = size_t(std::strtoull(line.c_str() + 1, &end, 10));
            if (number != body.ops.size())
                return fail(why, "line `" + line + "` is out of order");
            const std::string rhs = trim(line.substr(eq + 1));
            const size_t sp = rhs.find(' ');
            PipeOpDesc op;
            op.mnemonic = rhs.substr(0, sp);
            if (sp == std::string::npos || !parseOperandList(rhs.substr(sp + 1), op.operands))
                return fail(why, "cannot parse `" + line + "`");
            body.ops.push_back(op);
        }
        if (!returned)
            return fail(why, "the body returns nothing");
        return true;
    }

    // The instruction list and the bindings for `body` on inputs of these shapes, with its results combined as
    // `combines` says. False (and the reason in *why) if the body does not fit the kernel.
    static bool build(const PipeBodyDesc &body, const std::vector<PipeInputShape> &inputs, const std::vector<VectorCombine> &combines,
                      PipeProgram &out, std::string *why = nullptr) {
        out = PipeProgram{};
        // `cast` stands for its operand: replace every use of such a line by what the line refers to
        PipeBodyDesc resolved = body;
        {
            std::vector<PipeOperandRef> standsFor(resolved.ops.size());
            std::vector<bool> isAlias(resolved.ops.size(), false);
            auto follow = [&](PipeOperandRef &ref) {
                while (ref.kind == PipeOperandRef::RESULT && ref.index < isAlias.size() && isAlias[ref.index])
                    ref = standsFor[ref.index];
            };
            for (size_t n = 0; n < resolved.ops.size(); n++) {
                for (PipeOperandRef &ref : resolved.ops[n].operands) {
                    if (ref.kind == PipeOperandRef::RESULT && ref.index >= n)
                        return fail(why, "operator " + std::to_string(n) + " uses a value that is defined later");
                    follow(ref);
                }
                if (resolved.ops[n].mnemonic == "cast") {
                    if (resolved.ops[n].operands.size() != 1)
                        return fail(why, "cast takes one operand");
                    isAlias[n] = true;
                    standsFor[n] = resolved.ops[n].operands[0];
                }
            }
            for (PipeOperandRef &ref : resolved.results) {
                if (ref.kind == PipeOperandRef::RESULT && ref.index >= resolved.ops.size())
                    return fail(why, "the body returns a value that no line defines");
                follow(ref);
            }
        }
        return buildResolved(resolved, inputs, combines, out, why);
    }

  private:
    static bool buildResolved(const PipeBodyDesc &body, const std::vector<PipeInputShape> &inputs,
                              const std::vector<VectorCombine> &combines, PipeProgram &out, std::string *why) {
        if (body.results.size() != combines.size())
            return fail(why, "the body returns " + std::to_string(body.results.size()) + " values for " +
                                 std::to_string(combines.size()) + " pipeline outputs");
        const size_t NONE = size_t(-1);
        // what the machine holds: the operator whose result is in t / in r (NONE: nothing yet; t may hold the primary input)
        size_t in_t = NONE, in_r = NONE, primary = NONE;
        bool t_is_primary = false;
        size_t tileCols = 0;
        int nMatrix = 0, nRowvec = 0, nColvec = 0, nTileOut = 0, nRowOut = 0, nAllOut = 0;
        out.inputs.assign(inputs.size(), PipeInputBinding{PipeInput::SCALAR, -1});
        std::vector<bool> bound(inputs.size(), false);
        out.outputs.assign(body.results.size(), PipeOutputBinding{PipeOutput::TILE, -1});
        enum Kind { K_TILE, K_ROW, K_ALL };
        std::vector<Kind> kindOf(body.ops.size(), K_TILE);

        auto isTileInput = [&](size_t i) {
            return i < inputs.size() && !inputs[i].isScalar && inputs[i].split == VectorSplit::ROWS && inputs[i].rows > 1;
        };
        auto makePrimary = [&](size_t i) {
            primary = i;
            tileCols = inputs[i].cols;
            out.inputs[i] = {PipeInput::PRIMARY, 0};
            bound[i] = true;
            t_is_primary = true;
        };
        auto emit = [&](int kind, int op, int domain, int operand, int index, int swap, double scalar) {
            out.program.push_back(dh_pipe_instr{kind, op, domain, operand, index, swap, scalar});
            return int(out.program.size()) - 1;
        };
        // stores the result of operator `n` if the pipeline returns it
        auto storeIfReturned = [&](size_t n, std::string &err) {
            for (size_t o = 0; o < body.results.size(); o++) {
                const PipeOperandRef &r = body.results[o];
                if (r.kind != PipeOperandRef::RESULT || r.index != n)
                    continue;
                if (out.outputs[o].slot >= 0) // the same value returned twice shares nothing: each output has its own matrix
                    continue;
                if (kindOf[n] == K_ALL)
                    continue; // bound where the reduction is emitted
                if (combines[o] != VectorCombine::ROWS) {
                    err = "output " + std::to_string(o) + " is made row by row but is not combined by ROWS";
                    return false;
                }
                const bool tile = kindOf[n] == K_TILE;
                int &count = tile ? nTileOut : nRowOut;
                if (count >= DH_PIPE_MAX_OPERANDS) {
                    err = "more than " + std::to_string(DH_PIPE_MAX_OPERANDS) + " outputs of one kind";
                    return false;
                }
                out.outputs[o] = {tile ? PipeOutput::TILE : PipeOutput::ROW, count};
                emit(tile ? DH_PIPE_STORE_TILE : DH_PIPE_STORE_ROW, 0, tile ? 0 : 1, 0, count, 0, 0.0);
                count++;
            }
            return true;
        };
        // is `ref` the value that is in t (domain 0) / in r (domain 1) right now?
        auto isCurrent = [&](const PipeOperandRef &ref, int domain) {
            if (domain == 0) {
                if (ref.kind == PipeOperandRef::INPUT)
                    return t_is_primary && ref.index == primary;
                return ref.kind == PipeOperandRef::RESULT && !t_is_primary && ref.index == in_t;
            }
            return ref.kind == PipeOperandRef::RESULT && ref.index == in_r;
        };

        for (size_t n = 0; n < body.ops.size(); n++) {
            const PipeOpDesc &op = body.ops[n];
            if (op.mnemonic == "cast")
                continue; // every use of it was replaced by its operand
            for (const PipeOperandRef &ref : op.operands) {
                if (ref.kind == PipeOperandRef::RESULT && ref.index >= n)
                    return fail(why, "operator " + std::to_string(n) + " uses a value that is defined later");
                if (ref.kind == PipeOperandRef::INPUT && ref.index >= inputs.size())
                    return fail(why, "operator " + std::to_string(n) + " uses input " + std::to_string(ref.index) + " of " +
                                         std::to_string(inputs.size()));
                if (ref.kind == PipeOperandRef::RESULT && kindOf[ref.index] == K_ALL)
                    return fail(why, "operator " + std::to_string(n) + " uses the result of a full aggregation");
            }
            int code = 0;
            FullAgg fa{};
            std::string err;
            if (lookup(binaryOps(), op.mnemonic, code)) {
                if (op.operands.size() != 2)
                    return fail(why, op.mnemonic + " takes two operands");
                // the domain: whichever of t and r one of the operands is in; the first tile operator picks the primary
                int domain = -1, cur = -1;
                for (int k = 0; k < 2 && domain < 0; k++)
                    for (int d = 0; d < 2 && domain < 0; d++)
                        if (isCurrent(op.operands[k], d)) {
                            // r as an operand of a tile operator is ROWREG: prefer the tile domain if the other one is in t
                            if (d == 1 && isCurrent(op.operands[1 - k], 0))
                                continue;
                            domain = d;
                            cur = k;
                        }
                if (domain < 0 && primary == NONE)
                    for (int k = 0; k < 2 && domain < 0; k++)
                        if (op.operands[k].kind == PipeOperandRef::INPUT && isTileInput(op.operands[k].index) &&
                            (inputs[op.operands[k].index].cols > 1 ||
                             !(op.operands[1 - k].kind == PipeOperandRef::INPUT && isTileInput(op.operands[1 - k].index)))) {
                            makePrimary(op.operands[k].index);
                            domain = 0;
                            cur = k;
                        }
                if (domain < 0 && primary == NONE)
                    for (int k = 0; k < 2 && domain < 0; k++)
                        if (op.operands[k].kind == PipeOperandRef::INPUT && isTileInput(op.operands[k].index)) {
                            makePrimary(op.operands[k].index);
                            domain = 0;
                            cur = k;
                        }
                if (domain < 0)
                    return fail(why, "operator " + std::to_string(n) + " (" + op.mnemonic + ") takes neither the current tile nor the current row value");
                const PipeOperandRef &other = op.operands[1 - cur];
                int operand = DH_OPD_SCALAR, index = 0;
                double scalar = 0.0;
                size_t scalarInput = NONE;
                if (isCurrent(other, domain))
                    operand = DH_OPD_SELF;
                else if (other.kind == PipeOperandRef::CONSTANT)
                    scalar = other.constant;
                else if (other.kind == PipeOperandRef::RESULT) {
                    if (domain == 0 && isCurrent(other, 1))
                        operand = DH_OPD_ROWREG;
                    else
                        return fail(why, "operator " + std::to_string(n) + " (" + op.mnemonic + ") uses %" + std::to_string(other.index) +
                                             ", which is no longer held (one tile and one row value at a time)");
                } else {
                    const size_t i = other.index;
                    const PipeInputShape &s = inputs[i];
                    if (s.isScalar)
                        scalarInput = i;
                    else {
                        PipeInput role;
                        if (isTileInput(i) && s.cols == tileCols && domain == 0)
                            role = PipeInput::MATRIX;
                        else if (isTileInput(i) && s.cols == 1)
                            role = PipeInput::COLVEC;
                        else if (s.rows == 1 && s.cols == tileCols && domain == 0 && !isTileInput(i))
                            role = PipeInput::ROWVEC;
                        else
                            return fail(why, "input " + std::to_string(i) + " (" + std::to_string(s.rows) + "x" + std::to_string(s.cols) +
                                                 ") is neither a row-split matrix / column nor a broadcast row of the tile's width");
                        if (bound[i] && out.inputs[i].role != role)
                            return fail(why, "input " + std::to_string(i) + " is used in two roles");
                        if (!bound[i]) {
                            int &count = role == PipeInput::MATRIX ? nMatrix : role == PipeInput::COLVEC ? nColvec : nRowvec;
                            if (count >= DH_PIPE_MAX_OPERANDS)
                                return fail(why, "more than " + std::to_string(DH_PIPE_MAX_OPERANDS) + " operands of one kind");
                            out.inputs[i] = {role, count++};
                            bound[i] = true;
                        }
                        operand = role == PipeInput::MATRIX ? DH_OPD_MATRIX : role == PipeInput::COLVEC ? DH_OPD_COLVEC : DH_OPD_ROWVEC;
                        index = out.inputs[i].slot;
                    }
                }
                const int at = emit(DH_PIPE_EW_BINARY, code, domain, operand, index, cur == 1 ? 1 : 0, scalar);
                if (scalarInput != NONE) {
                    out.inputs[scalarInput].role = PipeInput::SCALAR;
                    out.inputs[scalarInput].instrs.push_back(at);
                    bound[scalarInput] = true;
                }
                kindOf[n] = domain == 0 ? K_TILE : K_ROW;
                if (domain == 0) {
                    in_t = n;
                    t_is_primary = false;
                } else
                    in_r = n;
            } else if (lookup(unaryOps(), op.mnemonic, code)) {
                if (op.operands.size() != 1)
                    return fail(why, op.mnemonic + " takes one operand");
                int domain = isCurrent(op.operands[0], 0) ? 0 : isCurrent(op.operands[0], 1) ? 1 : -1;
                if (domain < 0 && primary == NONE && op.operands[0].kind == PipeOperandRef::INPUT && isTileInput(op.operands[0].index)) {
                    makePrimary(op.operands[0].index);
                    domain = 0;
                }
                if (domain < 0)
                    return fail(why, "operator " + std::to_string(n) + " (" + op.mnemonic + ") takes neither the current tile nor the current row value");
                emit(DH_PIPE_EW_UNARY, code, domain, 0, 0, 0, 0.0);
                kindOf[n] = domain == 0 ? K_TILE : K_ROW;
                if (domain == 0) {
                    in_t = n;
                    t_is_primary = false;
                } else
                    in_r = n;
            } else if (lookup(rowAggs(), op.mnemonic, code)) {
                if (op.operands.size() != 1)
                    return fail(why, op.mnemonic + " takes one operand");
                if (!isCurrent(op.operands[0], 0)) {
                    if (primary == NONE && op.operands[0].kind == PipeOperandRef::INPUT && isTileInput(op.operands[0].index))
                        makePrimary(op.operands[0].index);
                    else
                        return fail(why, "operator " + std::to_string(n) + " (" + op.mnemonic + ") does not aggregate the current tile");
                }
                emit(DH_PIPE_ROW_AGG, code, 0, 0, 0, 0, 0.0);
                kindOf[n] = K_ROW;
                in_r = n; // t keeps its value
            } else if (fullAgg(op.mnemonic, fa)) {
                if (op.operands.size() != 1)
                    return fail(why, op.mnemonic + " takes one operand");
                int domain = isCurrent(op.operands[0], 1) ? 1 : isCurrent(op.operands[0], 0) ? 0 : -1;
                if (domain < 0 && primary == NONE && op.operands[0].kind == PipeOperandRef::INPUT && isTileInput(op.operands[0].index)) {
                    makePrimary(op.operands[0].index);
                    domain = 0;
                }
                if (domain < 0)
                    return fail(why, "operator " + std::to_string(n) + " (" + op.mnemonic + ") reduces neither the current tile nor the current row value");
                kindOf[n] = K_ALL;
                bool returned = false;
                for (size_t o = 0; o < body.results.size(); o++) {
                    const PipeOperandRef &r = body.results[o];
                    if (r.kind != PipeOperandRef::RESULT || r.index != n)
                        continue;
                    if (returned)
                        return fail(why, "a full aggregation is returned twice");
                    if (combines[o] != fa.combine)
                        return fail(why, "output " + std::to_string(o) + " (" + op.mnemonic + ") is not combined the way it is reduced");
                    if (nAllOut >= 2)
                        return fail(why, "more than two full aggregations");
                    out.outputs[o] = {PipeOutput::ALL, nAllOut};
                    emit(DH_PIPE_REDUCE_ALL, fa.op, domain, 0, nAllOut, 0, 0.0);
                    nAllOut++;
                    returned = true;
                }
                if (!returned)
                    return fail(why, "the result of " + op.mnemonic + " is not an output of the pipeline");
            } else
                return fail(why, "operator `" + op.mnemonic + "` has no instruction in the fused kernel");
            if (!storeIfReturned(n, err))
                return fail(why, err);
            if (out.program.size() > DH_PIPE_MAX_INSTR)
                return fail(why, "more than " + std::to_string(DH_PIPE_MAX_INSTR) + " instructions");
        }
        if (primary == NONE)
            return fail(why, "no operator works on a row-split input");
        for (size_t o = 0; o < out.outputs.size(); o++)
            if (out.outputs[o].slot < 0)
                return fail(why, "output " + std::to_string(o) + " is not the result of an operator of the body");
        for (size_t i = 0; i < inputs.size(); i++)
            if (!bound[i])
                return fail(why, "input " + std::to_string(i) + " is not used by the body");
        return true;
    }
};

} // namespace HIP
