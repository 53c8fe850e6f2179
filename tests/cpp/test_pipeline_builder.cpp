// Host-only tests of HIP::PipelineProgramBuilder: the text form of a device body to the instruction list of the fused
// pipeline kernel, or the reason why a body does not fit. No device and no device library involved.
#include <runtime/local/kernels/HIP/PipelineProgramBuilder.h>

#include <cstdio>
#include <string>
#include <vector>

static int g_fail = 0, g_checks = 0;
#define CHECK(cond)                                                                                 \
    do {                                                                                            \
        g_checks++;                                                                                 \
        if (!(cond)) {                                                                              \
            g_fail++;                                                                               \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
        }                                                                                           \
    } while (0)

using namespace HIP;

static bool same(const dh_pipe_instr &a, int kind, int op, int domain, int operand, int index, int swap, double scalar = 0) {
    return a.kind == kind && a.op == op && a.domain == domain && a.operand == operand && a.index == index && a.swap == swap &&
           a.scalar == scalar;
}
static bool buildText(const char *text, const std::vector<PipeInputShape> &in, const std::vector<VectorCombine> &comb, PipeProgram &p,
                      std::string &why) {
    PipeBodyDesc d;
    return PipelineProgramBuilder::parse(text, d, &why) && PipelineProgramBuilder::build(d, in, comb, p, &why);
}

int main() {
    const PipeInputShape X{false, VectorSplit::ROWS, 1000, 64}, rowvec{false, VectorSplit::NONE, 1, 64},
        colvec{false, VectorSplit::ROWS, 1000, 1}, scalar{true, VectorSplit::NONE, 1, 1};
    PipeProgram p;
    std::string why;

    // the z-score body: ((X - mu) / sd)^2 -> rowSums -> r > 64 -> sum; outputs r (ROWS) and the count (ADD)
    const char *zscore = "%0 = ewSub in0, in1\n%1 = ewDiv %0, in2\n%2 = ewMul %1, %1\n%3 = sumRow %2\n%4 = ewGt %3, #64\n%5 = sumAll %4\n"
                         "return %3, %5\n";
    CHECK(buildText(zscore, {X, rowvec, rowvec}, {VectorCombine::ROWS, VectorCombine::ADD}, p, why));
    CHECK(p.program.size() == 7);
    if (p.program.size() == 7) {
        CHECK(same(p.program[0], DH_PIPE_EW_BINARY, int(BinaryOpCode::SUB), 0, DH_OPD_ROWVEC, 0, 0));
        CHECK(same(p.program[1], DH_PIPE_EW_BINARY, int(BinaryOpCode::DIV), 0, DH_OPD_ROWVEC, 1, 0));
        CHECK(same(p.program[2], DH_PIPE_EW_BINARY, int(BinaryOpCode::MUL), 0, DH_OPD_SELF, 0, 0));
        CHECK(same(p.program[3], DH_PIPE_ROW_AGG, int(AggOpCode::SUM), 0, 0, 0, 0));
        CHECK(same(p.program[4], DH_PIPE_STORE_ROW, 0, 1, 0, 0, 0));
        CHECK(same(p.program[5], DH_PIPE_EW_BINARY, int(BinaryOpCode::GT), 1, DH_OPD_SCALAR, 0, 0, 64.0));
        CHECK(same(p.program[6], DH_PIPE_REDUCE_ALL, int(AggOpCode::SUM), 1, 0, 0, 0));
    }
    CHECK(p.inputs.size() == 3 && p.inputs[0].role == PipeInput::PRIMARY && p.inputs[1].role == PipeInput::ROWVEC &&
          p.inputs[1].slot == 0 && p.inputs[2].role == PipeInput::ROWVEC && p.inputs[2].slot == 1);
    CHECK(p.outputs.size() == 2 && p.outputs[0].role == PipeOutput::ROW && p.outputs[0].slot == 0 &&
          p.outputs[1].role == PipeOutput::ALL && p.outputs[1].slot == 0);

    // the threshold as a scalar input of the pipeline: its instruction is remembered, the immediate comes per call
    const char *zscoreThr = "%0 = ewSub in0, in1\n%1 = ewDiv %0, in2\n%2 = ewMul %1, %1\n%3 = sumRow %2\n%4 = ewGt %3, in3\n%5 = sumAll %4\n"
                            "return %3, %5\n";
    CHECK(buildText(zscoreThr, {X, rowvec, rowvec, scalar}, {VectorCombine::ROWS, VectorCombine::ADD}, p, why));
    CHECK(p.inputs.size() == 4 && p.inputs[3].role == PipeInput::SCALAR && p.inputs[3].instrs == std::vector<int>{5});

    // operand on the left: 1 / x, column vector times matrix (the matrix is the tile, the column the operand)
    CHECK(buildText("%0 = ewDiv #1, in0\n%1 = ewMul in1, %0\nreturn %1\n", {X, colvec}, {VectorCombine::ROWS}, p, why));
    CHECK(p.program.size() == 3 && same(p.program[0], DH_PIPE_EW_BINARY, int(BinaryOpCode::DIV), 0, DH_OPD_SCALAR, 0, 1, 1.0) &&
          same(p.program[1], DH_PIPE_EW_BINARY, int(BinaryOpCode::MUL), 0, DH_OPD_COLVEC, 0, 1) &&
          same(p.program[2], DH_PIPE_STORE_TILE, 0, 0, 0, 0, 0));
    CHECK(buildText("%0 = ewMul in0, in1\nreturn %0\n", {colvec, X}, {VectorCombine::ROWS}, p, why));
    CHECK(p.inputs[1].role == PipeInput::PRIMARY && p.inputs[0].role == PipeInput::COLVEC && p.program[0].swap == 1);

    // a tile returned and then overwritten is stored when it is made; the row value broadcast back over the tile
    CHECK(buildText("%0 = ewSub in0, in1\n%1 = maxRow %0\n%2 = ewSub %0, %1\n%3 = ewExp %2\n%4 = sumRow %3\n%5 = ewDiv %3, %4\n"
                    "return %0, %5\n",
                    {X, X}, {VectorCombine::ROWS, VectorCombine::ROWS}, p, why));
    CHECK(p.program.size() == 8 && p.program[1].kind == DH_PIPE_STORE_TILE && p.program[3].operand == DH_OPD_ROWREG &&
          p.program[6].operand == DH_OPD_ROWREG && p.program[7].kind == DH_PIPE_STORE_TILE && p.program[7].index == 1);
    CHECK(p.inputs[1].role == PipeInput::MATRIX);

    // full aggregation of the tile itself, minimum combined by MIN
    CHECK(buildText("%0 = ewAbs in0\n%1 = minAll %0\nreturn %1\n", {X}, {VectorCombine::MIN}, p, why));
    CHECK(p.program.size() == 2 && same(p.program[1], DH_PIPE_REDUCE_ALL, int(AggOpCode::MIN), 0, 0, 0, 0));

    // what does not fit, and why
    CHECK(!buildText("%0 = ewSub in0, in1\n%1 = ewMul %0, %0\n%2 = ewAdd %1, %0\nreturn %2\n", {X, rowvec}, {VectorCombine::ROWS}, p, why));
    CHECK(why.find("no longer held") != std::string::npos);
    CHECK(!buildText("%0 = matMul in0, in1\nreturn %0\n", {X, X}, {VectorCombine::ROWS}, p, why));
    CHECK(why.find("matMul") != std::string::npos);
    CHECK(!buildText("%0 = ewSub in0, in1\nreturn %0\n", {X, rowvec}, {VectorCombine::COLS}, p, why));
    CHECK(why.find("ROWS") != std::string::npos);
    CHECK(!buildText("%0 = sumRow in0\n%1 = sumAll %0\nreturn %1\n", {X}, {VectorCombine::MAX}, p, why));
    CHECK(why.find("combined") != std::string::npos);
    CHECK(!buildText("%0 = ewAdd in0, in1\nreturn %0\n", {X, PipeInputShape{false, VectorSplit::NONE, 1, 7}}, {VectorCombine::ROWS}, p, why));
    CHECK(why.find("input 1") != std::string::npos);
    CHECK(!buildText("%0 = ewAdd in0, in1\nreturn %0\n", {rowvec, rowvec}, {VectorCombine::ROWS}, p, why));
    CHECK(!buildText("%0 = meanAll in0\nreturn %0\n", {X}, {VectorCombine::ADD}, p, why));
    CHECK(!buildText("%0 = ewAdd in0 in1\nreturn %0\n", {X, X}, {VectorCombine::ROWS}, p, why));
    CHECK(!buildText("%1 = ewAdd in0, in1\nreturn %1\n", {X, X}, {VectorCombine::ROWS}, p, why));
    CHECK(!buildText("%0 = ewAdd in0, in1\n", {X, X}, {VectorCombine::ROWS}, p, why));
    {
        std::string text;
        for (int i = 0; i < 17; i++)
            text += "%" + std::to_string(i) + " = ewAdd " + (i ? "%" + std::to_string(i - 1) : std::string("in0")) + ", #1\n";
        text += "return %16\n";
        CHECK(!buildText(text.c_str(), {X}, {VectorCombine::ROWS}, p, why));
        CHECK(why.find("instructions") != std::string::npos);
    }
    std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
