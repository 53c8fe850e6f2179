// Host-only tests of the two lowerings that sit between DaphneIR operators and the multi-operator kernels:
// HIP::PipelineProgramBuilder (the text form of a pipeline's device body to the instruction list of the fused pipeline
// kernel, or the reason why a body does not fit) and HIP::OperatorChainMatcher (which operator chains one kernel of
// FusedOperators.h stands for). No device and no device library involved.
#include <runtime/local/kernels/HIP/OperatorChainMatcher.h>
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

static void run_chain_matcher() {
    // LeNet's second block and its head, as the DSL builtins produce them (values are numbered as they appear):
    //   (v20, v21, v22) = Convolution_Forward(x v1, W v2, b v3, N v4, C v5, H v6, W v7, 5 v8, 5 v9, 1 v10, 1 v11, 2 v12, 2 v13)
    //   v23 = NN_Relu_Forward(v20); (v24, v25, v26) = NN_Max_Forward(v23, v4, v14, v21, v22, 2 v15, 2 v15, 2 v15, 2 v15, 0 v16, 0 v16)
    //   v27 = NN_Affine_Forward(v24, v17, v18); v28 = NN_Relu_Forward(v27); v29 = NN_Affine_Forward(v28, v19, v30); v31 = Softmax(v29)
    ChainGraph g;
    g.ops = {{"Convolution_Forward", {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13}, {20, 21, 22}},
             {"NN_Relu_Forward", {20}, {23}},
             {"NN_Max_Forward", {23, 4, 14, 21, 22, 15, 15, 15, 15, 16, 16}, {24, 25, 26}},
             {"NN_Affine_Forward", {24, 17, 18}, {27}},
             {"NN_Relu_Forward", {27}, {28}},
             {"NN_Affine_Forward", {28, 19, 30}, {29}},
             {"Softmax", {29}, {31}}};
    g.constants = {{8, 5}, {9, 5}, {10, 1}, {11, 1}, {12, 2}, {13, 2}, {15, 2}, {16, 0}};
    g.escaping = {31};
    auto found = OperatorChainMatcher::match(g);
    CHECK(found.size() == 2);
    if (found.size() == 2) {
        CHECK(found[0].kind == ChainKind::CONV_RELU_POOL && found[0].epilogue == 3 && found[0].ops == (std::vector<size_t>{0, 1, 2}));
        CHECK(found[0].results == (std::vector<int>{24, 25, 26}) && found[0].args.at("filter") == 2 && found[0].args.at("pad_w") == 13);
        CHECK(found[1].kind == ChainKind::AFFINE_RELU && found[1].ops == (std::vector<size_t>{3, 4}) && found[1].results == (std::vector<int>{28}));
    }
    // the rectified activations are needed elsewhere: only the rectifier folds into the convolution
    ChainGraph g2 = g;
    g2.escaping.push_back(23);
    found = OperatorChainMatcher::match(g2);
    CHECK(found.size() == 2 && found[0].kind == ChainKind::CONV_RELU_POOL && found[0].epilogue == 1 &&
          found[0].results == (std::vector<int>{23, 21, 22}));
    // a 3 x 3 pooling window does not fold; a convolution with nothing behind it is left alone
    ChainGraph g3 = g;
    g3.constants[15] = 3;
    found = OperatorChainMatcher::match(g3);
    CHECK(found.size() == 2 && found[0].epilogue == 1);
    ChainGraph g4;
    g4.ops = {g.ops[0]};
    g4.escaping = {20};
    CHECK(OperatorChainMatcher::match(g4).empty());

    // lmDS: A = syrk(X); b = t(X) @ y; both spellings of the transposed product
    ChainGraph n;
    n.ops = {{"syrk", {1, 2}, {10}}, {"transpose", {1}, {11}}, {"matMul", {11, 3, 4, 4}, {12}}, {"ewAdd", {10, 5}, {13}}, {"solve", {13, 12}, {14}}};
    n.constants = {{2, 1}, {4, 0}};
    n.shapes = {{1, {100000, 100}}, {3, {100000, 1}}};
    n.escaping = {14};
    found = OperatorChainMatcher::match(n);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::NORMAL_EQUATIONS && found[0].ops == (std::vector<size_t>{0, 1, 2}) &&
          found[0].results == (std::vector<int>{10, 12}) && found[0].args.at("X") == 1 && found[0].args.at("y") == 3);
    n.ops[2] = {"matMul", {1, 3, 2, 4}, {12}}; // transa = true on X itself; the transpose stays (it has no other use, but is not ours)
    found = OperatorChainMatcher::match(n);
    CHECK(found.size() == 1 && found[0].ops == (std::vector<size_t>{0, 2}));
    n.shapes[3] = {100000, 7}; // a right-hand side of seven columns is a matrix product, not t(X) y
    CHECK(OperatorChainMatcher::match(n).empty());

    // k-means: D = (X @ t(C)) * -2 + xx + t(cc'); idx = idxminRow(D)
    ChainGraph k;
    k.ops = {{"transpose", {2}, {10}}, {"matMul", {1, 10, 5, 5}, {11}}, {"ewMul", {11, 6}, {12}}, {"ewAdd", {12, 3}, {13}},
             {"ewAdd", {13, 4}, {14}}, {"idxminRow", {14}, {15}}};
    k.constants = {{5, 0}, {6, -2}};
    k.shapes = {{1, {2000000, 64}}, {2, {16, 64}}, {3, {2000000, 1}}, {4, {1, 16}}};
    k.escaping = {15};
    found = OperatorChainMatcher::match(k);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_ASSIGN && found[0].ops.size() == 6 && found[0].args.at("C") == 2 &&
          found[0].args.at("xx") == 3 && found[0].args.at("cc") == 4 && found[0].results == (std::vector<int>{15}));
    // xx - 2 * (X @ t(C)) + cc rounds the same way; X @ t(C) * 2 + xx + cc does not compute the distances
    ChainGraph k2 = k;
    k2.ops[2] = {"ewMul", {7, 11}, {12}};
    k2.ops[3] = {"ewSub", {3, 12}, {13}};
    k2.ops[4] = {"ewAdd", {4, 13}, {14}};
    k2.constants[7] = 2;
    found = OperatorChainMatcher::match(k2);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_ASSIGN);
    ChainGraph k3 = k;
    k3.constants[6] = 2;
    CHECK(OperatorChainMatcher::match(k3).empty());
    ChainGraph k4 = k; // the distances are printed as well: they have to exist
    k4.escaping.push_back(14);
    CHECK(OperatorChainMatcher::match(k4).empty());

    // the whole Lloyd iteration: P = oneHot(idx, [16]); C' = (t(P) @ X) / t(sum(P, 1)) - labels and centroids from one pass
    ChainGraph s = k;
    s.ops.push_back({"cast", {15}, {16}});
    s.ops.push_back({"oneHot", {16, 8}, {17}});
    s.ops.push_back({"matMul", {17, 1, 9, 5}, {18}}); // transa = 1 (value 9), transb = 0 (value 5)
    s.ops.push_back({"sumCol", {17}, {19}});
    s.ops.push_back({"transpose", {19}, {20}});
    s.ops.push_back({"ewDiv", {18, 20}, {21}});
    s.constants[9] = 1;
    s.shapes[15] = {2000000, 1};
    s.shapes[16] = {2000000, 1};
    s.shapes[17] = {2000000, 16};
    s.escaping = {21};
    found = OperatorChainMatcher::match(s);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_STEP && found[0].ops.size() == 12 &&
          found[0].results == (std::vector<int>{15, 21, 19}) && found[0].args.at("X") == 1 && found[0].args.at("C") == 2);
    ChainGraph s2 = s; // the labels are returned as well: still one kernel, it makes them anyway
    s2.escaping.push_back(15);
    found = OperatorChainMatcher::match(s2);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_STEP);
    ChainGraph s3 = s; // t(P) written out
    s3.ops[8] = {"transpose", {17}, {22}};
    s3.ops.insert(s3.ops.begin() + 9, {"matMul", {22, 1, 5, 5}, {18}});
    found = OperatorChainMatcher::match(s3);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_STEP && found[0].ops.size() == 13);
    ChainGraph s4 = s; // the means of another matrix: the assignment alone is fused
    s4.ops[8] = {"matMul", {17, 30, 9, 5}, {18}};
    found = OperatorChainMatcher::match(s4);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_ASSIGN && found[0].results == (std::vector<int>{15}));
    ChainGraph s5 = s; // the encoding is printed: it has to exist
    s5.escaping.push_back(17);
    found = OperatorChainMatcher::match(s5);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_ASSIGN);
    ChainGraph s6 = s; // an encoding wider than C has rows is not an encoding of these labels
    s6.shapes[17] = {2000000, 20};
    found = OperatorChainMatcher::match(s6);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_ASSIGN);
    ChainGraph s7 = s; // the sums divided by something else than their counts
    s7.ops[11] = {"ewDiv", {18, 31}, {21}};
    found = OperatorChainMatcher::match(s7);
    CHECK(found.size() == 1 && found[0].kind == ChainKind::KMEANS_ASSIGN);
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
    run_chain_matcher();
    std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
