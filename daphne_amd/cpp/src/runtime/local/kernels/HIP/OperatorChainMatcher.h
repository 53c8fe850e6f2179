// OperatorChainMatcher: which chains of DaphneIR operators one kernel of FusedOperators.h can stand for.
//
// The reference's compiler turns every operator into one kernel call
// (src/compiler/lowering/RewriteToCallKernelOpPass.cpp:360-455). Four chains that its scripts and DNN builtins produce
// have a single kernel in libdaphne_hip.so instead; this file recognises them on a description of the operators that
// has nothing of MLIR in it - mnemonics (DaphneOps.td), operand and result value numbers, the constants and shapes
// that are known - so that it is compiled and tested with the rest of the kernel layer. The compiler pass
// src/compiler/lowering/FuseHIPOperatorChainsPass.cpp fills such a description from a function body, calls match() and
// rewrites what it returns.
//
//   CONV_RELU_POOL     Convolution_Forward -> NN_Relu_Forward -> NN_Max_Forward with a 2 x 2 window, stride 2, no
//                      padding, on the convolution's own output extents; either follower may be missing (not both)
//                      (scripts: conv2d(...), relu(...), max_pool2d(...), DaphneDSLBuiltins.cpp:883-896)
//   AFFINE_RELU        NN_Affine_Forward -> NN_Relu_Forward
//   NORMAL_EQUATIONS   syrk(X, transLeft) and matMul(t(X), y) with a one-column y, in either order
//                      (scripts/algorithms/lmDS_.daph:100-101 after the t(X) @ X -> syrk rewrite)
//   KMEANS_ASSIGN      idxminRow of (matMul(X, t(C)) * -2 + xx) + cc, written with ewMul / ewAdd / ewSub in any of the
//                      forms that round the same way (x * -2 + a, a - x * 2, operands of ewAdd / ewMul in either order)
//   KMEANS_STEP        KMEANS_ASSIGN whose labels go on (possibly through a cast) into oneHot(idx, info) -> P,
//                      matMul(t(P), X) / t(sumCol(P)) over the same X: a whole Lloyd iteration, labels and new centroids from
//                      one pass over X. The labels may have other users (the kernel returns them); P may not.
// An intermediate value must have no other user, or the chain's kernel could not leave it out.
#pragma once

#include <cstddef>
#include <map>
#include <string>
#include <utility>
#include <vector>

namespace HIP {

struct ChainOp {
    std::string mnemonic;      // as in DaphneOps.td: "Convolution_Forward", "ewAdd", "matMul", ...
    std::vector<int> operands; // value numbers
    std::vector<int> results;  // value numbers
};
struct ChainGraph {
    std::vector<ChainOp> ops;                      // in program order
    std::map<int, double> constants;               // values known at compile time (sizes, flags as 0 / 1, scalars)
    std::map<int, std::pair<long, long>> shapes;   // rows, cols where known (-1: unknown)
    std::vector<int> escaping;                     // values used outside the described operators (returned, stored, ...)
};

enum class ChainKind { CONV_RELU_POOL, AFFINE_RELU, NORMAL_EQUATIONS, KMEANS_ASSIGN, KMEANS_STEP };

struct ChainMatch {
    ChainKind kind;
    std::vector<size_t> ops;         // the operators the kernel stands for, in program order
    std::map<std::string, int> args; // the kernel's arguments by name -> value numbers
    std::vector<int> results;        // the values the kernel produces, in the kernel's result order
    size_t epilogue = 0;             // CONV_RELU_POOL / AFFINE_RELU: bit 0 rectifier, bit 1 pooling
};

class OperatorChainMatcher {
    const ChainGraph &g;
    std::map<int, std::vector<size_t>> users; // value -> operators that take it
    std::map<int, size_t> producer;           // value -> operator that makes it
    std::vector<bool> taken;

    explicit OperatorChainMatcher(const ChainGraph &graph) : g(graph), taken(graph.ops.size(), false) {
        for (size_t i = 0; i < g.ops.size(); i++) {
            for (int v : g.ops[i].operands)
                users[v].push_back(i);
            for (int v : g.ops[i].results)
                producer[v] = i;
        }
    }
    bool escapes(int v) const {
        for (int e : g.escaping)
            if (e == v)
                return true;
        return false;
    }
    // the one operator that uses v, if v has exactly one use and does not escape
    bool soleUser(int v, size_t &op) const {
        auto it = users.find(v);
        if (it == users.end() || it->second.size() != 1 || escapes(v))
            return false;
        op = it->second[0];
        return !taken[op];
    }
    bool unused(int v) const { return users.find(v) == users.end() && !escapes(v); }
    bool constantIs(int v, double want) const {
        auto it = g.constants.find(v);
        return it != g.constants.end() && it->second == want;
    }
    bool producedBy(int v, const char *mnemonic, size_t &op) const {
        auto it = producer.find(v);
        if (it == producer.end() || taken[it->second] || g.ops[it->second].mnemonic != mnemonic)
            return false;
        op = it->second;
        return true;
    }
    bool isOp(size_t i, const char *mnemonic, size_t numOperands) const {
        return g.ops[i].mnemonic == mnemonic && g.ops[i].operands.size() == numOperands;
    }
    long rowsOf(int v) const {
        auto it = g.shapes.find(v);
        return it == g.shapes.end() ? -1 : it->second.first;
    }
    long colsOf(int v) const {
        auto it = g.shapes.find(v);
        return it == g.shapes.end() ? -1 : it->second.second;
    }
    void take(const ChainMatch &m) {
        for (size_t i : m.ops)
            taken[i] = true;
    }
    static void sortOps(ChainMatch &m) {
        for (size_t a = 0; a < m.ops.size(); a++)
            for (size_t b = a + 1; b < m.ops.size(); b++)
                if (m.ops[b] < m.ops[a])
                    std::swap(m.ops[a], m.ops[b]);
    }

    // Convolution_Forward(input, filter, bias, N, C, H, W, Hf, Wf, sh, sw, ph, pw) -> (out, P, Q)
    bool matchConv(size_t i, ChainMatch &m) const {
        if (!isOp(i, "Convolution_Forward", 13) || g.ops[i].results.size() != 3)
            return false;
        const ChainOp &conv = g.ops[i];
        m = ChainMatch{ChainKind::CONV_RELU_POOL, {i}, {}, conv.results, 0};
        static const char *names[] = {"data", "filter", "bias", "batch_size", "num_channels", "img_h", "img_w",
                                      "filter_h", "filter_w", "stride_h", "stride_w", "pad_h", "pad_w"};
        for (size_t k = 0; k < 13; k++)
            m.args[names[k]] = conv.operands[k];
        int cur = conv.results[0];
        size_t next;
        if (soleUser(cur, next) && isOp(next, "NN_Relu_Forward", 1) && g.ops[next].results.size() == 1) {
            m.ops.push_back(next);
            m.epilogue |= 1;
            cur = g.ops[next].results[0];
        }
        // NN_Max_Forward(input, N, C, H, W, ph, pw, sh, sw, padh, padw) -> (out, h, w): on the convolution's extents
        if (soleUser(cur, next) && isOp(next, "NN_Max_Forward", 11) && g.ops[next].results.size() == 3) {
            const ChainOp &pool = g.ops[next];
            const bool window = constantIs(pool.operands[5], 2) && constantIs(pool.operands[6], 2) && constantIs(pool.operands[7], 2) &&
                                constantIs(pool.operands[8], 2) && constantIs(pool.operands[9], 0) && constantIs(pool.operands[10], 0);
            // its extents are the convolution's results: nobody else may need those once the pooled ones replace them
            const bool extents = pool.operands[3] == conv.results[1] && pool.operands[4] == conv.results[2] &&
                                 users.at(conv.results[1]).size() == 1 && users.at(conv.results[2]).size() == 1 &&
                                 !escapes(conv.results[1]) && !escapes(conv.results[2]);
            if (window && extents) {
                m.ops.push_back(next);
                m.epilogue |= 2;
                m.results = pool.results;
                cur = pool.results[0];
            }
        }
        m.results[0] = cur;
        return m.epilogue != 0;
    }

    // NN_Affine_Forward(data, weights, bias) -> out, NN_Relu_Forward(out)
    bool matchAffine(size_t i, ChainMatch &m) const {
        if (!isOp(i, "NN_Affine_Forward", 3) || g.ops[i].results.size() != 1)
            return false;
        size_t next;
        if (!(soleUser(g.ops[i].results[0], next) && isOp(next, "NN_Relu_Forward", 1) && g.ops[next].results.size() == 1))
            return false;
        m = ChainMatch{ChainKind::AFFINE_RELU, {i, next}, {}, {g.ops[next].results[0]}, 1};
        m.args = {{"data", g.ops[i].operands[0]}, {"weights", g.ops[i].operands[1]}, {"bias", g.ops[i].operands[2]}};
        return true;
    }

    // is `v` t(X) for this X, as the left operand of a matMul whose transa operand is `transa`?
    bool isTransposeOf(int v, int transa, int X, std::vector<size_t> &extraOps) const {
        if (v == X && constantIs(transa, 1))
            return true;
        size_t t;
        if (constantIs(transa, 0) && producedBy(v, "transpose", t) && g.ops[t].operands.size() == 1 && g.ops[t].operands[0] == X) {
            size_t only;
            if (soleUser(v, only)) // the transposed copy is not needed any more
                extraOps.push_back(t);
            return true;
        }
        return false;
    }
    // syrk(X, transLeft = true) -> A; matMul(t(X), y, ...) -> b with y of one column
    bool matchNormalEquations(size_t i, ChainMatch &m) const {
        if (!isOp(i, "syrk", 2) || !constantIs(g.ops[i].operands[1], 1) || g.ops[i].results.size() != 1)
            return false;
        const int X = g.ops[i].operands[0];
        for (size_t j = 0; j < g.ops.size(); j++) {
            if (taken[j] || !isOp(j, "matMul", 4) || g.ops[j].results.size() != 1 || !constantIs(g.ops[j].operands[3], 0))
                continue;
            const int y = g.ops[j].operands[1];
            if (colsOf(y) != 1)
                continue;
            std::vector<size_t> extra;
            if (!isTransposeOf(g.ops[j].operands[0], g.ops[j].operands[2], X, extra))
                continue;
            // the kernel is placed where the later of the two stands: what the earlier one makes must not be needed in between
            const size_t first = i < j ? i : j, last = i < j ? j : i;
            bool usedBetween = false;
            for (size_t k = first + 1; k < last && !usedBetween; k++)
                for (int v : g.ops[k].operands)
                    usedBetween |= v == g.ops[first].results[0];
            if (usedBetween)
                continue;
            m = ChainMatch{ChainKind::NORMAL_EQUATIONS, {i, j}, {{"X", X}, {"y", y}}, {g.ops[i].results[0], g.ops[j].results[0]}, 0};
            for (size_t t : extra)
                m.ops.push_back(t);
            sortOps(m);
            return true;
        }
        return false;
    }

    // v = x * s (ewMul with a constant, either order); returns x and s
    bool isScaled(int v, int &x, double &s, size_t &op) const {
        if (!producedBy(v, "ewMul", op) || g.ops[op].operands.size() != 2)
            return false;
        for (int k = 0; k < 2; k++) {
            auto c = g.constants.find(g.ops[op].operands[k]);
            if (c != g.constants.end()) {
                x = g.ops[op].operands[1 - k];
                s = c->second;
                return true;
            }
        }
        return false;
    }
    // idxminRow(D), D = (M * -2 + xx) + cc in one of its equally rounded spellings, M = matMul(X, t(C))
    bool matchKmeansAssign(size_t i, ChainMatch &m) const {
        if (!isOp(i, "idxminRow", 1) || g.ops[i].results.size() != 1)
            return false;
        size_t outer;
        if (!producedBy(g.ops[i].operands[0], "ewAdd", outer) || g.ops[outer].operands.size() != 2)
            return false;
        size_t only;
        if (!soleUser(g.ops[outer].results[0], only))
            return false;
        for (int k = 0; k < 2; k++) {
            // outer = inner + cc (either order), cc a row of k values
            const int cc = g.ops[outer].operands[k], innerV = g.ops[outer].operands[1 - k];
            if (rowsOf(cc) != 1)
                continue;
            size_t inner;
            if (!soleUser(innerV, only) || only != outer)
                continue;
            int xx = -1, scaledV = -1;
            double want = 0;
            if (producedBy(innerV, "ewAdd", inner) && g.ops[inner].operands.size() == 2) { // x * -2 + xx, either order
                for (int q = 0; q < 2; q++)
                    if (colsOf(g.ops[inner].operands[q]) == 1 && rowsOf(g.ops[inner].operands[q]) != 1) {
                        xx = g.ops[inner].operands[q];
                        scaledV = g.ops[inner].operands[1 - q];
                    }
                want = -2;
            } else if (producedBy(innerV, "ewSub", inner) && g.ops[inner].operands.size() == 2) { // xx - x * 2
                if (colsOf(g.ops[inner].operands[0]) == 1 && rowsOf(g.ops[inner].operands[0]) != 1) {
                    xx = g.ops[inner].operands[0];
                    scaledV = g.ops[inner].operands[1];
                }
                want = 2;
            }
            if (xx < 0)
                continue;
            int prod = -1;
            double s = 0;
            size_t mul, mm;
            if (!isScaled(scaledV, prod, s, mul) || s != want || !soleUser(scaledV, only) || only != inner)
                continue;
            if (!producedBy(prod, "matMul", mm) || g.ops[mm].operands.size() != 4 || !soleUser(prod, only) || only != mul)
                continue;
            if (!constantIs(g.ops[mm].operands[2], 0)) // X is not transposed
                continue;
            const int X = g.ops[mm].operands[0];
            int C = -1;
            std::vector<size_t> extra;
            size_t t;
            if (constantIs(g.ops[mm].operands[3], 1))
                C = g.ops[mm].operands[1];
            else if (constantIs(g.ops[mm].operands[3], 0) && producedBy(g.ops[mm].operands[1], "transpose", t) &&
                     g.ops[t].operands.size() == 1) {
                C = g.ops[t].operands[0];
                if (soleUser(g.ops[mm].operands[1], only))
                    extra.push_back(t);
            }
            if (C < 0)
                continue;
            m = ChainMatch{ChainKind::KMEANS_ASSIGN, {mm, mul, inner, outer, i}, {{"X", X}, {"C", C}, {"xx", xx}, {"cc", cc}},
                           {g.ops[i].results[0]}, 0};
            for (size_t e : extra)
                m.ops.push_back(e);
            sortOps(m);
            return true;
        }
        return false;
    }

    // m: a KMEANS_ASSIGN match. If the labels are one-hot encoded and the encoding is only used for the cluster means
    // of the same X - oneHot(idx, info) -> P, matMul(t(P), X) -> S, sumCol(P) -> n, S / t(n) - the match becomes
    // KMEANS_STEP with the results (idx, C_new, n). The labels come from an arg-min over C's rows, so they are valid
    // positions of the encoding whenever P is as wide as C has rows - which the shapes must show.
    bool extendToKmeansStep(ChainMatch &m) const {
        const int idx = m.results[0], X = m.args.at("X"), C = m.args.at("C");
        auto iu = users.find(idx);
        if (iu == users.end() || colsOf(idx) != 1)
            return false;
        for (size_t u : iu->second) {
            std::vector<size_t> chain;
            size_t oh = u;
            int labels = idx;
            size_t next;
            if (!taken[u] && isOp(u, "cast", 1) && g.ops[u].results.size() == 1 && soleUser(g.ops[u].results[0], next)) {
                chain.push_back(u);
                labels = g.ops[u].results[0];
                oh = next;
            }
            if (taken[oh] || !isOp(oh, "oneHot", 2) || g.ops[oh].operands[0] != labels || g.ops[oh].results.size() != 1)
                continue;
            const int P = g.ops[oh].results[0];
            auto pu = users.find(P);
            if (escapes(P) || pu == users.end() || pu->second.size() != 2 || colsOf(P) < 1 || colsOf(P) != rowsOf(C))
                continue;
            bool haveMm = false, haveSc = false;
            size_t mm = 0, sc = 0;
            std::vector<size_t> extra;
            for (size_t q : pu->second) {
                if (taken[q])
                    continue;
                const ChainOp &o = g.ops[q];
                if (isOp(q, "sumCol", 1) && o.results.size() == 1) {
                    sc = q;
                    haveSc = true;
                } else if (isOp(q, "matMul", 4) && o.results.size() == 1 && o.operands[0] == P && o.operands[1] == X &&
                           constantIs(o.operands[2], 1) && constantIs(o.operands[3], 0)) {
                    mm = q;
                    haveMm = true;
                } else if (isOp(q, "transpose", 1) && o.results.size() == 1 && soleUser(o.results[0], next) && isOp(next, "matMul", 4) &&
                           g.ops[next].results.size() == 1 && g.ops[next].operands[0] == o.results[0] && g.ops[next].operands[1] == X &&
                           constantIs(g.ops[next].operands[2], 0) && constantIs(g.ops[next].operands[3], 0)) {
                    mm = next;
                    haveMm = true;
                    extra.push_back(q);
                }
            }
            if (!haveMm || !haveSc)
                continue;
            const int S = g.ops[mm].results[0], n = g.ops[sc].results[0];
            size_t tn, dv, only;
            if (!soleUser(n, tn) || !isOp(tn, "transpose", 1) || g.ops[tn].results.size() != 1)
                continue;
            const int nT = g.ops[tn].results[0];
            if (!soleUser(nT, dv) || !isOp(dv, "ewDiv", 2) || g.ops[dv].results.size() != 1 || g.ops[dv].operands[0] != S ||
                g.ops[dv].operands[1] != nT || !soleUser(S, only) || only != dv)
                continue;
            m.kind = ChainKind::KMEANS_STEP;
            for (size_t o : chain)
                m.ops.push_back(o);
            for (size_t o : {oh, sc, mm, tn, dv})
                m.ops.push_back(o);
            for (size_t o : extra)
                m.ops.push_back(o);
            m.results = {idx, g.ops[dv].results[0], n};
            sortOps(m);
            return true;
        }
        return false;
    }

  public:
    // Every chain found, each operator in at most one of them.
    static std::vector<ChainMatch> match(const ChainGraph &graph) {
        OperatorChainMatcher self(graph);
        std::vector<ChainMatch> found;
        for (size_t i = 0; i < graph.ops.size(); i++) {
            if (self.taken[i])
                continue;
            ChainMatch m;
            if (self.matchConv(i, m) || self.matchAffine(i, m) || self.matchNormalEquations(i, m) || self.matchKmeansAssign(i, m)) {
                if (m.kind == ChainKind::KMEANS_ASSIGN)
                    self.extendToKmeansStep(m);
                self.take(m);
                found.push_back(m);
            }
        }
        return found;
    }
};

} // namespace HIP
