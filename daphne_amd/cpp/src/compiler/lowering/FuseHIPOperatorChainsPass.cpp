// FuseHIPOperatorChainsPass: replaces chains of operators that one kernel of libdaphne_hip.so computes by that kernel.
//
// NOT COMPILED IN THIS REPOSITORY (it needs MLIR and DAPHNE's IR). In DAPHNE this file is
// src/compiler/lowering/FuseHIPOperatorChainsPass.cpp; patches/0013-fuse-hip-operator-chains.patch lists it in
// src/compiler/lowering/CMakeLists.txt, declares it in Passes.h, defines the four operations it creates in
// DaphneOps.td and schedules it in DaphneIrExecutor right after MarkHIPOpsPass, i.e. before
// RewriteToCallKernelOpPass turns every operation into a kernel call
// (src/compiler/lowering/RewriteToCallKernelOpPass.cpp:360-455).
//
// What is a chain is not decided here: every block is written down as a HIP::ChainGraph - mnemonics, value numbers,
// the constants and shapes that are known - and handed to HIP::OperatorChainMatcher
// (src/runtime/local/kernels/HIP/OperatorChainMatcher.h), which is plain C++ and tested with the kernel layer. This
// file only translates: operations marked `hip_device` in (and, as links of a k-means iteration only, the one-hot
// encoding of the labels and a cast in front of it, which have no device kernels of their own), daphne.conv2DForwardFused /
// affineForwardFused / normalEquations / kmeansAssign / kmeansStep out. The new operations carry `hip_device` too, so RewriteToCallKernelOpPass finds
// their kernels in HIPcatalog.json by mnemonic like any other (HIP_conv2DForwardFused__..., kernels/HIP/FusedOperators.h).
#ifdef USE_HIP
#include "ir/daphneir/Daphne.h"
#include "ir/daphneir/Passes.h"

#include <runtime/local/kernels/HIP/OperatorChainMatcher.h>

#include <llvm/ADT/DenseMap.h>

#include <vector>

using namespace mlir;

namespace {

constexpr const char *ATTR_HIP_DEVICE = "hip_device";

struct FuseHIPOperatorChainsPass : public PassWrapper<FuseHIPOperatorChainsPass, OperationPass<func::FuncOp>> {
    void runOnOperation() final {
        std::vector<Block *> blocks;
        getOperation().walk([&](Block *b) { blocks.push_back(b); });
        for (Block *b : blocks)
            fuseBlock(*b);
    }

    static bool numericConstant(Operation &op, double &out) {
        auto c = llvm::dyn_cast<daphne::ConstantOp>(op);
        if (!c)
            return false;
        if (auto f = llvm::dyn_cast<FloatAttr>(c.getValue())) {
            out = f.getValueAsDouble();
            return true;
        }
        if (auto i = llvm::dyn_cast<IntegerAttr>(c.getValue())) {
            out = i.getType().isUnsignedInteger() ? static_cast<double>(i.getValue().getZExtValue())
                                                  : static_cast<double>(i.getValue().getSExtValue());
            return true;
        }
        return false;
    }

    void fuseBlock(Block &block) {
        llvm::DenseMap<Value, int> numberOf;
        std::vector<Value> valueOf;
        auto number = [&](Value v) {
            auto it = numberOf.find(v);
            if (it != numberOf.end())
                return it->second;
            const int n = static_cast<int>(valueOf.size());
            numberOf[v] = n;
            valueOf.push_back(v);
            return n;
        };
        HIP::ChainGraph g;
        std::vector<Operation *> listed;
        auto noteShape = [&](Value v) {
            if (auto mt = llvm::dyn_cast<daphne::MatrixType>(v.getType()))
                g.shapes[number(v)] = {static_cast<long>(mt.getNumRows()), static_cast<long>(mt.getNumCols())};
        };
        for (BlockArgument a : block.getArguments())
            noteShape(a);
        for (Operation &op : block) {
            double c = 0;
            if (op.getNumResults() == 1 && numericConstant(op, c))
                g.constants[number(op.getResult(0))] = c;
            for (Value r : op.getResults())
                noteShape(r);
            const bool isChainOp = llvm::isa<daphne::DaphneDialect>(op.getDialect()) && op.getNumRegions() == 0 &&
                                   (op.hasAttr(ATTR_HIP_DEVICE) || llvm::isa<daphne::OneHotOp, daphne::CastOp>(op));
            if (isChainOp) {
                HIP::ChainOp co;
                co.mnemonic = op.getName().stripDialect().str();
                for (Value v : op.getOperands())
                    co.operands.push_back(number(v));
                for (Value r : op.getResults())
                    co.results.push_back(number(r));
                g.ops.push_back(co);
                listed.push_back(&op);
            } else {
                // whatever this operation (or anything nested in it) reads has to exist: those values escape
                op.walk([&](Operation *inner) {
                    for (Value v : inner->getOperands())
                        g.escaping.push_back(number(v));
                });
            }
        }
        for (const HIP::ChainMatch &m : HIP::OperatorChainMatcher::match(g))
            rewrite(m, listed, valueOf);
    }

    void rewrite(const HIP::ChainMatch &m, const std::vector<Operation *> &listed, std::vector<Value> &valueOf) {
        Operation *last = listed[m.ops.back()];
        // the kernel goes where the chain's last operation stands; every user of what it makes must come after that
        for (int r : m.results)
            for (Operation *user : valueOf[r].getUsers())
                if (user->getBlock() == last->getBlock() && user->isBeforeInBlock(last))
                    return;
        OpBuilder builder(last);
        const Location loc = last->getLoc();
        auto arg = [&](const char *name) { return valueOf[m.args.at(name)]; };
        std::vector<Type> resultTypes;
        for (int r : m.results)
            resultTypes.push_back(valueOf[r].getType());
        Operation *fused = nullptr;
        switch (m.kind) {
        case HIP::ChainKind::CONV_RELU_POOL: {
            Value epilogue = builder.create<daphne::ConstantOp>(loc, builder.getIndexType(), builder.getIndexAttr(m.epilogue));
            fused = builder.create<daphne::Conv2DForwardFusedOp>(
                loc, resultTypes,
                ValueRange{arg("data"), arg("filter"), arg("bias"), arg("batch_size"), arg("num_channels"), arg("img_h"), arg("img_w"),
                           arg("filter_h"), arg("filter_w"), arg("stride_h"), arg("stride_w"), arg("pad_h"), arg("pad_w"), epilogue});
            break;
        }
        case HIP::ChainKind::AFFINE_RELU: {
            Value epilogue = builder.create<daphne::ConstantOp>(loc, builder.getIndexType(), builder.getIndexAttr(m.epilogue));
            fused = builder.create<daphne::AffineForwardFusedOp>(loc, resultTypes,
                                                                 ValueRange{arg("data"), arg("weights"), arg("bias"), epilogue});
            break;
        }
        case HIP::ChainKind::NORMAL_EQUATIONS: {
            auto vt = llvm::cast<daphne::MatrixType>(arg("X").getType()).getElementType();
            Value lambda = builder.create<daphne::ConstantOp>(loc, vt, builder.getFloatAttr(vt, 0.0));
            fused = builder.create<daphne::NormalEquationsOp>(loc, resultTypes, ValueRange{arg("X"), arg("y"), lambda});
            break;
        }
        case HIP::ChainKind::KMEANS_ASSIGN:
            fused = builder.create<daphne::KmeansAssignOp>(loc, resultTypes, ValueRange{arg("X"), arg("C"), arg("xx"), arg("cc")});
            break;
        case HIP::ChainKind::KMEANS_STEP: // results: the labels, the new centroids, the cluster sizes (the column sums of the encoding)
            fused = builder.create<daphne::KmeansStepOp>(loc, resultTypes, ValueRange{arg("X"), arg("C"), arg("xx"), arg("cc")});
            break;
        }
        fused->setAttr(ATTR_HIP_DEVICE, builder.getI32IntegerAttr(0));
        for (size_t k = 0; k < m.results.size(); k++) {
            valueOf[m.results[k]].replaceAllUsesWith(fused->getResult(k));
            valueOf[m.results[k]] = fused->getResult(k); // a later chain may take this value as its argument
        }
        // the chain's operations are dead now, last first (each one's only user was the next)
        for (size_t k = m.ops.size(); k-- > 0;)
            if (listed[m.ops[k]]->use_empty())
                listed[m.ops[k]]->erase();
    }
};

} // namespace

std::unique_ptr<Pass> daphne::createFuseHIPOperatorChainsPass() { return std::make_unique<FuseHIPOperatorChainsPass>(); }
#endif // USE_HIP
