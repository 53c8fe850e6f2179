// MarkHIPOpsPass: decides which operations of a compiled program run on the HIP device.
//
// NOT COMPILED IN THIS REPOSITORY (it needs MLIR and DAPHNE's IR). In DAPHNE this file is
// src/compiler/lowering/MarkHIPOpsPass.cpp, listed in src/compiler/lowering/CMakeLists.txt next to
// MarkCUDAOpsPass.cpp and scheduled by DaphneIrExecutor when --hip is given (see ../../../patches).
//
// It plays the part of MarkCUDAOpsPass (src/compiler/lowering/MarkCUDAOpsPass.cpp:26-205): an operation that is
// chosen gets the attribute `hip_device = 0`, which RewriteToCallKernelOpPass turns into a kernel lookup with
// backend "HIP". The choice differs in one point. The reference asks a trait that is compiled into the operation
// (`CUDASupport` in DaphneOps.td) and so has to be kept in step with the kernel library by hand; here the question
// is put to the kernel catalog itself: an operation is a candidate if HIPcatalog.json, loaded at start-up, holds a
// "HIP" kernel for its mnemonic and its result and argument types. Adding an instantiation to HIPkernels.json is
// then all it takes to move an operation to the device.
//
// The other conditions are the reference's: the operation computes on matrices, and, unless `force_hip` is set,
// at least one operand or result has a dimension of 256 or more and all of them together fit 90 % of the device's
// memory (unknown dimensions count as 256 for the first test and as 1 for the second).
// The body of a VectorizedPipelineOp is cloned into the op's device region when all of its operations qualify
// (or any of them, with `hip_fuse_any`), and the clones are marked. That region is the op's second region, which
// the reference names `cuda`; LowerToLLVMPass outlines it as `_vect_hip<N>`.
#ifdef USE_HIP
#include "compiler/utils/CompilerUtils.h"
#include "ir/daphneir/Daphne.h"
#include "ir/daphneir/Passes.h"
#include <compiler/catalog/KernelCatalog.h>

#include <daphne_hip.h>

#include <mlir/IR/IRMapping.h>

#include <cmath>
#include <vector>

using namespace mlir;

namespace {

constexpr const char *ATTR_HIP_DEVICE = "hip_device";
constexpr int64_t MIN_DIM = 256;

struct MatrixFootprint {
    bool any_large = false; // some matrix has a dimension >= MIN_DIM
    size_t bytes = 0;       // all matrices together
};

struct MarkHIPOpsPass : public PassWrapper<MarkHIPOpsPass, OperationPass<func::FuncOp>> {
    const DaphneUserConfig &cfg;
    size_t mem_budget = 0;
    std::shared_ptr<spdlog::logger> logger;

    explicit MarkHIPOpsPass(const DaphneUserConfig &cfg) : cfg(cfg) {
        logger = spdlog::get("compiler::hip");
        size_t free_bytes = 0, total_bytes = 0;
        if (dh_device_memory(0, &free_bytes, &total_bytes) != DH_OK)
            throw std::runtime_error(std::string("MarkHIPOpsPass: ") + dh_last_error());
        mem_budget = static_cast<size_t>(std::floor(0.9 * static_cast<double>(total_bytes)));
    }

    // Does the catalog hold a HIP kernel for this operation as it stands (mnemonic, types)?
    bool catalogHasKernel(Operation *op) const {
        std::vector<Type> argTys, resTys;
        for (Type t : op->getOperandTypes())
            argTys.push_back(KernelCatalog::normalizeTypeForKernelLookup(t));
        for (Type t : op->getResultTypes())
            resTys.push_back(KernelCatalog::normalizeTypeForKernelLookup(t));
        const std::string mnemonic = op->getName().stripDialect().str();
        return cfg.kernelCatalog.findKernel(mnemonic, argTys, resTys, "HIP").has_value();
    }

    static MatrixFootprint footprint(Operation *op) {
        MatrixFootprint f;
        auto add = [&f](Type type) {
            auto t = llvm::dyn_cast<daphne::MatrixType>(type);
            if (!t)
                return;
            const int64_t rows = t.getNumRows(), cols = t.getNumCols();
            f.any_large |= (rows < 0 ? MIN_DIM : rows) >= MIN_DIM || (cols < 0 ? MIN_DIM : cols) >= MIN_DIM;
            f.bytes += static_cast<size_t>(rows < 0 ? 1 : rows) * static_cast<size_t>(cols < 0 ? 1 : cols) *
                       (t.getElementType().getIntOrFloatBitWidth() / 8);
        };
        for (Type t : op->getOperandTypes())
            add(t);
        for (Type t : op->getResultTypes())
            add(t);
        return f;
    }

    bool runsOnDevice(Operation *op) const {
        if (!CompilerUtils::isMatrixComputation(op) || !catalogHasKernel(op))
            return false;
        if (cfg.force_hip)
            return true;
        const MatrixFootprint f = footprint(op);
        logger->trace("MarkHIPOpsPass: {}: large={} bytes={} budget={}", op->getName().getStringRef().str(), f.any_large,
                      f.bytes, mem_budget);
        return f.any_large && f.bytes < mem_budget;
    }

    void mark(Operation *op) const {
        OpBuilder b(op);
        op->setAttr(ATTR_HIP_DEVICE, b.getI32IntegerAttr(0));
    }

    void handlePipeline(daphne::VectorizedPipelineOp pipelineOp) const {
        size_t supported = 0, total = 0;
        for (Operation &o : pipelineOp.getBody().front().getOperations()) {
            if (llvm::isa<daphne::ReturnOp>(o))
                continue;
            total++;
            supported += runsOnDevice(&o);
        }
        const bool build = cfg.hip_fuse_any ? supported > 0 : (total > 0 && supported == total);
        if (!build)
            return;
        IRMapping mapper;
        pipelineOp.getBody().cloneInto(&pipelineOp.getCuda(), mapper); // the device region
        for (Operation &o : pipelineOp.getCuda().front().getOperations())
            if (!llvm::isa<daphne::ReturnOp>(o) && CompilerUtils::isMatrixComputation(&o) && catalogHasKernel(&o))
                mark(&o);
    }

    void runOnOperation() final {
        getOperation()->walk([&](Operation *op) {
            if (llvm::isa<daphne::ConstantOp>(op))
                return;
            if (auto pipelineOp = llvm::dyn_cast<daphne::VectorizedPipelineOp>(op)) {
                handlePipeline(pipelineOp);
                return;
            }
            // operations inside a pipeline body are handled with their pipeline
            if (llvm::isa<daphne::VectorizedPipelineOp>(op->getParentOp()))
                return;
            if (llvm::isa<daphne::CreateHIPContextOp>(op) || runsOnDevice(op))
                mark(op);
        });
    }
};

} // namespace

std::unique_ptr<Pass> daphne::createMarkHIPOpsPass(const DaphneUserConfig &cfg) { return std::make_unique<MarkHIPOpsPass>(cfg); }

#endif // USE_HIP
