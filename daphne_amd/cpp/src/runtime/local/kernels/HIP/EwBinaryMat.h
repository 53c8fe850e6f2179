// EwBinaryMat (kernels/CUDA/EwBinaryMat.h:31-47)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTLhs, class DTRhs> struct EwBinaryMat {
    static void apply(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) = delete;
};
template <typename VT> struct EwBinaryMat<DenseMatrix<VT>, DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(BinaryOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *lhs, const DenseMatrix<VT> *rhs,
                      DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(lhs->getNumRows(), lhs->getNumCols(), false, &alloc_desc);
        check(dh_ew_binary(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(&alloc_desc), res->getRowSkip(),
                           lhs->getValues(&alloc_desc), lhs->getNumRows(), lhs->getNumCols(), lhs->getRowSkip(), rhs->getValues(&alloc_desc),
                           rhs->getNumRows(), rhs->getNumCols(), rhs->getRowSkip()));
    }
};
template <class DTRes, class DTLhs, class DTRhs>
void ewBinaryMat(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
    EwBinaryMat<DTRes, DTLhs, DTRhs>::apply(opCode, res, lhs, rhs, ctx);
}

} // namespace HIP
