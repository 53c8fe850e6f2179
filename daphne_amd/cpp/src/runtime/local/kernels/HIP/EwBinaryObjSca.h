// EwBinaryObjSca (kernels/CUDA/EwBinaryObjSca.h:37-60)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTLhs, typename VTRhs> struct EwBinaryObjSca {
    static void apply(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, VTRhs rhs, DCTX(ctx)) = delete;
};
template <typename VT> struct EwBinaryObjSca<DenseMatrix<VT>, DenseMatrix<VT>, VT> {
    static void apply(BinaryOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *lhs, VT rhs, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(lhs->getNumRows(), lhs->getNumCols(), false, &alloc_desc);
        check(dh_ew_binary_sca(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(&alloc_desc), res->getRowSkip(),
                               lhs->getValues(&alloc_desc), lhs->getNumRows(), lhs->getNumCols(), lhs->getRowSkip(), rhs));
    }
};
template <class DTRes, class DTLhs, typename VTRhs>
void ewBinaryObjSca(BinaryOpCode opCode, DTRes *&res, const DTLhs *lhs, VTRhs rhs, DCTX(ctx)) {
    EwBinaryObjSca<DTRes, DTLhs, VTRhs>::apply(opCode, res, lhs, rhs, ctx);
}

} // namespace HIP
