// EwUnaryMat (kernels/EwUnaryMat.h:35-45; no device version in the reference)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct EwUnaryMat {
    static void apply(UnaryOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct EwUnaryMat<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(UnaryOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(arg->getNumRows(), arg->getNumCols(), false, &alloc_desc);
        check(dh_ew_unary(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(&alloc_desc), res->getRowSkip(),
                          arg->getValues(&alloc_desc), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void ewUnaryMat(UnaryOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    EwUnaryMat<DTRes, DTArg>::apply(opCode, res, arg, ctx);
}

} // namespace HIP
