// Syrk (kernels/Syrk.h:30-40 signature with transLeft; device: kernels/CUDA/Syrk.h:29-46)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct Syrk {
    static void apply(DTRes *&res, const DTArg *arg, bool transLeft, DCTX(ctx)) = delete;
};
template <typename VT> struct Syrk<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, bool transLeft, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        const size_t n = transLeft ? arg->getNumCols() : arg->getNumRows();
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(n, n, false, &alloc_desc);
        check(dh_syrk(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), arg->getValues(&alloc_desc), arg->getNumRows(),
                      arg->getNumCols(), arg->getRowSkip(), transLeft ? 1 : 0));
    }
};
template <class DTRes, class DTArg> void syrk(DTRes *&res, const DTArg *arg, bool transLeft, DCTX(ctx)) {
    Syrk<DTRes, DTArg>::apply(res, arg, transLeft, ctx);
}

} // namespace HIP
