// AggCol (kernels/CUDA/AggCol.h:30-52)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct AggCol {
    static void apply(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct AggCol<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(1, arg->getNumCols(), false, &alloc_desc);
        check(dh_agg_col(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(&alloc_desc), arg->getValues(&alloc_desc),
                         arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <typename VT> struct AggCol<DenseMatrix<size_t>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<size_t> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<size_t>>(1, arg->getNumCols(), false, &alloc_desc);
        check(dh_agg_col_idx(VT(), detail::raw(ctx), static_cast<int>(opCode), reinterpret_cast<uint64_t *>(res->getValues(&alloc_desc)),
                             arg->getValues(&alloc_desc), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void aggCol(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    AggCol<DTRes, DTArg>::apply(opCode, res, arg, ctx);
}

} // namespace HIP
