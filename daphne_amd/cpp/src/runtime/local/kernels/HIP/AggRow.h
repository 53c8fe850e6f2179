// AggRow (kernels/CUDA/AggRow.h:30-52; IDXMIN / IDXMAX: kernels/AggRow.h:71-94)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct AggRow {
    static void apply(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct AggRow<DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<VT> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(arg->getNumRows(), 1, false, &alloc_desc);
        check(dh_agg_row(VT(), detail::raw(ctx), static_cast<int>(opCode), res->getValues(&alloc_desc), res->getRowSkip(),
                         arg->getValues(&alloc_desc), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
// RowIdxMin / RowIdxMax: the op's result type is a matrix of size_t (ir/daphneir/DaphneOps.td:544)
template <typename VT> struct AggRow<DenseMatrix<size_t>, DenseMatrix<VT>> {
    static void apply(AggOpCode opCode, DenseMatrix<size_t> *&res, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        static_assert(sizeof(size_t) == sizeof(uint64_t), "indices are 64 bit");
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<size_t>>(arg->getNumRows(), 1, false, &alloc_desc);
        check(dh_agg_row_idx(VT(), detail::raw(ctx), static_cast<int>(opCode), reinterpret_cast<uint64_t *>(res->getValues(&alloc_desc)),
                             res->getRowSkip(), arg->getValues(&alloc_desc), arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void aggRow(AggOpCode opCode, DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    AggRow<DTRes, DTArg>::apply(opCode, res, arg, ctx);
}

} // namespace HIP
