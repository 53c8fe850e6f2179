// Solve (kernels/CUDA/Solve.h; checks of kernels/Solve.h:93-101)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTLhs, class DTRhs> struct Solve {
    static void apply(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) = delete;
};
template <typename VT> struct Solve<DenseMatrix<VT>, DenseMatrix<VT>, DenseMatrix<VT>> {
    static void apply(DenseMatrix<VT> *&res, const DenseMatrix<VT> *lhs, const DenseMatrix<VT> *rhs, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        if (lhs->getNumRows() != rhs->getNumRows())
            throw std::runtime_error("#rows of lhs and #rows of rhs must be the same");
        if (lhs->getNumRows() != lhs->getNumCols())
            throw std::runtime_error("#rows and #cols of lhs must be the same");
        if (lhs->getRowSkip() != lhs->getNumCols())
            throw std::runtime_error("#cols of lhs must match row skip");
        if (rhs->getNumCols() != 1)
            throw std::runtime_error("#cols of rhs must be 1");
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<VT>>(lhs->getNumRows(), 1, false, &alloc_desc);
        check(dh_solve(VT(), detail::raw(ctx), res->getValues(&alloc_desc), lhs->getValues(&alloc_desc), lhs->getNumRows(), lhs->getRowSkip(),
                       rhs->getValues(&alloc_desc)));
    }
};
template <class DTRes, class DTLhs, class DTRhs> void solve(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
    Solve<DTRes, DTLhs, DTRhs>::apply(res, lhs, rhs, ctx);
}

} // namespace HIP
