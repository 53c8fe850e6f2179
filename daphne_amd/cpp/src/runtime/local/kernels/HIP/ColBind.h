// ColBind (kernels/CUDA/ColBind.h:26-44)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTLhs, class DTRhs> struct ColBind {
    static void apply(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (lhs->getNumRows() != rhs->getNumRows())
            throw std::runtime_error("ColBind - the two operands must have the same number of rows, but lhs has " +
                                     std::to_string(lhs->getNumRows()) + " and rhs has " +
                                     std::to_string(rhs->getNumRows()) + " rows");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(lhs->getNumRows(), lhs->getNumCols() + rhs->getNumCols(), false, &alloc_desc);
        check(dh_col_bind(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), lhs->getValues(&alloc_desc), lhs->getNumRows(),
                          lhs->getNumCols(), lhs->getRowSkip(), rhs->getValues(&alloc_desc), rhs->getNumRows(), rhs->getNumCols(),
                          rhs->getRowSkip()));
    }
};
template <class DTRes, class DTLhs, class DTRhs> void colBind(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, DCTX(ctx)) {
    ColBind<DTRes, DTLhs, DTRhs>::apply(res, lhs, rhs, ctx);
}

} // namespace HIP
