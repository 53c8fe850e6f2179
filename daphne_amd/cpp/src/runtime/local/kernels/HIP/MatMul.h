// MatMul (kernels/CUDA/MatMul.h:31-51)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTLhs, class DTRhs> struct MatMul {
    static void apply(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, bool transa, bool transb, DCTX(ctx)) = delete;
};
template <typename T> struct MatMul<DenseMatrix<T>, DenseMatrix<T>, DenseMatrix<T>> {
    static void apply(DenseMatrix<T> *&res, const DenseMatrix<T> *lhs, const DenseMatrix<T> *rhs, bool transa,
                      bool transb, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        const size_t nr1 = transa ? lhs->getNumCols() : lhs->getNumRows();
        const size_t nc1 = transa ? lhs->getNumRows() : lhs->getNumCols();
        const size_t nr2 = transb ? rhs->getNumCols() : rhs->getNumRows();
        const size_t nc2 = transb ? rhs->getNumRows() : rhs->getNumCols();
        if (nc1 != nr2) // kernels/MatMul.cpp:256-259, before anything is allocated
            throw std::runtime_error("MatMul - #cols of lhs and #rows of rhs must be the same, but got" +
                                     std::to_string(nc1) + "and" + std::to_string(nr2));
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<T>>(nr1, nc2, false, &alloc_desc);
        check(dh_matmul(T(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), lhs->getValues(&alloc_desc), lhs->getNumRows(),
                        lhs->getNumCols(), lhs->getRowSkip(), rhs->getValues(&alloc_desc), rhs->getNumRows(), rhs->getNumCols(),
                        rhs->getRowSkip(), transa ? 1 : 0, transb ? 1 : 0));
    }
};
template <class DTRes, class DTLhs, class DTRhs>
void matMul(DTRes *&res, const DTLhs *lhs, const DTRhs *rhs, bool transa, bool transb, DCTX(ctx)) {
    MatMul<DTRes, DTLhs, DTRhs>::apply(res, lhs, rhs, transa, transb, ctx);
}

} // namespace HIP
