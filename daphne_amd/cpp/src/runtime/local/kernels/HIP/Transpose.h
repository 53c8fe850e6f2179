// Transpose (kernels/CUDA/Transpose.h:33-47)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct Transpose {
    static void apply(DTRes *&res, const DTArg *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(arg->getNumCols(), arg->getNumRows(), false, &alloc_desc);
        check(dh_transpose(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), arg->getValues(&alloc_desc),
                           arg->getNumRows(), arg->getNumCols(), arg->getRowSkip()));
    }
};
// positions and counts (size_t): moved as the 64-bit integers they are
template <> struct Transpose<DenseMatrix<size_t>, DenseMatrix<size_t>> {
    static void apply(DenseMatrix<size_t> *&res, const DenseMatrix<size_t> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        static_assert(sizeof(size_t) == sizeof(int64_t), "size_t is 64 bit");
        if (res == nullptr)
            res = DataObjectFactory::create<DenseMatrix<size_t>>(arg->getNumCols(), arg->getNumRows(), false, &alloc_desc);
        check(dh_transpose_si64(detail::raw(ctx), reinterpret_cast<int64_t *>(res->getValues(&alloc_desc)), res->getRowSkip(),
                                reinterpret_cast<const int64_t *>(arg->getValues(&alloc_desc)), arg->getNumRows(), arg->getNumCols(),
                                arg->getRowSkip()));
    }
};
template <class DTRes, class DTArg> void transpose(DTRes *&res, const DTArg *arg, DCTX(ctx)) {
    Transpose<DTRes, DTArg>::apply(res, arg, ctx);
}

} // namespace HIP
