// Gemv (kernels/CUDA/Gemv.h:34-48): res = t(mat) * vec
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTMat, class DTVec> struct Gemv {
    static void apply(DTRes *&res, const DTMat *mat, const DTVec *vec, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(mat->getNumCols(), 1, false, &alloc_desc);
        check(dh_gemv(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), mat->getValues(&alloc_desc), mat->getNumRows(),
                      mat->getNumCols(), mat->getRowSkip(), vec->getValues(&alloc_desc), vec->getNumRows(), vec->getRowSkip()));
    }
};
template <class DTRes, class DTMat, class DTVec> void gemv(DTRes *&res, const DTMat *mat, const DTVec *vec, DCTX(ctx)) {
    Gemv<DTRes, DTMat, DTVec>::apply(res, mat, vec, ctx);
}

} // namespace HIP
