// Fill (kernels/CUDA/Fill.h:30-47)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, typename VTArg> struct Fill {
    static void apply(DTRes *&res, VTArg arg, size_t numRows, size_t numCols, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(numRows, numCols, false, &alloc_desc);
        check(dh_fill(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), static_cast<VT>(arg), numRows, numCols));
    }
};
template <class DTRes, typename VTArg> void fill(DTRes *&res, VTArg arg, size_t numRows, size_t numCols, DCTX(ctx)) {
    Fill<DTRes, VTArg>::apply(res, arg, numRows, numCols, ctx);
}

} // namespace HIP
