// Softmax (kernels/CUDA/Softmax.h:32-34)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct Softmax {
    static void apply(DTRes *&res, const DTArg *data, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, &alloc_desc);
        check(dh_softmax(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), data->getValues(&alloc_desc),
                         data->getNumRows(), data->getNumCols(), data->getRowSkip()));
    }
};

} // namespace HIP
