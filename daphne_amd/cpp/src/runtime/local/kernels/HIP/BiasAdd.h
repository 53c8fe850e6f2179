// BiasAdd (kernels/CUDA/BiasAdd.h:26-28)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct BiasAdd {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *bias, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, &alloc_desc);
        check(dh_bias_add(VT(), detail::raw(ctx), res->getValues(&alloc_desc), data->getValues(&alloc_desc), data->getNumRows(),
                          data->getNumCols(), bias->getValues(&alloc_desc), bias->getNumItems()));
    }
};

} // namespace HIP
