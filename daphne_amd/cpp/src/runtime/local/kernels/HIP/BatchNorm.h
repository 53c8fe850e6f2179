// BatchNormInferenceForward (kernels/CUDA/BatchNorm.h:26-29)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct BatchNormInferenceForward {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *gamma, const DTArg *beta, const DTArg *ema_mean,
                      const DTArg *ema_var, const typename DTArg::VT eps, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, &alloc_desc);
        check(dh_batchnorm_inference(VT(), detail::raw(ctx), res->getValues(&alloc_desc), data->getValues(&alloc_desc), data->getNumRows(),
                                     data->getNumCols(), gamma->getValues(&alloc_desc), beta->getValues(&alloc_desc), ema_mean->getValues(&alloc_desc),
                                     ema_var->getValues(&alloc_desc), gamma->getNumRows(), eps, 0));
    }
};

} // namespace HIP
