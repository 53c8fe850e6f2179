// BatchNorm2DTrainForward (kernels/BatchNorm2DTrainForward.h:38-57). The four statistics results are C x 1 here
// (the reference allocates C x C and fills the first C values).
// The reference has this kernel on the CPU only; same template parameters and argument order.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct BatchNorm2DTrainForward {
    static void apply(DTRes *&res, DTRes *&new_emaMean, DTRes *&new_emaVar, DTRes *&mean, DTRes *&invVar, const DTArg *in,
                      const DTArg *gamma, const DTArg *beta, const DTArg *emaMean, const DTArg *emaVar,
                      const typename DTArg::VT eps, const typename DTArg::VT mu, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        const size_t C = gamma->getNumRows() * gamma->getNumCols();
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(in->getNumRows(), in->getNumCols(), false, &alloc_desc);
        for (DTRes **m : {&new_emaMean, &new_emaVar, &mean, &invVar})
            if (*m == nullptr)
                *m = DataObjectFactory::create<DTRes>(C, 1, false, &alloc_desc);
        check(dh_batchnorm_train_forward(VT(), detail::raw(ctx), res->getValues(&alloc_desc), new_emaMean->getValues(&alloc_desc),
                                         new_emaVar->getValues(&alloc_desc), mean->getValues(&alloc_desc), invVar->getValues(&alloc_desc), in->getValues(&alloc_desc),
                                         in->getNumRows(), in->getNumCols(), gamma->getValues(&alloc_desc), beta->getValues(&alloc_desc),
                                         emaMean->getValues(&alloc_desc), emaVar->getValues(&alloc_desc), C, eps, mu));
    }
};
template <class DTRes, class DTArg>
void batchNorm2DTrainForward(DTRes *&res, DTRes *&new_emaMean, DTRes *&new_emaVar, DTRes *&mean, DTRes *&invVar, const DTArg *in,
                             const DTArg *gamma, const DTArg *beta, const DTArg *emaMean, const DTArg *emaVar,
                             const typename DTArg::VT eps, const typename DTArg::VT mu, DCTX(ctx)) {
    BatchNorm2DTrainForward<DTRes, DTArg>::apply(res, new_emaMean, new_emaVar, mean, invVar, in, gamma, beta, emaMean, emaVar, eps,
                                                 mu, ctx);
}

} // namespace HIP
