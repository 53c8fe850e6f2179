// BatchNorm2DBackward (kernels/BatchNorm2DBackward.h:38-53)
// The reference has this kernel on the CPU only; same template parameters and argument order.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct BatchNorm2DBackward {
    static void apply(DTRes *&dX, DTRes *&dGamma, DTRes *&dBeta, const DTArg *mean, const DTArg *invVar, const DTArg *in,
                      const DTArg *dout, const DTArg *gamma, const typename DTArg::VT eps, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        const size_t C = gamma->getNumRows() * gamma->getNumCols();
        if (dX == nullptr)
            dX = DataObjectFactory::create<DTRes>(in->getNumRows(), in->getNumCols(), false, &alloc_desc);
        if (dGamma == nullptr)
            dGamma = DataObjectFactory::create<DTRes>(C, 1, false, &alloc_desc);
        if (dBeta == nullptr)
            dBeta = DataObjectFactory::create<DTRes>(C, 1, false, &alloc_desc);
        check(dh_batchnorm_backward(VT(), detail::raw(ctx), dX->getValues(&alloc_desc), dGamma->getValues(&alloc_desc), dBeta->getValues(&alloc_desc),
                                    mean->getValues(&alloc_desc), invVar->getValues(&alloc_desc), in->getValues(&alloc_desc), dout->getValues(&alloc_desc), in->getNumRows(),
                                    in->getNumCols(), gamma->getValues(&alloc_desc), C, eps));
    }
};
template <class DTRes, class DTArg>
void batchNorm2DBackward(DTRes *&dX, DTRes *&dGamma, DTRes *&dBeta, const DTArg *mean, const DTArg *invVar, const DTArg *in,
                         const DTArg *dout, const DTArg *gamma, const typename DTArg::VT eps, DCTX(ctx)) {
    BatchNorm2DBackward<DTRes, DTArg>::apply(dX, dGamma, dBeta, mean, invVar, in, dout, gamma, eps, ctx);
}

} // namespace HIP
