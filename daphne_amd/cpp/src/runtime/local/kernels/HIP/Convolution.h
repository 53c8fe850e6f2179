// Convolution::Forward (kernels/CUDA/Convolution.h:33-38)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

namespace Convolution {
template <class DTRes, class DTArg> struct Forward {
    static void apply(DTRes *&res, size_t *res_h, size_t *res_w, const DTArg *data, const DTArg *filter, const DTArg *bias,
                      const size_t batch_size, const size_t num_channels, const size_t img_h, const size_t img_w,
                      const size_t filter_h, const size_t filter_w, const size_t stride_h, const size_t stride_w,
                      const size_t pad_h, const size_t pad_w, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        const size_t F = filter->getNumRows();
        const size_t P = (img_h + 2 * pad_h - filter_h) / stride_h + 1, Q = (img_w + 2 * pad_w - filter_w) / stride_w + 1;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(batch_size, F * P * Q, false, &alloc_desc);
        // the CUDA kernel skips the bias when it is null or aliases the filter (Convolution.cpp:119-121)
        const VT *b = (bias && bias != filter) ? bias->getValues(&alloc_desc) : nullptr;
        check(dh_conv2d_forward(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res_h, res_w, data->getValues(&alloc_desc),
                                filter->getValues(&alloc_desc), filter->getNumRows(), filter->getNumCols(), b, batch_size,
                                num_channels, img_h, img_w, filter_h, filter_w, stride_h, stride_w, pad_h, pad_w));
    }
};
} // namespace Convolution

} // namespace HIP
