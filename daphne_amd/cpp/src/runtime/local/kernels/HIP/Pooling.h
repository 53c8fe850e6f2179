// NN::Pooling::Forward<MAX | AVG> (kernels/CUDA/Pooling.h:31-35)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

namespace NN::Pooling {
template <typename VT> struct MAX {};
template <typename VT> struct AVG {};
template <template <typename> class OP, class DTRes, class DTArg> struct Forward {
    static void apply(DTRes *&res, size_t &res_h, size_t &res_w, const DTArg *data, const size_t batch_size,
                      const size_t num_channels, const size_t img_h, const size_t img_w, const size_t pool_h,
                      const size_t pool_w, const size_t stride_h, const size_t stride_w, const size_t pad_h,
                      const size_t pad_w, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        const size_t P = (img_h + 2 * pad_h - pool_h) / stride_w + 1, Q = (img_w + 2 * pad_w - pool_w) / stride_h + 1;
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(batch_size, num_channels * P * Q, false, &alloc_desc);
        if constexpr (std::is_same<OP<VT>, MAX<VT>>::value)
            check(dh_maxpool_forward(VT(), detail::raw(ctx), res->getValues(&alloc_desc), &res_h, &res_w, data->getValues(&alloc_desc),
                                     batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h,
                                     pad_w));
        else
            check(dh_avgpool_forward(VT(), detail::raw(ctx), res->getValues(&alloc_desc), &res_h, &res_w, data->getValues(&alloc_desc),
                                     batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h,
                                     pad_w));
    }
};
} // namespace NN::Pooling

} // namespace HIP
