// MaxPoolBackward / AvgPoolBackward (kernels/MaxPoolBackward.h:35-40, AvgPoolBackward.h:35-40)
// The reference has this kernel on the CPU only; same template parameters and argument order.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

#define DH_POOL_BACKWARD(NAME, FN)                                                                                      \
    template <class DTRes, class DTArg> struct NAME {                                                                   \
        static void apply(DTRes *&res, const DTArg *input, const DTArg *dOut, const size_t batch_size,                  \
                          const size_t num_channels, const size_t img_h, const size_t img_w, const size_t pool_h,       \
                          const size_t pool_w, const size_t stride_h, const size_t stride_w, const size_t pad_h,        \
                          const size_t pad_w, DCTX(ctx)) {                                                              \
            AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);                                                  \
            using VT = typename DTArg::VT;                                                                              \
            if (res == nullptr)                                                                                         \
                res = DataObjectFactory::create<DTRes>(batch_size, num_channels * img_h * img_w, false, &alloc_desc);           \
            check(FN(VT(), detail::raw(ctx), res->getValues(&alloc_desc), input->getValues(&alloc_desc), dOut->getValues(&alloc_desc), batch_size,       \
                     num_channels, img_h, img_w, pool_h, pool_w, stride_h, stride_w, pad_h, pad_w));                    \
        }                                                                                                               \
    };
DH_POOL_BACKWARD(MaxPoolBackward, dh_maxpool_backward)
DH_POOL_BACKWARD(AvgPoolBackward, dh_avgpool_backward)
#undef DH_POOL_BACKWARD
#define DH_POOL_BACKWARD_FN(FN, NAME)                                                                                   \
    template <class DTRes, class DTArg>                                                                                 \
    void FN(DTRes *&res, const DTArg *input, const DTArg *dOut, const size_t batch_size, const size_t num_channels,     \
            const size_t img_h, const size_t img_w, const size_t pool_h, const size_t pool_w, const size_t stride_h,    \
            const size_t stride_w, const size_t pad_h, const size_t pad_w, DCTX(ctx)) {                                 \
        NAME<DTRes, DTArg>::apply(res, input, dOut, batch_size, num_channels, img_h, img_w, pool_h, pool_w, stride_h,   \
                                  stride_w, pad_h, pad_w, ctx);                                                         \
    }
DH_POOL_BACKWARD_FN(maxPoolBackward, MaxPoolBackward)
DH_POOL_BACKWARD_FN(avgPoolBackward, AvgPoolBackward)
#undef DH_POOL_BACKWARD_FN

} // namespace HIP
