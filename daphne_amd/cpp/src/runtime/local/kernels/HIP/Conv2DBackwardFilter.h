// Conv2DBackwardFilter (kernels/Conv2DBackwardFilter.h:35-46)
// The reference has this kernel on the CPU only; same template parameters and argument order.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct Conv2DBackwardFilter {
    static void apply(DTRes *&dFilter, const DTArg *input, const DTArg *output, const size_t stride_h, const size_t stride_w,
                      const size_t pad_h, const size_t pad_w, const size_t input_batch_size, const size_t input_num_channels,
                      const size_t input_h, const size_t input_w, const size_t filter_num_filters,
                      const size_t filter_num_channels, const size_t filter_h, const size_t filter_w, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        if (dFilter == nullptr)
            dFilter = DataObjectFactory::create<DTRes>(filter_num_filters, filter_num_channels * filter_h * filter_w, false, &alloc_desc);
        check(dh_conv2d_backward_filter(VT(), detail::raw(ctx), dFilter->getValues(&alloc_desc), input->getValues(&alloc_desc), output->getValues(&alloc_desc),
                                        input_batch_size, input_num_channels, input_h, input_w, filter_num_filters, filter_h,
                                        filter_w, stride_h, stride_w, pad_h, pad_w));
    }
};
template <class DTRes, class DTArg>
void conv2DBackwardFilter(DTRes *&dFilter, const DTArg *input, const DTArg *output, const size_t stride_h, const size_t stride_w,
                          const size_t pad_h, const size_t pad_w, const size_t input_batch_size, const size_t input_num_channels,
                          const size_t input_h, const size_t input_w, const size_t filter_num_filters,
                          const size_t filter_num_channels, const size_t filter_h, const size_t filter_w, DCTX(ctx)) {
    Conv2DBackwardFilter<DTRes, DTArg>::apply(dFilter, input, output, stride_h, stride_w, pad_h, pad_w, input_batch_size,
                                              input_num_channels, input_h, input_w, filter_num_filters, filter_num_channels,
                                              filter_h, filter_w, ctx);
}

} // namespace HIP
