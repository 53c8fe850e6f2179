// Conv2DBackwardData (kernels/Conv2DBackwardData.h:35-46): `output` is the gradient w.r.t. the convolution's result
// The reference has this kernel on the CPU only; same template parameters and argument order.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg> struct Conv2DBackwardData {
    static void apply(const DTArg *filter, const DTArg *output, const size_t stride_h, const size_t stride_w, const size_t pad_h,
                      const size_t pad_w, const size_t input_batch_size, const size_t input_num_channels, const size_t input_h,
                      const size_t input_w, const size_t filter_num_filters, const size_t filter_num_channels,
                      const size_t filter_h, const size_t filter_w, DTRes *&data, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        (void)filter_num_channels;
        if (data == nullptr)
            data = DataObjectFactory::create<DTRes>(input_batch_size, input_num_channels * input_h * input_w, false, &alloc_desc);
        check(dh_conv2d_backward_data(VT(), detail::raw(ctx), data->getValues(&alloc_desc), filter->getValues(&alloc_desc), output->getValues(&alloc_desc),
                                      input_batch_size, input_num_channels, input_h, input_w, filter_num_filters, filter_h,
                                      filter_w, stride_h, stride_w, pad_h, pad_w));
    }
};
template <class DTRes, class DTArg>
void conv2DBackwardData(const DTArg *filter, const DTArg *output, const size_t stride_h, const size_t stride_w, const size_t pad_h,
                        const size_t pad_w, const size_t input_batch_size, const size_t input_num_channels, const size_t input_h,
                        const size_t input_w, const size_t filter_num_filters, const size_t filter_num_channels,
                        const size_t filter_h, const size_t filter_w, DTRes *&data, DCTX(ctx)) {
    Conv2DBackwardData<DTRes, DTArg>::apply(filter, output, stride_h, stride_w, pad_h, pad_w, input_batch_size, input_num_channels,
                                            input_h, input_w, filter_num_filters, filter_num_channels, filter_h, filter_w, data, ctx);
}

} // namespace HIP
