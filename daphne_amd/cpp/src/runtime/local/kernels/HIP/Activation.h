// NN::Activation::Forward<ReLU> (kernels/CUDA/Activation.h:24-33)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

namespace NN::Activation {
struct ReLU {};
template <typename OP, typename DTRes, typename DTArg> struct Forward {
    static void apply(DTRes *&res, const DTArg *data, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        static_assert(std::is_same<OP, ReLU>::value, "ReLU is the only activation of the reference's kernel library");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), data->getNumCols(), false, &alloc_desc);
        check(dh_relu_forward(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), data->getValues(&alloc_desc),
                              data->getNumRows(), data->getNumCols(), data->getRowSkip()));
    }
};
} // namespace NN::Activation

} // namespace HIP
