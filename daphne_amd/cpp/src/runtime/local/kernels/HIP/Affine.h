// NN::Affine::Forward (kernels/CUDA/Affine.h:24-26)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

namespace NN::Affine {
template <class DTRes, class DTArg> struct Forward {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *weights, const DTArg *bias, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (data->getNumCols() != weights->getNumRows())
            throw std::runtime_error("CUDA::NN::Affine: #cols of lhs and #rows of rhs must be the same (" +
                                     std::to_string(data->getNumCols()) + " != " + std::to_string(weights->getNumRows()) + ")");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), weights->getNumCols(), false, &alloc_desc);
        check(dh_affine_forward(VT(), detail::raw(ctx), res->getValues(&alloc_desc), data->getValues(&alloc_desc), data->getNumRows(),
                                data->getNumCols(), weights->getValues(&alloc_desc), weights->getNumRows(), weights->getNumCols(),
                                bias ? bias->getValues(&alloc_desc) : nullptr, bias ? bias->getNumRows() : 0,
                                bias ? bias->getNumCols() : 0));
    }
};
} // namespace NN::Affine

} // namespace HIP
