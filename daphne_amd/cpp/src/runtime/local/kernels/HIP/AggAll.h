// AggAll (kernels/CUDA/AggAll.h:28-50)
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <typename VTRes, class DTArg> struct AggAll {
    static VTRes apply(AggOpCode opCode, const DTArg *arg, DCTX(ctx)) = delete;
};
template <typename VT> struct AggAll<VT, DenseMatrix<VT>> {
    static VT apply(AggOpCode opCode, const DenseMatrix<VT> *arg, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        VT out{};
        check(dh_agg_all(VT(), detail::raw(ctx), static_cast<int>(opCode), arg->getValues(&alloc_desc), arg->getNumRows(),
                         arg->getNumCols(), arg->getRowSkip(), &out));
        return out;
    }
};
template <typename VTRes, class DTArg> VTRes aggAll(AggOpCode opCode, const DTArg *arg, DCTX(ctx)) {
    return AggAll<VTRes, DTArg>::apply(opCode, arg, ctx);
}

} // namespace HIP
