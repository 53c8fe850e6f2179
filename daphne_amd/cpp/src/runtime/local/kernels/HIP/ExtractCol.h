// ExtractCol (kernels/CUDA/ExtractCol.h:26-45); positions as DenseMatrix<int64_t>
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <class DTRes, class DTArg, class DTSel> struct ExtractCol {
    static void apply(DTRes *&res, const DTArg *arg, const DTSel *sel, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        static_assert(std::is_same<typename DTSel::VT, int64_t>::value, "column positions are int64_t");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(arg->getNumRows(), sel->getNumRows(), false, &alloc_desc);
        check(dh_extract_col(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res->getRowSkip(), arg->getValues(&alloc_desc),
                             arg->getNumRows(), arg->getNumCols(), arg->getRowSkip(), sel->getValues(&alloc_desc), sel->getNumRows(),
                             sel->getNumCols(), sel->getRowSkip()));
    }
};
template <class DTRes, class DTArg, class DTSel> void extractCol(DTRes *&res, const DTArg *arg, const DTSel *sel, DCTX(ctx)) {
    ExtractCol<DTRes, DTArg, DTSel>::apply(res, arg, sel, ctx);
}

} // namespace HIP
