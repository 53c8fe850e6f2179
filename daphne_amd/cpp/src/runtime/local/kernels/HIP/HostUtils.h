// What every HIP kernel header needs: the data objects and op codes of the run-time, the device context and
// allocation descriptor, and the C ABI of libdaphne_hip.so overloaded on the value type.
// (The counterpart of src/runtime/local/kernels/CUDA/HostUtils.h, which carries the CUDA error-check macros.)
//
// Every kernel of this directory is a template struct with a static apply() plus a convenience function, with the
// template parameters, argument order and exception behaviour of the reference's device kernels
// (src/runtime/local/kernels/CUDA/*.h; signatures cited per kernel), in namespace HIP instead of CUDA.
// `DT *&res`: nullptr on entry makes the kernel allocate the result on the device, otherwise it writes in place
// (res may alias lhs). The last argument is the DaphneContext, from which the device context is taken like
// CUDAContext::get(dctx, deviceID).
//
// Device pointers come from the data objects exactly as in the reference's device kernels
// (e.g. kernels/CUDA/EwBinaryMat.cu:223-233): `AllocationDescriptorHIP alloc_desc(ctx, deviceID)`,
// `arg->getValues(&alloc_desc)` for inputs (const: the matrix uploads itself on first use and its other
// placements stay valid) and for the result (non-const: the device copy becomes the only current one);
// results are created with `DataObjectFactory::create<DT>(rows, cols, false, &alloc_desc)` and live on
// the device until somebody asks for their host values.
//
// All of this is host code for a plain C++17 compiler: nothing of HIP leaks through the C ABI.
#pragma once

#include <runtime/local/context/DaphneContext.h>
#include <runtime/local/context/HIPContext.h>
#include <runtime/local/datastructures/AllocationDescriptorHIP.h>
#include <runtime/local/datastructures/DataObjectFactory.h>
#include <runtime/local/datastructures/DenseMatrix.h>
#include <runtime/local/kernels/AggOpCode.h>
#include <runtime/local/kernels/BinaryOpCode.h>
#include <runtime/local/kernels/UnaryOpCode.h>

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include <daphne_hip.h>

namespace HIP {

namespace detail {
constexpr uint32_t deviceID = 0; // ToDo of the reference as well: multi device support
inline dh_ctx *raw(DCTX(ctx)) { return HIPContext::get(ctx, deviceID)->raw(); }
} // namespace detail

// The C ABI is overloaded on the value type here so that the templates below stay one-liners.
#define DH_OVERLOAD2(NAME)                                                                                              \
    template <typename... A> inline dh_status NAME(float, A... a) { return NAME##_f32(a...); }                          \
    template <typename... A> inline dh_status NAME(double, A... a) { return NAME##_f64(a...); }
DH_OVERLOAD2(dh_ew_binary)
DH_OVERLOAD2(dh_ew_binary_sca)
DH_OVERLOAD2(dh_ew_unary)
DH_OVERLOAD2(dh_agg_all)
DH_OVERLOAD2(dh_agg_row)
DH_OVERLOAD2(dh_agg_row_idx)
DH_OVERLOAD2(dh_agg_col)
DH_OVERLOAD2(dh_agg_col_idx)
DH_OVERLOAD2(dh_matmul)
DH_OVERLOAD2(dh_syrk)
DH_OVERLOAD2(dh_solve)
DH_OVERLOAD2(dh_conv2d_forward)
DH_OVERLOAD2(dh_maxpool_forward)
DH_OVERLOAD2(dh_affine_forward)
DH_OVERLOAD2(dh_bias_add)
DH_OVERLOAD2(dh_batchnorm_inference)
DH_OVERLOAD2(dh_softmax)
DH_OVERLOAD2(dh_avgpool_forward)
DH_OVERLOAD2(dh_relu_forward)
DH_OVERLOAD2(dh_fill)
DH_OVERLOAD2(dh_col_bind)
DH_OVERLOAD2(dh_extract_col)
DH_OVERLOAD2(dh_transpose)
DH_OVERLOAD2(dh_gemv)
DH_OVERLOAD2(dh_batchnorm_train_forward)
DH_OVERLOAD2(dh_batchnorm_backward)
DH_OVERLOAD2(dh_maxpool_backward)
DH_OVERLOAD2(dh_avgpool_backward)
DH_OVERLOAD2(dh_conv2d_backward_data)
DH_OVERLOAD2(dh_conv2d_backward_filter)
#undef DH_OVERLOAD2
// integer value types, as far as the reference instantiates its device kernels for them
// (kernels/CUDA/EwBinaryMat.cu:267-270, EwBinaryObjSca.cu:91-94, AggAll.cu:155, AggRow.cu:146, AggCol.cu:89,
// Fill.cu:47,49, ColBind.cu:75, ExtractCol.cu:58); any other combination fails to compile, like a missing
// instantiation fails to link there
#define DH_OVERLOAD_INT(NAME, SUF, T)                                                                                   \
    template <typename... A> inline dh_status NAME(T, A... a) { return NAME##_##SUF(a...); }
DH_OVERLOAD_INT(dh_ew_binary, si64, int64_t)
DH_OVERLOAD_INT(dh_ew_binary, ui64, uint64_t)
DH_OVERLOAD_INT(dh_ew_binary, si32, int32_t)
DH_OVERLOAD_INT(dh_ew_binary, ui32, uint32_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, si64, int64_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, ui64, uint64_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, si32, int32_t)
DH_OVERLOAD_INT(dh_ew_binary_sca, ui32, uint32_t)
DH_OVERLOAD_INT(dh_agg_all, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_row, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_row_idx, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_col, si64, int64_t)
DH_OVERLOAD_INT(dh_agg_col_idx, si64, int64_t)
DH_OVERLOAD_INT(dh_fill, si64, int64_t)
DH_OVERLOAD_INT(dh_fill, ui64, uint64_t)
DH_OVERLOAD_INT(dh_col_bind, si64, int64_t)
DH_OVERLOAD_INT(dh_extract_col, si64, int64_t)
DH_OVERLOAD_INT(dh_transpose, si64, int64_t)
#undef DH_OVERLOAD_INT

} // namespace HIP
