// Elementwise kernels, float instantiation. See ew_impl.h for the design and reference citations.
#include "ew_impl.h"

extern "C" dh_status dh_ew_binary_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *lhs, size_t lhs_rows,
                                     size_t lhs_cols, size_t ld_lhs, const float *rhs, size_t rhs_rows,
                                     size_t rhs_cols, size_t ld_rhs) {
    return dh_ew::ew_binary<float>(ctx, op, res, ld_res, lhs, lhs_rows, lhs_cols, ld_lhs, rhs, rhs_rows, rhs_cols,
                                ld_rhs);
}

extern "C" dh_status dh_ew_binary_sca_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *lhs, size_t rows,
                                         size_t cols, size_t ld_lhs, float rhs) {
    return dh_ew::ew_binary_sca<float>(ctx, op, res, ld_res, lhs, rows, cols, ld_lhs, rhs);
}

extern "C" dh_status dh_ew_unary_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *arg, size_t rows,
                                    size_t cols, size_t ld_arg) {
    return dh_ew::ew_unary<float>(ctx, op, res, ld_res, arg, rows, cols, ld_arg);
}

// CUDA::NN::Activation::Forward<ReLU,...>::apply (kernels/CUDA/Activation.cpp:21-47): max(0, x) with NaN
// passed through, which is std::max(x, 0) of the elementwise MAX.
extern "C" dh_status dh_relu_forward_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *data, size_t rows, size_t cols,
                                          size_t ld_data) {
    return dh_ew::ew_binary_sca<float>(ctx, DH_BIN_MAX, res, ld_res, data, rows, cols, ld_data, float(0));
}
