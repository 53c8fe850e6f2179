// DNN inference kernels, float instantiation. See dnn_impl.h for the design and reference citations.
#include "dnn_impl.h"

extern "C" dh_status dh_conv2d_forward_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w, const float *data,
                                          const float *filter, size_t filter_rows, size_t filter_cols, const float *bias,
                                          size_t batch, size_t channels, size_t img_h, size_t img_w, size_t filter_h,
                                          size_t filter_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                          size_t pad_w) {
    return dh_dnn::conv2d_forward<float>(ctx, res, res_h, res_w, data, filter, filter_rows, filter_cols, bias, batch,
                                      channels, img_h, img_w, filter_h, filter_w, stride_h, stride_w, pad_h, pad_w);
}

extern "C" dh_status dh_conv2d_forward_fused_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w, const float *data,
                                                const float *filter, size_t filter_rows, size_t filter_cols, const float *bias,
                                                size_t batch, size_t channels, size_t img_h, size_t img_w, size_t filter_h,
                                                size_t filter_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                                size_t pad_w, unsigned epilogue) {
    return dh_dnn::conv2d_forward<float>(ctx, res, res_h, res_w, data, filter, filter_rows, filter_cols, bias, batch,
                                      channels, img_h, img_w, filter_h, filter_w, stride_h, stride_w, pad_h, pad_w, epilogue);
}

extern "C" dh_status dh_maxpool_forward_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w, const float *data,
                                           size_t batch, size_t channels, size_t img_h, size_t img_w, size_t pool_h,
                                           size_t pool_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                           size_t pad_w) {
    return dh_dnn::maxpool_forward<float>(ctx, res, res_h, res_w, data, batch, channels, img_h, img_w, pool_h, pool_w,
                                       stride_h, stride_w, pad_h, pad_w);
}

extern "C" dh_status dh_bias_add_f32(dh_ctx *ctx, float *res, const float *data, size_t rows, size_t cols, const float *bias,
                                    size_t num_bias) {
    return dh_dnn::bias_add<float>(ctx, res, data, rows, cols, bias, num_bias);
}

extern "C" dh_status dh_batchnorm_inference_f32(dh_ctx *ctx, float *res, const float *data, size_t rows, size_t cols,
                                               const float *gamma, const float *beta, const float *ema_mean,
                                               const float *ema_var, size_t channels, float eps, int stat_index) {
    return dh_dnn::batchnorm_inference<float>(ctx, res, data, rows, cols, gamma, beta, ema_mean, ema_var, channels, eps,
                                           stat_index);
}

extern "C" dh_status dh_softmax_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows, size_t cols,
                                   size_t ld) {
    return dh_dnn::softmax<float>(ctx, res, ld_res, arg, rows, cols, ld);
}

extern "C" dh_status dh_avgpool_forward_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w, const float *data,
                                             size_t batch, size_t channels, size_t img_h, size_t img_w, size_t pool_h,
                                             size_t pool_w, size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w) {
    return dh_dnn::avgpool_forward<float>(ctx, res, res_h, res_w, data, batch, channels, img_h, img_w, pool_h, pool_w, stride_h,
                                       stride_w, pad_h, pad_w);
}
