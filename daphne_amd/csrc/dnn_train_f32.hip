// DNN training kernels, float instantiation. See dnn_train_impl.h for the design and reference citations.
#include "dnn_train_impl.h"

extern "C" dh_status dh_batchnorm_train_forward_f32(dh_ctx *ctx, float *res, float *new_ema_mean, float *new_ema_var, float *mean, float *inv_var,
                                                   const float *in, size_t rows, size_t cols, const float *gamma, const float *beta,
                                                   const float *ema_mean, const float *ema_var, size_t channels, float eps, float mu) {
    return dh_train::batchnorm_train_forward<float>(ctx, res, new_ema_mean, new_ema_var, mean, inv_var, in, rows, cols, gamma, beta,
                                                 ema_mean, ema_var, channels, eps, mu);
}
extern "C" dh_status dh_batchnorm_backward_f32(dh_ctx *ctx, float *dX, float *dGamma, float *dBeta, const float *mean, const float *inv_var,
                                              const float *in, const float *dout, size_t rows, size_t cols, const float *gamma,
                                              size_t channels, float eps) {
    (void)eps; // BatchNorm2DBackward.h:65 takes it and never uses it
    return dh_train::batchnorm_backward<float>(ctx, dX, dGamma, dBeta, mean, inv_var, in, dout, rows, cols, gamma, channels);
}
extern "C" dh_status dh_maxpool_backward_f32(dh_ctx *ctx, float *res, const float *input, const float *dOut, size_t N, size_t C, size_t H,
                                            size_t W, size_t pool_h, size_t pool_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                            size_t pad_w) {
    return dh_train::pool_backward<float, false>(ctx, res, input, dOut, N, C, H, W, pool_h, pool_w, stride_h, stride_w, pad_h, pad_w);
}
extern "C" dh_status dh_avgpool_backward_f32(dh_ctx *ctx, float *res, const float *input, const float *dOut, size_t N, size_t C, size_t H,
                                            size_t W, size_t pool_h, size_t pool_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                            size_t pad_w) {
    return dh_train::pool_backward<float, true>(ctx, res, input, dOut, N, C, H, W, pool_h, pool_w, stride_h, stride_w, pad_h, pad_w);
}
extern "C" dh_status dh_conv2d_backward_data_f32(dh_ctx *ctx, float *dX, const float *filter, const float *dY, size_t N, size_t C, size_t H,
                                                size_t W, size_t F, size_t Hf, size_t Wf, size_t stride_h, size_t stride_w,
                                                size_t pad_h, size_t pad_w) {
    return dh_train::conv2d_backward_data<float>(ctx, dX, filter, dY, N, C, H, W, F, Hf, Wf, stride_h, stride_w, pad_h, pad_w);
}
extern "C" dh_status dh_conv2d_backward_filter_f32(dh_ctx *ctx, float *dW, const float *input, const float *dY, size_t N, size_t C, size_t H,
                                                  size_t W, size_t F, size_t Hf, size_t Wf, size_t stride_h, size_t stride_w,
                                                  size_t pad_h, size_t pad_w) {
    return dh_train::conv2d_backward_filter<float>(ctx, dW, input, dY, N, C, H, W, F, Hf, Wf, stride_h, stride_w, pad_h, pad_w);
}
