// DNN training kernels, double instantiation. See dnn_train_impl.h for the design and reference citations.
#include "dnn_train_impl.h"

extern "C" dh_status dh_batchnorm_train_forward_f64(dh_ctx *ctx, double *res, double *new_ema_mean, double *new_ema_var, double *mean, double *inv_var,
                                                   const double *in, size_t rows, size_t cols, const double *gamma, const double *beta,
                                                   const double *ema_mean, const double *ema_var, size_t channels, double eps, double mu) {
    return dh_train::batchnorm_train_forward<double>(ctx, res, new_ema_mean, new_ema_var, mean, inv_var, in, rows, cols, gamma, beta,
                                                 ema_mean, ema_var, channels, eps, mu);
}
extern "C" dh_status dh_batchnorm_backward_f64(dh_ctx *ctx, double *dX, double *dGamma, double *dBeta, const double *mean, const double *inv_var,
                                              const double *in, const double *dout, size_t rows, size_t cols, const double *gamma,
                                              size_t channels, double eps) {
    (void)eps; // BatchNorm2DBackward.h:65 takes it and never uses it
    return dh_train::batchnorm_backward<double>(ctx, dX, dGamma, dBeta, mean, inv_var, in, dout, rows, cols, gamma, channels);
}
extern "C" dh_status dh_maxpool_backward_f64(dh_ctx *ctx, double *res, const double *input, const double *dOut, size_t N, size_t C, size_t H,
                                            size_t W, size_t pool_h, size_t pool_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                            size_t pad_w) {
    return dh_train::pool_backward<double, false>(ctx, res, input, dOut, N, C, H, W, pool_h, pool_w, stride_h, stride_w, pad_h, pad_w);
}
extern "C" dh_status dh_avgpool_backward_f64(dh_ctx *ctx, double *res, const double *input, const double *dOut, size_t N, size_t C, size_t H,
                                            size_t W, size_t pool_h, size_t pool_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                            size_t pad_w) {
    return dh_train::pool_backward<double, true>(ctx, res, input, dOut, N, C, H, W, pool_h, pool_w, stride_h, stride_w, pad_h, pad_w);
}
extern "C" dh_status dh_conv2d_backward_data_f64(dh_ctx *ctx, double *dX, const double *filter, const double *dY, size_t N, size_t C, size_t H,
                                                size_t W, size_t F, size_t Hf, size_t Wf, size_t stride_h, size_t stride_w,
                                                size_t pad_h, size_t pad_w) {
    return dh_train::conv2d_backward_data<double>(ctx, dX, filter, dY, N, C, H, W, F, Hf, Wf, stride_h, stride_w, pad_h, pad_w);
}
extern "C" dh_status dh_conv2d_backward_filter_f64(dh_ctx *ctx, double *dW, const double *input, const double *dY, size_t N, size_t C, size_t H,
                                                  size_t W, size_t F, size_t Hf, size_t Wf, size_t stride_h, size_t stride_w,
                                                  size_t pad_h, size_t pad_w) {
    return dh_train::conv2d_backward_filter<double>(ctx, dW, input, dY, N, C, H, W, F, Hf, Wf, stride_h, stride_w, pad_h, pad_w);
}
