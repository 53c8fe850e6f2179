// CPU oracle, part 3: the reference's DNN training kernels (forward of batch normalisation in training mode and the
// backward passes). TEST INFRASTRUCTURE ONLY - the product never links or calls this file.
//
// Restated from the reference's CPU kernels (it has no device versions of these):
//   BatchNorm2DTrainForward.h:66-118, BatchNorm2DBackward.h:63-120, MaxPoolBackward.h:35-82,
//   AvgPoolBackward.h:35-77, Padding.h:6-34, Conv2DBackwardData.h:70-158, Conv2DBackwardFilter.h:68-152.
//
// The loops keep the reference's order of floating-point operations. Two of the reference's kernels are only
// consistent for part of their argument space, and are restated for that part:
//  * Conv2DBackwardData copies the output gradient into its work matrix with the FILTER's extent as loop bounds
//    and row length (GetLossGradientMatrix, :72-82) and bounds its column loop with pad_h (:142): it computes the
//    data gradient only when the output extent equals the filter extent and pad_h == pad_w - the case its own
//    test covers (DNNConv2DBackwardTest.cpp:24-50). Here the gradient is the adjoint of Conv2DForward for every
//    shape, accumulated in the reference's order (filters ascending, filter rows and columns descending), which
//    coincides with the reference where that is consistent.
//  * Conv2DBackwardFilter addresses the filter gradient with p * filter_h + q (:140), correct for square filters;
//    here p * filter_w + q.
//  * Max / average pooling backward take P from stride_w and Q from stride_h like the forward kernels
//    (MaxPoolBackward.h:45-46); windows that would leave the padded image (possible only with unequal strides,
//    where the reference reads and writes out of bounds) are skipped.
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <vector>

namespace {
enum { ST_OK = 0, ST_RUNTIME = 1, ST_INVALID = 2 };

inline size_t get_pq(size_t img, size_t filter, size_t pad, size_t stride) { return (img + 2 * pad - filter) / stride + 1; }

// BatchNorm2DTrainForward.h:66-118. in: N x (C*HW); gamma, beta, ema_mean, ema_var: C values; outputs mean,
// inv_var, new_ema_mean, new_ema_var: C values (the reference allocates C x C matrices and fills the first C).
template <typename T>
int bn_train_forward(T *res, T *new_ema_mean, T *new_ema_var, T *mean_out, T *inv_var, const T *in, size_t N, size_t CHW,
                     const T *gamma, const T *beta, const T *ema_mean, const T *ema_var, size_t C, T eps, T mu) {
    if (C == 0 || CHW % C)
        return ST_INVALID;
    const size_t HW = CHW / C;
    const T m = static_cast<T>(N * HW);
    for (size_t c = 0; c < C; c++) {
        T mean = 0;
        for (size_t i = 0; i < N; i++)
            for (size_t j = 0; j < HW; j++)
                mean = mean + in[i * CHW + c * HW + j] / m;
        T var = 0;
        for (size_t i = 0; i < N; i++)
            for (size_t j = 0; j < HW; j++)
                var = var + std::pow(in[i * CHW + c * HW + j] - mean, T(2)) / m;
        mean_out[c] = mean;
        inv_var[c] = 1 / std::sqrt(var + eps);
        new_ema_mean[c] = (1 - mu) * ema_mean[c] + mu * mean;
        new_ema_var[c] = (1 - mu) * ema_var[c] + mu * var;
        for (size_t i = 0; i < N; i++)
            for (size_t j = 0; j < HW; j++) {
                const size_t off = i * CHW + c * HW + j;
                const T x_hat = (in[off] - mean) / std::sqrt(var + eps);
                res[off] = gamma[c] * x_hat + beta[c];
            }
    }
    return ST_OK;
}

// BatchNorm2DBackward.h:63-120
template <typename T>
int bn_backward(T *dX, T *dGamma, T *dBeta, const T *mean, const T *inv_var, const T *in, const T *dout, size_t N,
                size_t CHW, const T *gamma, size_t C) {
    if (C == 0 || CHW % C)
        return ST_INVALID;
    const size_t HW = CHW / C;
    const T m = static_cast<T>(N * HW);
    const T half = T(1) / T(2), const_2_m = T(2) / m;
    for (size_t c = 0; c < C; c++) {
        T sum_dBeta = 0, sum_dGamma = 0, dVar = 0, dMean = 0;
        for (size_t i = 0; i < N; i++)
            for (size_t j = 0; j < HW; j++) {
                const size_t off = i * CHW + c * HW + j;
                sum_dBeta += dout[off];
                sum_dGamma += dout[off] * (in[off] - mean[c]) * inv_var[c];
                const T dX_hat = dout[off] * gamma[c];
                dVar -= dX_hat * (in[off] - mean[c]) * half * std::pow(inv_var[c], T(3));
            }
        dBeta[c] = sum_dBeta;
        dGamma[c] = sum_dGamma;
        for (size_t i = 0; i < N; i++)
            for (size_t j = 0; j < HW; j++) {
                const size_t off = i * CHW + c * HW + j;
                const T dX_hat = dout[off] * gamma[c];
                dMean += dX_hat * (-inv_var[c]) + dVar * (-const_2_m) * (in[off] - mean[c]);
            }
        for (size_t i = 0; i < N; i++)
            for (size_t j = 0; j < HW; j++) {
                const size_t off = i * CHW + c * HW + j;
                const T dX_hat = dout[off] * gamma[c];
                dX[off] = dX_hat * inv_var[c] + dVar * const_2_m * (in[off] - mean[c]) + dMean / m;
            }
    }
    return ST_OK;
}

// MaxPoolBackward.h:35-82 (AVG = false) and AvgPoolBackward.h:35-77 (AVG = true), scatter form as in the reference
template <typename T, bool AVG>
int pool_backward(T *res, const T *input, const T *dOut, size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw,
                  size_t sh, size_t sw, size_t padh, size_t padw) {
    if (H + 2 * padh < ph || W + 2 * padw < pw || sh == 0 || sw == 0)
        return ST_INVALID;
    const size_t HW = H * W, CHW = C * HW;
    const size_t P = get_pq(H, ph, padh, sw), Q = get_pq(W, pw, padw, sh);
    const size_t CPQ = C * P * Q;
    const size_t pH = H + 2 * padh, pW = W + 2 * padw;
    const T plen = T(1) / static_cast<T>(pw * ph);
    std::vector<T> rp(pH * pW), ip(pH * pW);
    for (size_t i = 0; i < N; i++)
        for (size_t c = 0; c < C; c++) {
            const size_t off_input = i * CHW + c * HW;
            std::fill(rp.begin(), rp.end(), T(0));
            std::fill(ip.begin(), ip.end(), T(0));
            for (size_t h = 0; h < H; h++)
                for (size_t w = 0; w < W; w++)
                    ip[(h + padh) * pW + w + padw] = input[off_input + h * W + w];
            for (size_t p = 0; p < P; p++)
                for (size_t q = 0; q < Q; q++) {
                    if (p * sh + ph > pH || q * sw + pw > pW)
                        continue; // would leave the padded image
                    const T g = dOut[i * CPQ + c * P * Q + p * Q + q];
                    if (AVG) {
                        for (size_t h = 0; h < ph; h++)
                            for (size_t w = 0; w < pw; w++) {
                                const size_t o = (p * sh + h) * pW + q * sw + w;
                                rp[o] = rp[o] + plen * g;
                            }
                    } else {
                        size_t max_index = p * sh * pW + q * sw;
                        for (size_t h = 0; h < ph; h++)
                            for (size_t w = 0; w < pw; w++) {
                                const size_t o = (p * sh + h) * pW + q * sw + w;
                                if (ip[o] > ip[max_index])
                                    max_index = o;
                            }
                        rp[max_index] = rp[max_index] + g;
                    }
                }
            for (size_t h = 0; h < H; h++)
                for (size_t w = 0; w < W; w++)
                    res[off_input + h * W + w] = rp[(h + padh) * pW + w + padw];
        }
    return ST_OK;
}

// Data gradient of Conv2DForward (see the header comment for how this relates to Conv2DBackwardData.h:88-158):
// dX[n][c][h][w] = sum_f sum_r sum_s dY[n][f][p][q] * W[f][c][r][s] with p*sh + r = h + pad_h, q*sw + s = w + pad_w.
template <typename T>
int conv_backward_data(T *dX, const T *filter, const T *dY, size_t N, size_t C, size_t H, size_t W, size_t F, size_t Hf,
                       size_t Wf, size_t sh, size_t sw, size_t padh, size_t padw) {
    if (H + 2 * padh < Hf || W + 2 * padw < Wf || sh == 0 || sw == 0)
        return ST_INVALID;
    const size_t P = get_pq(H, Hf, padh, sh), Q = get_pq(W, Wf, padw, sw);
    for (size_t n = 0; n < N; n++)
        for (size_t c = 0; c < C; c++)
            for (size_t h = 0; h < H; h++)
                for (size_t w = 0; w < W; w++) {
                    T acc = 0;
                    for (size_t f = 0; f < F; f++)
                        for (size_t r = Hf; r-- > 0;)
                            for (size_t s = Wf; s-- > 0;) {
                                const size_t hh = h + padh, ww = w + padw;
                                if (hh < r || ww < s || (hh - r) % sh || (ww - s) % sw)
                                    continue;
                                const size_t p = (hh - r) / sh, q = (ww - s) / sw;
                                if (p >= P || q >= Q)
                                    continue;
                                acc = acc + dY[((n * F + f) * P + p) * Q + q] * filter[((f * C + c) * Hf + r) * Wf + s];
                            }
                    dX[((n * C + c) * H + h) * W + w] = acc;
                }
    return ST_OK;
}

// Conv2DBackwardFilter.h:68-152: dW[f][c][r][s] = sum_n sum_p sum_q Xpad[n][c][p*sh + r][q*sw + s] * dY[n][f][p][q],
// accumulated over images, then output rows, then output columns, as the reference does.
template <typename T>
int conv_backward_filter(T *dW, const T *input, const T *dY, size_t N, size_t C, size_t H, size_t W, size_t F, size_t Hf,
                         size_t Wf, size_t sh, size_t sw, size_t padh, size_t padw) {
    if (H + 2 * padh < Hf || W + 2 * padw < Wf || sh == 0 || sw == 0)
        return ST_INVALID;
    const size_t P = get_pq(H, Hf, padh, sh), Q = get_pq(W, Wf, padw, sw);
    for (size_t f = 0; f < F; f++)
        for (size_t c = 0; c < C; c++)
            for (size_t r = 0; r < Hf; r++)
                for (size_t s = 0; s < Wf; s++) {
                    T acc = 0;
                    for (size_t n = 0; n < N; n++)
                        for (size_t p = 0; p < P; p++)
                            for (size_t q = 0; q < Q; q++) {
                                const size_t hh = p * sh + r, ww = q * sw + s; // padded coordinates
                                if (hh < padh || ww < padw || hh - padh >= H || ww - padw >= W)
                                    continue; // zero border
                                acc = acc + input[((n * C + c) * H + hh - padh) * W + ww - padw] *
                                                dY[((n * F + f) * P + p) * Q + q];
                            }
                    dW[((f * C + c) * Hf + r) * Wf + s] = acc;
                }
    return ST_OK;
}
} // namespace

#define ORACLE_TRAIN_EXPORTS(SUF, T)                                                                                    \
    extern "C" int oracle_batchnorm_train_forward_##SUF(T *res, T *new_ema_mean, T *new_ema_var, T *mean, T *inv_var,   \
                                                        const T *in, size_t N, size_t CHW, const T *gamma,              \
                                                        const T *beta, const T *ema_mean, const T *ema_var, size_t C,   \
                                                        T eps, T mu) {                                                  \
        return bn_train_forward<T>(res, new_ema_mean, new_ema_var, mean, inv_var, in, N, CHW, gamma, beta, ema_mean,    \
                                   ema_var, C, eps, mu);                                                                \
    }                                                                                                                   \
    extern "C" int oracle_batchnorm_backward_##SUF(T *dX, T *dGamma, T *dBeta, const T *mean, const T *inv_var,         \
                                                   const T *in, const T *dout, size_t N, size_t CHW, const T *gamma,    \
                                                   size_t C) {                                                          \
        return bn_backward<T>(dX, dGamma, dBeta, mean, inv_var, in, dout, N, CHW, gamma, C);                            \
    }                                                                                                                   \
    extern "C" int oracle_maxpool_backward_##SUF(T *res, const T *input, const T *dOut, size_t N, size_t C, size_t H,   \
                                                 size_t W, size_t ph, size_t pw, size_t sh, size_t sw, size_t padh,     \
                                                 size_t padw) {                                                         \
        return pool_backward<T, false>(res, input, dOut, N, C, H, W, ph, pw, sh, sw, padh, padw);                       \
    }                                                                                                                   \
    extern "C" int oracle_avgpool_backward_##SUF(T *res, const T *input, const T *dOut, size_t N, size_t C, size_t H,   \
                                                 size_t W, size_t ph, size_t pw, size_t sh, size_t sw, size_t padh,     \
                                                 size_t padw) {                                                         \
        return pool_backward<T, true>(res, input, dOut, N, C, H, W, ph, pw, sh, sw, padh, padw);                        \
    }                                                                                                                   \
    extern "C" int oracle_conv2d_backward_data_##SUF(T *dX, const T *filter, const T *dY, size_t N, size_t C, size_t H, \
                                                     size_t W, size_t F, size_t Hf, size_t Wf, size_t sh, size_t sw,    \
                                                     size_t padh, size_t padw) {                                        \
        return conv_backward_data<T>(dX, filter, dY, N, C, H, W, F, Hf, Wf, sh, sw, padh, padw);                        \
    }                                                                                                                   \
    extern "C" int oracle_conv2d_backward_filter_##SUF(T *dW, const T *input, const T *dY, size_t N, size_t C,          \
                                                       size_t H, size_t W, size_t F, size_t Hf, size_t Wf, size_t sh,   \
                                                       size_t sw, size_t padh, size_t padw) {                           \
        return conv_backward_filter<T>(dW, input, dY, N, C, H, W, F, Hf, Wf, sh, sw, padh, padw);                       \
    }
ORACLE_TRAIN_EXPORTS(f32, float)
ORACLE_TRAIN_EXPORTS(f64, double)
