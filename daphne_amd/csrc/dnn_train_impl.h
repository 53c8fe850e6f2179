// DNN training kernels for DenseMatrix<float|double>: batch normalisation in training mode (forward) and the backward
// passes of batch normalisation, max / average pooling and 2-D convolution. The reference has these as CPU kernels
// only (src/runtime/local/kernels/BatchNorm2DTrainForward.h:66-118, BatchNorm2DBackward.h:63-120,
// MaxPoolBackward.h:35-82, AvgPoolBackward.h:35-77, Conv2DBackwardData.h:88-158, Conv2DBackwardFilter.h:68-152);
// these are their device counterparts, data NCHW as rows of images like the forward kernels.
//
// Per-channel statistics are deterministic two-stage reductions with double accumulators (every workgroup owns a
// channel and a slice of the images; a small second kernel folds the slices in order and derives the per-channel
// coefficients); the elementwise passes use one 16-byte vector per thread where the layout allows. No kernel uses
// atomics, so results do not depend on timing:
//   - pooling gradients are gathers (one thread per gradient element, or per vector of them for 2 x 2 windows),
//     visiting the contributions in the reference's order;
//   - the data gradient of a convolution is a forward convolution (stride 1, no border) of the dilated, framed
//     output gradient with the rotated, axis-swapped filters, on the matrix cores;
//   - the filter gradient keeps the image in LDS and contracts over images and pixels on the matrix cores
//     (conv_filter_resident_kernel; partial slabs per workgroup, added in order), or, for shapes that kernel does
//     not take, builds the patch matrix and calls the split-K GEMM;
//   - small problems take plain gather kernels (one thread per gradient element).
//
// Pooling keeps the forward kernels' quirk of taking the output height from stride_w and the width from stride_h
// (MaxPoolBackward.h:45-46). Conv2DBackwardData of the reference is only consistent where the output extent equals
// the filter extent; here it is the adjoint of the forward convolution for every shape, which coincides with the
// reference there (its test vector is reproduced).
#pragma once

#include "dnn_impl.h"

#include <cmath>
#include <type_traits>

namespace dh_train {

constexpr int THREADS = 256;

// ---------------------------------------------------------------------------------------
// per-channel reductions
// ---------------------------------------------------------------------------------------
// MODE 2: sum dy, sum dy*(x - mean[c]), sum (x - mean[c])
// MODE 3: sum (x - s), sum (x - s)^2 with s = the channel's first value: mean and variance from one pass
// A workgroup takes one channel of a slice of images. Its threads walk the (image, vector) positions of that channel
// with a stride of THREADS positions, kept as an (image, vector) pair that is advanced without divisions; four
// positions are loaded before the first is used, positions past the slice read its last image and count as zero.
template <typename T, int MODE, int VEC>
__global__ __launch_bounds__(THREADS) void chan_stage1(const T *x, const T *dy, const T *mean, size_t N, size_t C, size_t HW,
                                                       size_t imgs_per_slice, double *partials /* [C][S][3] */) {
    static_assert(MODE == 2 || MODE == 3, "unknown reduction");
    constexpr int K = MODE == 2 ? 3 : 2;
    constexpr int UN = 4;
    __shared__ double lds[K][THREADS / DH_WAVE];
    const size_t c = blockIdx.x, s = blockIdx.y;
    const size_t n0 = s * imgs_per_slice, n1 = (n0 + imgs_per_slice < N) ? n0 + imgs_per_slice : N;
    const size_t CHW = C * HW;
    const double mu = MODE == 3 ? static_cast<double>(x[c * HW]) : static_cast<double>(mean[c]);
    double a0 = 0.0, a1 = 0.0, a2 = 0.0;
    const size_t imgs = n1 > n0 ? n1 - n0 : 0;
    if (imgs > 0) {
        const size_t cvecs = HW / VEC;
        const size_t dn = THREADS / cvecs, dj = THREADS % cvecs; // one stride, as images and vectors
        size_t n = threadIdx.x / cvecs, j = threadIdx.x % cvecs;
        const T *xc = x + n0 * CHW + c * HW;
        const T *gc = MODE == 2 ? dy + n0 * CHW + c * HW : nullptr;
        while (n < imgs) {
            T v[UN][VEC], g[UN][VEC];
            bool valid[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                valid[u] = n < imgs;
                const size_t off = (valid[u] ? n : imgs - 1) * CHW + j * VEC;
                dh_load_vec<T, VEC>(xc + off, v[u]); // read again by the elementwise pass: no streaming hint
                if constexpr (MODE == 2)
                    dh_load_vec_stream<T, VEC>(gc + off, g[u]);
                n += dn;
                j += dj;
                const bool wrap = j >= cvecs;
                j -= wrap ? cvecs : 0;
                n += wrap ? 1 : 0;
            }
#pragma unroll
            for (int u = 0; u < UN; u++)
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    const double d = valid[u] ? static_cast<double>(v[u][e]) - mu : 0.0;
                    if constexpr (MODE == 3) {
                        a0 += d;
                        a1 += d * d;
                    } else {
                        const double gr = valid[u] ? static_cast<double>(g[u][e]) : 0.0;
                        a0 += gr;
                        a1 += gr * d;
                        a2 += d;
                    }
                }
        }
    }
    double a[3] = {a0, a1, a2};
#pragma unroll
    for (int k = 0; k < K; k++) {
        double v = a[k];
        dh_butterfly(DH_WAVE, [&](auto peer) { v += peer(v); });
        if (threadIdx.x % DH_WAVE == 0)
            lds[k][threadIdx.x / DH_WAVE] = v;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < K; k++) {
            double v = 0.0;
            for (int w = 0; w < THREADS / DH_WAVE; w++)
                v += lds[k][w];
            partials[(c * gridDim.y + s) * 3 + k] = v;
        }
    }
}

template <typename T, int MODE>
static inline void launch_stage1(dh_ctx *ctx, dim3 grid, const T *x, const T *dy, const T *mean, size_t N, size_t C, size_t HW,
                                 size_t imgs_per_slice, double *partials) {
    constexpr int V = dh_vec<T>::N;
    if (HW % V == 0 && dh_aligned(x, 16) && (MODE != 2 || dh_aligned(dy, 16)))
        hipLaunchKernelGGL((chan_stage1<T, MODE, V>), grid, dim3(THREADS), 0, ctx->stream, x, dy, mean, N, C, HW, imgs_per_slice,
                           partials);
    else
        hipLaunchKernelGGL((chan_stage1<T, MODE, 1>), grid, dim3(THREADS), 0, ctx->stream, x, dy, mean, N, C, HW, imgs_per_slice,
                           partials);
}

// Folds the slices of every channel (one thread per channel, slices in order) and derives what the next pass needs.
// STEP 0: mean[c] = sum / m.
// STEP 1: var = sum / m; inv_var, moving averages; coef[c] = sqrt(var + eps) for the normalisation pass.
// STEP 2: dBeta, dGamma and coef[c][0..1] = dVar * 2/m, dMean / m for the gradient pass.
// STEP 3: STEP 0 and STEP 1 from the shifted sums of MODE 3 (x0 = the input, whose first value per channel is the shift).
template <typename T, int STEP>
__global__ void chan_stage2(const double *partials, size_t C, size_t S, double m, T *mean, T *inv_var, T *new_ema_mean,
                            T *new_ema_var, const T *ema_mean, const T *ema_var, T eps, T mu_, const T *gamma, T *dGamma,
                            T *dBeta, T *coef, const T *x0 = nullptr, size_t HW = 0) {
    const size_t c = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= C)
        return;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0;
    for (size_t s = 0; s < S; s++) {
        s0 += partials[(c * S + s) * 3 + 0];
        if (STEP == 3)
            s1 += partials[(c * S + s) * 3 + 1];
        if (STEP == 2) {
            s1 += partials[(c * S + s) * 3 + 1];
            s2 += partials[(c * S + s) * 3 + 2];
        }
    }
    if constexpr (STEP == 0) {
        mean[c] = static_cast<T>(s0 / m);
    } else if constexpr (STEP == 1 || STEP == 3) {
        T var, mn;
        if constexpr (STEP == 3) {
            const double d = s0 / m; // mean - shift
            mn = static_cast<T>(static_cast<double>(x0[c * HW]) + d);
            const double v = s1 / m - d * d;
            var = static_cast<T>(v > 0.0 ? v : 0.0);
            mean[c] = mn;
        } else {
            var = static_cast<T>(s0 / m);
            mn = mean[c];
        }
        const T sd = sizeof(T) == 4 ? static_cast<T>(sqrtf(static_cast<float>(var + eps))) : static_cast<T>(sqrt(static_cast<double>(var + eps)));
        inv_var[c] = T(1) / sd;
        new_ema_mean[c] = (T(1) - mu_) * ema_mean[c] + mu_ * mn;
        new_ema_var[c] = (T(1) - mu_) * ema_var[c] + mu_ * var;
        coef[c] = sd;
    } else {
        // BatchNorm2DBackward.h:88-118 with the sums taken out of the loops
        const double iv = static_cast<double>(inv_var[c]), g = static_cast<double>(gamma[c]);
        dBeta[c] = static_cast<T>(s0);
        dGamma[c] = static_cast<T>(s1 * iv);
        const double dVar = -(g * s1) * 0.5 * iv * iv * iv;
        const double c2m = 2.0 / m;
        const double dMean = -(g * s0) * iv + dVar * (-c2m) * s2;
        coef[2 * c] = static_cast<T>(dVar * c2m);
        coef[2 * c + 1] = static_cast<T>(dMean / m);
    }
}

// Elementwise passes over the (N*C) x HW view. FWD: res = gamma * ((x - mean) / sd) + beta
// (BatchNorm2DTrainForward.h:108-115). Else: dX = (dy * gamma) * inv_var + coef0 * (x - mean) + coef1
// (BatchNorm2DBackward.h:110-118).
// The rows are taken from the last to the first: the reduction pass before it went through x from the first image to
// the last, so the end of x is what the memory-side cache still holds (8 % of the two passes' time at 4096 x 64 x 14 x 14).
template <typename T, int VEC, bool FWD>
__global__ __launch_bounds__(THREADS) void chan_apply(T *res, const T *x, const T *dy, size_t rows, size_t C, size_t HW,
                                                      const T *mean, const T *gamma, const T *beta, const T *inv_var,
                                                      const T *coef) {
    const size_t cvecs = HW / VEC;
    const size_t r = static_cast<size_t>(gridDim.x - 1 - blockIdx.x) * blockDim.y + threadIdx.y;
    if (r >= rows)
        return;
    // 32-bit remainder where the row count allows (uniform)
    const size_t c = rows <= 0xffffffffull ? static_cast<unsigned>(r) % static_cast<unsigned>(C) : r % C;
    const T mn = mean[c], g = gamma[c];
    const T p0 = FWD ? coef[c] : inv_var[c], p1 = FWD ? beta[c] : coef[2 * c], p2 = FWD ? T(0) : coef[2 * c + 1];
    for (size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x; cv < cvecs;
         cv += static_cast<size_t>(gridDim.y) * blockDim.x) {
        T a[VEC], b[VEC], o[VEC];
        dh_load_vec<T, VEC>(x + r * HW + cv * VEC, a);
        if constexpr (!FWD)
            dh_load_vec_stream<T, VEC>(dy + r * HW + cv * VEC, b);
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            if constexpr (FWD)
                o[i] = g * ((a[i] - mn) / p0) + p1;
            else
                o[i] = (b[i] * g) * p0 + p1 * (a[i] - mn) + p2;
        }
        dh_store_vec_stream<T, VEC>(res + r * HW + cv * VEC, o);
    }
}

// Both passes from ONE read where a channel's values (all images) fit a workgroup's LDS: the workgroup of a channel
// copies them in, adds up what the channel's statistics need (in double, threads in a fixed order), derives the
// channel's coefficients in one thread and applies them to the copy. FWD: the sums of chan_stage1 MODE 3 and the
// arithmetic of chan_stage2 STEP 3 and chan_apply; else MODE 2, STEP 2 and the gradient form, with dy in LDS beside x.
template <typename T, bool FWD>
__global__ __launch_bounds__(512) void chan_lds_kernel(T *res, const T *x, const T *dy, unsigned N, unsigned C, unsigned HW, T *mean,
                                                       T *inv_var, T *new_ema_mean, T *new_ema_var, const T *ema_mean,
                                                       const T *ema_var, T eps, T mu_, const T *gamma, const T *beta, T *dGamma,
                                                       T *dBeta) {
    extern __shared__ __attribute__((aligned(16))) unsigned char chan_lds[];
    T *sx = reinterpret_cast<T *>(chan_lds);
    __shared__ double red[3][8];
    __shared__ T coef[4];
    const unsigned c = blockIdx.x, tid = threadIdx.x, n_el = N * HW;
    T *sdy = sx + n_el;
    // a thread's positions, 512 apart, as (image, position in the plane) pairs advanced without divisions
    const unsigned dn = 512 / HW, dj = 512 % HW;
    {
        unsigned n = tid / HW, j = tid % HW;
        for (unsigned idx = tid; idx < n_el; idx += 512) {
            const size_t off = (static_cast<size_t>(n) * C + c) * HW + j;
            sx[idx] = x[off];
            if constexpr (!FWD)
                sdy[idx] = dy[off];
            n += dn;
            j += dj;
            const bool wrap = j >= HW;
            j -= wrap ? HW : 0;
            n += wrap ? 1 : 0;
        }
    }
    __syncthreads();
    const double shift = FWD ? static_cast<double>(sx[0]) : static_cast<double>(mean[c]);
    double a[3] = {0.0, 0.0, 0.0};
    for (unsigned idx = tid; idx < n_el; idx += 512) {
        const double d = static_cast<double>(sx[idx]) - shift;
        if constexpr (FWD) {
            a[0] += d;
            a[1] += d * d;
        } else {
            const double gr = static_cast<double>(sdy[idx]);
            a[0] += gr;
            a[1] += gr * d;
            a[2] += d;
        }
    }
#pragma unroll
    for (int k = 0; k < 3; k++) {
        double v = a[k];
        dh_butterfly(DH_WAVE, [&](auto peer) { v += peer(v); });
        if (tid % DH_WAVE == 0)
            red[k][tid / DH_WAVE] = v;
    }
    __syncthreads();
    if (tid == 0) {
        double s[3];
#pragma unroll
        for (int k = 0; k < 3; k++) {
            s[k] = 0.0;
            for (int w = 0; w < 8; w++)
                s[k] += red[k][w];
        }
        const double m = static_cast<double>(n_el);
        if constexpr (FWD) {
            // BatchNorm2DTrainForward.h:84-106 from the shifted sums
            const double d = s[0] / m; // mean - shift
            const T mn = static_cast<T>(shift + d);
            const double v = s[1] / m - d * d;
            const T var = static_cast<T>(v > 0.0 ? v : 0.0);
            const T sd = sizeof(T) == 4 ? static_cast<T>(sqrtf(static_cast<float>(var + eps))) : static_cast<T>(sqrt(static_cast<double>(var + eps)));
            mean[c] = mn;
            inv_var[c] = T(1) / sd;
            new_ema_mean[c] = (T(1) - mu_) * ema_mean[c] + mu_ * mn;
            new_ema_var[c] = (T(1) - mu_) * ema_var[c] + mu_ * var;
            coef[0] = mn;
            coef[1] = sd;
        } else {
            // BatchNorm2DBackward.h:88-118 with the sums taken out of the loops
            const double iv = static_cast<double>(inv_var[c]), g = static_cast<double>(gamma[c]);
            dBeta[c] = static_cast<T>(s[0]);
            dGamma[c] = static_cast<T>(s[1] * iv);
            const double dVar = -(g * s[1]) * 0.5 * iv * iv * iv;
            const double c2m = 2.0 / m;
            const double dMean = -(g * s[0]) * iv + dVar * (-c2m) * s[2];
            coef[0] = static_cast<T>(dVar * c2m);
            coef[1] = static_cast<T>(dMean / m);
        }
    }
    __syncthreads();
    const T g = gamma[c];
    const T p0 = coef[0], p1 = coef[1];
    const T mn = FWD ? p0 : mean[c], ivc = FWD ? T(0) : inv_var[c], bt = FWD ? beta[c] : T(0);
    unsigned n = tid / HW, j = tid % HW;
    for (unsigned idx = tid; idx < n_el; idx += 512) {
        const size_t off = (static_cast<size_t>(n) * C + c) * HW + j;
        const T xv = sx[idx];
        if constexpr (FWD)
            res[off] = g * ((xv - mn) / p1) + bt;
        else
            res[off] = (sdy[idx] * g) * ivc + p0 * (xv - mn) + p1;
        n += dn;
        j += dj;
        const bool wrap = j >= HW;
        j -= wrap ? HW : 0;
        n += wrap ? 1 : 0;
    }
}

// Whether a channel's values fit: at most 64 KB of LDS (two workgroups a CU), enough channels to occupy the device or a
// tensor so small that the launches of the general path would cost more than idle CUs.
static inline bool chan_fits_lds(const dh_ctx *ctx, size_t N, size_t C, size_t HW, size_t elem, int arrays) {
    const size_t slice = N * HW * elem * arrays;
    return slice <= (size_t(64) << 10) && N * HW < (size_t(1) << 31) && C < (size_t(1) << 31) &&
           (C * 4 >= static_cast<size_t>(ctx->num_cus) || slice * C <= (size_t(8) << 20));
}

struct ChanPlan {
    size_t S, imgs_per_slice;
};
static inline ChanPlan chan_plan(const dh_ctx *ctx, size_t N, size_t C) {
    // about eight workgroups per CU over all channels, every slice at least one image
    size_t S = dh_ceil_div(static_cast<size_t>(ctx->num_cus) * 8, C);
    if (S > N)
        S = N;
    if (S < 1)
        S = 1;
    if (S > 65535)
        S = 65535;
    ChanPlan p;
    p.imgs_per_slice = dh_ceil_div(N, S);
    p.S = dh_ceil_div(N, p.imgs_per_slice);
    return p;
}

template <typename T, bool FWD>
static inline void launch_apply(dh_ctx *ctx, T *res, const T *x, const T *dy, size_t rows, size_t C, size_t HW, const T *mean,
                                const T *gamma, const T *beta, const T *inv_var, const T *coef) {
    constexpr int V = dh_vec<T>::N;
    const bool vec_ok = HW % V == 0 && dh_aligned(res, 16) && dh_aligned(x, 16) && (FWD || dh_aligned(dy, 16));
    const size_t cvecs = vec_ok ? HW / V : HW;
    unsigned tx = 1;
    while (tx < THREADS && tx < cvecs)
        tx <<= 1;
    const unsigned ty = THREADS / tx;
    size_t gy = dh_ceil_div(cvecs, tx);
    if (gy > 65535)
        gy = 65535;
    const dim3 grid(static_cast<unsigned>(dh_ceil_div(rows, static_cast<size_t>(ty))), static_cast<unsigned>(gy)), block(tx, ty);
    if (vec_ok)
        hipLaunchKernelGGL((chan_apply<T, V, FWD>), grid, block, 0, ctx->stream, res, x, dy, rows, C, HW, mean, gamma, beta,
                           inv_var, coef);
    else
        hipLaunchKernelGGL((chan_apply<T, 1, FWD>), grid, block, 0, ctx->stream, res, x, dy, rows, C, HW, mean, gamma, beta,
                           inv_var, coef);
}

template <typename T>
dh_status batchnorm_train_forward(dh_ctx *ctx, T *res, T *new_ema_mean, T *new_ema_var, T *mean, T *inv_var, const T *in,
                                  size_t rows, size_t cols, const T *gamma, const T *beta, const T *ema_mean, const T *ema_var,
                                  size_t C, T eps, T mu) {
    DH_REQUIRE_CTX(ctx);
    if (C == 0 || cols % C != 0)
        return dh_fail(DH_ERR_INVALID_ARG, "BatchNorm2DTrainForward - the number of columns (%zu) is not a multiple of the channel count (%zu)", cols, C);
    if (rows == 0 || cols == 0)
        return DH_OK;
    if (rows * (cols / C) >= (size_t(1) << 31) * C && rows >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "BatchNorm2DTrainForward - too many images");
    const size_t HW = cols / C;
    if (chan_fits_lds(ctx, rows, C, HW, sizeof(T), 1)) {
        hipLaunchKernelGGL((chan_lds_kernel<T, true>), dim3(static_cast<unsigned>(C)), dim3(512), rows * HW * sizeof(T), ctx->stream, res, in,
                           static_cast<const T *>(nullptr), static_cast<unsigned>(rows), static_cast<unsigned>(C),
                           static_cast<unsigned>(HW), mean, inv_var, new_ema_mean, new_ema_var, ema_mean, ema_var, eps, mu, gamma, beta,
                           static_cast<T *>(nullptr), static_cast<T *>(nullptr));
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    const ChanPlan p = chan_plan(ctx, rows, C);
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, C * p.S * 3 * sizeof(double) + 2 * C * sizeof(T) + 256, &wsv);
    if (st != DH_OK)
        return st;
    double *partials = static_cast<double *>(wsv);
    T *coef = reinterpret_cast<T *>(partials + C * p.S * 3);
    const double m = static_cast<double>(rows) * static_cast<double>(HW);
    const dim3 g1(static_cast<unsigned>(C), static_cast<unsigned>(p.S)), g2(static_cast<unsigned>(dh_ceil_div(C, 64)));
    // mean and variance from ONE pass: sums of (x - s) and (x - s)^2 around the channel's first value, in double
    launch_stage1<T, 3>(ctx, g1, in, nullptr, nullptr, rows, C, HW, p.imgs_per_slice, partials);
    hipLaunchKernelGGL((chan_stage2<T, 3>), g2, dim3(64), 0, ctx->stream, partials, C, p.S, m, mean, inv_var, new_ema_mean,
                       new_ema_var, ema_mean, ema_var, eps, mu, gamma, nullptr, nullptr, coef, in, HW);
    launch_apply<T, true>(ctx, res, in, nullptr, rows * C, C, HW, mean, gamma, beta, inv_var, coef);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T>
dh_status batchnorm_backward(dh_ctx *ctx, T *dX, T *dGamma, T *dBeta, const T *mean, const T *inv_var, const T *in, const T *dout,
                             size_t rows, size_t cols, const T *gamma, size_t C) {
    DH_REQUIRE_CTX(ctx);
    if (C == 0 || cols % C != 0)
        return dh_fail(DH_ERR_INVALID_ARG, "BatchNorm2DBackward - the number of columns (%zu) is not a multiple of the channel count (%zu)", cols, C);
    if (rows == 0 || cols == 0)
        return DH_OK;
    const size_t HW = cols / C;
    if (chan_fits_lds(ctx, rows, C, HW, sizeof(T), 2)) {
        hipLaunchKernelGGL((chan_lds_kernel<T, false>), dim3(static_cast<unsigned>(C)), dim3(512), 2 * rows * HW * sizeof(T), ctx->stream, dX,
                           in, dout, static_cast<unsigned>(rows), static_cast<unsigned>(C), static_cast<unsigned>(HW),
                           const_cast<T *>(mean), const_cast<T *>(inv_var), static_cast<T *>(nullptr), static_cast<T *>(nullptr),
                           static_cast<const T *>(nullptr), static_cast<const T *>(nullptr), T(0), T(0), gamma,
                           static_cast<const T *>(nullptr), dGamma, dBeta);
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    const ChanPlan p = chan_plan(ctx, rows, C);
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, C * p.S * 3 * sizeof(double) + 2 * C * sizeof(T) + 256, &wsv);
    if (st != DH_OK)
        return st;
    double *partials = static_cast<double *>(wsv);
    T *coef = reinterpret_cast<T *>(partials + C * p.S * 3);
    const double m = static_cast<double>(rows) * static_cast<double>(HW);
    const dim3 g1(static_cast<unsigned>(C), static_cast<unsigned>(p.S)), g2(static_cast<unsigned>(dh_ceil_div(C, 64)));
    launch_stage1<T, 2>(ctx, g1, in, dout, mean, rows, C, HW, p.imgs_per_slice, partials);
    hipLaunchKernelGGL((chan_stage2<T, 2>), g2, dim3(64), 0, ctx->stream, partials, C, p.S, m, const_cast<T *>(mean),
                       const_cast<T *>(inv_var), nullptr, nullptr, nullptr, nullptr, T(0), T(0), gamma, dGamma, dBeta, coef);
    launch_apply<T, false>(ctx, dX, in, dout, rows * C, C, HW, mean, gamma, nullptr, inv_var, coef);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// pooling backward (gather form)
// ---------------------------------------------------------------------------------------
struct PoolBwdArgs {
    unsigned C, H, W, P, Q, ph, pw, sh, sw, padh, padw;
    size_t total; // N*C*H*W
};

template <typename T, bool AVG>
__global__ __launch_bounds__(THREADS) void pool_backward_kernel(T *res, const T *input, const T *dOut, PoolBwdArgs g) {
#pragma clang fp contract(off) // plen * g is rounded before it is added, as on the host
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= g.total)
        return;
    const unsigned HW = g.H * g.W;
    size_t img; // (n, c) plane
    unsigned hw;
    if (g.total <= 0xffffffffull) { // 32-bit divisions suffice (uniform)
        img = static_cast<unsigned>(idx) / HW;
        hw = static_cast<unsigned>(idx) % HW;
    } else {
        img = idx / HW;
        hw = static_cast<unsigned>(idx % HW);
    }
    const unsigned h = hw / g.W, w = hw % g.W;
    const unsigned hp = h + g.padh, wp = w + g.padw; // position in the zero-padded plane
    const unsigned pH = g.H + 2 * g.padh, pW = g.W + 2 * g.padw;
    const T *plane = input + img * HW;
    const T *dplane = dOut + img * (static_cast<size_t>(g.P) * g.Q);
    const T plen = T(1) / static_cast<T>(g.pw * g.ph);
    // windows (p, q) that contain (hp, wp): p*sh <= hp < p*sh + ph
    const unsigned p_lo = hp + 1 > g.ph ? (hp + 1 - g.ph + g.sh - 1) / g.sh : 0, q_lo = wp + 1 > g.pw ? (wp + 1 - g.pw + g.sw - 1) / g.sw : 0;
    unsigned p_hi = hp / g.sh, q_hi = wp / g.sw;
    if (p_hi >= g.P)
        p_hi = g.P - 1;
    if (q_hi >= g.Q)
        q_hi = g.Q - 1;
    auto val = [&](unsigned a, unsigned b) -> T { // padded plane
        return (a >= g.padh && b >= g.padw && a - g.padh < g.H && b - g.padw < g.W) ? plane[(a - g.padh) * g.W + (b - g.padw)] : T(0);
    };
    T acc = T(0);
    for (unsigned p = p_lo; p <= p_hi && p < g.P; p++)
        for (unsigned q = q_lo; q <= q_hi && q < g.Q; q++) {
            if (p * g.sh + g.ph > pH || q * g.sw + g.pw > pW)
                continue; // window would leave the padded plane
            const T gr = dplane[p * g.Q + q];
            if constexpr (AVG) {
                acc = acc + plen * gr;
            } else {
                // first maximum in row-major order, found with a strict comparison starting from the window origin
                unsigned ma = p * g.sh, mb = q * g.sw;
                T mv = val(ma, mb);
                for (unsigned a = 0; a < g.ph; a++)
                    for (unsigned b = 0; b < g.pw; b++) {
                        const T v = val(p * g.sh + a, q * g.sw + b);
                        if (v > mv) {
                            mv = v;
                            ma = p * g.sh + a;
                            mb = q * g.sw + b;
                        }
                    }
                if (ma == hp && mb == wp)
                    acc = acc + gr;
            }
        }
    res[idx] = acc;
}

// AvgPool gradient of 2x2 windows with stride 2 (no padding, even H and W). Planes are contiguous, so the result is
// a flat list of value pairs, Q = W / 2 to an image row, and pair (row, q) is twice a quarter of gradient
// (row / 2, q). A thread writes ONE vector of VI / 2 pairs and consecutive threads write consecutive vectors; both
// image rows of a window row read the same Q gradients.
template <typename T, int VI>
__global__ __launch_bounds__(THREADS) void avgpool2x2_backward_kernel(T *res, const T *dOut, unsigned Q, size_t total) {
#pragma clang fp contract(off)
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total)
        return;
    const bool small = total * (VI / 2) <= 0xffffffffull; // 32-bit divisions suffice (uniform)
    T g[VI / 2];
#pragma unroll
    for (int k = 0; k < VI / 2; k++) {
        const size_t pair = idx * (VI / 2) + k;
        size_t row; // image row over all planes
        unsigned q;
        if (small) {
            row = static_cast<unsigned>(pair) / Q;
            q = static_cast<unsigned>(pair) % Q;
        } else {
            row = pair / Q;
            q = static_cast<unsigned>(pair % Q);
        }
        g[k] = dOut[(row >> 1) * Q + q];
    }
    typedef T vec_t __attribute__((ext_vector_type(VI)));
    vec_t w;
#pragma unroll
    for (int k = 0; k < VI / 2; k++)
        w[2 * k] = w[2 * k + 1] = (T(1) / T(4)) * g[k];
    __builtin_nontemporal_store(w, reinterpret_cast<vec_t *>(res + idx * VI));
}

// MaxPool gradient of 2x2 windows with stride 2 (no padding, even H and W), flat like the average above: a thread
// writes one vector of VI / 2 value pairs of the result. For each pair it reads both rows of the pair's window (the
// other image row of the window asks for the same values; they come from the cache) and the window's gradient, and
// keeps the gradient where the first maximum of the window (row-major order, strict comparison,
// MaxPoolBackward.h:62-69) lies in its own row.
template <typename T, int VI>
__global__ __launch_bounds__(THREADS) void maxpool2x2_backward_kernel(T *res, const T *input, const T *dOut, unsigned Q,
                                                                           size_t total) {
    typedef T pair_t __attribute__((ext_vector_type(2)));
    typedef T vec_t __attribute__((ext_vector_type(VI)));
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total)
        return;
    const bool small = total * (VI / 2) <= 0xffffffffull; // 32-bit divisions suffice (uniform)
    pair_t top[VI / 2], bot[VI / 2];
    T g[VI / 2];
    bool lower[VI / 2]; // this pair lies in the window's second row
#pragma unroll
    for (int k = 0; k < VI / 2; k++) {
        const size_t pair = idx * (VI / 2) + k;
        size_t row; // image row over all planes
        unsigned q;
        if (small) {
            row = static_cast<unsigned>(pair) / Q;
            q = static_cast<unsigned>(pair) % Q;
        } else {
            row = pair / Q;
            q = static_cast<unsigned>(pair % Q);
        }
        const size_t wrow = row >> 1;
        const T *x0 = input + wrow * 4 * Q + 2 * q; // an image row holds 2 * Q values
        top[k] = *reinterpret_cast<const pair_t *>(x0);
        bot[k] = *reinterpret_cast<const pair_t *>(x0 + 2 * Q);
        g[k] = dOut[wrow * Q + q];
        lower[k] = (row & 1) != 0;
    }
    vec_t w;
#pragma unroll
    for (int k = 0; k < VI / 2; k++) {
        int best = 0;
        T m = top[k][0];
        if (top[k][1] > m) {
            m = top[k][1];
            best = 1;
        }
        if (bot[k][0] > m) {
            m = bot[k][0];
            best = 2;
        }
        if (bot[k][1] > m)
            best = 3;
        const int first = lower[k] ? 2 : 0;
        w[2 * k] = best == first ? g[k] : T(0);
        w[2 * k + 1] = best == first + 1 ? g[k] : T(0);
    }
    __builtin_nontemporal_store(w, reinterpret_cast<vec_t *>(res + idx * VI));
}

template <typename T, bool AVG>
dh_status pool_backward(dh_ctx *ctx, T *res, const T *input, const T *dOut, size_t N, size_t C, size_t H, size_t W, size_t ph,
                        size_t pw, size_t sh, size_t sw, size_t padh, size_t padw) {
    DH_REQUIRE_CTX(ctx);
    if (H + 2 * padh < ph || W + 2 * padw < pw || sh == 0 || sw == 0 || ph == 0 || pw == 0)
        return dh_fail(DH_ERR_INVALID_ARG, "Pooling backward - window, stride and padding do not fit the image");
    if ((H | W | C | ph | pw | sh | sw | padh | padw) >> 30)
        return dh_fail(DH_ERR_RUNTIME, "Pooling backward - extents beyond 2^30 are not supported");
    PoolBwdArgs g;
    g.C = C, g.H = H, g.W = W, g.ph = ph, g.pw = pw, g.sh = sh, g.sw = sw, g.padh = padh, g.padw = padw;
    g.P = static_cast<unsigned>((H + 2 * padh - ph) / sw + 1); // stride_w for the height, as in the reference
    g.Q = static_cast<unsigned>((W + 2 * padw - pw) / sh + 1);
    g.total = N * C * H * W;
    if (g.total == 0)
        return DH_OK;
    constexpr int VFULL = dh_vec<T>::N;
    if (ph == 2 && pw == 2 && sh == 2 && sw == 2 && padh == 0 && padw == 0 && H % 2 == 0 && W % 2 == 0 &&
        dh_aligned(res, 16) && (AVG || dh_aligned(input, 2 * sizeof(T)))) {
        const size_t total = g.total / VFULL; // H and W are even: H * W is a multiple of four
        if (dh_ceil_div(total, THREADS) < (size_t(1) << 31)) {
            const dim3 grid(static_cast<unsigned>(dh_ceil_div(total, THREADS)));
            if constexpr (AVG)
                hipLaunchKernelGGL((avgpool2x2_backward_kernel<T, VFULL>), grid, dim3(THREADS), 0, ctx->stream, res, dOut,
                                   static_cast<unsigned>(W / 2), total);
            else
                hipLaunchKernelGGL((maxpool2x2_backward_kernel<T, VFULL>), grid, dim3(THREADS), 0, ctx->stream, res, input,
                                   dOut, static_cast<unsigned>(W / 2), total);
            DH_CHECK_LAUNCH();
            return DH_OK;
        }
    }
    const size_t blocks = dh_ceil_div(g.total, THREADS);
    if (blocks >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Pooling backward - too many elements for one launch");
    hipLaunchKernelGGL((pool_backward_kernel<T, AVG>), dim3(static_cast<unsigned>(blocks)), dim3(THREADS), 0, ctx->stream, res,
                       input, dOut, g);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// convolution backward
// ---------------------------------------------------------------------------------------
struct ConvBwdArgs {
    unsigned N, C, H, W, F, Hf, Wf, P, Q, sh, sw, padh, padw;
};

// dX[n][c][h][w] = sum_f sum_r sum_s dY[n][f][p][q] * Wt[f][c][r][s], p*sh + r = h + padh, q*sw + s = w + padw;
// one thread per element, filters ascending and filter rows / columns descending like the reference's rotated filter.
template <typename T> __global__ __launch_bounds__(THREADS) void conv_backward_data_kernel(T *dX, const T *filter, const T *dY, ConvBwdArgs g) {
    const size_t total = static_cast<size_t>(g.N) * g.C * g.H * g.W;
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total)
        return;
    const unsigned HW = g.H * g.W, PQ = g.P * g.Q;
    const size_t nc = idx / HW;
    const unsigned n = static_cast<unsigned>(nc / g.C), c = static_cast<unsigned>(nc % g.C);
    const unsigned hw = static_cast<unsigned>(idx % HW), hh = hw / g.W + g.padh, ww = hw % g.W + g.padw;
    const T *dyn = dY + static_cast<size_t>(n) * g.F * PQ;
    T acc = T(0);
    for (unsigned f = 0; f < g.F; f++) {
        const T *wf = filter + (static_cast<size_t>(f) * g.C + c) * g.Hf * g.Wf;
        const T *dyf = dyn + static_cast<size_t>(f) * PQ;
        for (unsigned r = g.Hf; r-- > 0;) {
            if (hh < r || (hh - r) % g.sh)
                continue;
            const unsigned p = (hh - r) / g.sh;
            if (p >= g.P)
                continue;
            for (unsigned s = g.Wf; s-- > 0;) {
                if (ww < s || (ww - s) % g.sw)
                    continue;
                const unsigned q = (ww - s) / g.sw;
                if (q >= g.Q)
                    continue;
                acc = acc + dyf[p * g.Q + q] * wf[r * g.Wf + s];
            }
        }
    }
    dX[idx] = acc;
}

// dW[f][c][r][s] = sum_n sum_p sum_q Xpad[n][c][p*sh + r][q*sw + s] * dY[n][f][p][q]. One workgroup per (f, c): its
// threads walk over (n, p, q), each keeping the partial sums of up to TAPS filter taps in registers (larger filters
// take several rounds); the partial sums are folded through LDS in a fixed order, in double.
template <typename T, int TAPS>
__global__ __launch_bounds__(THREADS) void conv_backward_filter_kernel(T *dW, const T *input, const T *dY, ConvBwdArgs g) {
    __shared__ double lds[THREADS / DH_WAVE][TAPS];
    const unsigned f = blockIdx.x / g.C, c = blockIdx.x % g.C;
    const unsigned HW = g.H * g.W, PQ = g.P * g.Q, taps = g.Hf * g.Wf;
    const size_t items = static_cast<size_t>(g.N) * PQ;
    for (unsigned t0 = 0; t0 < taps; t0 += TAPS) {
        double acc[TAPS];
#pragma unroll
        for (int t = 0; t < TAPS; t++)
            acc[t] = 0.0;
        for (size_t i = threadIdx.x; i < items; i += THREADS) {
            const unsigned n = static_cast<unsigned>(i / PQ), pq = static_cast<unsigned>(i % PQ), p = pq / g.Q, q = pq % g.Q;
            const double gr = static_cast<double>(dY[(static_cast<size_t>(n) * g.F + f) * PQ + pq]);
            const T *plane = input + (static_cast<size_t>(n) * g.C + c) * HW;
#pragma unroll
            for (int t = 0; t < TAPS; t++) {
                const unsigned tap = t0 + t;
                if (tap < taps) {
                    const unsigned hh = p * g.sh + tap / g.Wf, ww = q * g.sw + tap % g.Wf;
                    if (hh >= g.padh && ww >= g.padw && hh - g.padh < g.H && ww - g.padw < g.W)
                        acc[t] += static_cast<double>(plane[(hh - g.padh) * g.W + (ww - g.padw)]) * gr;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < TAPS; t++) {
            double v = acc[t];
            dh_butterfly(DH_WAVE, [&](auto peer) { v += peer(v); });
            if (threadIdx.x % DH_WAVE == 0)
                lds[threadIdx.x / DH_WAVE][t] = v;
        }
        __syncthreads();
        if (threadIdx.x < TAPS && t0 + threadIdx.x < taps) {
            double v = 0.0;
            for (int w = 0; w < THREADS / DH_WAVE; w++)
                v += lds[w][threadIdx.x];
            dW[(static_cast<size_t>(f) * g.C + c) * taps + t0 + threadIdx.x] = static_cast<T>(v);
        }
        __syncthreads();
    }
}

static inline dh_status conv_bwd_args(ConvBwdArgs *g, size_t N, size_t C, size_t H, size_t W, size_t F, size_t Hf, size_t Wf,
                                      size_t sh, size_t sw, size_t padh, size_t padw) {
    if (H + 2 * padh < Hf || W + 2 * padw < Wf || sh == 0 || sw == 0 || Hf == 0 || Wf == 0)
        return dh_fail(DH_ERR_INVALID_ARG, "Conv2D backward - filter, stride and padding do not fit the image");
    if ((N | C | H | W | F | Hf | Wf | sh | sw | padh | padw) >> 30)
        return dh_fail(DH_ERR_RUNTIME, "Conv2D backward - extents beyond 2^30 are not supported");
    g->N = N, g->C = C, g->H = H, g->W = W, g->F = F, g->Hf = Hf, g->Wf = Wf, g->sh = sh, g->sw = sw, g->padh = padh, g->padw = padw;
    g->P = static_cast<unsigned>((H + 2 * padh - Hf) / sh + 1);
    g->Q = static_cast<unsigned>((W + 2 * padw - Wf) / sw + 1);
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// convolution gradients on the matrix cores
// ---------------------------------------------------------------------------------------
// Both gradients are contractions, so they are handed to the kernels that already run them on the matrix cores:
//  * data:   dX = forward convolution (stride 1, no padding) of the output gradient - dilated by the stride and
//            placed in a zero frame of (H + Hf - 1) x (W + Wf - 1) - with the filters rotated by 180 degrees and
//            their filter / channel axes exchanged;
//  * filter: dW (F x C*Hf*Wf) = dY as an F x (N*P*Q) matrix times the patch matrix (N*P*Q) x (C*Hf*Wf) of the input.
// The sums then run in the order of those kernels (results agree with the gather kernels above to rounding). The
// temporaries come from the context's block cache; shapes whose temporaries would be very large, or padding beyond
// the filter extent, take the gather kernels.
static inline dh_status conv_fwd(dh_ctx *ctx, float *res, size_t *rh, size_t *rw, const float *data, const float *filter, size_t fr,
                                 size_t fc, size_t N, size_t C, size_t H, size_t W, size_t Hf, size_t Wf, size_t padh = 0,
                                 size_t padw = 0) {
    return dh_conv2d_forward_f32(ctx, res, rh, rw, data, filter, fr, fc, nullptr, N, C, H, W, Hf, Wf, 1, 1, padh, padw);
}
static inline dh_status conv_fwd(dh_ctx *ctx, double *res, size_t *rh, size_t *rw, const double *data, const double *filter, size_t fr,
                                 size_t fc, size_t N, size_t C, size_t H, size_t W, size_t Hf, size_t Wf, size_t padh = 0,
                                 size_t padw = 0) {
    return dh_conv2d_forward_f64(ctx, res, rh, rw, data, filter, fr, fc, nullptr, N, C, H, W, Hf, Wf, 1, 1, padh, padw);
}
static inline dh_status mat_mul(dh_ctx *ctx, float *res, size_t ldr, const float *a, size_t ar, size_t ac, size_t lda, const float *b,
                                size_t br, size_t bc, size_t ldb) {
    return dh_matmul_f32(ctx, res, ldr, a, ar, ac, lda, b, br, bc, ldb, 0, 0);
}
static inline dh_status mat_mul(dh_ctx *ctx, double *res, size_t ldr, const double *a, size_t ar, size_t ac, size_t lda, const double *b,
                                size_t br, size_t bc, size_t ldb) {
    return dh_matmul_f64(ctx, res, ldr, a, ar, ac, lda, b, br, bc, ldb, 0, 0);
}

// frame[n][f][a][b], a < H + Hf - 1, b < W + Wf - 1: dY[n][f][p][q] at (p*sh + Hf-1-padh, q*sw + Wf-1-padw), else 0
template <typename T> __global__ __launch_bounds__(THREADS) void dilate_frame_kernel(T *frame, const T *dY, ConvBwdArgs g, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total)
        return;
    const unsigned FH = g.H + g.Hf - 1, FW = g.W + g.Wf - 1;
    size_t plane; // (n, f)
    unsigned ab;
    if (total <= 0xffffffffull) { // 32-bit divisions suffice (uniform)
        plane = static_cast<unsigned>(idx) / (FH * FW);
        ab = static_cast<unsigned>(idx) % (FH * FW);
    } else {
        plane = idx / (static_cast<size_t>(FH) * FW);
        ab = static_cast<unsigned>(idx % (static_cast<size_t>(FH) * FW));
    }
    const unsigned a = ab / FW, b = ab % FW;
    const unsigned oh = g.Hf - 1 - g.padh, ow = g.Wf - 1 - g.padw;
    T v = T(0);
    if (a >= oh && b >= ow && (a - oh) % g.sh == 0 && (b - ow) % g.sw == 0) {
        const unsigned p = (a - oh) / g.sh, q = (b - ow) / g.sw;
        if (p < g.P && q < g.Q)
            v = dY[plane * (static_cast<size_t>(g.P) * g.Q) + p * g.Q + q];
    }
    frame[idx] = v;
}
// wr[c][(f, r, s)] = w[f][(c, Hf-1-r, Wf-1-s)]
template <typename T> __global__ __launch_bounds__(THREADS) void rotate_filter_kernel(T *wr, const T *w, ConvBwdArgs g) {
    const unsigned taps = g.Hf * g.Wf;
    const size_t total = static_cast<size_t>(g.C) * g.F * taps;
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total)
        return;
    const unsigned t = static_cast<unsigned>(idx % taps), f = static_cast<unsigned>((idx / taps) % g.F), c = static_cast<unsigned>(idx / (static_cast<size_t>(taps) * g.F));
    wr[idx] = w[(static_cast<size_t>(f) * g.C + c) * taps + (taps - 1 - t)];
}
// patch[(n, p, q)][(c, r, s)] = Xpad[n][c][p*sh + r][q*sw + s]; a thread writes VEC consecutive (c, r, s) of one row
template <typename T, int VEC> __global__ __launch_bounds__(THREADS) void im2col_kernel(T *patch, const T *input, ConvBwdArgs g, size_t total_vecs) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total_vecs)
        return;
    const unsigned taps = g.Hf * g.Wf, Kp = g.C * taps, PQ = g.P * g.Q, kvecs = Kp / VEC;
    const size_t row = idx / kvecs;
    const unsigned k0 = static_cast<unsigned>(idx % kvecs) * VEC;
    const unsigned n = static_cast<unsigned>(row / PQ), pq = static_cast<unsigned>(row % PQ), p = pq / g.Q, q = pq % g.Q;
    const T *img = input + static_cast<size_t>(n) * g.C * g.H * g.W;
    unsigned c = k0 / taps, t = k0 % taps, r = t / g.Wf, s_ = t % g.Wf;
    T v[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const unsigned hh = p * g.sh + r, ww = q * g.sw + s_;
        v[e] = (hh >= g.padh && ww >= g.padw && hh - g.padh < g.H && ww - g.padw < g.W)
                   ? img[(static_cast<size_t>(c) * g.H + (hh - g.padh)) * g.W + (ww - g.padw)]
                   : T(0);
        if (++s_ == g.Wf) { // next (c, r, s) without divisions
            s_ = 0;
            if (++r == g.Hf) {
                r = 0;
                c++;
            }
        }
    }
    dh_store_vec<T, VEC>(patch + row * Kp + k0, v);
}
// a[f][(n, pq)] = dY[n][f][pq]
template <typename T> __global__ __launch_bounds__(THREADS) void dy_rows_kernel(T *a, const T *dY, ConvBwdArgs g, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (idx >= total)
        return;
    const unsigned PQ = g.P * g.Q;
    const size_t L = static_cast<size_t>(g.N) * PQ;
    const unsigned f = static_cast<unsigned>(idx / L);
    const size_t l = idx % L;
    const unsigned n = static_cast<unsigned>(l / PQ), pq = static_cast<unsigned>(l % PQ);
    a[idx] = dY[(static_cast<size_t>(n) * g.F + f) * PQ + pq];
}

constexpr size_t TRAIN_TEMP_LIMIT = size_t(24) << 30; // bytes of temporaries beyond which the gather kernels are used

static inline unsigned blocks_for(size_t total) { return static_cast<unsigned>(dh_ceil_div(total, static_cast<size_t>(THREADS))); }

template <typename T> static bool conv_backward_data_mfma(dh_ctx *ctx, T *dX, const T *filter, const T *dY, const ConvBwdArgs &g, dh_status *st) {
    if (g.padh > g.Hf - 1 || g.padw > g.Wf - 1)
        return false;
    const size_t FH = g.H + g.Hf - 1, FW = g.W + g.Wf - 1;
    const size_t frame_elems = static_cast<size_t>(g.N) * g.F * FH * FW, wr_elems = static_cast<size_t>(g.C) * g.F * g.Hf * g.Wf;
    // too little work to pay for the extra passes, or too large temporaries
    if (static_cast<size_t>(g.N) * g.C * g.H * g.W < (size_t(1) << 16) || frame_elems * sizeof(T) > TRAIN_TEMP_LIMIT ||
        dh_ceil_div(frame_elems, static_cast<size_t>(THREADS)) >= (size_t(1) << 31))
        return false;
    void *frame = nullptr, *wr = nullptr;
    if (g.sh == 1 && g.sw == 1 && g.P + g.Hf - 1 == g.H + 2 * g.padh && g.Q + g.Wf - 1 == g.W + 2 * g.padw) {
        // nothing to dilate: the frame is dY with Hf - 1 - padh rows and Wf - 1 - padw columns of zeros on every side,
        // which is the forward convolution's own padding
        *st = dh_malloc(ctx, wr_elems * sizeof(T), 0, &wr);
        if (*st != DH_OK)
            return true;
        hipLaunchKernelGGL((rotate_filter_kernel<T>), dim3(blocks_for(wr_elems)), dim3(THREADS), 0, ctx->stream, static_cast<T *>(wr), filter, g);
        size_t rh = 0, rw = 0;
        *st = conv_fwd(ctx, dX, &rh, &rw, dY, static_cast<const T *>(wr), g.C, static_cast<size_t>(g.F) * g.Hf * g.Wf, g.N, g.F, g.P, g.Q,
                       g.Hf, g.Wf, g.Hf - 1 - g.padh, g.Wf - 1 - g.padw);
        dh_free(ctx, wr);
        if (*st == DH_OK && (rh != g.H || rw != g.W))
            *st = dh_fail(DH_ERR_RUNTIME, "Conv2D backward - internal extent mismatch (%zu x %zu for %u x %u)", rh, rw, g.H, g.W);
        return true;
    }
    *st = dh_malloc(ctx, frame_elems * sizeof(T), 0, &frame);
    if (*st != DH_OK)
        return true;
    *st = dh_malloc(ctx, wr_elems * sizeof(T), 0, &wr);
    if (*st != DH_OK) {
        dh_free(ctx, frame);
        return true;
    }
    hipLaunchKernelGGL((dilate_frame_kernel<T>), dim3(blocks_for(frame_elems)), dim3(THREADS), 0, ctx->stream, static_cast<T *>(frame), dY, g,
                       frame_elems);
    hipLaunchKernelGGL((rotate_filter_kernel<T>), dim3(blocks_for(wr_elems)), dim3(THREADS), 0, ctx->stream, static_cast<T *>(wr), filter, g);
    size_t rh = 0, rw = 0;
    *st = conv_fwd(ctx, dX, &rh, &rw, static_cast<const T *>(frame), static_cast<const T *>(wr), g.C, static_cast<size_t>(g.F) * g.Hf * g.Wf,
                   g.N, g.F, FH, FW, g.Hf, g.Wf);
    // blocks go back to the cache; reuse is ordered by the context's stream
    dh_free(ctx, frame);
    dh_free(ctx, wr);
    if (*st == DH_OK && (rh != g.H || rw != g.W))
        *st = dh_fail(DH_ERR_RUNTIME, "Conv2D backward - internal extent mismatch (%zu x %zu for %u x %u)", rh, rw, g.H, g.W);
    return true;
}

// ---------------------------------------------------------------------------------------
// Filter gradient with the image resident in LDS (the forward convolution's layout with the roles swapped):
//     dW[f][k] = sum over images n and pixels pq of dY[n][f][pq] * patch_n[k][pq],   k = (c, hy, hx)
// A workgroup of 8 waves keeps 16 * MFW filters x `chunk` filter columns as accumulators of the 16x16x4 matrix
// instruction for its whole run over the images n = blockIdx.x, blockIdx.x + gridDim.x, ...: per image it copies
// the padded image into LDS, reads dY rows from global memory (a 16-byte vector of consecutive pixels per lane)
// and gathers the patch values from LDS at "column offset + pixel offset". Every workgroup leaves one partial
// F x K slab; a second kernel adds the slabs in order.
// DB (small planes, two images fit LDS): the next image is copied into a second LDS frame while the current one is
// contracted - a few channels per pixel block of the contraction, loaded at its start and stored at its end - so
// that a workgroup that has its CU to itself never waits for an image, and an image costs one barrier, not two.
// ---------------------------------------------------------------------------------------
struct ConvFilterResidentArgs {
    const void *x;     // N x C x H x W
    const void *dy;    // N x F x P x Q
    const int *koff;   // column k -> c*Hp*Wp + hy*Wp + hx, padded with zeros to the columns all chunks cover
    const int *pixtab; // pixel pq -> p*sh*Wp + q*sw, padded with zeros to PQpad
    void *slabs;       // [gridDim.x][F][K]
    unsigned N, C, H, W, Wp, ph, pw, F, K, PQ, PQpad, HpWp, frame, chunk;
};

static __global__ __launch_bounds__(256) void conv_filter_tables_kernel(int *koff, int *pixtab, unsigned K, unsigned Kcols, unsigned PQ,
                                                                        unsigned PQpad, unsigned HpWp, unsigned Wp, unsigned Hf,
                                                                        unsigned Wf, unsigned Q, unsigned sh, unsigned sw) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x, nt = gridDim.x * 256;
    for (unsigned k = t; k < Kcols; k += nt) {
        int off = 0;
        if (k < K) {
            const unsigned c = k / (Hf * Wf), hw = k % (Hf * Wf);
            off = static_cast<int>(c * HpWp + (hw / Wf) * Wp + hw % Wf);
        }
        koff[k] = off;
    }
    for (unsigned i = t; i < PQpad; i += nt)
        pixtab[i] = i < PQ ? static_cast<int>((i / Q) * sh * Wp + (i % Q) * sw) : 0;
}

constexpr int CONV_FILTER_STAGE_CH = 4; // DB: channels of the next image that one pixel block of the contraction brings in, at most
template <typename T, int MFW, int WAVES, int NF, bool DB>
__global__ __launch_bounds__(64 * WAVES) void conv_filter_resident_kernel(ConvFilterResidentArgs g) {
    using M = dh_gemm::Mfma16<T>;
    constexpr int VEC = 16 / sizeof(T), NPARTS = WAVES / MFW, NT = 64 * WAVES;
    static_assert(WAVES % MFW == 0, "waves per filter block");
    extern __shared__ __attribute__((aligned(16))) unsigned char conv_lds[];
    int *pixtab = reinterpret_cast<int *>(conv_lds); // PQpad entries: a multiple of 16 bytes
    T *frame = reinterpret_cast<T *>(conv_lds + g.PQpad * sizeof(int));
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const unsigned f0 = blockIdx.y * (16 * MFW), col0 = blockIdx.z * g.chunk;
    // both tables as byte offsets into the LDS image: a gather's address is then one addition (every ordinary vector
    // instruction issued beside the matrix instructions takes a pass out of the matrix pipe)
    for (unsigned i = tid; i < g.PQpad; i += NT)
        pixtab[i] = g.pixtab[i] * static_cast<int>(sizeof(T));

    const int mf = wave % MFW, part = wave / MFW;
    const int li = lane % 16, lk = lane / 16;
    // this lane's filter column in each of the wave's column blocks (dealt round-robin over the waves)
    int koffs[NF];
    int nfv = 0;
#pragma unroll
    for (int j = 0; j < NF; j++) {
        const unsigned first = col0 + (j * NPARTS + part) * 16;
        koffs[j] = g.koff[first + li] * static_cast<int>(sizeof(T));
        if (first < g.K)
            nfv = j + 1;
    }
    typename M::acc_t acc[NF];
#pragma unroll
    for (int j = 0; j < NF; j++)
        acc[j] = typename M::acc_t{0, 0, 0, 0};

    const unsigned frow = f0 + mf * 16 + li;
    const bool rowok = frow < g.F;
    const T *dy = static_cast<const T *>(g.dy);
    const int *pixl = pixtab + lk * VEC;
    const char *frame_b = reinterpret_cast<const char *>(frame);
    // DB: this thread's position in the padded plane (planes of at most NT positions), where it lies in the image
    // (position 0 for the border, which is stored as zero), and the channels a pixel block brings in
    const unsigned HW = g.H * g.W;
    const unsigned sy = static_cast<unsigned>(tid) / g.Wp - g.ph, sxx = static_cast<unsigned>(tid) % g.Wp - g.pw; // wrap inside the border
    const bool s_plane = static_cast<unsigned>(tid) < g.HpWp, s_in = s_plane && sy < g.H && sxx < g.W;
    const unsigned s_src = s_in ? sy * g.W + sxx : 0;
    const unsigned cpi = (g.C + g.PQpad / (4 * VEC) - 1) / (g.PQpad / (4 * VEC));
    unsigned cur = 0;
    if constexpr (DB) {
        dh_dnn::conv_stage_frame<T, 32>(frame, static_cast<const T *>(g.x) + static_cast<size_t>(blockIdx.x) * g.C * HW, g.C, g.H, g.W,
                                    g.Wp, g.ph, g.pw, g.HpWp, g.frame, tid, NT);
        __syncthreads();
    }

    for (unsigned img = blockIdx.x; img < g.N; img += gridDim.x) {
        if constexpr (!DB) {
            __syncthreads(); // every wave is done with the previous image
            dh_dnn::conv_stage_frame<T, 32>(frame, static_cast<const T *>(g.x) + static_cast<size_t>(img) * g.C * HW, g.C, g.H, g.W,
                                        g.Wp, g.ph, g.pw, g.HpWp, g.frame, tid, NT);
            __syncthreads();
        }
        // DB: the frame being contracted, the frame being filled, and the image that fills it (the last image of
        // the workgroup brings itself in again; nobody reads that copy)
        const char *fb = DB ? frame_b + static_cast<size_t>(cur) * g.frame * sizeof(T) : frame_b;
        T *fill = frame + static_cast<size_t>(cur ^ 1u) * g.frame;
        const T *xnext = static_cast<const T *>(g.x) + static_cast<size_t>(img + gridDim.x < g.N ? img + gridDim.x : img) * g.C * HW;
        const T *arow = dy + (static_cast<size_t>(img) * g.F + (rowok ? frow : 0)) * g.PQ + lk * VEC;
        // dY values of pixel block q0 for this lane; lanes past the row end (or past F) read the tensor's first
        // vector instead and are zeroed when the values are taken into use
        auto a_ok = [&](unsigned q0) { return rowok && q0 + lk * VEC < g.PQ; };
        auto contract = [&](auto nv_tag) {
            constexpr int NV = decltype(nv_tag)::value;
            // dY comes from HBM: its vectors are asked for two pixel blocks ahead
            // the patch values alternate between two register sets from step to step (an even number of steps per
            // pixel block), so that none is copied
            static_assert(VEC % 2 == 0, "the two sets of patch registers alternate from step to step");
            T a_cur[VEC], a_nxt[VEC], b_even[NV], b_odd[NV];
            int pt[VEC];
            const unsigned q1 = (4 * VEC < g.PQpad) ? 4 * VEC : 0;
            bool ok_nxt = a_ok(q1);
            {
                const bool ok = a_ok(0);
                dh_load_vec<T, VEC>(ok ? arow : dy, a_cur);
                dh_load_vec<T, VEC>(ok_nxt ? arow + q1 : dy, a_nxt);
#pragma unroll
                for (int s_ = 0; s_ < VEC; s_++)
                    a_cur[s_] = ok ? a_cur[s_] : T(0);
            }
#pragma unroll
            for (int s_ = 0; s_ < VEC; s_++)
                pt[s_] = pixl[s_];
#pragma unroll
            for (int j = 0; j < NV; j++)
                b_even[j] = *reinterpret_cast<const T *>(fb + (koffs[j] + pt[0]));
            unsigned c_lo = 0; // DB: first channel this pixel block brings in
            for (unsigned q0 = 0; q0 < g.PQpad; q0 += 4 * VEC) {
                T sv[CONV_FILTER_STAGE_CH];
                if constexpr (DB) {
#pragma unroll
                    for (int u = 0; u < CONV_FILTER_STAGE_CH; u++) {
                        const unsigned c = c_lo + u;
                        sv[u] = xnext[s_src + (c < g.C ? c : 0) * HW];
                    }
                }
                const unsigned qn = (q0 + 4 * VEC < g.PQpad) ? q0 + 4 * VEC : q0;
                const unsigned qnn = (q0 + 8 * VEC < g.PQpad) ? q0 + 8 * VEC : q0;
                const bool ok_nn = a_ok(qnn);
                T a_nn[VEC];
                int pt_nxt[VEC];
                dh_load_vec<T, VEC>(ok_nn ? arow + qnn : dy, a_nn);
#pragma unroll
                for (int s_ = 0; s_ < VEC; s_++)
                    pt_nxt[s_] = pixl[qn + s_];
#pragma unroll
                for (int s_ = 0; s_ < VEC; s_++) {
                    const int pt_after = (s_ + 1 < VEC) ? pt[s_ + 1] : pt_nxt[0];
                    __builtin_amdgcn_sched_barrier(0); // a gather must not sink to its use in the next step
                    if (s_ % 2 == 0) {
#pragma unroll
                        for (int j = 0; j < NV; j++)
                            b_odd[j] = *reinterpret_cast<const T *>(fb + (koffs[j] + pt_after));
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int j = 0; j < NV; j++)
                            acc[j] = M::mma(a_cur[s_], b_even[j], acc[j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < NV; j++)
                            b_even[j] = *reinterpret_cast<const T *>(fb + (koffs[j] + pt_after));
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int j = 0; j < NV; j++)
                            acc[j] = M::mma(a_cur[s_], b_odd[j], acc[j]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int s_ = 0; s_ < VEC; s_++) {
                    a_cur[s_] = ok_nxt ? a_nxt[s_] : T(0);
                    a_nxt[s_] = a_nn[s_];
                    pt[s_] = pt_nxt[s_];
                }
                ok_nxt = ok_nn;
                if constexpr (DB) {
#pragma unroll
                    for (int u = 0; u < CONV_FILTER_STAGE_CH; u++) {
                        const unsigned c = c_lo + u;
                        if (s_plane && static_cast<unsigned>(u) < cpi && c < g.C)
                            fill[c * g.HpWp + tid] = s_in ? sv[u] : T(0);
                    }
                    c_lo += cpi;
                }
            }
        };
        if (nfv == NF - 1)
            contract(std::integral_constant<int, NF - 1>{});
        else if (nfv > 0)
            contract(std::integral_constant<int, NF>{});
        if constexpr (DB) {
            // a wave without column blocks (nfv == 0) has to bring in its share of the next image all the same
            if (nfv == 0) {
                for (unsigned c = 0; c < g.C; c++)
                    if (s_plane)
                        fill[c * g.HpWp + tid] = s_in ? xnext[s_src + c * HW] : T(0);
            }
            __syncthreads(); // the next image is in place, and every wave is done with this one
            cur ^= 1u;
        }
    }

    T *slab = static_cast<T *>(g.slabs) + static_cast<size_t>(blockIdx.x) * g.F * g.K;
#pragma unroll
    for (int j = 0; j < NF; j++) {
        const unsigned col = col0 + (j * NPARTS + part) * 16 + li;
        if (j < nfv && col < g.K) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const unsigned f = f0 + mf * 16 + M::row(lane, v);
                if (f < g.F)
                    slab[static_cast<size_t>(f) * g.K + col] = acc[j][v];
            }
        }
    }
}

// res[i] = slabs[0][i] + slabs[1][i] + ... in slab order
template <typename T> __global__ __launch_bounds__(THREADS) void slab_sum_kernel(T *res, const T *slabs, unsigned nslabs, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * THREADS + threadIdx.x;
    if (i >= n)
        return;
    T sum = T(0);
    unsigned z = 0;
    for (; z + 4 <= nslabs; z += 4) {
        const T a0 = slabs[z * n + i], a1 = slabs[(z + 1) * n + i], a2 = slabs[(z + 2) * n + i], a3 = slabs[(z + 3) * n + i];
        sum = (((sum + a0) + a1) + a2) + a3;
    }
    for (; z < nslabs; z++)
        sum += slabs[z * n + i];
    res[i] = sum;
}

template <typename T, int MFW, int WAVES, int NF, bool DB>
static inline dh_status conv_filter_resident_launch(dh_ctx *ctx, const ConvFilterResidentArgs &g, dim3 grid, size_t lds) {
    // dynamic LDS beyond 64 KiB has to be asked for, per kernel and device (the call is cheap next to the kernel)
    if (lds > 65536) {
        DH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_filter_resident_kernel<T, MFW, WAVES, NF, DB>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    }
    hipLaunchKernelGGL((conv_filter_resident_kernel<T, MFW, WAVES, NF, DB>), grid, dim3(64 * WAVES), lds, ctx->stream, g);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T> static bool conv_backward_filter_resident(dh_ctx *ctx, T *dW, const T *input, const T *dY, const ConvBwdArgs &g, dh_status *st) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr size_t NFMAX = 13; // column blocks per wave: 13 accumulator blocks and their operands fit 2 waves per SIMD
    const size_t PQ = static_cast<size_t>(g.P) * g.Q, K = static_cast<size_t>(g.C) * g.Hf * g.Wf;
    const size_t Hp = g.H + 2 * g.padh, Wp = g.W + 2 * g.padw, frame = g.C * Hp * Wp;
    const size_t PQpad = dh_ceil_div(PQ, static_cast<size_t>(4 * VEC)) * (4 * VEC);
    size_t lds = PQpad * sizeof(int) + frame * sizeof(T);
    const int mfw = g.F <= 16 ? 1 : (g.F <= 32 ? 2 : 4);
    const size_t waves = 8;
    const size_t parts = waves / mfw, fgroups = dh_ceil_div(static_cast<size_t>(g.F), static_cast<size_t>(16 * mfw));
    const size_t blocks16 = dh_ceil_div(K, 16);
    const size_t chunks = dh_ceil_div(blocks16, parts * NFMAX);
    const size_t nf = dh_ceil_div(blocks16, parts * chunks);
    const size_t chunk = parts * nf * 16;
    if (PQ % VEC != 0 || !dh_aligned(dY, 16) || lds > 150 * 1024 || nf < 3 || PQ < 32 || static_cast<size_t>(g.N) * PQ < 4096 ||
        fgroups >= 65536 || chunks >= 65536 || frame >= (size_t(1) << 31))
        return false;
    // up to 7 column blocks per wave take few enough registers for two workgroups per CU, LDS permitting
    const size_t per_cu = (nf <= 7 && lds <= 80 * 1024) ? 2 : 1;
    // A workgroup alone on its CU has nothing to cover the copy-in of an image with: it brings the next image in
    // beside the contraction, where a plane has no more positions than the workgroup has threads, a pixel block's
    // share of the channels is small, and two images fit LDS.
    const bool db = per_cu == 1 && Hp * Wp <= waves * 64 && dh_ceil_div(static_cast<size_t>(g.C), PQpad / (4 * VEC)) <= CONV_FILTER_STAGE_CH &&
                    PQpad * sizeof(int) + 2 * frame * sizeof(T) <= 150 * 1024;
    if (db)
        lds = PQpad * sizeof(int) + 2 * frame * sizeof(T);
    size_t groups = static_cast<size_t>(ctx->num_cus) * per_cu / (fgroups * chunks);
    if (groups < 1)
        groups = 1;
    if (groups > g.N)
        groups = g.N;
    const size_t kcols = chunks * chunk;
    void *tabs = nullptr, *slabs = nullptr;
    *st = dh_malloc(ctx, (kcols + PQpad) * sizeof(int), 0, &tabs);
    if (*st != DH_OK)
        return true;
    *st = dh_malloc(ctx, groups * g.F * K * sizeof(T), 0, &slabs);
    if (*st != DH_OK) {
        dh_free(ctx, tabs);
        return true;
    }
    int *koff = static_cast<int *>(tabs), *pixtab = koff + kcols;
    hipLaunchKernelGGL(conv_filter_tables_kernel, dim3(static_cast<unsigned>(dh_ceil_div(kcols + PQpad, 256))), dim3(256), 0, ctx->stream,
                       koff, pixtab, static_cast<unsigned>(K), static_cast<unsigned>(kcols), static_cast<unsigned>(PQ),
                       static_cast<unsigned>(PQpad), static_cast<unsigned>(Hp * Wp), static_cast<unsigned>(Wp), g.Hf, g.Wf, g.Q, g.sh, g.sw);
    ConvFilterResidentArgs r{};
    r.x = input;
    r.dy = dY;
    r.koff = koff;
    r.pixtab = pixtab;
    r.slabs = slabs;
    r.N = g.N;
    r.C = g.C;
    r.H = g.H;
    r.W = g.W;
    r.Wp = static_cast<unsigned>(Wp);
    r.ph = g.padh;
    r.pw = g.padw;
    r.F = g.F;
    r.K = static_cast<unsigned>(K);
    r.PQ = static_cast<unsigned>(PQ);
    r.PQpad = static_cast<unsigned>(PQpad);
    r.HpWp = static_cast<unsigned>(Hp * Wp);
    r.frame = static_cast<unsigned>(frame);
    r.chunk = static_cast<unsigned>(chunk);
    const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(fgroups), static_cast<unsigned>(chunks));
#define DH_CONV_FILTER_NF(MFW_, WAVES_)                                                                                   \
    (nf <= 7 ? conv_filter_resident_launch<T, MFW_, WAVES_, 7, false>(ctx, r, grid, lds)                                  \
             : (nf <= 10 ? (db ? conv_filter_resident_launch<T, MFW_, WAVES_, 10, true>(ctx, r, grid, lds)                \
                               : conv_filter_resident_launch<T, MFW_, WAVES_, 10, false>(ctx, r, grid, lds))              \
                         : (db ? conv_filter_resident_launch<T, MFW_, WAVES_, 13, true>(ctx, r, grid, lds)                \
                               : conv_filter_resident_launch<T, MFW_, WAVES_, 13, false>(ctx, r, grid, lds))))
#define DH_CONV_FILTER_RES(MFW_) DH_CONV_FILTER_NF(MFW_, 8)
    *st = mfw == 1 ? DH_CONV_FILTER_RES(1) : (mfw == 2 ? DH_CONV_FILTER_RES(2) : DH_CONV_FILTER_RES(4));
#undef DH_CONV_FILTER_RES
#undef DH_CONV_FILTER_NF
    if (*st == DH_OK) {
        const size_t n = static_cast<size_t>(g.F) * K;
        hipLaunchKernelGGL((slab_sum_kernel<T>), dim3(blocks_for(n)), dim3(THREADS), 0, ctx->stream, dW, static_cast<const T *>(slabs),
                           static_cast<unsigned>(groups), n);
    }
    dh_free(ctx, tabs);
    dh_free(ctx, slabs);
    return true;
}

template <typename T> static bool conv_backward_filter_mfma(dh_ctx *ctx, T *dW, const T *input, const T *dY, const ConvBwdArgs &g, dh_status *st) {
    const size_t L = static_cast<size_t>(g.N) * g.P * g.Q, Kp = static_cast<size_t>(g.C) * g.Hf * g.Wf;
    const size_t patch_elems = L * Kp, a_elems = static_cast<size_t>(g.F) * L;
    if (L < 4096 || (patch_elems + a_elems) * sizeof(T) > TRAIN_TEMP_LIMIT || dh_ceil_div(patch_elems, static_cast<size_t>(THREADS)) >= (size_t(1) << 31))
        return false;
    void *patch = nullptr, *a = nullptr;
    *st = dh_malloc(ctx, patch_elems * sizeof(T), 0, &patch);
    if (*st != DH_OK)
        return true;
    *st = dh_malloc(ctx, a_elems * sizeof(T), 0, &a);
    if (*st != DH_OK) {
        dh_free(ctx, patch);
        return true;
    }
    constexpr int V = dh_vec<T>::N;
    if (Kp % V == 0)
        hipLaunchKernelGGL((im2col_kernel<T, V>), dim3(blocks_for(patch_elems / V)), dim3(THREADS), 0, ctx->stream, static_cast<T *>(patch),
                           input, g, patch_elems / V);
    else
        hipLaunchKernelGGL((im2col_kernel<T, 1>), dim3(blocks_for(patch_elems)), dim3(THREADS), 0, ctx->stream, static_cast<T *>(patch), input,
                           g, patch_elems);
    hipLaunchKernelGGL((dy_rows_kernel<T>), dim3(blocks_for(a_elems)), dim3(THREADS), 0, ctx->stream, static_cast<T *>(a), dY, g, a_elems);
    *st = mat_mul(ctx, dW, Kp, static_cast<const T *>(a), g.F, L, L, static_cast<const T *>(patch), L, Kp, Kp);
    dh_free(ctx, patch);
    dh_free(ctx, a);
    return true;
}

template <typename T>
dh_status conv2d_backward_data(dh_ctx *ctx, T *dX, const T *filter, const T *dY, size_t N, size_t C, size_t H, size_t W, size_t F,
                               size_t Hf, size_t Wf, size_t sh, size_t sw, size_t padh, size_t padw, bool use_mfma = true) {
    DH_REQUIRE_CTX(ctx);
    ConvBwdArgs g;
    dh_status st = conv_bwd_args(&g, N, C, H, W, F, Hf, Wf, sh, sw, padh, padw);
    if (st != DH_OK)
        return st;
    const size_t total = N * C * H * W;
    if (total == 0)
        return DH_OK;
    if (use_mfma && conv_backward_data_mfma<T>(ctx, dX, filter, dY, g, &st))
        return st;
    const size_t blocks = dh_ceil_div(total, THREADS);
    if (blocks >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Conv2D backward - too many elements for one launch");
    hipLaunchKernelGGL((conv_backward_data_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(THREADS), 0, ctx->stream, dX, filter,
                       dY, g);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T>
dh_status conv2d_backward_filter(dh_ctx *ctx, T *dW, const T *input, const T *dY, size_t N, size_t C, size_t H, size_t W, size_t F,
                                 size_t Hf, size_t Wf, size_t sh, size_t sw, size_t padh, size_t padw, bool use_mfma = true) {
    DH_REQUIRE_CTX(ctx);
    ConvBwdArgs g;
    dh_status st = conv_bwd_args(&g, N, C, H, W, F, Hf, Wf, sh, sw, padh, padw);
    if (st != DH_OK)
        return st;
    if (F * C == 0)
        return DH_OK;
    if (F * C >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Conv2D backward - too many filter planes for one launch");
    if (use_mfma && conv_backward_filter_resident<T>(ctx, dW, input, dY, g, &st))
        return st;
    if (use_mfma && conv_backward_filter_mfma<T>(ctx, dW, input, dY, g, &st))
        return st;
    hipLaunchKernelGGL((conv_backward_filter_kernel<T, 16>), dim3(static_cast<unsigned>(F * C)), dim3(THREADS), 0, ctx->stream, dW,
                       input, dY, g);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

} // namespace dh_train
