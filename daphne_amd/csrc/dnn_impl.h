// DNN inference kernels for DenseMatrix<float|double> (one NCHW image per matrix row):
// Conv2D forward (im2col-free implicit GEMM on MFMA), MaxPool forward, BiasAdd, BatchNorm
// inference, Softmax. Instantiated per value type by dnn_f32.hip / dnn_f64.hip.
//
// Arithmetic follows the reference's CPU kernels (paths relative to
// src/runtime/local/kernels/): Conv2DForward.h:77-140, Pooling.cpp:28-107 + Pooling.h:33-58,
// BiasAdd.h:34-52, BatchNorm2DTestForward.h:77-101, Softmax.h:22-58; the entry points stand in
// for the CUDA wrappers in kernels/CUDA/{Convolution,Pooling,BiasAdd,BatchNorm,Softmax}.cpp.
//
// Conv2D as a GEMM without materialising im2col:
//     out_n[f][pixel] = sum_k W[f][k] * patch[k][pixel],   k = (c, h, w), pixel = (n, p, q)
// The filter matrix (F x K, K contiguous) is the row operand; the patch matrix is never built:
// each workgroup gathers its BK x BN slice straight from the NCHW input into LDS (zero outside
// the image), with consecutive lanes on consecutive output pixels so that both the gather and
// the final store are contiguous along q. Pixels of all images form one long N dimension, so a
// tile may span image boundaries and small images still fill the 128-pixel tile.
#pragma once

#include "gemm_impl.h"

#include <limits>

namespace dh_dnn {

using dh_gemm::Mfma;
using dh_gemm::TileLayout;
using dh_gemm::TileMover;

struct ConvArgs {
    const void *data, *filter, *bias;
    void *res;
    unsigned N, C, H, W, F, Hf, Wf, sh, sw, ph, pw, P, Q;
    unsigned K;          // C*Hf*Wf
    int aligned_w;       // filter rows can be read with 16-byte loads
    size_t pixels;       // N*P*Q
    const int *ktab;     // per k (padded to a multiple of the K tile): offset of (c, hy, hx) in an image,
                         // then hy << 16 | hx; entries beyond K are zero
};

// k = (c, hy, hx) -> { c*H*W + hy*W + hx, hy << 16 | hx }, so that the gather does no divisions.
static __global__ void conv_table_kernel(int *tab, unsigned K, unsigned Kpad, unsigned HW, unsigned W, unsigned Hf,
                                         unsigned Wf) {
    for (unsigned k = blockIdx.x * blockDim.x + threadIdx.x; k < Kpad; k += gridDim.x * blockDim.x) {
        int off = 0, yx = 0;
        if (k < K) {
            const unsigned c = k / (Hf * Wf), hw = k % (Hf * Wf);
            const unsigned hy = hw / Wf, hx = hw % Wf;
            off = static_cast<int>(c * HW + hy * W + hx);
            yx = static_cast<int>(hy << 16 | hx);
        }
        tab[k] = off;
        tab[Kpad + k] = yx;
    }
}

template <typename T, int BM, int BN, int BK, int WN>
__global__ __launch_bounds__(64 * WN) void conv2d_kernel(ConvArgs g) {
    using M = Mfma<T>;
    constexpr int THREADS = 64 * WN;
    constexpr int TN = BN / WN;
    constexpr int FM = BM / M::MT, FN = TN / M::NT;
    static_assert(BM % M::MT == 0 && TN % M::NT == 0 && BK % M::KT == 0, "tile shape");
    static_assert(THREADS % BN == 0 && BK % (THREADS / BN) == 0, "gather mapping");
    using LA = TileLayout<T, BM, BK, true>;  // filter tile [f][k]
    using LB = TileLayout<T, BN, BK, false>; // patch tile  [k][pixel]
    __shared__ __attribute__((aligned(16))) T lds_a[2][LA::ELEMS];
    __shared__ __attribute__((aligned(16))) T lds_b[2][LB::ELEMS];

    const T *X = static_cast<const T *>(g.data);
    const T *Wt = static_cast<const T *>(g.filter);
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const size_t pix0 = static_cast<size_t>(blockIdx.x) * BN;
    const size_t f0 = static_cast<size_t>(blockIdx.y) * BM;
    const unsigned PQ = g.P * g.Q, HW = g.H * g.W;

    // the pixel this thread gathers for, decoded once
    constexpr int KG = THREADS / BN;      // K groups among the threads
    constexpr int KPT = BK / KG;          // K values per thread and tile
    const int gj = tid % BN, gkg = tid / BN;
    const size_t gpix = pix0 + gj;
    const bool pix_ok = gpix < g.pixels;
    const bool small = g.pixels <= 0xffffffffull; // 32-bit divisions suffice (uniform)
    unsigned img = 0, p = 0, q = 0;
    if (pix_ok) {
        unsigned pq;
        if (small) {
            img = static_cast<unsigned>(gpix) / PQ;
            pq = static_cast<unsigned>(gpix) % PQ;
        } else {
            img = static_cast<unsigned>(gpix / PQ);
            pq = static_cast<unsigned>(gpix % PQ);
        }
        p = pq / g.Q;
        q = pq % g.Q;
    }
    const int y0 = static_cast<int>(p * g.sh) - static_cast<int>(g.ph);
    // a pixel beyond the end gets a row origin that fails every bounds check
    const int x0 = pix_ok ? static_cast<int>(q * g.sw) - static_cast<int>(g.pw) : -0x10000000;
    const T *xpix = X + static_cast<size_t>(img) * g.C * HW + static_cast<ptrdiff_t>(y0) * static_cast<int>(g.W) + x0;
    const unsigned Kpad = (g.K + BK - 1) / BK * BK;
    const int *tab_off = g.ktab + gkg * KPT, *tab_yx = g.ktab + Kpad + gkg * KPT;

    TileMover<T, BM, BK, true, THREADS> mv_a;
    T gb[KPT];
    auto fetch = [&](unsigned k0) {
        mv_a.load(Wt, g.K, f0, k0, g.F, g.K, g.aligned_w != 0, tid);
        int off[KPT], yx[KPT];
#pragma unroll
        for (int i = 0; i < KPT; i++) {
            off[i] = tab_off[k0 + i];
            yx[i] = tab_yx[k0 + i];
        }
#pragma unroll
        for (int i = 0; i < KPT; i++) {
            // unsigned compares fold the lower bound in: a negative coordinate wraps to a huge value
            const unsigned y = static_cast<unsigned>(y0 + (yx[i] >> 16)), x = static_cast<unsigned>(x0 + (yx[i] & 0xffff));
            gb[i] = (y < g.H && x < g.W && k0 + gkg * KPT + i < g.K) ? xpix[off[i]] : T(0);
        }
    };
    auto stash = [&](int buf) {
        mv_a.store(lds_a[buf], tid);
#pragma unroll
        for (int i = 0; i < KPT; i++)
            lds_b[buf][LB::at(gj, gkg * KPT + i)] = gb[i];
    };

    typename M::acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
            acc[i][j] = M::zero();

    const int frag_row = lane % M::ROWS, frag_k = lane / M::ROWS;
    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (unsigned k0 = 0; k0 < g.K; k0 += BK) {
        const bool more = k0 + BK < g.K;
        if (more)
            fetch(k0 + BK);
        const T *la = lds_a[buf];
        const T *lb = lds_b[buf];
#pragma unroll
        for (int kk = 0; kk < BK; kk += M::KT) {
            T fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; i++)
                fa[i] = la[LA::at(i * M::MT + frag_row, kk + frag_k)];
#pragma unroll
            for (int j = 0; j < FN; j++)
                fb[j] = lb[LB::at(wave * TN + j * M::NT + frag_row, kk + frag_k)];
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++)
                    acc[i][j] = M::mma(fa[i], fb[j], acc[i][j]);
        }
        if (more)
            stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // out[img][f][pq]: lanes along pixels -> contiguous stores
    T *out = static_cast<T *>(g.res);
    const T *bias = static_cast<const T *>(g.bias);
#pragma unroll
    for (int j = 0; j < FN; j++) {
        const size_t pix = pix0 + wave * TN + j * M::NT + M::col(lane);
        if (pix < g.pixels) {
            size_t oimg, opq;
            if (small) {
                oimg = static_cast<unsigned>(pix) / PQ;
                opq = static_cast<unsigned>(pix) % PQ;
            } else {
                oimg = pix / PQ;
                opq = pix % PQ;
            }
            T *obase = out + oimg * g.F * PQ + opq;
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int v = 0; v < M::ACC; v++) {
                    const size_t f = f0 + i * M::MT + M::row(lane, v);
                    if (f < g.F)
                        obase[f * PQ] = acc[i][j][v] + (bias ? bias[f] : T(0));
                }
        }
    }
}

template <typename T>
dh_status conv2d_forward(dh_ctx *ctx, T *res, size_t *res_h, size_t *res_w, const T *data, const T *filter,
                         size_t filter_rows, size_t filter_cols, const T *bias, size_t N, size_t C, size_t H,
                         size_t W, size_t Hf, size_t Wf, size_t sh, size_t sw, size_t ph, size_t pw) {
    DH_REQUIRE_CTX(ctx);
    const size_t F = filter_rows;
    if (filter_rows * filter_cols != F * C * Hf * Wf)
        // kernels/CUDA/Convolution.cpp:32-39
        return dh_fail(DH_ERR_INVALID_ARG,
                       "Convolution kernel dimension mismatch: expected %zu elements [%zux%zux%zux%zu] but got %zu.",
                       F * C * Hf * Wf, F, C, Hf, Wf, filter_rows * filter_cols);
    if (sh == 0 || sw == 0 || H + 2 * ph < Hf || W + 2 * pw < Wf)
        return dh_fail(DH_ERR_INVALID_ARG, "Convolution: filter %zux%zu does not fit the padded image %zux%zu",
                       Hf, Wf, H + 2 * ph, W + 2 * pw);
    const size_t P = (H + 2 * ph - Hf) / sh + 1, Q = (W + 2 * pw - Wf) / sw + 1; // Padding.h:6-9
    if (res_h)
        *res_h = P;
    if (res_w)
        *res_w = Q;
    const size_t pixels = N * P * Q;
    if (pixels == 0 || F == 0)
        return DH_OK;
    if (C * H * W >= (size_t(1) << 31) || C * Hf * Wf >= (size_t(1) << 31) || P * Q >= (size_t(1) << 31) ||
        N >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Convolution: image or filter extents exceed 2^31 elements");
    ConvArgs g{};
    g.data = data;
    g.filter = filter;
    g.bias = bias;
    g.res = res;
    g.N = N; g.C = C; g.H = H; g.W = W; g.F = F; g.Hf = Hf; g.Wf = Wf;
    g.sh = sh; g.sw = sw; g.ph = ph; g.pw = pw; g.P = P; g.Q = Q;
    g.K = static_cast<unsigned>(C * Hf * Wf);
    g.pixels = pixels;
    g.aligned_w = dh_aligned(filter, 16) && (g.K % (16 / sizeof(T)) == 0);
    constexpr int BK = dh_gemm::GemmBK<T>::value;
    constexpr int BN = 128;
    const size_t gx = dh_ceil_div(pixels, BN);
    if (gx >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Convolution: too many output pixels for one launch");
    if (Hf >= 0x8000 || Wf >= 0x10000 || H >= (size_t(1) << 28) || W >= (size_t(1) << 28))
        return dh_fail(DH_ERR_RUNTIME, "Convolution: filter or image side too large");
    const unsigned Kpad = static_cast<unsigned>(dh_ceil_div(g.K, BK) * BK);
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, 2 * static_cast<size_t>(Kpad) * sizeof(int), &wsv);
    if (st != DH_OK)
        return st;
    g.ktab = static_cast<const int *>(wsv);
    hipLaunchKernelGGL(conv_table_kernel, dim3(static_cast<unsigned>(dh_ceil_div(Kpad, 256) > 64 ? 64 : dh_ceil_div(Kpad, 256))),
                       dim3(256), 0, ctx->stream, static_cast<int *>(wsv), g.K, Kpad, static_cast<unsigned>(H * W),
                       static_cast<unsigned>(W), static_cast<unsigned>(Hf), static_cast<unsigned>(Wf));
    if (F <= 32) {
        hipLaunchKernelGGL((conv2d_kernel<T, 32, BN, BK, 4>), dim3(static_cast<unsigned>(gx), 1), dim3(256), 0,
                           ctx->stream, g);
    } else {
        const unsigned gy = static_cast<unsigned>(dh_ceil_div(F, 64));
        hipLaunchKernelGGL((conv2d_kernel<T, 64, BN, BK, 4>), dim3(static_cast<unsigned>(gx), gy), dim3(256), 0,
                           ctx->stream, g);
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// MaxPool forward. One thread per output; consecutive threads on consecutive q.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void maxpool_kernel(T *res, const T *data, size_t total, unsigned planes_dummy,
                                                      unsigned H, unsigned W, unsigned P, unsigned Q, unsigned ph,
                                                      unsigned pw, unsigned sh, unsigned sw, unsigned padh,
                                                      unsigned padw) {
    const unsigned PQ = P * Q, HW = H * W;
    for (size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; idx < total;
         idx += static_cast<size_t>(gridDim.x) * 256) {
        const size_t plane = idx / PQ;
        const unsigned pq = static_cast<unsigned>(idx % PQ);
        const unsigned p = pq / Q, q = pq % Q;
        const T *in = data + plane * HW;
        // window in image coordinates, clipped at the border (Pooling.cpp:77,89,102); the padding
        // ring holds zeros, and the output starts at zero anyway (Pooling.cpp:57, Pooling.h:46-54)
        const int y_lo = static_cast<int>(p * sh) - static_cast<int>(padh);
        const int x_lo = static_cast<int>(q * sw) - static_cast<int>(padw);
        const int y0 = y_lo < 0 ? 0 : y_lo, x0 = x_lo < 0 ? 0 : x_lo;
        int y1 = y_lo + static_cast<int>(ph), x1 = x_lo + static_cast<int>(pw);
        if (y1 > static_cast<int>(H))
            y1 = H;
        if (x1 > static_cast<int>(W))
            x1 = W;
        T m = T(0);
        for (int y = y0; y < y1; y++)
            for (int x = x0; x < x1; x++) {
                const T v = in[static_cast<unsigned>(y) * W + static_cast<unsigned>(x)];
                m = (m < v) ? v : m; // std::max(m, v)
            }
        res[idx] = m;
    }
}

// Non-overlapping 2x2 windows (stride 2, no padding, even H and W): the tensor is a flat list of row
// pairs [R][2][W] -> [R][W/2]. Each thread loads VI consecutive values of both rows of a pair and
// writes VI/2 outputs, all as single vector accesses.
template <typename T, int VI>
__global__ __launch_bounds__(256) void maxpool2x2_kernel(T *res, const T *data, size_t items, unsigned W,
                                                         unsigned wvecs) {
    const size_t item = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (item >= items)
        return;
    size_t r;
    unsigned j;
    if (items <= 0xffffffffull) {
        r = static_cast<unsigned>(item) / wvecs;
        j = static_cast<unsigned>(item) % wvecs;
    } else {
        r = item / wvecs;
        j = static_cast<unsigned>(item % wvecs);
    }
    const T *in = data + r * 2 * W + static_cast<size_t>(j) * VI;
    T a[VI], b[VI], o[VI / 2];
    dh_load_vec_stream<T, VI>(in, a);
    dh_load_vec_stream<T, VI>(in + W, b);
#pragma unroll
    for (int i = 0; i < VI / 2; i++) {
        // window order of Pooling.cpp:77-105 with the accumulator starting at zero
        T m = T(0);
        m = (m < a[2 * i]) ? a[2 * i] : m;
        m = (m < a[2 * i + 1]) ? a[2 * i + 1] : m;
        m = (m < b[2 * i]) ? b[2 * i] : m;
        m = (m < b[2 * i + 1]) ? b[2 * i + 1] : m;
        o[i] = m;
    }
    T *out = res + r * (W / 2) + static_cast<size_t>(j) * (VI / 2);
    if constexpr (VI / 2 == 1) {
        *out = o[0];
    } else {
        typedef T half_vec __attribute__((ext_vector_type(VI / 2)));
        half_vec t;
#pragma unroll
        for (int i = 0; i < VI / 2; i++)
            t[i] = o[i];
        *reinterpret_cast<half_vec *>(out) = t;
    }
}

template <typename T> __global__ __launch_bounds__(256) void fill_kernel(T *p, size_t n, T v) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256)
        p[i] = v;
}

template <typename T>
dh_status maxpool_forward(dh_ctx *ctx, T *res, size_t *res_h, size_t *res_w, const T *data, size_t N, size_t C,
                          size_t H, size_t W, size_t ph, size_t pw, size_t sh, size_t sw, size_t padh, size_t padw) {
    DH_REQUIRE_CTX(ctx);
    if (sh == 0 || sw == 0 || H + 2 * padh < ph || W + 2 * padw < pw)
        return dh_fail(DH_ERR_INVALID_ARG, "Pooling: window %zux%zu does not fit the padded image %zux%zu", ph, pw,
                       H + 2 * padh, W + 2 * padw);
    // Pooling.cpp:38-39: P is derived with stride_w and Q with stride_h.
    const size_t P = (H + 2 * padh - ph) / sw + 1, Q = (W + 2 * padw - pw) / sh + 1;
    if (res_h)
        *res_h = P;
    if (res_w)
        *res_w = Q;
    const size_t total = N * C * P * Q;
    if (total == 0)
        return DH_OK;
    if (H * W >= (size_t(1) << 31) || P * Q >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Pooling: image extents exceed 2^31 elements");
    size_t grid = dh_ceil_div(total, 256);
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 32;
    if (grid > cap)
        grid = cap;
    constexpr int VI = 16 / sizeof(T);
    if (ph == 2 && pw == 2 && sh == 2 && sw == 2 && padh == 0 && padw == 0 && H % 2 == 0 && W % VI == 0 &&
        dh_aligned(data, 16) && dh_aligned(res, 8) && total * 2 / VI < (size_t(1) << 39)) {
        const size_t items = N * C * P * (W / VI);
        hipLaunchKernelGGL((maxpool2x2_kernel<T, VI>), dim3(static_cast<unsigned>(dh_ceil_div(items, 256))), dim3(256), 0,
                           ctx->stream, res, data, items, static_cast<unsigned>(W), static_cast<unsigned>(W / VI));
    } else if (P == 1 && Q == 1 && W == 1) {
        // Pooling.cpp:57-66: this quick path folds the window into numeric_limits::max(), so that
        // value is what the CPU kernel returns for every output.
        hipLaunchKernelGGL((fill_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, total,
                           std::numeric_limits<T>::max());
    } else {
        hipLaunchKernelGGL((maxpool_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, data,
                           total, 0u, static_cast<unsigned>(H), static_cast<unsigned>(W), static_cast<unsigned>(P),
                           static_cast<unsigned>(Q), static_cast<unsigned>(ph), static_cast<unsigned>(pw),
                           static_cast<unsigned>(sh), static_cast<unsigned>(sw), static_cast<unsigned>(padh),
                           static_cast<unsigned>(padw));
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// Per-channel streaming ops: BiasAdd and BatchNorm inference. The matrix is viewed as
// (rows * C) x HW: every view row has one channel, so the statistics are fetched once per row.
// ---------------------------------------------------------------------------------------
template <typename T, int VEC, bool BATCHNORM>
__global__ __launch_bounds__(256) void channel_kernel(T *res, const T *data, size_t vrows, size_t hw_vecs, unsigned C,
                                                      const T *a0 /* bias | gamma */, const T *beta, const T *mean,
                                                      const T *var, T eps) {
    const size_t HW = hw_vecs * VEC;
    for (size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x; cv < hw_vecs;
         cv += static_cast<size_t>(gridDim.y) * blockDim.x) {
        for (size_t r = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y; r < vrows;
             r += static_cast<size_t>(gridDim.x) * blockDim.y) {
            const unsigned ch = static_cast<unsigned>(r % C);
            T x[VEC];
            dh_load_vec<T, VEC>(data + r * HW + cv * VEC, x);
            T o[VEC];
            if constexpr (BATCHNORM) {
                // BatchNorm2DTestForward.h:96-97, same operation order
                const T sd = sizeof(T) == 4 ? sqrtf(var[ch] + eps) : sqrt(var[ch] + eps);
                const T g = a0[ch], b = beta[ch], mu = mean[ch];
#pragma unroll
                for (int i = 0; i < VEC; i++) {
                    const T x_hat = (x[i] - mu) / sd;
                    o[i] = g * x_hat + b;
                }
            } else {
                const T b = a0[ch];
#pragma unroll
                for (int i = 0; i < VEC; i++)
                    o[i] = x[i] + b;
            }
            dh_store_vec<T, VEC>(res + r * HW + cv * VEC, o);
        }
    }
}

template <typename T, bool BATCHNORM>
static inline dh_status channel_launch(dh_ctx *ctx, T *res, const T *data, size_t vrows, size_t HW, size_t C,
                                       const T *a0, const T *beta, const T *mean, const T *var, T eps) {
    if (vrows == 0 || HW == 0)
        return DH_OK;
    constexpr int V = 16 / sizeof(T);
    const bool vec_ok = (HW % V == 0) && dh_aligned(res, 16) && dh_aligned(data, 16);
    const size_t cvecs = vec_ok ? HW / V : HW;
    unsigned tx = 1;
    while (tx < 256 && tx < cvecs)
        tx <<= 1;
    const unsigned ty = 256 / tx;
    size_t gy = dh_ceil_div(cvecs, tx);
    if (gy > 1024)
        gy = 1024;
    size_t gx = dh_ceil_div(vrows, ty);
    size_t cap = static_cast<size_t>(ctx->num_cus) * 32 / gy;
    if (cap < 1)
        cap = 1;
    if (gx > cap)
        gx = cap;
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), block(tx, ty);
    if (vec_ok)
        hipLaunchKernelGGL((channel_kernel<T, V, BATCHNORM>), grid, block, 0, ctx->stream, res, data, vrows, cvecs,
                           static_cast<unsigned>(C), a0, beta, mean, var, eps);
    else
        hipLaunchKernelGGL((channel_kernel<T, 1, BATCHNORM>), grid, block, 0, ctx->stream, res, data, vrows, cvecs,
                           static_cast<unsigned>(C), a0, beta, mean, var, eps);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T>
dh_status bias_add(dh_ctx *ctx, T *res, const T *data, size_t rows, size_t cols, const T *bias, size_t num_bias) {
    DH_REQUIRE_CTX(ctx);
    if (num_bias == 0 || cols % num_bias != 0 || num_bias >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "BiasAdd: %zu columns cannot be split into %zu channels", cols, num_bias);
    return channel_launch<T, false>(ctx, res, data, rows * num_bias, cols / num_bias, num_bias, bias, nullptr, nullptr,
                                    nullptr, T(0));
}

template <typename T>
dh_status batchnorm_inference(dh_ctx *ctx, T *res, const T *data, size_t rows, size_t cols, const T *gamma,
                              const T *beta, const T *mean, const T *var, size_t channels, T eps, int stat_index) {
    DH_REQUIRE_CTX(ctx);
    if (stat_index == 1) {
        // statistics indexed by the image (row) like the reference's CPU loop
        if (rows >= (size_t(1) << 31))
            return dh_fail(DH_ERR_RUNTIME, "BatchNorm: too many rows");
        return channel_launch<T, true>(ctx, res, data, rows, cols, rows ? rows : 1, gamma, beta, mean, var, eps);
    }
    if (stat_index != 0)
        return dh_fail(DH_ERR_RUNTIME, "BatchNorm: stat_index must be 0 (channel) or 1 (row)");
    if (channels == 0 || cols % channels != 0 || channels >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "BatchNorm: %zu columns cannot be split into %zu channels", cols, channels);
    return channel_launch<T, true>(ctx, res, data, rows * channels, cols / channels, channels, gamma, beta, mean, var,
                                   eps);
}

// ---------------------------------------------------------------------------------------
// Softmax: G lanes per row; max, exp and sum, scale (Softmax.h:36-52).
// ---------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ T dev_exp(T a);
template <> __device__ __forceinline__ float dev_exp<float>(float a) { return expf(a); }
template <> __device__ __forceinline__ double dev_exp<double>(double a) { return exp(a); }

template <typename T>
__global__ __launch_bounds__(256) void softmax_kernel(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,
                                                      size_t ld, int G) {
    const int lane = threadIdx.x % G;
    const size_t rpb = 256 / G;
    for (size_t r = static_cast<size_t>(blockIdx.x) * rpb + threadIdx.x / G; r < rows;
         r += static_cast<size_t>(gridDim.x) * rpb) {
        const T *in = arg + r * ld;
        T *out = res + r * ld_res;
        // max: NaN anywhere in the row ends up in every output through the sum, as on the CPU
        T mx = -std::numeric_limits<T>::infinity();
        for (size_t c = lane; c < cols; c += G) {
            const T v = in[c];
            mx = (mx < v) ? v : mx;
        }
        for (int off = G / 2; off >= 1; off >>= 1) {
            const T o = dh_shfl_xor(mx, off);
            mx = (mx < o) ? o : mx;
        }
        const T first = in[0];
        if (first != first)
            mx = first;
        T sum = T(0);
        for (size_t c = lane; c < cols; c += G) {
            const T e = dev_exp<T>(in[c] - mx);
            out[c] = e;
            sum += e;
        }
        for (int off = G / 2; off >= 1; off >>= 1)
            sum += dh_shfl_xor(sum, off);
        const T inv = T(1) / sum;
        for (size_t c = lane; c < cols; c += G)
            out[c] *= inv;
    }
}

template <typename T>
dh_status softmax(dh_ctx *ctx, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols || ld_res < cols)
        return dh_fail(DH_ERR_RUNTIME, "Softmax - a leading dimension is smaller than the column count");
    if (rows == 0 || cols == 0)
        return DH_OK;
    int G = 1;
    while (G < 64 && static_cast<size_t>(G) < cols)
        G <<= 1;
    size_t grid = dh_ceil_div(rows, 256 / G);
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 16;
    if (grid > cap)
        grid = cap;
    hipLaunchKernelGGL((softmax_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, ld_res,
                       arg, rows, cols, ld, G);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

} // namespace dh_dnn
