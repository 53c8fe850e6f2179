// Kernels that stand for a CHAIN of DaphneIR operators, each computed in one pass (or one launch) by libdaphne_hip.so:
//   conv2DForwardFused   Convolution_Forward -> NN_Relu_Forward -> NN_Max_Forward (2 x 2 window, stride 2, no padding);
//                        epilogue bit 0: the rectifier, bit 1: the pooling (either may be missing from the chain)
//   affineForwardFused   NN_Affine_Forward -> NN_Relu_Forward
//   normalEquations      syrk(X) [+ lambda on the diagonal] and matMul(t(X), y) from one pass over X
//   kmeansAssign         idxminRow(((matMul(X, t(C)) * -2) + xx) + cc) without the rows x k distances in memory
//   kmeansUpdate         per-cluster means of the rows of X by label (t(P) X / counts with P = one-hot(idx), P never built)
//   kmeansStep           kmeansAssign followed by kmeansUpdate, from one pass over X where the library has that kernel
// The reference has no kernel for any of them: its compiler emits one kernel call per operator
// (src/compiler/lowering/RewriteToCallKernelOpPass.cpp:360-455). Which chain of operators may be replaced by which of
// these is decided by HIP::OperatorChainMatcher (OperatorChainMatcher.h); the compiler pass that applies it is
// src/compiler/lowering/FuseHIPOperatorChainsPass.cpp. Results: the convolution, affine and assignment kernels give the
// bits of the chain they replace; normalEquations and kmeansUpdate add in another order (within rounding).
// Signatures follow the kernels they start from (kernels/CUDA/Convolution.h:33-38, kernels/CUDA/Affine.h:24-26,
// kernels/Syrk.h:51, kernels/AggRow.h:71-94), with the result(s) first and the DaphneContext last.
#pragma once

#include <runtime/local/kernels/HIP/HostUtils.h>

namespace HIP {

template <typename... A> inline dh_status dh_conv2d_forward_fused(float, A... a) { return dh_conv2d_forward_fused_f32(a...); }
template <typename... A> inline dh_status dh_conv2d_forward_fused(double, A... a) { return dh_conv2d_forward_fused_f64(a...); }
template <typename... A> inline dh_status dh_affine_forward_fused(float, A... a) { return dh_affine_forward_fused_f32(a...); }
template <typename... A> inline dh_status dh_affine_forward_fused(double, A... a) { return dh_affine_forward_fused_f64(a...); }
template <typename... A> inline dh_status dh_normal_equations(float, A... a) { return dh_normal_equations_f32(a...); }
template <typename... A> inline dh_status dh_normal_equations(double, A... a) { return dh_normal_equations_f64(a...); }
template <typename... A> inline dh_status dh_kmeans_assign(float, A... a) { return dh_kmeans_assign_f32(a...); }
template <typename... A> inline dh_status dh_kmeans_assign(double, A... a) { return dh_kmeans_assign_f64(a...); }
template <typename... A> inline dh_status dh_kmeans_update(float, A... a) { return dh_kmeans_update_f32(a...); }
template <typename... A> inline dh_status dh_kmeans_update(double, A... a) { return dh_kmeans_update_f64(a...); }
template <typename... A> inline dh_status dh_kmeans_step(float, A... a) { return dh_kmeans_step_f32(a...); }
template <typename... A> inline dh_status dh_kmeans_step(double, A... a) { return dh_kmeans_step_f64(a...); }

// epilogue bits of conv2DForwardFused / affineForwardFused (dh_epilogue of the C ABI)
constexpr size_t EPILOGUE_RELU = 1, EPILOGUE_MAXPOOL_2X2 = 2;

template <class DTRes, class DTArg> struct Conv2DForwardFused {
    static void apply(DTRes *&res, size_t *res_h, size_t *res_w, const DTArg *data, const DTArg *filter, const DTArg *bias,
                      const size_t batch_size, const size_t num_channels, const size_t img_h, const size_t img_w,
                      const size_t filter_h, const size_t filter_w, const size_t stride_h, const size_t stride_w,
                      const size_t pad_h, const size_t pad_w, const size_t epilogue, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        const size_t F = filter->getNumRows();
        size_t P = (img_h + 2 * pad_h - filter_h) / stride_h + 1, Q = (img_w + 2 * pad_w - filter_w) / stride_w + 1;
        if (epilogue & EPILOGUE_MAXPOOL_2X2) {
            P /= 2;
            Q /= 2;
        }
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(batch_size, F * P * Q, false, &alloc_desc);
        const VT *b = (bias && bias != filter) ? bias->getValues(&alloc_desc) : nullptr; // as Convolution::Forward
        check(dh_conv2d_forward_fused(VT(), detail::raw(ctx), res->getValues(&alloc_desc), res_h, res_w, data->getValues(&alloc_desc),
                                      filter->getValues(&alloc_desc), filter->getNumRows(), filter->getNumCols(), b, batch_size,
                                      num_channels, img_h, img_w, filter_h, filter_w, stride_h, stride_w, pad_h, pad_w,
                                      static_cast<unsigned>(epilogue)));
    }
};
template <class DTRes, class DTArg>
void conv2DForwardFused(DTRes *&res, size_t *res_h, size_t *res_w, const DTArg *data, const DTArg *filter, const DTArg *bias,
                        size_t batch_size, size_t num_channels, size_t img_h, size_t img_w, size_t filter_h, size_t filter_w,
                        size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t epilogue, DCTX(ctx)) {
    Conv2DForwardFused<DTRes, DTArg>::apply(res, res_h, res_w, data, filter, bias, batch_size, num_channels, img_h, img_w, filter_h,
                                            filter_w, stride_h, stride_w, pad_h, pad_w, epilogue, ctx);
}

template <class DTRes, class DTArg> struct AffineForwardFused {
    static void apply(DTRes *&res, const DTArg *data, const DTArg *weights, const DTArg *bias, const size_t epilogue, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        if (data->getNumCols() != weights->getNumRows())
            throw std::runtime_error("HIP::affineForwardFused: #cols of lhs and #rows of rhs must be the same (" +
                                     std::to_string(data->getNumCols()) + " != " + std::to_string(weights->getNumRows()) + ")");
        if (res == nullptr)
            res = DataObjectFactory::create<DTRes>(data->getNumRows(), weights->getNumCols(), false, &alloc_desc);
        check(dh_affine_forward_fused(VT(), detail::raw(ctx), res->getValues(&alloc_desc), data->getValues(&alloc_desc),
                                      data->getNumRows(), data->getNumCols(), weights->getValues(&alloc_desc), weights->getNumRows(),
                                      weights->getNumCols(), bias ? bias->getValues(&alloc_desc) : nullptr,
                                      bias ? bias->getNumRows() : 0, bias ? bias->getNumCols() : 0, static_cast<unsigned>(epilogue)));
    }
};
template <class DTRes, class DTArg>
void affineForwardFused(DTRes *&res, const DTArg *data, const DTArg *weights, const DTArg *bias, size_t epilogue, DCTX(ctx)) {
    AffineForwardFused<DTRes, DTArg>::apply(res, data, weights, bias, epilogue, ctx);
}

// A = t(X) X + lambda I (cols x cols), b = t(X) y (cols x 1)
template <class DTRes, class DTArg> struct NormalEquations {
    static void apply(DTRes *&A, DTRes *&b, const DTArg *X, const DTArg *y, const typename DTArg::VT lambda, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTRes::VT;
        const size_t rows = X->getNumRows(), cols = X->getNumCols();
        if (y->getNumRows() != rows || y->getNumCols() != 1)
            throw std::runtime_error("HIP::normalEquations: y must be " + std::to_string(rows) + " x 1, it is " +
                                     std::to_string(y->getNumRows()) + " x " + std::to_string(y->getNumCols()));
        if (A == nullptr)
            A = DataObjectFactory::create<DTRes>(cols, cols, false, &alloc_desc);
        if (b == nullptr)
            b = DataObjectFactory::create<DTRes>(cols, 1, false, &alloc_desc);
        check(dh_normal_equations(VT(), detail::raw(ctx), A->getValues(&alloc_desc), A->getRowSkip(), b->getValues(&alloc_desc),
                                  b->getRowSkip(), X->getValues(&alloc_desc), rows, cols, X->getRowSkip(), y->getValues(&alloc_desc),
                                  y->getRowSkip(), lambda));
    }
};
template <class DTRes, class DTArg>
void normalEquations(DTRes *&A, DTRes *&b, const DTArg *X, const DTArg *y, typename DTArg::VT lambda, DCTX(ctx)) {
    NormalEquations<DTRes, DTArg>::apply(A, b, X, y, lambda, ctx);
}

// idx (rows x 1, size_t): first position of the minimum of ((X t(C))[i][c] * -2 + xx[i]) + cc[c]; xx rows x 1, cc 1 x k
template <class DTIdx, class DTArg> struct KmeansAssign {
    static void apply(DTIdx *&idx, const DTArg *X, const DTArg *C, const DTArg *xx, const DTArg *cc, DCTX(ctx)) {
        static_assert(sizeof(typename DTIdx::VT) == sizeof(uint64_t), "the labels are 64-bit positions");
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        checkShapes(X, C, xx, cc);
        if (idx == nullptr)
            idx = DataObjectFactory::create<DTIdx>(X->getNumRows(), 1, false, &alloc_desc);
        if (idx->getRowSkip() != 1 || xx->getRowSkip() != 1)
            throw std::runtime_error("HIP::kmeansAssign: the labels and the row norms must be contiguous columns");
        check(dh_kmeans_assign(VT(), detail::raw(ctx), reinterpret_cast<uint64_t *>(idx->getValues(&alloc_desc)),
                               X->getValues(&alloc_desc), X->getNumRows(), X->getNumCols(), X->getRowSkip(), C->getValues(&alloc_desc),
                               C->getNumRows(), C->getRowSkip(), xx->getValues(&alloc_desc), cc->getValues(&alloc_desc)));
    }
    static void checkShapes(const DTArg *X, const DTArg *C, const DTArg *xx, const DTArg *cc) {
        if (C->getNumCols() != X->getNumCols())
            throw std::runtime_error("HIP::kmeans: X and C must have the same number of columns");
        if (xx->getNumRows() != X->getNumRows() || xx->getNumCols() != 1)
            throw std::runtime_error("HIP::kmeans: xx must be #rows(X) x 1");
        if (cc->getNumRows() != 1 || cc->getNumCols() != C->getNumRows())
            throw std::runtime_error("HIP::kmeans: cc must be 1 x #rows(C)");
    }
};
template <class DTIdx, class DTArg> void kmeansAssign(DTIdx *&idx, const DTArg *X, const DTArg *C, const DTArg *xx, const DTArg *cc, DCTX(ctx)) {
    KmeansAssign<DTIdx, DTArg>::apply(idx, X, C, xx, cc, ctx);
}

// Cnew (k x cols): mean of the rows of X with label c; counts (1 x k): their number (an empty cluster: 0 / 0)
template <class DTRes, class DTArg, class DTIdx> struct KmeansUpdate {
    static void apply(DTRes *&Cnew, DTRes *&counts, const DTArg *X, const DTIdx *idx, const size_t k, DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        if (idx->getNumRows() != X->getNumRows() || idx->getNumCols() != 1 || idx->getRowSkip() != 1)
            throw std::runtime_error("HIP::kmeansUpdate: idx must be a contiguous #rows(X) x 1 column");
        if (Cnew == nullptr)
            Cnew = DataObjectFactory::create<DTRes>(k, X->getNumCols(), false, &alloc_desc);
        if (counts == nullptr)
            counts = DataObjectFactory::create<DTRes>(1, k, false, &alloc_desc);
        check(dh_kmeans_update(VT(), detail::raw(ctx), Cnew->getValues(&alloc_desc), Cnew->getRowSkip(), counts->getValues(&alloc_desc),
                               X->getValues(&alloc_desc), X->getNumRows(), X->getNumCols(), X->getRowSkip(),
                               reinterpret_cast<const uint64_t *>(idx->getValues(&alloc_desc)), k));
    }
};
template <class DTRes, class DTArg, class DTIdx>
void kmeansUpdate(DTRes *&Cnew, DTRes *&counts, const DTArg *X, const DTIdx *idx, size_t k, DCTX(ctx)) {
    KmeansUpdate<DTRes, DTArg, DTIdx>::apply(Cnew, counts, X, idx, k, ctx);
}

template <class DTIdx, class DTRes, class DTArg> struct KmeansStep {
    static void apply(DTIdx *&idx, DTRes *&Cnew, DTRes *&counts, const DTArg *X, const DTArg *C, const DTArg *xx, const DTArg *cc,
                      DCTX(ctx)) {
        AllocationDescriptorHIP alloc_desc(ctx, detail::deviceID);
        using VT = typename DTArg::VT;
        KmeansAssign<DTIdx, DTArg>::checkShapes(X, C, xx, cc);
        const size_t k = C->getNumRows();
        if (idx == nullptr)
            idx = DataObjectFactory::create<DTIdx>(X->getNumRows(), 1, false, &alloc_desc);
        if (Cnew == nullptr)
            Cnew = DataObjectFactory::create<DTRes>(k, X->getNumCols(), false, &alloc_desc);
        if (counts == nullptr)
            counts = DataObjectFactory::create<DTRes>(1, k, false, &alloc_desc);
        if (idx->getRowSkip() != 1 || xx->getRowSkip() != 1)
            throw std::runtime_error("HIP::kmeansStep: the labels and the row norms must be contiguous columns");
        check(dh_kmeans_step(VT(), detail::raw(ctx), reinterpret_cast<uint64_t *>(idx->getValues(&alloc_desc)),
                             Cnew->getValues(&alloc_desc), Cnew->getRowSkip(), counts->getValues(&alloc_desc), X->getValues(&alloc_desc),
                             X->getNumRows(), X->getNumCols(), X->getRowSkip(), C->getValues(&alloc_desc), k, C->getRowSkip(),
                             xx->getValues(&alloc_desc), cc->getValues(&alloc_desc)));
    }
};
template <class DTIdx, class DTRes, class DTArg>
void kmeansStep(DTIdx *&idx, DTRes *&Cnew, DTRes *&counts, const DTArg *X, const DTArg *C, const DTArg *xx, const DTArg *cc, DCTX(ctx)) {
    KmeansStep<DTIdx, DTRes, DTArg>::apply(idx, Cnew, counts, X, C, xx, cc, ctx);
}

} // namespace HIP
