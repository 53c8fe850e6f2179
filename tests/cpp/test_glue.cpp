// Exercises the C++ kernel interface (daphne_amd/cpp/daphne_hip_kernels.h) the way the reference's
// Catch2 unit tests exercise its device kernels: contexts built by hand, Kernel<...>::apply called
// directly (reference: test/run_tests.cpp:28-49, test/runtime/local/kernels/CUDA/*.cpp). The
// literals are the reference's own test vectors. Built with a plain host compiler.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <functional>
#include <memory>
#include <stdexcept>
#include <vector>

#include <daphne_hip_kernels.h>

#define TEST_ON_DEVICE 1 // the C ABI under the tests is libdaphne_hip.so on a GPU
#include "dm_access.h"
#include "placement_and_tasks.h"
#include "zscore_via_wrappers.h"

template <typename VT> void run_all(DaphneContext *dctx) {
    using DT = DenseMatrix<VT>;
    auto G = [&](size_t rows, std::vector<VT> v) { return given<DT>(rows, v); };

    // CUDA/MatMulTest.cpp:37-123
    {
        auto m1 = G(3, {1, 2, 3, 3, 1, 2, 2, 3, 1}), m2v = G(3, {13, 13, 10, 10, 13, 13, 13, 10, 13});
        auto m3 = G(2, {1, 0, 3, 0, 0, 0, 2, 0}), m4 = G(4, {0, 1, 2, 0, 1, 1, 0, 0});
        auto v2 = G(3, {1, 2, 3});
        DT *res = nullptr;
        HIP::matMul(res, m1, m1, false, false, dctx);
        CHECK(equals(res, toHost(m2v)));
        DataObjectFactory::destroy(res);
        res = nullptr;
        HIP::matMul(res, m3, m4, false, false, dctx);
        CHECK(equals(res, {3, 4, 2, 2}));
        DataObjectFactory::destroy(res);
        res = nullptr;
        HIP::matMul(res, m1, v2, false, false, dctx);
        CHECK(equals(res, {14, 11, 11}));
        DataObjectFactory::destroy(res);
        // CUDA/MatMulTest.cpp:125-228 (transposed): m3 * m3^T
        res = nullptr;
        HIP::matMul(res, m3, m3, false, true, dctx);
        CHECK(res->getNumRows() == 2 && res->getNumCols() == 2 && equals(res, {10, 6, 6, 4}));
        DataObjectFactory::destroy(res);
        res = nullptr;
        CHECK_THROWS_AS(HIP::matMul(res, m3, m3, false, false, dctx), std::runtime_error);
        CHECK(res == nullptr);
        for (auto *m : {m1, m2v, m3, m4, v2})
            DataObjectFactory::destroy(m);
    }
    // AggRowTest.cpp:221-277 (idxmin incl. ties), result type size_t
    {
        auto m1 = G(3, {4, 6, 3, 9, 2, 5, 0, 1, 7, 4, 5, 4});
        DenseMatrix<size_t> *idx = nullptr;
        HIP::aggRow(AggOpCode::IDXMIN, idx, m1, dctx);
        CHECK(equals(idx, {2, 2, 1}));
        DT *sum = nullptr;
        HIP::aggRow(AggOpCode::SUM, sum, m1, dctx);
        CHECK(equals(sum, {22, 8, 20}));
        DT *cs = nullptr;
        HIP::aggCol(AggOpCode::MAX, cs, m1, dctx);
        CHECK(equals(cs, {7, 6, 5, 9}));
        CHECK((HIP::aggAll<VT, DT>(AggOpCode::SUM, m1, dctx) == VT(50)));
        CHECK_THROWS_AS(HIP::aggRow(static_cast<AggOpCode>(99), sum, m1, dctx), std::runtime_error);
        DataObjectFactory::destroy(idx);
        DataObjectFactory::destroy(sum);
        DataObjectFactory::destroy(cs);
        DataObjectFactory::destroy(m1);
    }
    // EwBinaryMatTest.cpp: add, broadcasting, invalid op code (:611), shape mismatch (EwBinaryMat.h:98-106)
    {
        auto m = G(2, {1, 2, 3, 4, 5, 6}), rv = G(1, {10, 20, 30}), cv = G(2, {100, 200}), bad = G(3, {1, 2, 3});
        DT *res = nullptr;
        HIP::ewBinaryMat(BinaryOpCode::ADD, res, m, rv, dctx);
        CHECK(equals(res, {11, 22, 33, 14, 25, 36}));
        HIP::ewBinaryMat(BinaryOpCode::ADD, res, res, cv, dctx); // in place, res aliases lhs (TasksCUDA.cpp:109)
        CHECK(equals(res, {111, 122, 133, 214, 225, 236}));
        DT *sca = nullptr;
        HIP::ewBinaryObjSca(BinaryOpCode::GT, sca, m, VT(3), dctx);
        CHECK(equals(sca, {0, 0, 0, 1, 1, 1}));
        CHECK_THROWS_AS(HIP::ewBinaryMat(static_cast<BinaryOpCode>(999), res, m, m, dctx), std::runtime_error);
        CHECK_THROWS_AS(HIP::ewBinaryMat(BinaryOpCode::ADD, res, m, bad, dctx), std::runtime_error);
        // a view with rowSkip > numCols
        DT *view = m->slice(0, 2, 1, 3);
        DT *vres = nullptr;
        HIP::ewBinaryObjSca(BinaryOpCode::MUL, vres, view, VT(2), dctx);
        CHECK(equals(vres, {4, 6, 10, 12}));
        for (auto *x : {view, m, rv, cv, bad, res, sca, vres})
            DataObjectFactory::destroy(x);
    }
    // EwUnaryMatTest.cpp:148 sqrt domain_error, :62 abs
    {
        auto a = G(1, {-1, 4, 9}), b = G(1, {1, 4, 9});
        DT *res = nullptr;
        CHECK_THROWS_AS(HIP::ewUnaryMat(UnaryOpCode::SQRT, res, a, dctx), std::domain_error);
        DataObjectFactory::destroy(res);
        res = nullptr;
        HIP::ewUnaryMat(UnaryOpCode::SQRT, res, b, dctx);
        CHECK(equals(res, {1, 2, 3}));
        HIP::ewUnaryMat(UnaryOpCode::ABS, res, a, dctx);
        CHECK(equals(res, {1, 4, 9}));
        CHECK_THROWS_AS(HIP::ewUnaryMat(static_cast<UnaryOpCode>(999), res, a, dctx), std::runtime_error);
        for (auto *x : {a, b, res})
            DataObjectFactory::destroy(x);
    }
    // DNNConv2DForwardTest.cpp:32-65 and CUDA/DNNConvolutionTest.cpp:36-43
    {
        std::vector<VT> img;
        for (int r = 0; r < 2; r++)
            for (int i = 1; i <= 27; i++)
                img.push_back(VT(i));
        auto input = G(2, img), filter = G(1, {1, 0, 0, 1, 1, 0, 0, 1, 1, 0, 0, 1}), bias = G(1, {0});
        DT *res = nullptr;
        size_t oh = 0, ow = 0;
        HIP::Convolution::Forward<DT, DT>::apply(res, &oh, &ow, input, filter, bias, 2, 3, 3, 3, 2, 2, 2, 2, 1, 1, dctx);
        CHECK(oh == 2 && ow == 2 && equals(res, {30, 36, 48, 96, 30, 36, 48, 96}));
        auto in1 = G(1, {1, 2, 3, 4, 5, 6, 7, 8, 9}), f1 = G(1, {1, 0, 0, 1});
        DT *res1 = nullptr;
        HIP::Convolution::Forward<DT, DT>::apply(res1, &oh, &ow, in1, f1, nullptr, 1, 1, 3, 3, 2, 2, 1, 1, 0, 0, dctx);
        CHECK(equals(res1, {6, 8, 12, 14}));
        DT *res2 = nullptr;
        CHECK_THROWS_AS((HIP::Convolution::Forward<DT, DT>::apply(res2, &oh, &ow, in1, f1, nullptr, 1, 1, 3, 3, 3, 3, 1, 1,
                                                                  0, 0, dctx)),
                        std::invalid_argument);
        for (auto *x : {input, filter, bias, res, in1, f1, res1, res2})
            DataObjectFactory::destroy(x);
    }
    // DNNPoolingTestForward.cpp:74-123 (2x2, stride 2, pad 1 on two 3x5x5 images)
    {
        std::vector<VT> v;
        for (int i = 1; i <= 150; i++)
            v.push_back(VT(i));
        auto in = G(2, v);
        DT *res = nullptr;
        size_t oh = 0, ow = 0;
        HIP::NN::Pooling::Forward<HIP::NN::Pooling::MAX, DT, DT>::apply(res, oh, ow, in, 2, 3, 5, 5, 2, 2, 2, 2, 1, 1, dctx);
        std::vector<VT> exp;
        for (int img = 0; img < 2; img++)
            for (int c = 0; c < 3; c++)
                for (int p : {0, 2, 4})
                    for (int q : {0, 2, 4})
                        exp.push_back(VT(img * 75 + c * 25 + p * 5 + q + 1));
        CHECK(oh == 3 && ow == 3 && equals(res, exp));
        DataObjectFactory::destroy(in);
        DataObjectFactory::destroy(res);
    }
    // DNNBiasAddForwardTest.cpp:32-50, SoftmaxTest.cpp:17-34, CUDA/DNNAffineTest.cpp:28-45,
    // DNNBatchNorm2DForwardTest.cpp:32-49
    {
        auto x = G(2, {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}), b = G(3, {1, 2, 3});
        DT *res = nullptr;
        HIP::BiasAdd<DT, DT>::apply(res, x, b, dctx);
        CHECK(equals(res, {2, 3, 4, 5, 7, 8, 9, 10, 12, 13, 14, 15, 2, 3, 4, 5, 7, 8, 9, 10, 12, 13, 14, 15}));
        auto s = G(3, {-3, -2, -1, 0, 1, 2, 3, 4, 5});
        DT *sm = nullptr;
        HIP::Softmax<DT, DT>::apply(sm, s, dctx);
        CHECK(approx(sm, {VT(0.09003057317038046), VT(0.24472847105479764), VT(0.6652409557748218), VT(0.09003057317038046),
                          VT(0.24472847105479764), VT(0.6652409557748218), VT(0.09003057317038046), VT(0.24472847105479764),
                          VT(0.6652409557748218)},
                     1e-6));
        auto in = G(1, {-3, -2, -1, 0, 1, 2, 3, 4, 5}), w = G(9, {1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6, 7, 7, 8, 8, 9, 9}),
             b0 = G(1, {0});
        DT *aff = nullptr;
        HIP::NN::Affine::Forward<DT, DT>::apply(aff, in, w, b0, dctx);
        CHECK(equals(aff, {105, 105}));
        auto one = G(1, {1}), zero = G(1, {0});
        DT *bn = nullptr;
        HIP::BatchNormInferenceForward<DT, DT>::apply(bn, in, one, zero, zero, one, VT(1e-5), dctx);
        CHECK(approx(bn, {-3, -2, -1, 0, 1, 2, 3, 4, 5}, 1e-4));
        for (auto *m : {x, b, res, s, sm, in, w, b0, aff, one, zero, bn})
            DataObjectFactory::destroy(m);
    }
    // TransposeTest.cpp (3x4), ColBindTest.cpp, ExtractColTest.cpp:159-197, CUDA/DNNActivationTest.cpp:34-40,
    // DNNPoolingTestForward.cpp AVG (first plane of the 2x2 / stride 2 / pad 1 result), FillTest.cpp
    {
        auto m = G(3, {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12});
        DT *mt = nullptr;
        HIP::transpose(mt, m, dctx);
        CHECK(mt->getNumRows() == 4 && mt->getNumCols() == 3);
        CHECK(equals(mt, {1, 5, 9, 2, 6, 10, 3, 7, 11, 4, 8, 12}));
        auto m0 = G(3, {1, 2, 3, 4, 5, 6}), m1 = G(3, {10, 20, 30, 40, 50, 60, 70, 80, 90});
        DT *cb = nullptr;
        HIP::colBind(cb, m0, m1, dctx);
        CHECK(equals(cb, {1, 2, 10, 20, 30, 3, 4, 40, 50, 60, 5, 6, 70, 80, 90}));
        bool threw = false;
        try {
            DT *bad = nullptr;
            HIP::colBind(bad, m0, mt, dctx);
        } catch (const std::runtime_error &) {
            threw = true;
        }
        CHECK(threw);
        auto arg = G(3, {1, 2, 3, 4, 5, 6, 7, 8, 9});
        using DTSel = DenseMatrix<int64_t>;
        auto sel = given<DTSel>(8, {1, 2, 2, 0, 1, 0, 1, 2});
        DT *ex = nullptr;
        HIP::extractCol(ex, arg, sel, dctx);
        CHECK(equals(ex, {2, 3, 3, 1, 2, 1, 2, 3, 5, 6, 6, 4, 5, 4, 5, 6, 8, 9, 9, 7, 8, 7, 8, 9}));
        auto selbad = given<DTSel>(2, {1, 3});
        threw = false;
        try {
            DT *bad = nullptr;
            HIP::extractCol(bad, arg, selbad, dctx);
        } catch (const std::out_of_range &) {
            threw = true;
        }
        CHECK(threw);
        auto in = G(1, {-3, -2, -1, 0, 1, 2, 3, 4, 5});
        DT *rl = nullptr;
        HIP::NN::Activation::Forward<HIP::NN::Activation::ReLU, DT, DT>::apply(rl, in, dctx);
        CHECK(equals(rl, {0, 0, 0, 0, 1, 2, 3, 4, 5}));
        DT *f = nullptr;
        HIP::fill(f, VT(2.5), 3, 4, dctx);
        CHECK(equals(f, std::vector<VT>(12, VT(2.5))));
        std::vector<VT> img(150);
        for (int i = 0; i < 150; i++)
            img[i] = VT(i + 1);
        auto pin = G(2, img);
        DT *avg = nullptr;
        size_t oh = 0, ow = 0;
        HIP::NN::Pooling::Forward<HIP::NN::Pooling::AVG, DT, DT>::apply(avg, oh, ow, pin, 2, 3, 5, 5, 2, 2, 2, 2, 1, 1, dctx);
        CHECK(oh == 3 && ow == 3);
        auto av = toHost(avg);
        const VT first[9] = {0.25, 1.25, 2.25, 4.25, 10, 12, 9.25, 20, 22};
        bool ok = av.size() == 54;
        for (int i = 0; ok && i < 9; i++)
            ok = av[i] == first[i];
        CHECK(ok);
        auto X = G(7, {1, 4, 5, 3, 7, 1, 2, 3, 5, 9, 8, 1, 1, 2, 3, 5, 1, 9, 2, 3, 1}), yv = G(7, {1, 2, 3, 4, 5, 6, 7});
        DT *gv = nullptr, *gm = nullptr;
        HIP::gemv(gv, X, yv, dctx);
        HIP::matMul(gm, X, yv, true, false, dctx);
        CHECK(equals(gv, toHost(gm)));
        for (auto *q : {m, mt, m0, m1, cb, arg, ex, in, rl, f, pin, avg, X, yv, gv, gm})
            DataObjectFactory::destroy(q);
        DataObjectFactory::destroy(sel);
        DataObjectFactory::destroy(selbad);
    }
    // SyrkTest.cpp:32-58 (syrk == t(X) X) and SolveTest.cpp:42-68 (normal equations)
    {
        auto X = G(7, {1, 4, 5, 3, 7, 1, 2, 3, 5, 9, 8, 1, 1, 2, 3, 5, 1, 9, 2, 3, 1}), w = G(3, {1, 2, 3});
        DT *y = nullptr, *A = nullptr, *A2 = nullptr, *b = nullptr, *sol = nullptr;
        HIP::matMul(y, X, w, false, false, dctx);
        HIP::syrk(A, X, true, dctx);
        HIP::matMul(A2, X, X, true, false, dctx);
        CHECK(equals(A, toHost(A2)));
        HIP::matMul(b, X, y, true, false, dctx);
        HIP::solve(sol, A, b, dctx);
        CHECK(approx(sol, {1, 2, 3}, sizeof(VT) == 4 ? 1e-3 : 1e-6));
        for (auto *m : {X, w, y, A, A2, b, sol})
            DataObjectFactory::destroy(m);
    }
}

// DNN training kernels with the reference's own vectors (DNNConv2DBackwardTest.cpp:23-95, DNNPoolingBackwardTest.cpp:25-110,
// DNNBatchNorm2DBackwardTest.cpp:22-70, DNNBatchNorm2DForwardTest.cpp:51-90)
template <typename VT> void run_training(DaphneContext *dctx) {
    using DT = DenseMatrix<VT>;
    auto G = [&](size_t rows, std::vector<VT> v) { return given<DT>(rows, v); };
    {
        auto dy = G(1, {1, 2, 3, 4, 5, 6, 7, 8});
        auto filter = G(2, {1, 0, 0, 2, 2, 0, 0, 3, 3, 0, 0, 4, 5, 0, 0, 6, 6, 0, 0, 7, 7, 0, 0, 8});
        DT *dx = nullptr, *dw = nullptr;
        HIP::Conv2DBackwardData<DT, DT>::apply(filter, dy, 2, 2, 1, 1, 1, 3, 3, 3, 2, 3, 2, 2, dx, dctx);
        CHECK(equals(dx, {32, 0, 40, 0, 44, 0, 48, 0, 56, 38, 0, 48, 0, 56, 0, 58, 0, 68, 44, 0, 56, 0, 68, 0, 68, 0, 80}));
        auto in = G(1, {1, 2, 3, 4, 5, 6, 7, 8, 9, 1, 2, 3, 4, 5, 6, 7, 8, 9, 1, 2, 3, 4, 5, 6, 7, 8, 9});
        HIP::Conv2DBackwardFilter<DT, DT>::apply(dw, in, dy, 2, 2, 1, 1, 1, 3, 3, 3, 2, 3, 2, 2, dctx);
        CHECK(equals(dw, {20, 36, 36, 64, 20, 36, 36, 64, 20, 36, 36, 64, 40, 76, 76, 144, 40, 76, 76, 144, 40, 76, 76, 144}));
        for (auto *m : {dy, filter, dx, dw, in})
            DataObjectFactory::destroy(m);
    }
    {
        std::vector<VT> iv(54), dv;
        for (int i = 0; i < 54; i++)
            iv[i] = VT(i + 1);
        for (int r = 0; r < 2; r++)
            for (int i = 1; i <= 12; i++)
                dv.push_back(VT(i));
        auto in = G(2, iv), dout = G(2, dv);
        DT *rmax = nullptr, *ravg = nullptr;
        HIP::MaxPoolBackward<DT, DT>::apply(rmax, in, dout, 2, 3, 3, 3, 2, 2, 2, 2, 1, 1, dctx);
        std::vector<VT> emax, eavg, one = {1, 0, 2, 0, 0, 0, 3, 0, 4, 5, 0, 6, 0, 0, 0, 7, 0, 8, 9, 0, 10, 0, 0, 0, 11, 0, 12};
        std::vector<VT> onea = {0.25, 0.50, 0.50, 0.75, 1.00, 1.00, 0.75, 1.00, 1.00, 1.25, 1.50, 1.50, 1.75, 2.00,
                                2.00, 1.75, 2.00, 2.00, 2.25, 2.50, 2.50, 2.75, 3.00, 3.00, 2.75, 3.00, 3.00};
        for (int r = 0; r < 2; r++) {
            emax.insert(emax.end(), one.begin(), one.end());
            eavg.insert(eavg.end(), onea.begin(), onea.end());
        }
        CHECK(equals(rmax, emax));
        HIP::AvgPoolBackward<DT, DT>::apply(ravg, in, dout, 2, 3, 3, 3, 2, 2, 2, 2, 1, 1, dctx);
        CHECK(equals(ravg, eavg));
        for (auto *m : {in, dout, rmax, ravg})
            DataObjectFactory::destroy(m);
    }
    {
        std::vector<VT> v;
        for (int r = 0; r < 2; r++)
            for (int i = 1; i <= 12; i++)
                v.push_back(VT(i));
        auto in = G(2, v), dout = G(2, v), gamma = G(3, {1, 1, 1}), mean = G(3, {2.5, 6.5, 10.5});
        const VT ivv = VT(1 / std::sqrt(1.25f + 1e-5f));
        auto invVar = G(3, {ivv, ivv, ivv});
        DT *dX = nullptr, *dG = nullptr, *dB = nullptr;
        HIP::BatchNorm2DBackward<DT, DT>::apply(dX, dG, dB, mean, invVar, in, dout, gamma, VT(1e-5), dctx);
        CHECK(approx(dG, {8.9442, 8.9442, 8.9442}, 1e-3));
        CHECK(approx(dB, {20, 52, 84}, 1e-4));
        CHECK(std::fabs(double(toHost(dX)[0]) + 1.0733e-05) < 1e-5);
        // training forward: statistics of the batch, output normalised per channel
        DT *res = nullptr, *nm = nullptr, *nv = nullptr, *mn = nullptr, *iv2 = nullptr;
        auto zeros = G(3, {0, 0, 0}), ones = G(3, {1, 1, 1});
        HIP::BatchNorm2DTrainForward<DT, DT>::apply(res, nm, nv, mn, iv2, in, gamma, zeros, zeros, ones, VT(1e-5), VT(1), dctx);
        CHECK(approx(mn, {2.5, 6.5, 10.5}, 1e-5));
        CHECK(approx(nv, {1.25, 1.25, 1.25}, 1e-5));
        CHECK(approx(iv2, {ivv, ivv, ivv}, 1e-5));
        CHECK(std::fabs(double(toHost(res)[0]) - (1 - 2.5) * double(ivv)) < 1e-5);
        for (auto *m : {in, dout, gamma, mean, invVar, dX, dG, dB, res, nm, nv, mn, iv2, zeros, ones})
            DataObjectFactory::destroy(m);
    }
}

// Integer instantiations (EwBinaryMatTest.cpp:34, EwBinaryObjScaTest.cpp:36 run with uint32_t; AggAllTest.cpp:32 with
// int64_t among others): the reference's literals where they are integers, plus integer-only behaviour.
template <typename VT> void run_integer_elementwise(DaphneContext *dctx) {
    using DT = DenseMatrix<VT>;
    auto G = [&](size_t rows, std::vector<VT> v) { return given<DT>(rows, v); };
    // EwBinaryMatTest.cpp:69-102 (add), :104-125 (mul), :178-222 (div), :523-557 (max)
    auto m1 = G(2, {1, 2, 0, 0, 1, 3}), m2 = G(2, {0, 9, 0, 0, 3, 4}), m3 = G(2, {1, 11, 0, 0, 4, 7});
    DT *res = nullptr;
    HIP::ewBinaryMat(BinaryOpCode::ADD, res, m1, m2, dctx);
    CHECK(equals(res, toHost(m3)));
    HIP::ewBinaryMat(BinaryOpCode::MUL, res, m1, m2, dctx);
    CHECK(equals(res, {0, 18, 0, 0, 3, 12}));
    HIP::ewBinaryMat(BinaryOpCode::MAX, res, m1, m2, dctx);
    CHECK(equals(res, {1, 9, 0, 0, 3, 4}));
    auto d1 = G(2, {7, 9, 20, 0, 1, 100}), d2 = G(2, {2, 3, 6, 5, 1, 7});
    HIP::ewBinaryMat(BinaryOpCode::DIV, res, d1, d2, dctx);
    CHECK(equals(res, {3, 3, 3, 0, 1, 14})); // truncating division
    HIP::ewBinaryMat(BinaryOpCode::MOD, res, d1, d2, dctx);
    CHECK(equals(res, {1, 0, 2, 0, 0, 2}));
    HIP::ewBinaryObjSca(BinaryOpCode::POW, res, d2, VT(3), dctx);
    CHECK(equals(res, {8, 27, 216, 125, 1, 343}));
    HIP::ewBinaryObjSca(BinaryOpCode::GE, res, d1, VT(9), dctx);
    CHECK(equals(res, {0, 1, 1, 0, 0, 1}));
    // a zero divisor is reported instead of trapping the process
    CHECK_THROWS_AS(HIP::ewBinaryMat(BinaryOpCode::DIV, res, d1, m1, dctx), std::domain_error);
    CHECK_THROWS_AS(HIP::ewBinaryObjSca(BinaryOpCode::MOD, res, d1, VT(0), dctx), std::domain_error);
    for (auto *m : {m1, m2, m3, d1, d2, res})
        DataObjectFactory::destroy(m);
}

// A pipeline body with one integer division, the way the compiler outlines it.
static void funDivSi64(DenseMatrix<int64_t> ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *a = dynamic_cast<DenseMatrix<int64_t> *>(inputs[0]), *b = dynamic_cast<DenseMatrix<int64_t> *>(inputs[1]);
    HIP::ewBinaryMat(BinaryOpCode::DIV, *outputs[0], a, b, ctx);
    DataObjectFactory::destroy(a);
    DataObjectFactory::destroy(b);
}

// Kernels that validate their arguments on the device, called batch after batch by a pipeline task: no batch waits
// for its verdict, and the task's execute() still throws what the failing kernel would have thrown.
// COLS on a pipeline shared with the CPU workers: a batch of rows becomes a batch of columns (t(x)); the device's
// columns come home with one pitched copy (MTWrapper_dense.cpp:355-368 copies them row by row)
template <class DT> void funTranspose(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *x = static_cast<DT *>(inputs[0]);
    HIP::transpose(*outputs[0], x, ctx);
    DataObjectFactory::destroy(x);
}
template <class DT> void hostTranspose(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *x = static_cast<DT *>(inputs[0]);
    const size_t n = x->getNumRows(), c = x->getNumCols();
    const auto *xv = static_cast<const DT *>(x)->getValues();
    auto *t = DataObjectFactory::create<DT>(c, n, false);
    for (size_t i = 0; i < n; i++)
        for (size_t j = 0; j < c; j++)
            t->getValues()[j * n + i] = xv[i * x->getRowSkip() + j];
    *outputs[0] = t;
    DataObjectFactory::destroy(x);
}
template <typename VT> void run_hybrid_cols(DaphneContext *dctx) {
    using DT = DenseMatrix<VT>;
    using Fn = void (*)(DT ***, Structure **, DCTX(ctx));
    const size_t rows = 777, cols = 6;
    std::vector<VT> a(rows * cols);
    for (size_t i = 0; i < a.size(); i++)
        a[i] = VT(i % 1000) * VT(0.5);
    auto *x = given<DT>(rows, a);
    std::vector<VT> want(rows * cols);
    for (size_t i = 0; i < rows; i++)
        for (size_t j = 0; j < cols; j++)
            want[j * rows + i] = a[i * cols + j];
    bool isScalar[] = {false};
    Structure *inputs[] = {x};
    int64_t outRows[] = {int64_t(cols)}, outCols[] = {int64_t(rows)};
    int64_t splits[] = {int64_t(VectorSplit::ROWS)}, combines[] = {int64_t(VectorCombine::COLS)};
    void *fun[] = {reinterpret_cast<void *>(Fn(&hostTranspose<DT>)), reinterpret_cast<void *>(Fn(&funTranspose<DT>))};
    for (double share : {0.25, 0.6, 1.0}) {
        dctx->config.hip_vect_device_share = share;
        dctx->config.hip_vect_shares = 2;
        dctx->config.hip_vect_batch_rows = 64;
        dctx->config.numberOfThreads = 3;
        dctx->config.phyBatchSize = 2048;
        DT *out[] = {nullptr};
        HIP::vectorizedPipeline<DT>(out, 1, isScalar, inputs, 1, outRows, outCols, splits, combines, 2, fun, dctx);
        CHECK(whereIs(out[0]) == (share < 1.0 ? 1 : 2));
        CHECK(toHost(out[0]) == want);
        DataObjectFactory::destroy(out[0]);
    }
    dctx->config.hip_vect_device_share = 1.0;
    dctx->config.hip_vect_shares = 1;
    dctx->config.hip_vect_batch_rows = 0;
    dctx->config.numberOfThreads = -1;
    dctx->config.phyBatchSize = 96 * 1024;
    CHECK(x->getRefCounter() == 1);
    DataObjectFactory::destroy(x);
}

static void run_deferred_verdicts(DaphneContext *dctx) {
    using DT = DenseMatrix<int64_t>;
    dh_ctx *raw = HIPContext::get(dctx, 0)->raw();
    const size_t rows = 700, cols = 4;
    std::vector<int64_t> num(rows * cols), den(rows * cols);
    for (size_t i = 0; i < num.size(); i++) {
        num[i] = int64_t(i) * 7 - 1000;
        den[i] = int64_t(i % 9) + 1;
    }
    auto a = given<DT>(rows, num), good = given<DT>(rows, den);
    den[250 * cols + 1] = 0; // batch 3 of 7 with 100 rows to a batch
    auto bad = given<DT>(rows, den);
    auto result = DataObjectFactory::create<DT>(rows, cols, false);
    DT **resPtr = &result;
    bool isScalar[] = {false, false};
    int64_t outRows[] = {int64_t(rows)}, outCols[] = {int64_t(cols)};
    const VectorSplit splits[] = {VectorSplit::ROWS, VectorSplit::ROWS};
    const VectorCombine combines[] = {VectorCombine::ROWS};
    std::mutex resLock;
    auto task = [&](DT *divisor) {
        Structure *inputs[] = {a, divisor};
        CompiledPipelineTaskData<DT> data{{&funDivSi64}, isScalar, inputs, 2, 1, outRows, outCols, splits, combines, 0, rows, outRows, outCols, 0, dctx};
        CompiledPipelineTaskHIP<DT> t(data, resLock, &resPtr);
        t.execute(0, 100);
    };
    // result is written on the device by the task: say so, as the pipeline kernel does before it starts its tasks
    {
        AllocationDescriptorHIP alloc_desc(dctx, 0);
        (void)result->getValues(&alloc_desc);
    }
    task(good);
    {
        const auto got = toHost(result);
        bool ok = got.size() == num.size();
        for (size_t i = 0; ok && i < got.size(); i++)
            ok = got[i] == num[i] / (int64_t(i % 9) + 1);
        CHECK(ok);
    }
    CHECK_THROWS_AS(task(bad), std::domain_error);
    // the verdict went with the exception: the next task on the context starts clean, and so does a direct call
    CHECK(dh_check_deferred(raw) == DH_OK);
    task(good);
    DT *direct = nullptr;
    CHECK_THROWS_AS(HIP::ewBinaryMat(BinaryOpCode::MOD, direct, a, bad, dctx), std::domain_error); // immediate outside a task
    HIP::ewBinaryMat(BinaryOpCode::MOD, direct, a, good, dctx);
    CHECK(direct != nullptr);

    // the C ABI directly: first failure in stream order wins, its status and message are those of the immediate form
    {
        AllocationDescriptorHIP alloc_desc(dctx, 0);
        const int64_t *pa = a->getValues(&alloc_desc), *pbad = bad->getValues(&alloc_desc);
        int64_t *pres = result->getValues(&alloc_desc);
        DenseMatrix<double> *neg = given<DenseMatrix<double>>(1, {4.0, -1.0, 9.0}), *root = DataObjectFactory::create<DenseMatrix<double>>(1, 3, false);
        const double *pneg = neg->getValues(&alloc_desc);
        double *proot = root->getValues(&alloc_desc);
        auto sel = given<DT>(2, {1, 17});
        const int64_t *psel = sel->getValues(&alloc_desc);
        auto picked = DataObjectFactory::create<DT>(rows, 2, false);
        int64_t *ppicked = picked->getValues(&alloc_desc);
        CHECK(dh_defer_checks(raw, 1) == DH_OK);
        CHECK(dh_defer_checks(raw, 1) == DH_OK); // nests
        CHECK(dh_ew_unary_f64(raw, DH_UN_SQRT, proot, 3, pneg, 1, 3, 3) == DH_OK);
        CHECK(dh_ew_binary_si64(raw, DH_BIN_MOD, pres, cols, pa, rows, cols, cols, pbad, rows, cols, cols) == DH_OK);
        CHECK(dh_extract_col_si64(raw, ppicked, 2, pa, rows, cols, cols, psel, 2, 1, 1) == DH_OK);
        CHECK(dh_defer_checks(raw, 0) == DH_OK);
        CHECK(dh_defer_checks(raw, 0) == DH_OK);
        CHECK(dh_defer_checks(raw, 0) != DH_OK); // left more often than entered
        CHECK(dh_check_deferred(raw) == DH_ERR_DOMAIN);
        CHECK(std::string(dh_last_error()).find("SQRT") != std::string::npos);
        CHECK(dh_check_deferred(raw) == DH_OK); // cleared
        // ExtractCol alone: the position and the bounds are in the message, the extraction itself stayed in bounds
        CHECK(dh_defer_checks(raw, 1) == DH_OK);
        CHECK(dh_extract_col_si64(raw, ppicked, 2, pa, rows, cols, cols, psel, 2, 1, 1) == DH_OK);
        CHECK(dh_defer_checks(raw, 0) == DH_OK);
        CHECK(dh_check_deferred(raw) == DH_ERR_OUT_OF_RANGE);
        CHECK(std::string(dh_last_error()).find("'17'") != std::string::npos && std::string(dh_last_error()).find("[0, 4)") != std::string::npos);
        // immediate mode again
        CHECK(dh_extract_col_si64(raw, ppicked, 2, pa, rows, cols, cols, psel, 2, 1, 1) == DH_ERR_OUT_OF_RANGE);
        for (auto *m : {sel, picked})
            DataObjectFactory::destroy(m);
        DataObjectFactory::destroy(neg);
        DataObjectFactory::destroy(root);
    }
    for (auto *m : {a, good, bad, result, direct})
        DataObjectFactory::destroy(m);
}

static void run_si64(DaphneContext *dctx) {
    using DT = DenseMatrix<int64_t>;
    auto G = [&](size_t rows, std::vector<int64_t> v) { return given<DT>(rows, v); };
    // AggRowTest.cpp / AggColTest.cpp literal, AggAllTest.cpp:62-75
    auto m = G(3, {3, 0, 2, 0, 0, 0, 1, 0, 0, 1, 0, 3});
    CHECK(HIP::aggAll<int64_t>(AggOpCode::SUM, m, dctx) == 10);
    CHECK(HIP::aggAll<int64_t>(AggOpCode::MAX, m, dctx) == 3);
    CHECK(HIP::aggAll<int64_t>(AggOpCode::MIN, m, dctx) == 0);
    DT *r = nullptr, *c = nullptr, *t = nullptr, *b = nullptr, *f = nullptr;
    HIP::aggRow(AggOpCode::SUM, r, m, dctx);
    CHECK(equals(r, {5, 1, 4}));
    HIP::aggCol(AggOpCode::MAX, c, m, dctx);
    CHECK(equals(c, {3, 1, 2, 3}));
    DenseMatrix<size_t> *idx = nullptr;
    HIP::aggRow(AggOpCode::IDXMAX, idx, m, dctx);
    CHECK(equals(idx, {0, 2, 3}));
    CHECK_THROWS_AS(HIP::aggAll<int64_t>(AggOpCode::MEAN, m, dctx), std::runtime_error);
    HIP::transpose(t, m, dctx);
    CHECK(equals(t, {3, 0, 0, 0, 0, 1, 2, 1, 0, 0, 0, 3}));
    HIP::colBind(b, m, r, dctx);
    CHECK(equals(b, {3, 0, 2, 0, 5, 0, 0, 1, 0, 1, 0, 1, 0, 3, 4}));
    HIP::fill(f, int64_t(-7), 2, 3, dctx);
    CHECK(equals(f, {-7, -7, -7, -7, -7, -7}));
    for (auto *x : {m, r, c, t, b, f})
        DataObjectFactory::destroy(x);
    DataObjectFactory::destroy(idx);
}

#include <dlfcn.h>
template <typename VT> static void run_zscore_via_wrappers(DaphneContext *dctx, void *lib) {
    using DT = DenseMatrix<VT>;
    using Z = ZscoreViaWrappers<VT>;
    CHECK(Z::load(lib));
    if (!Z::load(lib))
        return;
    {
        {
            const size_t rows = 5000, cols = 64;
            std::vector<VT> xv(rows * cols);
            uint32_t seed = 777u;
            for (auto &v : xv) {
                seed = seed * 1664525u + 1013904223u;
                v = VT(5.0 + 4.0 * ((seed >> 8) * (1.0 / 16777216.0) - 0.5));
            }
            auto x = given<DT>(rows, xv);
            DT *mu = nullptr, *var = nullptr, *sd = nullptr;
            HIP::aggCol(AggOpCode::MEAN, mu, x, dctx);
            HIP::aggCol(AggOpCode::VAR, var, x, dctx);
            HIP::ewUnaryMat(UnaryOpCode::SQRT, sd, var, dctx);
            const int kPipe = dctx->dispatchMapping.registerKernel("_vect_hip1", "script.daphne", 9, 1);
            DT *byOps[] = {nullptr, nullptr}, *asOne[] = {nullptr, nullptr};
            dctx->config.hip_vect_shares = 2;
            dctx->config.hip_vect_batch_rows = 1000;
            Z::run(byOps, x, mu, sd, 64.0, false, kPipe, dctx);
            CHECK(Z::entry().lastMode() == 0);
            Z::run(asOne, x, mu, sd, 64.0, true, kPipe, dctx);
            CHECK(Z::entry().lastMode() == 1);
            if (Z::entry().lastMode() != 1)
                std::printf("fusedPipeline ran operator by operator: %s\n", Z::entry().lastReason());
            CHECK(dh_vectorized_pipeline_last_mode() == 1);
            // r: the same IEEE operations per element, and for float also the same order of additions over a row of
            // 64 (both kernels give a row to 16 lanes of four values): bit for bit. For double the row-sum kernel takes
            // 32 lanes of two values where the fused kernel takes 16 lanes of four: equal within rounding.
            if (std::is_same<VT, float>::value)
                CHECK(toHost(asOne[0]) == toHost(byOps[0]));
            else {
                const auto got = toHost(asOne[0]), want = toHost(byOps[0]);
                bool ok = got.size() == want.size();
                for (size_t i = 0; ok && i < got.size(); i++)
                    ok = std::fabs(double(got[i]) - double(want[i])) <= 1e-14 * std::fabs(double(want[i]));
                CHECK(ok);
            }
            CHECK(toHost(asOne[1]) == toHost(byOps[1]));
            const double count = double(toHost(asOne[1])[0]);
            CHECK(count > 0 && count < double(rows));
            dctx->config.hip_vect_shares = 1;
            dctx->config.hip_vect_batch_rows = 0;
            DataObjectFactory::destroy(byOps[0], byOps[1], asOne[0], asOne[1]);
            DataObjectFactory::destroy(x, mu, var, sd);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// The generated entry points of libHIPKernels.so, called the way a compiled program calls them
// (genKernelInst.py:132-154, 236-262; ErrorHandler.cpp:80-90)
// ------------------------------------------------------------------------------------------------
#include <dlfcn.h>
static void run_generated_wrappers(DaphneContext *dctx, const char *lib_path) {
    using DT = DenseMatrix<double>;
    void *lib = dlopen(lib_path, RTLD_NOW | RTLD_LOCAL);
    if (!lib) {
        std::printf("FAILED to load %s: %s\n", lib_path, dlerror());
        g_fail++;
        return;
    }
    using EwFn = void (*)(DT **, const DT *, const DT *, int, DaphneContext *);
    using AggFn = void (*)(double *, const DT *, int, DaphneContext *);
    using UnFn = void (*)(DT **, const DT *, int, DaphneContext *);
    auto ewAdd = reinterpret_cast<EwFn>(dlsym(lib, "HIP_ewAdd__DenseMatrix_double__DenseMatrix_double__DenseMatrix_double"));
    auto sumAll = reinterpret_cast<AggFn>(dlsym(lib, "HIP_sumAll__double__DenseMatrix_double"));
    auto ewSqrt = reinterpret_cast<UnFn>(dlsym(lib, "HIP_ewSqrt__DenseMatrix_double__DenseMatrix_double"));
    CHECK(ewAdd && sumAll && ewSqrt);
    if (!(ewAdd && sumAll && ewSqrt))
        return;
    const int kAdd = dctx->dispatchMapping.registerKernel("HIP_ewAdd__DenseMatrix_double__DenseMatrix_double__DenseMatrix_double",
                                                          "script.daphne", 3, 7);
    const int kSum = dctx->dispatchMapping.registerKernel("HIP_sumAll__double__DenseMatrix_double", "script.daphne", 4, 1);
    const int kSqrt = dctx->dispatchMapping.registerKernel("HIP_ewSqrt__DenseMatrix_double__DenseMatrix_double", "script.daphne", 5, 2);
    auto a = given<DT>(2, {1, 2, 3, 4}), b = given<DT>(2, {10, 20, 30, 40}), bad = given<DT>(3, {1, 2, 3});
    dctx->config.enable_statistics = true;
    DT *res = nullptr;
    ewAdd(&res, a, b, kAdd, dctx);
    CHECK(res != nullptr && equals(res, {11, 22, 33, 44}));
    double total = 0;
    sumAll(&total, res, kSum, dctx);
    CHECK(total == 110);
    CHECK(dctx->kernel_stats[kAdd].first == 1 && dctx->kernel_stats[kSum].first == 1);
    dctx->config.enable_statistics = false;
    // a kernel's exception comes out as the run-time error of the call site: kernel name, message, position
    std::string what;
    try {
        DT *r2 = nullptr;
        ewAdd(&r2, a, bad, kAdd, dctx);
    } catch (const std::runtime_error &e) {
        what = e.what();
    }
    CHECK(what.find("The kernel-function HIP_ewAdd__DenseMatrix_double__DenseMatrix_double__DenseMatrix_double failed during runtime") == 0);
    CHECK(what.find("script.daphne:3:7") != std::string::npos);
    what.clear();
    auto neg = given<DT>(1, {4, -1});
    try {
        DT *r3 = nullptr;
        ewSqrt(&r3, neg, kSqrt, dctx);
    } catch (const std::runtime_error &e) { // the domain error of the kernel, re-thrown as the call site's error
        what = e.what();
    }
    CHECK(what.find("HIP_ewSqrt__DenseMatrix_double__DenseMatrix_double") != std::string::npos &&
          what.find("script.daphne:5:2") != std::string::npos);
    DataObjectFactory::destroy(a, b, bad, res, neg);

    // The z-score pipeline the way a compiled program runs it with patch 0012: HIP_fusedPipeline gets the outlined
    // device body - a function that calls the generated HIP_<mnemonic> entry points one after the other - and the
    // text of the same operators. With the text every batch is ONE launch of the specialised kernel; without it the
    // outlined body runs. ROWS results are equal bit for bit.
    {
        run_zscore_via_wrappers<float>(dctx, lib);
        run_zscore_via_wrappers<double>(dctx, lib);
    }
    dlclose(lib);
}


int main(int argc, char **argv) {
    // test/runtime/local/kernels/CUDA_ContextTest.cpp:25-30
    auto dctx = std::make_unique<DaphneContext>();
    try {
        HIP::createHIPContext(dctx.get());
    } catch (const std::exception &e) {
        std::printf("FAILED to create the HIP context: %s\n", e.what());
        return 2;
    }
    CHECK(dctx->useHIP());
    CHECK(HIPContext::get(dctx.get(), 0)->getMemBudget() > 0);
    run_all<float>(dctx.get());
    run_all<double>(dctx.get());
    run_training<float>(dctx.get());
    run_training<double>(dctx.get());
    run_integer_elementwise<int64_t>(dctx.get());
    run_integer_elementwise<uint64_t>(dctx.get());
    run_integer_elementwise<int32_t>(dctx.get());
    run_integer_elementwise<uint32_t>(dctx.get());
    run_si64(dctx.get());
    run_placement(dctx.get());
    run_pipeline_tasks<float>(dctx.get());
    run_pipeline_tasks<double>(dctx.get());
    run_hybrid_pipeline<float>(dctx.get());
    run_hybrid_pipeline<double>(dctx.get());
    run_hybrid_cols<float>(dctx.get());
    run_hybrid_cols<double>(dctx.get());
    run_deferred_verdicts(dctx.get());
    if (argc > 1) // path of libHIPKernels.so
        run_generated_wrappers(dctx.get(), argv[1]);
    std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
