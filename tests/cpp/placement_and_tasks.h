// Tests of the placement model and of the vectorized-pipeline tasks, written against the interface that DAPHNE's
// own data structures have. test_glue.cpp runs them on the device over the stand-in data structures;
// test_glue_reference.cpp compiles the same code against the reference's DenseMatrix / MetaDataObject / Structure
// sources over a host-memory implementation of the C ABI.
#pragma once

#include "dm_access.h"

#ifndef DAPHNE_HIP_KERNELS_INCLUDED_PIECEWISE
#include <daphne_hip_kernels.h>
#endif

#include <cmath>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

// ------------------------------------------------------------------------------------------------
// Data placement: what DenseMatrix::getValues(&alloc_desc) and AllocationDescriptorHIP do together
// (DenseMatrix.cpp:126-234, AllocationDescriptorCUDA.h:24-75)
// ------------------------------------------------------------------------------------------------
// Views and device placements (DenseMatrix.cpp:98-115 with the device-view patch): a view addresses its parent's device
// buffer at its own offset, for reading and for writing, also as a view of a view and as a column range.
static void run_views(DaphneContext *dctx) {
    using DT = DenseMatrix<float>;
    HIPContext *hc = HIPContext::get(dctx, 0);
    const size_t allocs0 = hc->numAllocations();
    AllocationDescriptorHIP alloc_desc(dctx, 0);
    auto p = given<DT>(4, {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20});
    // (1) parent current on host and device; row, column and nested views read their own elements on the device
    CHECK(static_cast<const DT *>(p)->getValues(&alloc_desc) != nullptr && whereIs(p) == 3);
    DT *rows = p->sliceRow(1, 4), *cols = p->sliceCol(1, 4), *inner = rows->slice(1, 3, 2, 5);
    CHECK(whereIs(rows) == 3 && numDataPlacements(rows) == 2 && hc->numAllocations() == allocs0 + 1);
    DT *r1 = nullptr, *r2 = nullptr, *r3 = nullptr;
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, r1, rows, 2.0f, dctx);
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, r2, cols, 2.0f, dctx);
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, r3, inner, 2.0f, dctx);
    CHECK(equals(r1, {12, 14, 16, 18, 20, 22, 24, 26, 28, 30, 32, 34, 36, 38, 40}));
    CHECK(equals(r2, {4, 6, 8, 14, 16, 18, 24, 26, 28, 34, 36, 38}));
    CHECK(equals(r3, {26, 28, 30, 36, 38, 40}));
    CHECK(hc->numAllocations() == allocs0 + 4); // three results, no copy of any view
    // the host side of the same views: the parent's host buffer at the view's offset
    CHECK(equals(inner, {13, 14, 15, 18, 19, 20}));
    DataObjectFactory::destroy(r1, r2, r3);

    // (2) a result that exists on the device only, written through views of its rows and of its columns
    DT *res = DataObjectFactory::create<DT>(4, 5, false, &alloc_desc);
    DT *whole = res;
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, whole, p, 0.0f, dctx); // zeros
    DT *top = res->sliceRow(0, 2), *bottom = res->sliceRow(2, 4), *pt = p->sliceRow(0, 2), *pb = p->sliceRow(2, 4);
    CHECK(whereIs(top) == 2 && numDataPlacements(top) == 1);
    HIP::ewBinaryObjSca(BinaryOpCode::ADD, bottom, pb, 100.0f, dctx); // bottom first: a base pointer would hit row 0
    HIP::ewBinaryObjSca(BinaryOpCode::ADD, top, pt, 0.5f, dctx);
    CHECK(equals(res, {1.5f, 2.5f, 3.5f, 4.5f, 5.5f, 6.5f, 7.5f, 8.5f, 9.5f, 10.5f, 111, 112, 113, 114, 115, 116, 117, 118, 119, 120}));
    // a view of a device-only matrix read on the host: downloaded from its offset into a buffer of its own
    DT *res2 = DataObjectFactory::create<DT>(4, 5, false, &alloc_desc);
    DT *whole2 = res2;
    HIP::ewBinaryObjSca(BinaryOpCode::ADD, whole2, p, 0.0f, dctx);
    DT *tail = res2->slice(2, 4, 3, 5);
    CHECK(whereIs(tail) == 2);
    CHECK(equals(tail, {14, 15, 19, 20}));
    CHECK(whereIs(tail) == 3 && whereIs(res2) == 2);
    DT *midv = res2->sliceCol(1, 3);
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, midv, midv, -1.0f, dctx); // in place through a column view
    CHECK(equals(res2, {1, -2, -3, 4, 5, 6, -7, -8, 9, 10, 11, -12, -13, 14, 15, 16, -17, -18, 19, 20}));
    DataObjectFactory::destroy(top, bottom, pt, pb, tail, midv);
    DataObjectFactory::destroy(res, res2);

    // (3) a view of a matrix that exists on the host only gets a device buffer of its own (the view's rows, strided
    // like the parent); the parent learns nothing of it
    auto q = given<DT>(3, {1, 2, 3, 4, 5, 6, 7, 8, 9});
    DT *qv = q->slice(1, 3, 1, 3);
    DT *rq = nullptr;
    const size_t before = hc->numAllocations();
    HIP::ewBinaryObjSca(BinaryOpCode::ADD, rq, qv, 10.0f, dctx);
    CHECK(equals(rq, {15, 16, 18, 19}));
    CHECK(numDataPlacements(q) == 1 && numDataPlacements(qv) == 2 && hc->numAllocations() == before + 2);
    // (4) an inherited device placement that has gone stale is refreshed at the view's offset
    CHECK(static_cast<const DT *>(q)->getValues(&alloc_desc) != nullptr);
    DT *qr = q->sliceRow(2, 3);
    qr->set(0, 1, 80.f); // host write through the view: its device placement is stale now
    CHECK(whereIs(qr) == 1);
    DT *rr = nullptr;
    HIP::ewBinaryObjSca(BinaryOpCode::ADD, rr, qr, 1.0f, dctx);
    CHECK(equals(rr, {8, 81, 10}));
    CHECK(equals(q, {1, 2, 3, 4, 5, 6, 7, 80, 9})); // the view's host buffer is the parent's
    DataObjectFactory::destroy(qv, rq, qr, rr, q);
    DataObjectFactory::destroy(rows, cols, inner, p);
    CHECK(hc->numAllocations() == allocs0);
}

static void run_placement(DaphneContext *dctx) {
    using DT = DenseMatrix<float>;
    HIPContext *hc = HIPContext::get(dctx, 0);
    const size_t allocs0 = hc->numAllocations();
    const size_t used0 = hc->getMemInUse();
    auto a = given<DT>(2, {1, 2, 3, 4, 5, 6});
    CHECK(whereIs(a) == 1 && numDataPlacements(a) == 1); // host only, nothing uploaded yet
    CHECK(hc->numAllocations() == allocs0);
    DT *r = nullptr;
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, r, a, 2.0f, dctx);
    // the input was uploaded on first use and both copies stay valid; the result exists on the device only
    CHECK(whereIs(a) == 3 && numDataPlacements(a) == 2);
    CHECK(whereIs(r) == 2 && numDataPlacements(r) == 1);
    CHECK(hc->numAllocations() == allocs0 + 2);
    // a second use finds the device copy: no further placement, no further allocation
    DT *r2 = nullptr;
    HIP::ewBinaryMat(BinaryOpCode::ADD, r2, a, r, dctx);
    CHECK(numDataPlacements(a) == 2 && hc->numAllocations() == allocs0 + 3);
    // reading the result on the host downloads it once; both copies are then current
    CHECK(equals(r2, {3, 6, 9, 12, 15, 18}));
    CHECK(whereIs(r2) == 3);
    // writing on the host makes the device copy stale; the next kernel uploads again and sees the new value
    a->set(0, 0, 10.f);
    CHECK(whereIs(a) == 1);
    HIP::ewBinaryObjSca(BinaryOpCode::MUL, r, a, 2.0f, dctx); // in place into r
    CHECK(whereIs(a) == 3 && whereIs(r) == 2);
    CHECK(equals(r, {20, 4, 6, 8, 10, 12}));
    // a kernel that writes into a matrix makes its host copy stale
    HIP::ewBinaryObjSca(BinaryOpCode::ADD, a, a, 1.0f, dctx);
    CHECK(whereIs(a) == 2);
    CHECK(equals(a, {11, 3, 4, 5, 6, 7}));
    // a view inherits its parent's placements: a kernel on a view of a device-current matrix reads the view's own
    // rows from the parent's device buffer, without another upload or allocation
    DT *v = a->sliceRow(1, 2);
    DT *rv = nullptr;
    HIP::ewBinaryObjSca(BinaryOpCode::SUB, rv, v, 1.0f, dctx);
    CHECK(equals(rv, {4, 5, 6}));
    CHECK(numDataPlacements(a) == 2 && hc->numAllocations() == allocs0 + 4);
    DataObjectFactory::destroy(v);
    run_views(dctx);
    // destroying the matrices gives the device memory back
    DataObjectFactory::destroy(a, r, r2, rv);
    CHECK(hc->numAllocations() == allocs0);
    CHECK(hc->getMemInUse() == used0);
}

// ------------------------------------------------------------------------------------------------
// Vectorized pipeline on the device: tasks over row shares, outputs combined
// (MultiThreadedKernelTest.cpp:30-154 bodies; TasksCUDA.cpp:21-119; MTWrapper_dense.cpp:339-373)
// ------------------------------------------------------------------------------------------------
// bodies as the compiler outlines them: operator by operator, results through *outputs[i], inputs given back
template <class DT> void funAdd(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *l = static_cast<DT *>(inputs[0]), *r = static_cast<DT *>(inputs[1]);
    HIP::ewBinaryMat(BinaryOpCode::ADD, *outputs[0], l, r, ctx);
    DataObjectFactory::destroy(l, r);
}
template <class DT> void funMul(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *l = static_cast<DT *>(inputs[0]), *r = static_cast<DT *>(inputs[1]);
    HIP::ewBinaryMat(BinaryOpCode::MUL, *outputs[0], l, r, ctx);
    DataObjectFactory::destroy(l, r);
}
// a body that ignores the offered output and returns a matrix of its own, like the reference's compiled bodies
template <class DT> void funAddFresh(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *l = static_cast<DT *>(inputs[0]), *r = static_cast<DT *>(inputs[1]);
    DT *fresh = nullptr;
    HIP::ewBinaryMat(BinaryOpCode::ADD, fresh, l, r, ctx);
    *outputs[0] = fresh;
    DataObjectFactory::destroy(l, r);
}
// outputs: 0 = (x - mu) * (x - mu) by ROWS, 1 = column sums by ADD, 2 = column minima by MIN, 3 = column maxima by MAX
template <class DT> void funStats(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *x = static_cast<DT *>(inputs[0]), *mu = static_cast<DT *>(inputs[1]);
    DT *c = nullptr;
    HIP::ewBinaryMat(BinaryOpCode::SUB, c, x, mu, ctx);
    HIP::ewBinaryMat(BinaryOpCode::MUL, *outputs[0], c, c, ctx);
    HIP::aggCol(AggOpCode::SUM, *outputs[1], x, ctx);
    HIP::aggCol(AggOpCode::MIN, *outputs[2], x, ctx);
    HIP::aggCol(AggOpCode::MAX, *outputs[3], x, ctx);
    DataObjectFactory::destroy(c, x, mu);
}

// the z-score body as the compiler outlines it for the device: one kernel per operator; inputs x, mu, sd and the
// threshold as a scalar in the place of a pointer (the bits of a double); outputs r by ROWS, count by ADD
template <class DT> void funZscoreOpByOp(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    using VT = typename DT::VT;
    auto *x = static_cast<DT *>(inputs[0]), *mu = static_cast<DT *>(inputs[1]), *sd = static_cast<DT *>(inputs[2]);
    const VT thr = HIP::FusedPipelineBody<VT>::scalarOf(inputs[3]);
    DT *c = nullptr, *z = nullptr, *zz = nullptr, *gt = nullptr;
    HIP::ewBinaryMat(BinaryOpCode::SUB, c, x, mu, ctx);
    HIP::ewBinaryMat(BinaryOpCode::DIV, z, c, sd, ctx);
    HIP::ewBinaryMat(BinaryOpCode::MUL, zz, z, z, ctx);
    HIP::aggRow(AggOpCode::SUM, *outputs[0], zz, ctx);
    HIP::ewBinaryObjSca(BinaryOpCode::GT, gt, *outputs[0], thr, ctx);
    const VT count = HIP::aggAll<VT, DT>(AggOpCode::SUM, gt, ctx);
    HIP::fill(*outputs[1], count, 1, 1, ctx);
    DataObjectFactory::destroy(c, z, zz, gt);
    DataObjectFactory::destroy(x, mu, sd);
}
static const char *const kZscoreBody = "%0 = ewSub in0, in1\n%1 = ewDiv %0, in2\n%2 = ewMul %1, %1\n%3 = sumRow %2\n"
                                       "%4 = ewGt %3, in3\n%5 = sumAll %4\n%6 = cast %5\nreturn %3, %6\n";
// a body that keeps two tiles alive (x - mu is used again after it was squared): it cannot run as one kernel
template <class DT> void funTwoTilesOpByOp(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    auto *x = static_cast<DT *>(inputs[0]), *mu = static_cast<DT *>(inputs[1]);
    DT *c = nullptr, *sq = nullptr;
    HIP::ewBinaryMat(BinaryOpCode::SUB, c, x, mu, ctx);
    HIP::ewBinaryMat(BinaryOpCode::MUL, sq, c, c, ctx);
    HIP::ewBinaryMat(BinaryOpCode::ADD, *outputs[0], sq, c, ctx);
    DataObjectFactory::destroy(c, sq, x, mu);
}
static const char *const kTwoTilesBody = "%0 = ewSub in0, in1\n%1 = ewMul %0, %0\n%2 = ewAdd %1, %0\nreturn %2\n";

template <typename VT> void run_pipeline_tasks(DaphneContext *dctx) {
    using DT = DenseMatrix<VT>;
    using Fn = void (*)(DT ***, Structure **, DCTX(ctx));
    const size_t rows = 1234, cols = 10;
    std::vector<VT> a(rows * cols), b(rows * cols);
    uint32_t s = 12345u;
    auto rnd = [&] { // values in [0, 1), as randMatrix(..., 0.0, 1.0, ...) in the reference's test
        s = s * 1664525u + 1013904223u;
        return VT((s >> 8) * (1.0 / 16777216.0));
    };
    for (auto &v : a)
        v = rnd();
    for (auto &v : b)
        v = rnd();
    auto m1 = given<DT>(rows, a), m2 = given<DT>(rows, b);
    bool isScalar[] = {false, false};
    Structure *inputs[] = {m1, m2};
    int64_t outRows[] = {int64_t(rows)}, outCols[] = {int64_t(cols)};
    int64_t splits[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::ROWS)};
    int64_t combines[] = {int64_t(VectorCombine::ROWS)};
    struct Case {
        uint64_t shares, batch;
    };
    const Case cases[] = {{1, 0}, {2, 0}, {7, 0}, {3, 100}, {1, 1000}};
    for (Fn fn : {Fn(&funAdd<DT>), Fn(&funMul<DT>), Fn(&funAddFresh<DT>)}) {
        DT *whole = nullptr; // single call on the whole matrices
        HIP::ewBinaryMat(fn == Fn(&funMul<DT>) ? BinaryOpCode::MUL : BinaryOpCode::ADD, whole, m1, m2, dctx);
        const auto expect = toHost(whole);
        bool host_ok = true;
        for (size_t i = 0; i < expect.size(); i++)
            host_ok &= expect[i] == (fn == Fn(&funMul<DT>) ? a[i] * b[i] : a[i] + b[i]);
        CHECK(host_ok);
        for (const Case &c : cases) {
            dctx->config.hip_vect_shares = c.shares;
            dctx->config.hip_vect_batch_rows = c.batch;
            DT *out[] = {nullptr};
            void *fun[] = {reinterpret_cast<void *>(fn)};
            HIP::vectorizedPipeline<DT>(out, 1, isScalar, inputs, 2, outRows, outCols, splits, combines, 1, fun, dctx);
            CHECK(out[0] != nullptr && out[0]->getNumRows() == rows && out[0]->getNumCols() == cols);
            CHECK(whereIs(out[0]) == 2); // combined on the device, not through the host
            CHECK(toHost(out[0]) == expect); // ROWS: bit for bit the whole-matrix result
            DataObjectFactory::destroy(out[0]);
        }
        DataObjectFactory::destroy(whole);
    }
    CHECK(m1->getRefCounter() == 1 && m2->getRefCounter() == 1);

    // ROWS + ADD + MIN + MAX in one pipeline, a broadcast input, op-by-op body
    {
        DT *mu = nullptr;
        HIP::aggCol(AggOpCode::MEAN, mu, m1, dctx);
        DT *c = nullptr, *sq = nullptr, *sum = nullptr, *mn = nullptr, *mx = nullptr;
        HIP::ewBinaryMat(BinaryOpCode::SUB, c, m1, mu, dctx);
        HIP::ewBinaryMat(BinaryOpCode::MUL, sq, c, c, dctx);
        HIP::aggCol(AggOpCode::SUM, sum, m1, dctx);
        HIP::aggCol(AggOpCode::MIN, mn, m1, dctx);
        HIP::aggCol(AggOpCode::MAX, mx, m1, dctx);
        bool isScalar2[] = {false, false};
        Structure *inputs2[] = {m1, mu};
        int64_t outRows2[] = {int64_t(rows), 1, 1, 1}, outCols2[] = {int64_t(cols), int64_t(cols), int64_t(cols), int64_t(cols)};
        int64_t splits2[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE)};
        int64_t combines2[] = {int64_t(VectorCombine::ROWS), int64_t(VectorCombine::ADD), int64_t(VectorCombine::MIN),
                               int64_t(VectorCombine::MAX)};
        const double tol = std::is_same<VT, float>::value ? 1e-4 : 1e-12; // sums of 1234 values in [0,1) in another order
        for (const Case &cs : cases) {
            dctx->config.hip_vect_shares = cs.shares;
            dctx->config.hip_vect_batch_rows = cs.batch;
            DT *out[] = {nullptr, nullptr, nullptr, nullptr};
            void *fun[] = {reinterpret_cast<void *>(Fn(&funStats<DT>))};
            HIP::vectorizedPipeline<DT>(out, 4, isScalar2, inputs2, 2, outRows2, outCols2, splits2, combines2, 1, fun, dctx);
            CHECK(toHost(out[0]) == toHost(sq));
            const auto got = toHost(out[1]), want = toHost(sum);
            bool ok = got.size() == want.size();
            for (size_t i = 0; ok && i < got.size(); i++)
                ok = std::fabs(double(got[i]) - double(want[i])) <= tol * std::fabs(double(want[i]));
            CHECK(ok);
            CHECK(toHost(out[2]) == toHost(mn)); // MIN / MAX do not depend on the order
            CHECK(toHost(out[3]) == toHost(mx));
            DataObjectFactory::destroy(out[0], out[1], out[2], out[3]);
        }
        CHECK(mu->getRefCounter() == 1);
        DataObjectFactory::destroy(mu, c, sq, sum, mn, mx);
    }

    // the same shape of work as ONE kernel per batch: z = (x - mu) / sd by ROWS, r = rowSums(z * z) by ROWS,
    // count of r > thr by ADD, largest r by MAX
    {
        DT *mu = nullptr, *var = nullptr, *sd = nullptr;
        HIP::aggCol(AggOpCode::MEAN, mu, m1, dctx);
        HIP::aggCol(AggOpCode::VAR, var, m1, dctx);
        HIP::ewUnaryMat(UnaryOpCode::SQRT, sd, var, dctx);
        const VT thr = VT(10);
        auto I = [](int kind, int op, int domain, int operand, int index, double scalar = 0) {
            return dh_pipe_instr{kind, op, domain, operand, index, 0, scalar};
        };
        HIP::FusedPipelineBody<VT> body;
        body.program = {I(DH_PIPE_EW_BINARY, int(BinaryOpCode::SUB), 0, DH_OPD_ROWVEC, 0),
                        I(DH_PIPE_EW_BINARY, int(BinaryOpCode::DIV), 0, DH_OPD_ROWVEC, 1),
                        I(DH_PIPE_STORE_TILE, 0, 0, 0, 0),
                        I(DH_PIPE_EW_BINARY, int(BinaryOpCode::MUL), 0, DH_OPD_SELF, 0),
                        I(DH_PIPE_ROW_AGG, int(AggOpCode::SUM), 0, 0, 0),
                        I(DH_PIPE_STORE_ROW, 0, 1, 0, 0),
                        I(DH_PIPE_REDUCE_ALL, int(AggOpCode::MAX), 1, 0, 1),
                        I(DH_PIPE_EW_BINARY, int(BinaryOpCode::GT), 1, DH_OPD_SCALAR, 0, double(thr)),
                        I(DH_PIPE_REDUCE_ALL, int(AggOpCode::SUM), 1, 0, 0)};
        body.inputs = {{HIP::PipeInput::PRIMARY, 0}, {HIP::PipeInput::ROWVEC, 0}, {HIP::PipeInput::ROWVEC, 1}};
        body.outputs = {{HIP::PipeOutput::TILE, 0}, {HIP::PipeOutput::ROW, 0}, {HIP::PipeOutput::ALL, 0}, {HIP::PipeOutput::ALL, 1}};
        // op by op on the whole matrix
        DT *c = nullptr, *z = nullptr, *zz = nullptr, *r = nullptr, *gt = nullptr;
        HIP::ewBinaryMat(BinaryOpCode::SUB, c, m1, mu, dctx);
        HIP::ewBinaryMat(BinaryOpCode::DIV, z, c, sd, dctx);
        HIP::ewBinaryMat(BinaryOpCode::MUL, zz, z, z, dctx);
        HIP::aggRow(AggOpCode::SUM, r, zz, dctx);
        HIP::ewBinaryObjSca(BinaryOpCode::GT, gt, r, thr, dctx);
        const VT count = HIP::aggAll<VT, DT>(AggOpCode::SUM, gt, dctx), rmax = HIP::aggAll<VT, DT>(AggOpCode::MAX, r, dctx);
        CHECK(count > VT(0) && count < VT(rows)); // the threshold splits the rows
        bool isScalar3[] = {false, false, false};
        Structure *inputs3[] = {m1, mu, sd};
        int64_t outRows3[] = {int64_t(rows), int64_t(rows), 1, 1}, outCols3[] = {int64_t(cols), 1, 1, 1};
        int64_t splits3[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE)};
        VectorCombine combines3[] = {VectorCombine::ROWS, VectorCombine::ROWS, VectorCombine::ADD, VectorCombine::MAX};
        const double tol = std::is_same<VT, float>::value ? 1e-5 : 1e-13;
        for (const Case &cs : cases) {
            dctx->config.hip_vect_shares = cs.shares;
            dctx->config.hip_vect_batch_rows = cs.batch;
            DT *out[] = {nullptr, nullptr, nullptr, nullptr};
            std::vector<std::function<void(DT ***, Structure **, DCTX(ctx))>> funcs{body};
            HIP::VectorizedPipeline<DT>::apply(out, 4, isScalar3, inputs3, 3, outRows3, outCols3,
                                               reinterpret_cast<const VectorSplit *>(splits3), combines3, funcs, dctx);
            CHECK(toHost(out[0]) == toHost(z)); // same IEEE operations per element: bit for bit
            const auto got = toHost(out[1]), want = toHost(r);
            bool ok = got.size() == want.size();
            for (size_t i = 0; ok && i < got.size(); i++)
                ok = std::fabs(double(got[i]) - double(want[i])) <= tol * std::fabs(double(want[i]));
            CHECK(ok);
            // rows whose r is within rounding of the threshold may fall on either side
            size_t ambiguous = 0;
            for (VT v : want)
                ambiguous += std::fabs(double(v) - double(thr)) <= tol * double(thr);
            CHECK(std::fabs(double(toHost(out[2])[0]) - double(count)) <= double(ambiguous));
            CHECK(std::fabs(double(toHost(out[3])[0]) - double(rmax)) <= tol * double(rmax));
            DataObjectFactory::destroy(out[0], out[1], out[2], out[3]);
        }
        DataObjectFactory::destroy(mu, var, sd, c, z);
        DataObjectFactory::destroy(zz, r, gt);
    }
    // HIP::fusedPipeline: the same pipeline given as the outlined device body AND as the text of its operators. The
    // text is lowered to the fused kernel's instruction list on the first call: every batch is ONE launch, and what it
    // stores by ROWS equals, bit for bit, what the body stores when it runs operator by operator.
    {
        using Fn4 = void (*)(DT ***, Structure **, DCTX(ctx));
        DT *mu = nullptr, *var = nullptr, *sd = nullptr;
        HIP::aggCol(AggOpCode::MEAN, mu, m1, dctx);
        HIP::aggCol(AggOpCode::VAR, var, m1, dctx);
        HIP::ewUnaryMat(UnaryOpCode::SQRT, sd, var, dctx);
        const double thr = 10.0;
        Structure *thrDisguised;
        std::memcpy(&thrDisguised, &thr, sizeof(thr));
        bool isScalar4[] = {false, false, false, true};
        Structure *inputs4[] = {m1, mu, sd, thrDisguised};
        int64_t outRows4[] = {int64_t(rows), 1}, outCols4[] = {1, 1};
        int64_t splits4[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE)};
        int64_t combines4[] = {int64_t(VectorCombine::ROWS), int64_t(VectorCombine::ADD)};
        void *fun[] = {nullptr, reinterpret_cast<void *>(Fn4(&funZscoreOpByOp<DT>))}; // {host body, device body}
        // operator by operator, whole matrix at once: the reference result
        dctx->config.hip_vect_shares = 1;
        dctx->config.hip_vect_batch_rows = 0;
        DT *ref[] = {nullptr, nullptr};
        HIP::fusedPipeline<DT>(ref, 2, isScalar4, inputs4, 4, outRows4, outCols4, splits4, combines4, 2, fun, nullptr, dctx);
        CHECK(HIP::fusedPipelineLastMode() == 0);
        const auto r_ref = toHost(ref[0]);
        const VT count_ref = toHost(ref[1])[0];
        CHECK(count_ref > VT(0) && count_ref < VT(rows));
        for (const Case &cs : cases) {
            dctx->config.hip_vect_shares = cs.shares;
            dctx->config.hip_vect_batch_rows = cs.batch;
            DT *out[] = {nullptr, nullptr};
            HIP::fusedPipeline<DT>(out, 2, isScalar4, inputs4, 4, outRows4, outCols4, splits4, combines4, 2, fun, kZscoreBody, dctx);
            CHECK(HIP::fusedPipelineLastMode() == 1);
#ifdef TEST_ON_DEVICE
            CHECK(dh_vectorized_pipeline_last_mode() == 1); // the specialised kernel: one launch per batch
#endif
            CHECK(whereIs(out[0]) == 2);
            // ten columns: the fused kernel and the row-sum kernel add a row's values in different orders (at the
            // 64-column shape of the configuration they add them alike: test_glue.cpp checks that one bit for bit)
            const auto got = toHost(out[0]);
            const double tol4 = std::is_same<VT, float>::value ? 1e-5 : 1e-13;
            bool ok = got.size() == r_ref.size();
            size_t ambiguous = 0;
            for (size_t i = 0; ok && i < got.size(); i++) {
                ok = std::fabs(double(got[i]) - double(r_ref[i])) <= tol4 * std::fabs(double(r_ref[i]));
                ambiguous += std::fabs(double(r_ref[i]) - thr) <= tol4 * thr;
            }
            CHECK(ok);
            CHECK(std::fabs(double(toHost(out[1])[0]) - double(count_ref)) <= double(ambiguous));
            DataObjectFactory::destroy(out[0], out[1]);
        }
        // a body that does not fit runs operator by operator, with the reason on record
        {
            bool isScalar2[] = {false, false};
            Structure *inputs2[] = {m1, mu};
            int64_t outRows2[] = {int64_t(rows)}, outCols2[] = {int64_t(cols)};
            int64_t splits2[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE)};
            int64_t combines2[] = {int64_t(VectorCombine::ROWS)};
            void *fun2[] = {nullptr, reinterpret_cast<void *>(Fn4(&funTwoTilesOpByOp<DT>))};
            dctx->config.hip_vect_shares = 3;
            dctx->config.hip_vect_batch_rows = 100;
            DT *out[] = {nullptr};
            HIP::fusedPipeline<DT>(out, 1, isScalar2, inputs2, 2, outRows2, outCols2, splits2, combines2, 2, fun2, kTwoTilesBody, dctx);
            CHECK(HIP::fusedPipelineLastMode() == 0);
            CHECK(HIP::fusedPipelineLastReason().find("no longer held") != std::string::npos);
            DT *c = nullptr, *sq = nullptr, *want = nullptr;
            HIP::ewBinaryMat(BinaryOpCode::SUB, c, m1, mu, dctx);
            HIP::ewBinaryMat(BinaryOpCode::MUL, sq, c, c, dctx);
            HIP::ewBinaryMat(BinaryOpCode::ADD, want, sq, c, dctx);
            CHECK(toHost(out[0]) == toHost(want));
            DataObjectFactory::destroy(out[0], c, sq, want);
        }
        CHECK(mu->getRefCounter() == 1 && sd->getRefCounter() == 1);
        DataObjectFactory::destroy(ref[0], ref[1], mu, var, sd);
    }
    dctx->config.hip_vect_shares = 1;
    dctx->config.hip_vect_batch_rows = 0;
    CHECK(m1->getRefCounter() == 1);
    DataObjectFactory::destroy(m1, m2);
}


// ------------------------------------------------------------------------------------------------
// One pipeline shared between the device and CPU workers
// (MTWrapper_dense.cpp:203-336 executeQueuePerDeviceType, 339-373 combineOutputs; WorkerGPU.h:22-52)
// ------------------------------------------------------------------------------------------------
// the host body of funStats: the same four results by loops in host memory, as fresh matrices
template <class DT> void hostStats(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    using VT = typename DT::VT;
    auto *x = static_cast<DT *>(inputs[0]), *mu = static_cast<DT *>(inputs[1]);
    const size_t n = x->getNumRows(), c = x->getNumCols();
    const VT *xv = static_cast<const DT *>(x)->getValues(), *mv = static_cast<const DT *>(mu)->getValues();
    auto *sq = DataObjectFactory::create<DT>(n, c, false), *sum = DataObjectFactory::create<DT>(1, c, false);
    auto *mn = DataObjectFactory::create<DT>(1, c, false), *mx = DataObjectFactory::create<DT>(1, c, false);
    for (size_t j = 0; j < c; j++) {
        sum->getValues()[j] = VT(0);
        mn->getValues()[j] = std::numeric_limits<VT>::infinity();
        mx->getValues()[j] = -std::numeric_limits<VT>::infinity();
    }
    for (size_t i = 0; i < n; i++)
        for (size_t j = 0; j < c; j++) {
            const VT v = xv[i * x->getRowSkip() + j], d = v - mv[j];
            sq->getValues()[i * c + j] = d * d;
            sum->getValues()[j] += v;
            mn->getValues()[j] = std::min(mn->getValues()[j], v);
            mx->getValues()[j] = std::max(mx->getValues()[j], v);
        }
    *outputs[0] = sq;
    *outputs[1] = sum;
    *outputs[2] = mn;
    *outputs[3] = mx;
    DataObjectFactory::destroy(x, mu);
}
// the host body of the z-score pipeline (funZscoreOpByOp): r by ROWS, the count of r > thr by ADD
template <class DT> void hostZscore(DT ***outputs, Structure **inputs, DCTX(ctx)) {
    using VT = typename DT::VT;
    auto *x = static_cast<DT *>(inputs[0]), *mu = static_cast<DT *>(inputs[1]), *sd = static_cast<DT *>(inputs[2]);
    const VT thr = HIP::FusedPipelineBody<VT>::scalarOf(inputs[3]);
    const size_t n = x->getNumRows(), c = x->getNumCols();
    const VT *xv = static_cast<const DT *>(x)->getValues(), *mv = static_cast<const DT *>(mu)->getValues(),
             *sv = static_cast<const DT *>(sd)->getValues();
    auto *r = DataObjectFactory::create<DT>(n, 1, false), *count = DataObjectFactory::create<DT>(1, 1, true);
    for (size_t i = 0; i < n; i++) {
        VT acc = VT(0);
        for (size_t j = 0; j < c; j++) {
            const VT z = (xv[i * x->getRowSkip() + j] - mv[j]) / sv[j];
            acc += z * z;
        }
        r->getValues()[i] = acc;
        count->getValues()[0] += acc > thr ? VT(1) : VT(0);
    }
    *outputs[0] = r;
    *outputs[1] = count;
    DataObjectFactory::destroy(x, mu, sd);
}
// a device body that fails after it has given its inputs back
template <class DT> void funFails(DT ***, Structure **inputs, DCTX(ctx)) {
    DataObjectFactory::destroy(static_cast<DT *>(inputs[0]), static_cast<DT *>(inputs[1]));
    throw std::domain_error("the device body failed");
}

template <typename VT> void run_hybrid_pipeline(DaphneContext *dctx) {
    using DT = DenseMatrix<VT>;
    using Fn = void (*)(DT ***, Structure **, DCTX(ctx));
    HIPContext *hc = HIPContext::get(dctx, 0);
    const size_t rows = 1234, cols = 10;
    std::vector<VT> a(rows * cols);
    uint32_t s = 777u;
    for (auto &v : a) {
        s = s * 1664525u + 1013904223u;
        v = VT((s >> 8) * (1.0 / 16777216.0));
    }
    auto m1 = given<DT>(rows, a);
    // the whole matrix on the device, operator by operator: what every division of the rows has to give
    DT *mu = nullptr, *c = nullptr, *sq = nullptr, *sum = nullptr, *mn = nullptr, *mx = nullptr;
    HIP::aggCol(AggOpCode::MEAN, mu, m1, dctx); // lives on the device only: the CPU workers need it brought home
    HIP::ewBinaryMat(BinaryOpCode::SUB, c, m1, mu, dctx);
    HIP::ewBinaryMat(BinaryOpCode::MUL, sq, c, c, dctx);
    HIP::aggCol(AggOpCode::SUM, sum, m1, dctx);
    HIP::aggCol(AggOpCode::MIN, mn, m1, dctx);
    HIP::aggCol(AggOpCode::MAX, mx, m1, dctx);
    const auto sq_want = toHost(sq), sum_want = toHost(sum), mn_want = toHost(mn), mx_want = toHost(mx);
    const size_t allocs0 = hc->numAllocations();

    bool isScalar[] = {false, false};
    Structure *inputs[] = {m1, mu};
    int64_t outRows[] = {int64_t(rows), 1, 1, 1}, outCols[] = {int64_t(cols), int64_t(cols), int64_t(cols), int64_t(cols)};
    int64_t splits[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE)};
    int64_t combines[] = {int64_t(VectorCombine::ROWS), int64_t(VectorCombine::ADD), int64_t(VectorCombine::MIN),
                          int64_t(VectorCombine::MAX)};
    void *fun[] = {reinterpret_cast<void *>(Fn(&hostStats<DT>)), reinterpret_cast<void *>(Fn(&funStats<DT>))}; // {host, device}
    const double tol = std::is_same<VT, float>::value ? 1e-4 : 1e-12; // sums of 1234 values in [0,1) in another order
    struct Case {
        double share;
        uint64_t shares, batch;
        int threads;
        size_t phyBatch;
    };
    // a quarter as the reference fixes it; one row; all but one row; nothing at all for the device
    const Case cases[] = {{0.25, 1, 0, 3, 96 * 1024}, {0.25, 3, 100, 1, 4096}, {0.5, 2, 0, 8, 1024},
                          {0.0005, 1, 0, 2, 96 * 1024}, {0.9995, 7, 50, 4, 96 * 1024}, {0.0, 1, 0, 2, 2048}};
    for (const Case &cs : cases) {
        dctx->config.hip_vect_device_share = cs.share;
        dctx->config.hip_vect_shares = cs.shares;
        dctx->config.hip_vect_batch_rows = cs.batch;
        dctx->config.numberOfThreads = cs.threads;
        dctx->config.phyBatchSize = cs.phyBatch;
        DT *out[] = {nullptr, nullptr, nullptr, nullptr};
        HIP::vectorizedPipeline<DT>(out, 4, isScalar, inputs, 2, outRows, outCols, splits, combines, 2, fun, dctx);
        CHECK(out[0] != nullptr && out[0]->getNumRows() == rows && out[0]->getNumCols() == cols);
        CHECK(whereIs(out[0]) == 1); // combined in host memory
        CHECK(toHost(out[0]) == sq_want); // ROWS: the same IEEE operations per element on either side
        const auto got = toHost(out[1]);
        bool ok = got.size() == sum_want.size();
        for (size_t i = 0; ok && i < got.size(); i++)
            ok = std::fabs(double(got[i]) - double(sum_want[i])) <= tol * std::fabs(double(sum_want[i]));
        CHECK(ok);
        CHECK(toHost(out[2]) == mn_want);
        CHECK(toHost(out[3]) == mx_want);
        DataObjectFactory::destroy(out[0], out[1], out[2], out[3]);
        CHECK(m1->getRefCounter() == 1 && mu->getRefCounter() == 1);
    }
    // a result that the caller brings along, wider than what the pipeline fills: the other columns stay
    {
        dctx->config.hip_vect_device_share = 0.3;
        dctx->config.hip_vect_shares = 2;
        dctx->config.hip_vect_batch_rows = 0;
        dctx->config.numberOfThreads = 3;
        auto *wide = DataObjectFactory::create<DT>(rows, cols + 3, false);
        std::fill(wide->getValues(), wide->getValues() + rows * (cols + 3), VT(-7));
        DT *out[] = {wide->sliceCol(0, cols), nullptr, nullptr, nullptr};
        HIP::vectorizedPipeline<DT>(out, 4, isScalar, inputs, 2, outRows, outCols, splits, combines, 2, fun, dctx);
        const VT *w = static_cast<const DT *>(wide)->getValues();
        bool ok = true;
        for (size_t i = 0; i < rows; i++)
            for (size_t j = 0; j < cols + 3; j++)
                ok &= w[i * (cols + 3) + j] == (j < cols ? sq_want[i * cols + j] : VT(-7));
        CHECK(ok);
        DataObjectFactory::destroy(out[0], out[1], out[2], out[3], wide);
    }
    // the device's share as ONE kernel per batch (the body's operators as text beside the outlined bodies)
    {
        DT *var = nullptr, *sd = nullptr;
        HIP::aggCol(AggOpCode::VAR, var, m1, dctx);
        HIP::ewUnaryMat(UnaryOpCode::SQRT, sd, var, dctx);
        const double thr = 10.0;
        Structure *thrDisguised;
        std::memcpy(&thrDisguised, &thr, sizeof(thr));
        bool isScalar4[] = {false, false, false, true};
        Structure *inputs4[] = {m1, mu, sd, thrDisguised};
        int64_t outRows4[] = {int64_t(rows), 1}, outCols4[] = {1, 1};
        int64_t splits4[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE)};
        int64_t combines4[] = {int64_t(VectorCombine::ROWS), int64_t(VectorCombine::ADD)};
        void *fun4[] = {reinterpret_cast<void *>(Fn(&hostZscore<DT>)), reinterpret_cast<void *>(Fn(&funZscoreOpByOp<DT>))};
        dctx->config.hip_vect_device_share = 1.0;
        dctx->config.hip_vect_shares = 1;
        dctx->config.hip_vect_batch_rows = 0;
        DT *ref[] = {nullptr, nullptr};
        HIP::fusedPipeline<DT>(ref, 2, isScalar4, inputs4, 4, outRows4, outCols4, splits4, combines4, 2, fun4, kZscoreBody, dctx);
        CHECK(HIP::fusedPipelineLastMode() == 1 && whereIs(ref[0]) == 2);
        const auto r_ref = toHost(ref[0]);
        const VT count_ref = toHost(ref[1])[0];
        const double rtol = std::is_same<VT, float>::value ? 1e-5 : 1e-13;
        size_t ambiguous = 0;
        for (VT v : r_ref)
            ambiguous += std::fabs(double(v) - thr) <= rtol * thr;
        for (double share : {0.25, 0.7}) {
            dctx->config.hip_vect_device_share = share;
            dctx->config.hip_vect_shares = 2;
            dctx->config.hip_vect_batch_rows = 128;
            dctx->config.numberOfThreads = 4;
            DT *out[] = {nullptr, nullptr};
            HIP::fusedPipeline<DT>(out, 2, isScalar4, inputs4, 4, outRows4, outCols4, splits4, combines4, 2, fun4, kZscoreBody, dctx);
            CHECK(HIP::fusedPipelineLastMode() == 1 && whereIs(out[0]) == 1);
            const auto got = toHost(out[0]);
            bool ok = got.size() == r_ref.size();
            for (size_t i = 0; ok && i < got.size(); i++)
                ok = std::fabs(double(got[i]) - double(r_ref[i])) <= rtol * std::fabs(double(r_ref[i]));
            CHECK(ok);
            CHECK(std::fabs(double(toHost(out[1])[0]) - double(count_ref)) <= double(ambiguous));
            DataObjectFactory::destroy(out[0], out[1]);
        }
        // no host body, and rows left for the CPU: refused before any worker starts
        {
            void *none[] = {nullptr, reinterpret_cast<void *>(Fn(&funZscoreOpByOp<DT>))};
            DT *out[] = {nullptr, nullptr};
            bool thrown = false;
            try {
                HIP::fusedPipeline<DT>(out, 2, isScalar4, inputs4, 4, outRows4, outCols4, splits4, combines4, 2, none, nullptr, dctx);
            } catch (const std::runtime_error &e) {
                thrown = std::string(e.what()).find("no host body") != std::string::npos;
            }
            CHECK(thrown);
            for (DT *o : out)
                if (o != nullptr)
                    DataObjectFactory::destroy(o);
        }
        CHECK(sd->getRefCounter() == 1);
        DataObjectFactory::destroy(ref[0], ref[1], var, sd);
    }
    // a device task that throws: the exception reaches the caller once every worker has finished, nothing is left behind
    {
        void *bad[] = {reinterpret_cast<void *>(Fn(&hostStats<DT>)), reinterpret_cast<void *>(Fn(&funFails<DT>))};
        dctx->config.hip_vect_device_share = 0.25;
        dctx->config.hip_vect_shares = 3;
        DT *out[] = {nullptr, nullptr, nullptr, nullptr};
        bool thrown = false;
        try {
            HIP::vectorizedPipeline<DT>(out, 4, isScalar, inputs, 2, outRows, outCols, splits, combines, 2, bad, dctx);
        } catch (const std::domain_error &e) {
            thrown = std::string(e.what()) == "the device body failed";
        }
        CHECK(thrown);
        for (DT *o : out)
            if (o != nullptr)
                DataObjectFactory::destroy(o);
        CHECK(m1->getRefCounter() == 1 && mu->getRefCounter() == 1);
    }
    CHECK(hc->numAllocations() == allocs0); // the device's views and results are gone
    dctx->config.hip_vect_device_share = 1.0;
    dctx->config.hip_vect_shares = 1;
    dctx->config.hip_vect_batch_rows = 0;
    dctx->config.numberOfThreads = -1;
    dctx->config.phyBatchSize = 96 * 1024;
    DataObjectFactory::destroy(m1, mu, c, sq, sum);
    DataObjectFactory::destroy(mn, mx);
}
