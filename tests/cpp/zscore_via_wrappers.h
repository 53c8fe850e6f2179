// The z-score pipeline (r = rowSums(((X - mu) / sd)^2), count = sum(r > thr)) the way a DAPHNE program compiled with
// --hip runs it: through the generated HIP_<mnemonic>__<types> entry points of libHIPKernels.so, looked up by name.
// vect_hip() is the device body as the compiler outlines it (one entry point per operator); HIP_fusedPipeline gets that
// body plus the text of the same operators. Used by the glue test (results) and by the harness that bench.py loads
// (timings). Test infrastructure only.
#pragma once

#include <daphne_hip_kernels.h>

#include <dlfcn.h>

#include <cstring>
#include <string>
#include <type_traits>

template <typename VT> struct ZscoreViaWrappers {
    using DT = DenseMatrix<VT>;
    using BinFn = void (*)(DT **, const DT *, const DT *, int, DaphneContext *);
    using ScaFn = void (*)(DT **, const DT *, VT, int, DaphneContext *);
    using RowFn = void (*)(DT **, const DT *, int, DaphneContext *);
    using AllFn = void (*)(VT *, const DT *, int, DaphneContext *);
    using FillFn = void (*)(DT **, VT, size_t, size_t, int, DaphneContext *);
    using PipeFn = void (*)(DT **, size_t, bool *, Structure **, size_t, int64_t *, int64_t *, int64_t *, int64_t *, size_t, void **,
                            const char *, int, DaphneContext *);
    struct Entry {
        BinFn sub = nullptr, div = nullptr, mul = nullptr;
        RowFn sumRow = nullptr;
        ScaFn gt = nullptr;
        AllFn sumAll = nullptr;
        FillFn fill = nullptr;
        PipeFn fusedPipeline = nullptr;
        int (*lastMode)() = nullptr;           // of the library's last fusedPipeline call on this thread
        const char *(*lastReason)() = nullptr; // why it ran operator by operator, if it did
    };
    static Entry &entry() {
        static Entry e;
        return e;
    }
    static const char *body() {
        return "%0 = ewSub in0, in1\n%1 = ewDiv %0, in2\n%2 = ewMul %1, %1\n%3 = sumRow %2\n%4 = ewGt %3, in3\n%5 = sumAll %4\n"
               "%6 = cast %5\nreturn %3, %6\n";
    }
    static bool load(void *lib) {
        const std::string vt = std::is_same<VT, float>::value ? "float" : "double", m = "DenseMatrix_" + vt;
        auto sym = [&](const std::string &name) { return dlsym(lib, name.c_str()); };
        Entry &e = entry();
        e.sub = reinterpret_cast<BinFn>(sym("HIP_ewSub__" + m + "__" + m + "__" + m));
        e.div = reinterpret_cast<BinFn>(sym("HIP_ewDiv__" + m + "__" + m + "__" + m));
        e.mul = reinterpret_cast<BinFn>(sym("HIP_ewMul__" + m + "__" + m + "__" + m));
        e.sumRow = reinterpret_cast<RowFn>(sym("HIP_sumRow__" + m + "__" + m));
        e.gt = reinterpret_cast<ScaFn>(sym("HIP_ewGt__" + m + "__" + m + "__" + vt));
        e.sumAll = reinterpret_cast<AllFn>(sym("HIP_sumAll__" + vt + "__" + m));
        e.fill = reinterpret_cast<FillFn>(sym("HIP_fill__" + m + "__" + vt + "__size_t__size_t"));
        e.fusedPipeline = reinterpret_cast<PipeFn>(sym("HIP_fusedPipeline__" + m + "_variadic__size_t__bool__Structure_variadic__size_t__"
                                                       "int64_t__int64_t__int64_t__int64_t__size_t__void_variadic__char"));
        e.lastMode = reinterpret_cast<int (*)()>(sym("HIP_fusedPipeline_lastMode"));
        e.lastReason = reinterpret_cast<const char *(*)()>(sym("HIP_fusedPipeline_lastReason"));
        return e.sub && e.div && e.mul && e.sumRow && e.gt && e.sumAll && e.fill && e.fusedPipeline && e.lastMode && e.lastReason;
    }
    // `_vect_hip<N>` as LowerToLLVMPass outlines it (calls inside a body carry no registered dispatch id here);
    // inputs x, mu, sd and the threshold as a scalar in the place of a pointer; outputs r (ROWS) and the count (ADD)
    static void vect_hip(DT ***outputs, Structure **inputs, DaphneContext *ctx) {
        const Entry &e = entry();
        const int kId = ErrorHandler::UNREGISTERED;
        auto *x = static_cast<DT *>(inputs[0]), *mu = static_cast<DT *>(inputs[1]), *sd = static_cast<DT *>(inputs[2]);
        const VT thr = HIP::FusedPipelineBody<VT>::scalarOf(inputs[3]);
        DT *c = nullptr, *z = nullptr, *zz = nullptr, *gt = nullptr;
        e.sub(&c, x, mu, kId, ctx);
        e.div(&z, c, sd, kId, ctx);
        e.mul(&zz, z, z, kId, ctx);
        e.sumRow(outputs[0], zz, kId, ctx);
        e.gt(&gt, *outputs[0], thr, kId, ctx);
        VT count = 0;
        e.sumAll(&count, gt, kId, ctx);
        e.fill(outputs[1], count, 1, 1, kId, ctx);
        DataObjectFactory::destroy(c, z, zz, gt);
        DataObjectFactory::destroy(x, mu, sd);
    }
    // One run of the pipeline over x (rows x cols) through HIP_fusedPipeline; `described`: with the body's text.
    // out[0] = r, out[1] = count; created when null, written in place otherwise.
    static void run(DT *out[2], DT *x, DT *mu, DT *sd, double thr, bool described, int kId, DaphneContext *ctx) {
        Structure *thrDisguised;
        std::memcpy(&thrDisguised, &thr, sizeof(thr));
        bool isScalar[] = {false, false, false, true};
        Structure *inputs[] = {x, mu, sd, thrDisguised};
        int64_t outRows[] = {int64_t(x->getNumRows()), 1}, outCols[] = {1, 1};
        int64_t splits[] = {int64_t(VectorSplit::ROWS), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE), int64_t(VectorSplit::NONE)};
        int64_t combines[] = {int64_t(VectorCombine::ROWS), int64_t(VectorCombine::ADD)};
        void *fun[] = {nullptr, reinterpret_cast<void *>(&vect_hip)}; // {host body, device body}
        entry().fusedPipeline(out, 2, isScalar, inputs, 4, outRows, outCols, splits, combines, 2, fun, described ? body() : "", kId, ctx);
    }
};
