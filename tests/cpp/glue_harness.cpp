// Test support: a C interface to the run-time objects that the generated kernel entry points take, so that pytest
// can call `HIP_<mnemonic>__<types>(results, arguments, kId, ctx)` out of libHIPKernels.so by the names its catalog
// lists. DAPHNE's compiled programs hand those functions DenseMatrix and DaphneContext pointers; here ctypes does,
// and this file is where such objects are made from numpy arrays and read back.
// Also runs a fused pipeline body through HIP::VectorizedPipeline (tasks over row shares, outputs combined), which
// is template code without a C entry point of its own.
// Built with the plain host compiler against the stand-in run-time headers, like libHIPKernels.so itself.
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include <daphne_hip_kernels.h>

#include "zscore_via_wrappers.h"

namespace {
thread_local std::string g_error;
template <class F> int guarded(F &&f) {
    try {
        f();
        return 0;
    } catch (const std::exception &e) {
        g_error = e.what();
    } catch (...) {
        g_error = "unknown exception";
    }
    return 1;
}
} // namespace

extern "C" {

const char *th_last_error() { return g_error.c_str(); }

void *th_ctx_create() {
    DaphneContext *ctx = nullptr;
    if (guarded([&] {
            ctx = new DaphneContext();
            try {
                HIP::createHIPContext(ctx);
            } catch (...) {
                delete ctx;
                ctx = nullptr;
                throw;
            }
        }))
        return nullptr;
    return ctx;
}
// a DaphneContext without a device context yet, as the compiled program has it before it calls createHIPContext
void *th_ctx_create_bare() { return new DaphneContext(); }
int th_ctx_uses_hip(void *ctx) { return static_cast<DaphneContext *>(ctx)->useHIP() ? 1 : 0; }
void th_ctx_destroy(void *ctx) { delete static_cast<DaphneContext *>(ctx); }
int th_register_kernel(void *ctx, const char *name, const char *file, int line, int column) {
    return static_cast<DaphneContext *>(ctx)->dispatchMapping.registerKernel(name, file, line, column);
}
void th_set_statistics(void *ctx, int on) { static_cast<DaphneContext *>(ctx)->config.enable_statistics = on != 0; }
uint64_t th_kernel_calls(void *ctx, int kId) {
    auto *c = static_cast<DaphneContext *>(ctx);
    std::lock_guard<std::mutex> g(c->stats_lock);
    auto it = c->kernel_stats.find(kId);
    return it == c->kernel_stats.end() ? 0 : it->second.first;
}
void th_set_vect(void *ctx, uint64_t shares, uint64_t batch_rows) {
    auto *c = static_cast<DaphneContext *>(ctx);
    c->config.hip_vect_shares = shares;
    c->config.hip_vect_batch_rows = batch_rows;
}
size_t th_device_allocations(void *ctx) { return HIPContext::get(static_cast<DaphneContext *>(ctx), 0)->numAllocations(); }

#define TH_MATRIX(SUF, T)                                                                                               \
    void *th_mat_from_host_##SUF(size_t rows, size_t cols, const T *data) {                                             \
        auto *m = DataObjectFactory::create<DenseMatrix<T>>(rows, cols, false);                                         \
        if (rows && cols)                                                                                              \
            std::memcpy(m->getValues(), data, rows * cols * sizeof(T));                                                 \
        return m;                                                                                                       \
    }                                                                                                                   \
    size_t th_mat_rows_##SUF(const void *m) { return static_cast<const DenseMatrix<T> *>(m)->getNumRows(); }            \
    size_t th_mat_cols_##SUF(const void *m) { return static_cast<const DenseMatrix<T> *>(m)->getNumCols(); }            \
    /* where the matrix's current contents are: bit 0 host, bit 1 device */                                            \
    int th_mat_where_##SUF(const void *m) {                                                                             \
        const MetaDataObject *mdo = static_cast<const DenseMatrix<T> *>(m)->getMetaDataObject();                        \
        int where = 0;                                                                                                  \
        for (size_t id : mdo->getLatest())                                                                              \
            where |= mdo->getDataPlacementByID(id)->allocation->getType() == ALLOCATION_TYPE::HOST ? 1 : 2;             \
        return where;                                                                                                   \
    }                                                                                                                   \
    int th_mat_to_host_##SUF(const void *m, T *out) {                                                                   \
        return guarded([&] {                                                                                            \
            const auto *dm = static_cast<const DenseMatrix<T> *>(m);                                                    \
            const T *h = dm->getValues();                                                                               \
            for (size_t r = 0; r < dm->getNumRows(); r++)                                                               \
                std::memcpy(out + r * dm->getNumCols(), h + r * dm->getRowSkip(), dm->getNumCols() * sizeof(T));        \
        });                                                                                                             \
    }                                                                                                                   \
    void *th_mat_slice_##SUF(const void *m, size_t rl, size_t ru, size_t cl, size_t cu) {                               \
        void *v = nullptr;                                                                                              \
        if (guarded([&] { v = static_cast<const DenseMatrix<T> *>(m)->slice(rl, ru, cl, cu); }))                        \
            return nullptr;                                                                                             \
        return v;                                                                                                       \
    }                                                                                                                   \
    void th_mat_destroy_##SUF(void *m) { DataObjectFactory::destroy(static_cast<DenseMatrix<T> *>(m)); }
TH_MATRIX(f32, float)
TH_MATRIX(f64, double)
TH_MATRIX(si64, int64_t)
TH_MATRIX(ui64, uint64_t)
TH_MATRIX(si32, int32_t)
TH_MATRIX(ui32, uint32_t)
#undef TH_MATRIX

// One fused body over `shares` row shares. in_roles: HIP::PipeInput per input, out_roles: HIP::PipeOutput per output.
// outputs[o] receives a new matrix handle.
#define TH_PIPELINE(SUF, T)                                                                                             \
    int th_run_fused_pipeline_##SUF(void *ctx, const dh_pipe_instr *program, int num_instr, void **inputs,              \
                                    const int *in_roles, const int *in_slots, const int64_t *splits, size_t num_inputs, \
                                    void **outputs, const int *out_roles, const int *out_slots, const int64_t *out_rows, \
                                    const int64_t *out_cols, const int64_t *combines, size_t num_outputs) {             \
        return guarded([&] {                                                                                            \
            using DT = DenseMatrix<T>;                                                                                  \
            HIP::FusedPipelineBody<T> body;                                                                             \
            body.program.assign(program, program + num_instr);                                                          \
            for (size_t i = 0; i < num_inputs; i++)                                                                     \
                body.inputs.push_back({static_cast<HIP::PipeInput>(in_roles[i]), in_slots[i]});                         \
            for (size_t o = 0; o < num_outputs; o++)                                                                    \
                body.outputs.push_back({static_cast<HIP::PipeOutput>(out_roles[o]), out_slots[o]});                     \
            std::vector<Structure *> ins(num_inputs);                                                                   \
            std::vector<char> is_scalar(num_inputs, 0);                                                                 \
            for (size_t i = 0; i < num_inputs; i++)                                                                     \
                ins[i] = static_cast<DT *>(inputs[i]);                                                                  \
            std::vector<DT *> outs(num_outputs, nullptr);                                                               \
            std::vector<std::function<void(DT ***, Structure **, DCTX(ctx))>> funcs{body};                              \
            HIP::VectorizedPipeline<DT>::apply(outs.data(), num_outputs, reinterpret_cast<const bool *>(is_scalar.data()), \
                                               ins.data(), num_inputs, out_rows, out_cols,                              \
                                               reinterpret_cast<const VectorSplit *>(splits),                           \
                                               reinterpret_cast<const VectorCombine *>(combines), funcs,                \
                                               static_cast<DaphneContext *>(ctx));                                      \
            for (size_t o = 0; o < num_outputs; o++)                                                                    \
                outputs[o] = outs[o];                                                                                   \
        });                                                                                                             \
    }
TH_PIPELINE(f32, float)
TH_PIPELINE(f64, double)
#undef TH_PIPELINE

// Times the fused stage of the z-score pipeline over x (rows x cols floats in device memory) the two ways a DAPHNE
// program compiled with --hip can run it, both through the generated entry points of the kernel library at
// `kernel_lib`: HIP_fusedPipeline without the body's text (the outlined body: one HIP_<mnemonic> call per operator,
// every intermediate in memory) and with it (one launch). Milliseconds per run from the context's stream stopwatch.
int th_time_zscore_stage_f32(void *ctx, const char *kernel_lib, const float *x_dev, size_t rows, size_t cols, float thr, int warmup,
                             int steps, double *ms_by_operators, double *ms_as_one_kernel, double *count_by_operators,
                             double *count_as_one_kernel) {
    return guarded([&] {
        using Z = ZscoreViaWrappers<float>;
        using DT = DenseMatrix<float>;
        auto *dctx = static_cast<DaphneContext *>(ctx);
        void *lib = dlopen(kernel_lib, RTLD_NOW | RTLD_LOCAL);
        if (!lib)
            throw std::runtime_error(std::string("cannot load the kernel library: ") + dlerror());
        if (!Z::load(lib))
            throw std::runtime_error("the kernel library lacks an entry point of the z-score pipeline");
        AllocationDescriptorHIP alloc_desc(dctx, 0);
        dh_ctx *raw = HIPContext::get(dctx, 0)->raw();
        DT *x = DataObjectFactory::create<DT>(rows, cols, false, &alloc_desc);
        HIP::check(dh_d2d(raw, x->getValues(&alloc_desc), x_dev, rows * cols * sizeof(float)));
        DT *mu = nullptr, *var = nullptr, *sd = nullptr;
        HIP::aggCol(AggOpCode::MEAN, mu, x, dctx);
        HIP::aggCol(AggOpCode::VAR, var, x, dctx);
        HIP::ewUnaryMat(UnaryOpCode::SQRT, sd, var, dctx);
        const int kId = dctx->dispatchMapping.registerKernel("_vect_hip1", "bench", 0, 0);
        double *ms_out[] = {ms_by_operators, ms_as_one_kernel}, *count_out[] = {count_by_operators, count_as_one_kernel};
        for (int described = 0; described < 2; described++) {
            DT *out[] = {nullptr, nullptr};
            for (int i = 0; i < warmup + steps; i++) {
                if (i == warmup)
                    HIP::check(dh_timer_start(raw));
                if (out[1] != nullptr) { // the count is folded into its result: start it from nothing each run
                    DataObjectFactory::destroy(out[1]);
                    out[1] = nullptr;
                }
                Z::run(out, x, mu, sd, double(thr), described != 0, kId, dctx);
            }
            float ms = 0;
            HIP::check(dh_timer_stop_ms(raw, &ms));
            if (Z::entry().lastMode() != described)
                throw std::runtime_error(std::string("the fused stage did not run the way it was asked to: ") + Z::entry().lastReason());
            *ms_out[described] = double(ms) / double(steps);
            *count_out[described] = double(static_cast<const DT *>(out[1])->getValues()[0]);
            DataObjectFactory::destroy(out[0], out[1]);
        }
        DataObjectFactory::destroy(x, mu, var, sd);
        dlclose(lib);
    });
}

} // extern "C"
