// Host side of the fused vectorized pipeline: validation, launch of the generic interpreter
// kernel (pipeline_kernel.h), second-stage reduction. See pipeline_kernel.h for the design.
#pragma once

#include "agg_impl.h"
#include "ew_impl.h"
#include "pipeline_kernel.h"

#include <cstdlib>
#include <memory>
#include <string>

namespace dh_pipe {

// pipeline_jit.hip
bool jit_enabled();
bool jit_lookup(int device, const char *tname, int vec, int kv, size_t cols, int G, int S, const dh_pipe_instr *prog, int n,
                hipFunction_t *fn, std::shared_ptr<const void> *keep, std::string *err, bool compile_only);
void jit_set_last_mode(int m);
size_t jit_cache_size();

// Folds the per-workgroup partials of a full reduction. One workgroup of 1024 threads; every thread keeps 16
// loads in flight (indices past the end are clamped for the load and replaced by the identity afterwards) and
// four independent accumulators; the association is fixed by the partial count alone.
constexpr int STAGE2_THREADS = 1024;
template <typename T>
__global__ __launch_bounds__(STAGE2_THREADS) void pipeline_all_stage2(const T *partials_all, size_t np_all, size_t chunk, int op,
                                                                      T *out) {
    // workgroup b folds the partials [b * chunk, (b + 1) * chunk) into out[b]
    const size_t begin = static_cast<size_t>(blockIdx.x) * chunk;
    const T *partials = partials_all + begin;
    const size_t np = (begin + chunk < np_all) ? chunk : np_all - begin;
    __shared__ T lds[STAGE2_THREADS / DH_WAVE];
    constexpr int UN = 16;
    const T id = (op == DH_AGG_SUM) ? T(0) : (op == DH_AGG_MIN) ? dh_inf<T>() : -dh_inf<T>();
    auto comb = [op](T a, T v) {
        return (op == DH_AGG_SUM) ? a + v : (op == DH_AGG_MIN) ? ((v < a) ? v : a) : ((a < v) ? v : a);
    };
    T a0 = id, a1 = id, a2 = id, a3 = id;
    for (size_t i = threadIdx.x; i < np; i += static_cast<size_t>(UN) * STAGE2_THREADS) {
        T v[UN];
#pragma unroll
        for (int k = 0; k < UN; k++) {
            const size_t j = i + static_cast<size_t>(k) * STAGE2_THREADS;
            v[k] = partials[j < np ? j : np - 1];
        }
#pragma unroll
        for (int k = 0; k < UN; k++)
            if (i + static_cast<size_t>(k) * STAGE2_THREADS >= np)
                v[k] = id;
#pragma unroll
        for (int k = 0; k < UN; k += 4) {
            a0 = comb(a0, v[k]);
            a1 = comb(a1, v[k + 1]);
            a2 = comb(a2, v[k + 2]);
            a3 = comb(a3, v[k + 3]);
        }
    }
    T a = comb(comb(a0, a1), comb(a2, a3));
    dh_butterfly(DH_WAVE, [&](auto peer) { a = comb(a, peer(a)); });
    if ((threadIdx.x % DH_WAVE) == 0)
        lds[threadIdx.x / DH_WAVE] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < STAGE2_THREADS / DH_WAVE; w++)
            a = comb(a, lds[w]);
        out[blockIdx.x] = a;
    }
}

static __global__ void pipe_clear_flag(int *flag) { *flag = 0; }

template <typename T, typename IO_C>
dh_status run(dh_ctx *ctx, const dh_pipe_instr *prog, int n, const IO_C *cio, size_t rows, size_t cols) {
    DH_REQUIRE_CTX(ctx);
    if (prog == nullptr || cio == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: program or io is null");
    if (n < 0 || n > DH_PIPE_MAX_INSTR)
        return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: %d instructions, at most %d are supported", n, DH_PIPE_MAX_INSTR);
    if (rows == 0 || cols == 0)
        return DH_OK;
    Program P{};
    P.n = n;
    PipeIO<T> io{};
    io.x = cio->x;
    io.ld_x = cio->ld_x;
    if (io.x == nullptr || io.ld_x < cols)
        return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: the primary input is null or its leading dimension is too small");
    for (int i = 0; i < DH_PIPE_MAX_OPERANDS; i++) {
        io.matrix[i] = cio->matrix[i];
        io.ld_matrix[i] = cio->ld_matrix[i];
        io.rowvec[i] = cio->rowvec[i];
        io.colvec[i] = cio->colvec[i];
        io.ld_colvec[i] = cio->ld_colvec[i];
        io.out_tile[i] = cio->out_tile[i];
        io.ld_out_tile[i] = cio->ld_out_tile[i];
        io.out_row[i] = cio->out_row[i];
        io.ld_out_row[i] = cio->ld_out_row[i];
    }
    constexpr int V = 16 / sizeof(T);
    bool vec_ok = (cols % V == 0) && (io.ld_x % V == 0) && dh_aligned(io.x, 16);
    bool rowvec_used[4] = {false, false, false, false};
    bool checks = false;
    int reduce_ops[2] = {-1, -1};
    T *reduce_out[2] = {nullptr, nullptr};
    for (int i = 0; i < n; i++) {
        const dh_pipe_instr &in = prog[i];
        P.ins[i] = in;
        const int idx = in.index;
        auto bad_index = [&]() { return idx < 0 || idx >= DH_PIPE_MAX_OPERANDS; };
        switch (in.kind) {
        case DH_PIPE_EW_BINARY:
            if (in.op < DH_BIN_ADD || in.op > DH_BIN_OR)
                return dh_fail(DH_ERR_RUNTIME, "unknown BinaryOpCode: %d", in.op);
            switch (in.operand) {
            case DH_OPD_SCALAR:
            case DH_OPD_SELF:
                break;
            case DH_OPD_ROWREG:
                if (in.domain != 0)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: ROWREG operand needs the tile domain", i);
                break;
            case DH_OPD_ROWVEC:
                if (in.domain != 0 || bad_index() || io.rowvec[idx] == nullptr)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: row-vector operand %d is not bound", i, idx);
                vec_ok = vec_ok && dh_aligned(io.rowvec[idx], 16);
                rowvec_used[idx] = true;
                break;
            case DH_OPD_COLVEC:
                if (bad_index() || io.colvec[idx] == nullptr || io.ld_colvec[idx] < 1)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: column-vector operand %d is not bound", i, idx);
                break;
            case DH_OPD_MATRIX:
                if (in.domain != 0 || bad_index() || io.matrix[idx] == nullptr || io.ld_matrix[idx] < cols)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: matrix operand %d is not bound", i, idx);
                vec_ok = vec_ok && (io.ld_matrix[idx] % V == 0) && dh_aligned(io.matrix[idx], 16);
                break;
            default:
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: unknown operand kind %d", i, in.operand);
            }
            break;
        case DH_PIPE_EW_UNARY:
            if (in.op < DH_UN_MINUS || in.op > DH_UN_ISNAN)
                return dh_fail(DH_ERR_RUNTIME, "unknown UnaryOpCode: %d", in.op);
            checks |= (in.op == DH_UN_SQRT || in.op == DH_UN_LN || in.op == DH_UN_ASIN || in.op == DH_UN_ACOS);
            break;
        case DH_PIPE_ROW_AGG:
            if (in.op < DH_AGG_SUM || in.op > DH_AGG_VAR)
                return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode");
            break;
        case DH_PIPE_STORE_TILE:
            if (bad_index() || io.out_tile[idx] == nullptr || io.ld_out_tile[idx] < cols)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: tile output %d is not bound", i, idx);
            vec_ok = vec_ok && (io.ld_out_tile[idx] % V == 0) && dh_aligned(io.out_tile[idx], 16);
            break;
        case DH_PIPE_STORE_ROW:
        case DH_PIPE_STORE_ROW_IDX:
            if (bad_index() || io.out_row[idx] == nullptr || io.ld_out_row[idx] < 1)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: row output %d is not bound", i, idx);
            break;
        case DH_PIPE_REDUCE_ALL:
            // the combines a vectorized pipeline knows: ADD MIN MAX
            // (ir/daphneir/DaphneVectorizableOpInterface.cpp:306-311)
            if (in.op != DH_AGG_SUM && in.op != DH_AGG_MIN && in.op != DH_AGG_MAX)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: REDUCE_ALL supports SUM, MIN and MAX");
            if (idx < 0 || idx > 1 || cio->out_all[idx] == nullptr)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: scalar output %d is not bound", i, idx);
            if (reduce_ops[idx] != -1)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: scalar output %d is reduced twice", idx);
            reduce_ops[idx] = in.op;
            reduce_out[idx] = cio->out_all[idx];
            break;
        default:
            return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: unknown kind %d", i, in.kind);
        }
    }
    for (int k = 0; k < 4; k++)
        if (!rowvec_used[k])
            io.rowvec[k] = nullptr; // the kernel loads every bound row vector
    PipeShape sh;
    if (!pipe_shape(cols, vec_ok ? V : 1, &sh))
        return dh_fail(DH_ERR_RUNTIME,
                       "vectorizedPipeline: rows of %zu values do not fit the register tile (at most %d per row here); "
                       "run the operators one by one instead",
                       cols, 64 * (vec_ok ? V : 1) * 4);
    const int vec = sh.vec, G = sh.G, KV = sh.KV, U = sh.U, S = sh.S;
    const size_t groups_per_block = THREADS / G;
    // One run of S steps per wavefront wherever the grid can express it (S from pipe_shape: one step for float
    // rows, four for double). A wavefront asks for its first tile before the operand vectors, so that the
    // values it derives from them once are computed under the tile's latency; with that, the shortest
    // wavefronts do best for float (6.4 TB/s on the 20M x 64 z-score body).
    size_t grid = dh_ceil_div(rows, groups_per_block * U * S);
    const size_t cap = 0x7fffffffull;
    if (grid > cap)
        grid = cap;
    void *wsv = nullptr;
    // one partial per wavefront and REDUCE_ALL slot, then room for the first of two folding rounds
    const size_t np = grid * (THREADS / DH_WAVE);
    constexpr size_t FOLD_BLOCKS = 64;
    dh_status st = dh_workspace(ctx, (2 * np + 2 * FOLD_BLOCKS) * sizeof(T) + 256, &wsv);
    if (st != DH_OK)
        return st;
    T *partials = static_cast<T *>(wsv);
    if (checks)
        hipLaunchKernelGGL(pipe_clear_flag, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev);
    // Preferred path: the body specialised at run time (pipeline_jit.hip). The generic interpreter
    // kernel below is the fallback when specialisation is switched off or fails.
    hipFunction_t jit_fn = nullptr;
    std::shared_ptr<const void> jit_keep; // the module stays loaded at least until the launch below is queued
    std::string jit_err;
    // the context's setting wins over the environment's (dh_ctx_set_pipeline_mode)
    const bool want_jit = n >= 1 && (ctx->pipeline_mode < 0 ? jit_enabled() : ctx->pipeline_mode == 1);
    const bool use_jit = want_jit && jit_lookup(ctx->device, sizeof(T) == 4 ? "float" : "double", vec, KV, cols, G, S, P.ins, n,
                                                &jit_fn, &jit_keep, &jit_err, false);
    if (want_jit && !use_jit) {
        // The body still runs (interpreted, at a fraction of the rate); the reason stays readable through
        // dh_last_error() and dh_vectorized_pipeline_last_mode() says 0. Reported once per process on stderr.
        dh_set_error("vectorizedPipeline: run-time specialisation failed, the body is interpreted instead: %s", jit_err.c_str());
        static bool warned = false;
        if (!warned) {
            warned = true;
            fprintf(stderr, "libdaphne_hip: %s\n", dh_last_error());
        }
    }
    const dim3 g(static_cast<unsigned>(grid)), b(THREADS);
    {
    DhKernelStopwatch stopwatch(ctx); // around the body kernel alone (dh_kernel_timing)
    if (use_jit) {
        size_t a_rows = rows, a_cols = cols;
        int a_G = G;
        int *a_flag = ctx->flag_dev;
        Immediates imm{};
        for (int i = 0; i < n; i++)
            imm.v[i] = prog[i].scalar;
        void *args[] = {&io, &a_rows, &a_cols, &a_G, &partials, &a_flag, &imm};
        DH_CHECK_HIP(hipModuleLaunchKernel(jit_fn, g.x, 1, 1, b.x, 1, 1, 0, ctx->stream, args, nullptr));
        jit_set_last_mode(1);
    } else {
        jit_set_last_mode(0);
#define DH_LAUNCH(VEC_, KV_)                                                                       \
    hipLaunchKernelGGL((pipeline_kernel<T, VEC_, KV_>), g, b, 0, ctx->stream, P, io, rows, cols, G, S, partials,        \
                       ctx->flag_dev)
        if (vec_ok) {
            if (KV == 1)
                DH_LAUNCH(V, 1);
            else if (KV == 2)
                DH_LAUNCH(V, 2);
            else
                DH_LAUNCH(V, 4);
        } else {
            if (KV == 1)
                DH_LAUNCH(1, 1);
            else if (KV == 2)
                DH_LAUNCH(1, 2);
            else
                DH_LAUNCH(1, 4);
        }
#undef DH_LAUNCH
    }
    }
    DH_CHECK_LAUNCH();
    for (int s = 0; s < 2; s++)
        if (reduce_ops[s] != -1) {
            const T *src = partials + s * np;
            size_t count = np;
            if (np > 4 * static_cast<size_t>(STAGE2_THREADS) * 16) {
                // many partials: 64 workgroups fold a contiguous share each, one workgroup folds their results
                T *mid = partials + 2 * np + s * FOLD_BLOCKS;
                const size_t chunk = dh_ceil_div(np, FOLD_BLOCKS);
                const size_t blocks = dh_ceil_div(np, chunk);
                hipLaunchKernelGGL((pipeline_all_stage2<T>), dim3(static_cast<unsigned>(blocks)), dim3(STAGE2_THREADS), 0, ctx->stream, src,
                                   np, chunk, reduce_ops[s], mid);
                DH_CHECK_LAUNCH();
                src = mid;
                count = blocks;
            }
            hipLaunchKernelGGL((pipeline_all_stage2<T>), dim3(1), dim3(STAGE2_THREADS), 0, ctx->stream, src, count, count,
                               reduce_ops[s], reduce_out[s]);
            DH_CHECK_LAUNCH();
        }
    if (checks) {
        if (ctx->deferred_depth > 0) // the verdict waits for dh_check_deferred
            return dh_latch_deferred(ctx, 0, DH_DEFERRED_PIPELINE_DOMAIN, 0, nullptr, 0, 0);
        DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        if (*ctx->flag_host != 0)
            return dh_fail_pipeline_domain();
    }
    return DH_OK;
}

} // namespace dh_pipe
