// A host-memory implementation of the part of the C ABI (include/daphne_hip.h) that the placement and
// vectorized-pipeline tests reach. "Device" memory is ordinary heap memory, kernels are plain loops. It exists so
// that the C++ kernel layer (HIPContext, AllocationDescriptorHIP, HIP::*::apply, CompiledPipelineTaskHIP) can be
// compiled and run against the reference's own DenseMatrix / MetaDataObject / Structure sources on a machine
// without a GPU: what is under test there is which pointers, leading dimensions and shapes the layer hands to the
// C ABI, not the kernels. Test infrastructure only; nothing of the product links it.
#include <daphne_hip.h>

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <string>
#include <vector>

struct dh_ctx {
    std::mutex m;
    std::map<void *, size_t> blocks;
    size_t in_use = 0;
};

namespace {
thread_local std::string g_error;
dh_status fail(dh_status st, const std::string &msg) {
    g_error = msg;
    return st;
}

template <typename T> bool binary(int op, T l, T r, T &out) {
    switch (op) {
    case DH_BIN_ADD: out = l + r; return true;
    case DH_BIN_SUB: out = l - r; return true;
    case DH_BIN_MUL: out = l * r; return true;
    case DH_BIN_DIV: out = l / r; return true;
    case DH_BIN_POW: out = std::pow(l, r); return true;
    case DH_BIN_MOD: out = std::fmod(l, r); return true;
    case DH_BIN_LOG: out = std::log(l) / std::log(r); return true;
    case DH_BIN_EQ: out = l == r; return true;
    case DH_BIN_NEQ: out = l != r; return true;
    case DH_BIN_LT: out = l < r; return true;
    case DH_BIN_LE: out = l <= r; return true;
    case DH_BIN_GT: out = l > r; return true;
    case DH_BIN_GE: out = l >= r; return true;
    case DH_BIN_MIN: out = std::min(l, r); return true;
    case DH_BIN_MAX: out = std::max(l, r); return true;
    case DH_BIN_AND: out = l && r; return true;
    case DH_BIN_OR: out = l || r; return true;
    default: return false;
    }
}
template <typename T> bool unary(int op, T a, T &out) {
    switch (op) {
    case DH_UN_SQRT: out = std::sqrt(a); return true;
    case DH_UN_ABS: out = std::fabs(a); return true;
    case DH_UN_EXP: out = std::exp(a); return true;
    default: return false;
    }
}
// one value from n values at stride `step`
template <typename T> bool aggregate(int op, const T *v, size_t n, size_t step, T &out) {
    if (n == 0)
        return false;
    if (op == DH_AGG_MEAN || op == DH_AGG_VAR || op == DH_AGG_STDDEV) {
        double s = 0;
        for (size_t i = 0; i < n; i++)
            s += double(v[i * step]);
        const double mean = s / double(n);
        if (op == DH_AGG_MEAN) {
            out = T(mean);
            return true;
        }
        double q = 0;
        for (size_t i = 0; i < n; i++)
            q += (double(v[i * step]) - mean) * (double(v[i * step]) - mean);
        out = T(op == DH_AGG_VAR ? q / double(n) : std::sqrt(q / double(n)));
        return true;
    }
    T acc = v[0];
    for (size_t i = 1; i < n; i++) {
        const T x = v[i * step];
        switch (op) {
        case DH_AGG_SUM: acc += x; break;
        case DH_AGG_PROD: acc *= x; break;
        case DH_AGG_MIN: acc = std::min(acc, x); break;
        case DH_AGG_MAX: acc = std::max(acc, x); break;
        default: return false;
        }
    }
    out = acc;
    return true;
}

template <typename T>
dh_status ew_binary(int op, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs, const T *rhs, size_t rr,
                    size_t rc, size_t ld_rhs) {
    const bool same = rr == lr && rc == lc, rowvec = rr == 1 && rc == lc, colvec = rr == lr && rc == 1;
    if (!(same || rowvec || colvec))
        return fail(DH_ERR_RUNTIME, "EwBinaryMat: lhs and rhs must have the same shape, or rhs must be a row / column vector");
    for (size_t r = 0; r < lr; r++)
        for (size_t c = 0; c < lc; c++) {
            const T b = same ? rhs[r * ld_rhs + c] : rowvec ? rhs[c] : rhs[r * ld_rhs];
            if (!binary(op, lhs[r * ld_lhs + c], b, res[r * ld_res + c]))
                return fail(DH_ERR_RUNTIME, "unknown BinaryOpCode");
        }
    return DH_OK;
}
template <typename T> dh_status ew_binary_sca(int op, T *res, size_t ld_res, const T *lhs, size_t rows, size_t cols, size_t ld, T rhs) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++)
            if (!binary(op, lhs[r * ld + c], rhs, res[r * ld_res + c]))
                return fail(DH_ERR_RUNTIME, "unknown BinaryOpCode");
    return DH_OK;
}
template <typename T> dh_status ew_unary(int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++)
            if (!unary(op, arg[r * ld + c], res[r * ld_res + c]))
                return fail(DH_ERR_RUNTIME, "UnaryOpCode outside the mock");
    return DH_OK;
}
template <typename T> dh_status agg_col(int op, T *res, const T *arg, size_t rows, size_t cols, size_t ld) {
    for (size_t c = 0; c < cols; c++)
        if (!aggregate(op, arg + c, rows, ld, res[c]))
            return fail(DH_ERR_RUNTIME, "AggOpCode outside the mock");
    return DH_OK;
}
template <typename T> dh_status agg_row(int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    for (size_t r = 0; r < rows; r++)
        if (!aggregate(op, arg + r * ld, cols, size_t(1), res[r * ld_res]))
            return fail(DH_ERR_RUNTIME, "AggOpCode outside the mock");
    return DH_OK;
}
template <typename T> dh_status agg_all(int op, const T *arg, size_t rows, size_t cols, size_t ld, T *out) {
    std::vector<T> flat(rows * cols);
    for (size_t r = 0; r < rows; r++)
        std::copy(arg + r * ld, arg + r * ld + cols, flat.begin() + r * cols);
    return aggregate(op, flat.data(), flat.size(), size_t(1), *out) ? DH_OK : fail(DH_ERR_RUNTIME, "AggOpCode outside the mock");
}

// the accumulator machine of the fused pipeline: per row a tile t (cols values) and a scalar r
template <typename T, typename IO> dh_status pipeline(const dh_pipe_instr *prog, int n, const IO *io, size_t rows, size_t cols) {
    if (n < 0 || n > DH_PIPE_MAX_INSTR)
        return fail(DH_ERR_RUNTIME, "pipeline: too many instructions");
    std::vector<T> t(cols);
    T all[2] = {T(0), T(0)};
    bool all_set[2] = {false, false};
    for (size_t row = 0; row < rows; row++) {
        std::copy(io->x + row * io->ld_x, io->x + row * io->ld_x + cols, t.begin());
        T r = T(0);
        for (int i = 0; i < n; i++) {
            const dh_pipe_instr &in = prog[i];
            switch (in.kind) {
            case DH_PIPE_EW_BINARY: {
                const size_t items = in.domain == 0 ? cols : 1;
                for (size_t c = 0; c < items; c++) {
                    T &cur = in.domain == 0 ? t[c] : r;
                    T opd;
                    switch (in.operand) {
                    case DH_OPD_SCALAR: opd = T(in.scalar); break;
                    case DH_OPD_SELF: opd = cur; break;
                    case DH_OPD_ROWVEC: opd = io->rowvec[in.index][c]; break;
                    case DH_OPD_COLVEC: opd = io->colvec[in.index][row * io->ld_colvec[in.index]]; break;
                    case DH_OPD_MATRIX: opd = io->matrix[in.index][row * io->ld_matrix[in.index] + c]; break;
                    case DH_OPD_ROWREG: opd = r; break;
                    default: return fail(DH_ERR_RUNTIME, "pipeline: unknown operand kind");
                    }
                    T out;
                    if (!(in.swap ? binary(in.op, opd, cur, out) : binary(in.op, cur, opd, out)))
                        return fail(DH_ERR_RUNTIME, "pipeline: unknown BinaryOpCode");
                    cur = out;
                }
                break;
            }
            case DH_PIPE_EW_UNARY: {
                const size_t items = in.domain == 0 ? cols : 1;
                for (size_t c = 0; c < items; c++) {
                    T &cur = in.domain == 0 ? t[c] : r;
                    if (!unary(in.op, cur, cur))
                        return fail(DH_ERR_RUNTIME, "pipeline: UnaryOpCode outside the mock");
                }
                break;
            }
            case DH_PIPE_ROW_AGG:
                if (!aggregate(in.op, t.data(), cols, size_t(1), r))
                    return fail(DH_ERR_RUNTIME, "pipeline: AggOpCode outside the mock");
                break;
            case DH_PIPE_STORE_TILE:
                std::copy(t.begin(), t.end(), io->out_tile[in.index] + row * io->ld_out_tile[in.index]);
                break;
            case DH_PIPE_STORE_ROW:
                static_cast<T *>(io->out_row[in.index])[row * io->ld_out_row[in.index]] = r;
                break;
            case DH_PIPE_STORE_ROW_IDX:
                static_cast<uint64_t *>(io->out_row[in.index])[row * io->ld_out_row[in.index]] = uint64_t(r);
                break;
            case DH_PIPE_REDUCE_ALL: {
                const size_t items = in.domain == 0 ? cols : 1;
                for (size_t c = 0; c < items; c++) {
                    const T v = in.domain == 0 ? t[c] : r;
                    T &acc = all[in.index];
                    if (!all_set[in.index]) {
                        acc = v;
                        all_set[in.index] = true;
                    } else if (in.op == DH_AGG_SUM)
                        acc += v;
                    else if (in.op == DH_AGG_MIN)
                        acc = std::min(acc, v);
                    else if (in.op == DH_AGG_MAX)
                        acc = std::max(acc, v);
                    else
                        return fail(DH_ERR_RUNTIME, "pipeline: REDUCE_ALL takes SUM, MIN or MAX");
                }
                break;
            }
            default:
                return fail(DH_ERR_RUNTIME, "pipeline: unknown instruction kind");
            }
        }
    }
    for (int k = 0; k < 2; k++)
        if (io->out_all[k] != nullptr && all_set[k])
            *io->out_all[k] = all[k];
    return DH_OK;
}
} // namespace

extern "C" {

const char *dh_last_error(void) { return g_error.c_str(); }

dh_status dh_ctx_create(int device, dh_ctx **out) {
    if (device != 0)
        return fail(DH_ERR_HIP, "the mock has one device");
    *out = new dh_ctx();
    return DH_OK;
}
dh_status dh_ctx_destroy(dh_ctx *ctx) {
    for (auto &b : ctx->blocks)
        std::free(b.first);
    delete ctx;
    return DH_OK;
}
size_t dh_ctx_mem_budget(const dh_ctx *) { return size_t(1) << 34; }
size_t dh_ctx_mem_in_use(const dh_ctx *ctx) { return ctx->in_use; }

dh_status dh_malloc(dh_ctx *ctx, size_t bytes, int zero, void **out) {
    void *p = zero ? std::calloc(std::max<size_t>(bytes, 1), 1) : std::malloc(std::max<size_t>(bytes, 1));
    if (!p)
        return fail(DH_ERR_OOM, "out of host memory");
    if (!zero)
        std::memset(p, 0xCD, bytes); // garbage, so that rows nobody wrote show
    std::lock_guard<std::mutex> g(ctx->m);
    ctx->blocks[p] = bytes;
    ctx->in_use += bytes;
    *out = p;
    return DH_OK;
}
dh_status dh_free(dh_ctx *ctx, void *ptr) {
    std::lock_guard<std::mutex> g(ctx->m);
    auto it = ctx->blocks.find(ptr);
    if (it == ctx->blocks.end())
        return fail(DH_ERR_RUNTIME, "dh_free: unknown pointer");
    ctx->in_use -= it->second;
    ctx->blocks.erase(it);
    std::free(ptr);
    return DH_OK;
}
// transfers must stay inside one block handed out by dh_malloc: an offset that runs past its allocation fails here
static bool inside(dh_ctx *ctx, const void *p, size_t bytes) {
    std::lock_guard<std::mutex> g(ctx->m);
    const char *q = static_cast<const char *>(p);
    for (auto &b : ctx->blocks) {
        const char *lo = static_cast<const char *>(b.first);
        if (q >= lo && q + bytes <= lo + std::max<size_t>(b.second, 1))
            return true;
    }
    return bytes == 0;
}
dh_status dh_h2d(dh_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    if (!inside(ctx, dst_dev, bytes))
        return fail(DH_ERR_HIP, "dh_h2d: destination outside any device allocation");
    std::memcpy(dst_dev, src_host, bytes);
    return DH_OK;
}
dh_status dh_d2h(dh_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if (!inside(ctx, src_dev, bytes))
        return fail(DH_ERR_HIP, "dh_d2h: source outside any device allocation");
    std::memcpy(dst_host, src_dev, bytes);
    return DH_OK;
}
// The mock's kernels have nothing to validate on a device: no verdict is ever pending.
dh_status dh_kernel_timing(dh_ctx *, int) { return DH_OK; }
dh_status dh_kernel_timing_read(dh_ctx *, double *total_ms, size_t *launches) {
    if (total_ms)
        *total_ms = 0.0;
    if (launches)
        *launches = 0;
    return DH_OK;
}
dh_status dh_defer_checks(dh_ctx *, int) { return DH_OK; }
dh_status dh_check_deferred(dh_ctx *) { return DH_OK; }
dh_status dh_d2d_2d(dh_ctx *, void *dst_dev, size_t dst_pitch, const void *src_dev, size_t src_pitch, size_t width_bytes,
                    size_t rows) {
    for (size_t r = 0; r < rows; r++)
        std::memcpy(static_cast<char *>(dst_dev) + r * dst_pitch, static_cast<const char *>(src_dev) + r * src_pitch, width_bytes);
    return DH_OK;
}
dh_status dh_d2h_2d(dh_ctx *ctx, void *dst_host, size_t dst_pitch, const void *src_dev, size_t src_pitch, size_t width_bytes,
                    size_t rows) {
    if (rows != 0 && width_bytes != 0 && !inside(ctx, src_dev, (rows - 1) * src_pitch + width_bytes))
        return fail(DH_ERR_HIP, "dh_d2h_2d: source outside any device allocation");
    for (size_t r = 0; r < rows; r++)
        std::memcpy(static_cast<char *>(dst_host) + r * dst_pitch, static_cast<const char *>(src_dev) + r * src_pitch, width_bytes);
    return DH_OK;
}

#define MOCK_KERNELS(SUF, T)                                                                                            \
    dh_status dh_ew_binary_##SUF(dh_ctx *, int op, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs,      \
                                 const T *rhs, size_t rr, size_t rc, size_t ld_rhs) {                                   \
        return ew_binary<T>(op, res, ld_res, lhs, lr, lc, ld_lhs, rhs, rr, rc, ld_rhs);                                 \
    }                                                                                                                   \
    dh_status dh_ew_binary_sca_##SUF(dh_ctx *, int op, T *res, size_t ld_res, const T *lhs, size_t rows, size_t cols,   \
                                     size_t ld_lhs, T rhs) {                                                            \
        return ew_binary_sca<T>(op, res, ld_res, lhs, rows, cols, ld_lhs, rhs);                                         \
    }                                                                                                                   \
    dh_status dh_ew_unary_##SUF(dh_ctx *, int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,        \
                                size_t ld_arg) {                                                                        \
        return ew_unary<T>(op, res, ld_res, arg, rows, cols, ld_arg);                                                   \
    }                                                                                                                   \
    dh_status dh_agg_all_##SUF(dh_ctx *, int op, const T *arg, size_t rows, size_t cols, size_t ld, T *result_host) {   \
        return agg_all<T>(op, arg, rows, cols, ld, result_host);                                                        \
    }                                                                                                                   \
    dh_status dh_agg_row_##SUF(dh_ctx *, int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,         \
                               size_t ld) {                                                                             \
        return agg_row<T>(op, res, ld_res, arg, rows, cols, ld);                                                        \
    }                                                                                                                   \
    dh_status dh_agg_col_##SUF(dh_ctx *, int op, T *res, const T *arg, size_t rows, size_t cols, size_t ld) {           \
        return agg_col<T>(op, res, arg, rows, cols, ld);                                                                \
    }                                                                                                                   \
    dh_status dh_fill_##SUF(dh_ctx *, T *res, size_t ld_res, T value, size_t rows, size_t cols) {                       \
        for (size_t r = 0; r < rows; r++)                                                                               \
            std::fill(res + r * ld_res, res + r * ld_res + cols, value);                                                \
        return DH_OK;                                                                                                   \
    }                                                                                                                   \
    dh_status dh_vectorized_pipeline_##SUF(dh_ctx *, const dh_pipe_instr *program, int num_instr,                       \
                                           const dh_pipe_io_##SUF *io, size_t rows, size_t cols) {                      \
        return pipeline<T>(program, num_instr, io, rows, cols);                                                         \
    }
MOCK_KERNELS(f32, float)
MOCK_KERNELS(f64, double)
#undef MOCK_KERNELS

} // extern "C"
