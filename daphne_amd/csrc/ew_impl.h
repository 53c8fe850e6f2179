// Elementwise binary / unary kernels for DenseMatrix<float|double>, instantiated once per value
// type by ew_f32.hip and ew_f64.hip.
//
// Semantics follow the reference's CPU kernels, not its CUDA ones:
//   EwBinaryMat   runtime/local/kernels/EwBinaryMat.h:54-108   (broadcast rules, res = lhs shape)
//   EwBinarySca   runtime/local/kernels/EwBinarySca.h:143-167  (the 17 floating-point ops)
//   EwBinaryObjSca runtime/local/kernels/EwBinaryObjSca.h:57-79
//   EwUnaryMat    runtime/local/kernels/EwUnaryMat.h:57-77
//   EwUnarySca    runtime/local/kernels/EwUnarySca.h:129-206   (19 numeric ops, domain errors)
//
// One kernel shape serves every case. Threads form a (TX, TY) tile: TX lanes walk the 16-byte
// column vectors of a row, TY rows are covered per workgroup, and each
// thread handles exactly one vector and exits (one-shot grid: measured on MI355X, millions of
// short-lived workgroups copy at ~6.2 TB/s where a grid-stride loop reaches ~4.7 TB/s). A
// row-vector operand is a cached 16-byte load per thread; a column-vector operand is one scalar
// per row; no integer division or modulo is executed per element. Contiguous
// same-shape / scalar / unary inputs are viewed as a matrix that is one block-row (256 vectors)
// wide, which turns the flat array into the same 2-D walk.
#pragma once

#include "common.h"
#include "ew_ops.h"

#include <cmath>
#include <limits>

namespace dh_ew {

// ---------------------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------------------
enum Mode { SAME = 0, ROWVEC = 1, COLVEC = 2, SCALAR = 3, UNARY = 4 };

template <typename T, int VEC> struct Pack {
    T v[VEC];
};
template <typename T, int VEC> __device__ __forceinline__ Pack<T, VEC> load_pack(const T *p) {
    Pack<T, VEC> r;
    if constexpr (VEC == 1) {
        r.v[0] = *p;
    } else {
        using V = typename dh_vec<T>::type;
        V t = *reinterpret_cast<const V *>(p);
        const T *tp = reinterpret_cast<const T *>(&t);
#pragma unroll
        for (int i = 0; i < VEC; i++)
            r.v[i] = tp[i];
    }
    return r;
}
template <typename T, int VEC> __device__ __forceinline__ void store_pack(T *p, const Pack<T, VEC> &r) {
    if constexpr (VEC == 1) {
        *p = r.v[0];
    } else {
        using V = typename dh_vec<T>::type;
        V t;
        T *tp = reinterpret_cast<T *>(&t);
#pragma unroll
        for (int i = 0; i < VEC; i++)
            tp[i] = r.v[i];
        *reinterpret_cast<V *>(p) = t;
    }
}

constexpr int EW_THREADS = 256;

template <typename T, int VEC, template <typename> class F, int MODE>
__global__ __launch_bounds__(EW_THREADS) void ew_kernel(T *res, size_t ld_res, const T *lhs, size_t ld_lhs,
                                                        const T *rhs, size_t ld_rhs, T sca, size_t rows,
                                                        size_t cvecs, int *flag) {
    // One 16-byte vector per thread and no loop: on MI355X a very large grid of short-lived
    // workgroups sustains markedly more copy bandwidth than a grid-stride loop over few of them.
    // blockIdx.x (up to 2^31 - 1) covers the rows, blockIdx.y the column vectors beyond one block.
    const size_t r = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y;
    if (r >= rows)
        return;
    bool any_bad = false;
    for (size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x; cv < cvecs;
         cv += static_cast<size_t>(gridDim.y) * blockDim.x) {
        const size_t c = cv * VEC;
        T a[VEC], b[VEC], o[VEC];
        dh_load_vec_stream<T, VEC>(lhs + r * ld_lhs + c, a);
        if constexpr (MODE == SAME)
            dh_load_vec_stream<T, VEC>(rhs + r * ld_rhs + c, b);
        if constexpr (MODE == ROWVEC)
            dh_load_vec<T, VEC>(rhs + c, b);
        if constexpr (MODE == COLVEC) {
            const T s = rhs[r * ld_rhs];
#pragma unroll
            for (int i = 0; i < VEC; i++)
                b[i] = s;
        }
        if constexpr (MODE == SCALAR || MODE == UNARY) {
#pragma unroll
            for (int i = 0; i < VEC; i++)
                b[i] = sca;
        }
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            o[i] = F<T>::apply(a[i], b[i]);
            if constexpr (F<T>::checks) {
                if constexpr (MODE == UNARY)
                    any_bad |= F<T>::bad(a[i]);
                else
                    any_bad |= F<T>::bad(a[i], b[i]);
            }
        }
        dh_store_vec_stream<T, VEC>(res + r * ld_res + c, o);
    }
    if constexpr (F<T>::checks) {
        if (any_bad)
            *flag = 1;
    }
}

static __global__ void set_flag_kernel(int *flag, int v) { *flag = v; }

// Checked unary operator on a small matrix (a vector of column statistics, say): one workgroup computes the results
// and sets the flag to whether any argument lay outside the domain - no separate launch to clear the flag first.
constexpr size_t EW_SMALL_CHECKED = 4096; // elements
template <typename T, template <typename> class F>
__global__ __launch_bounds__(EW_THREADS) void ew_unary_small_checked_kernel(T *res, size_t ld_res, const T *arg, size_t ld_arg,
                                                                            unsigned rows, unsigned cols, int *flag) {
    static_assert(F<T>::checks, "only for operators with a domain");
    int any_bad = 0;
    for (unsigned i = threadIdx.x; i < rows * cols; i += EW_THREADS) {
        const unsigned r = i / cols, c = i % cols;
        const T a = arg[static_cast<size_t>(r) * ld_arg + c];
        any_bad |= F<T>::bad(a) ? 1 : 0;
        res[static_cast<size_t>(r) * ld_res + c] = F<T>::apply(a, T(0));
    }
    const int any = __syncthreads_or(any_bad);
    if (threadIdx.x == 0)
        *flag = any ? 1 : 0;
}

// C++ names of the value types as the reference prints them (ValueTypeUtils::cppNameFor)
template <typename T> static inline const char *type_name();
template <> inline const char *type_name<float>() { return "float"; }
template <> inline const char *type_name<double>() { return "double"; }
template <> inline const char *type_name<int>() { return "int32_t"; }
template <> inline const char *type_name<unsigned>() { return "uint32_t"; }
template <> inline const char *type_name<long>() { return "int64_t"; }
template <> inline const char *type_name<unsigned long>() { return "uint64_t"; }

// ---------------------------------------------------------------------------------------
// host-side launch
// ---------------------------------------------------------------------------------------
struct Shape {
    size_t rows, cvecs;
    dim3 grid, block;
};

// Picks the (TX, TY) thread tile and the grid for `rows` x `cvecs` vectors.
static inline Shape plan(const dh_ctx *ctx, size_t rows, size_t cvecs) {
    unsigned tx = 1;
    while (tx < EW_THREADS && tx < cvecs)
        tx <<= 1;
    unsigned ty = EW_THREADS / tx;
    size_t gy = dh_ceil_div(cvecs, tx);
    if (gy > 65535)
        gy = 65535; // the kernel strides over the remaining column vectors
    size_t gx = dh_ceil_div(rows, static_cast<size_t>(ty));
    if (gx < 1)
        gx = 1;
    (void)ctx;
    Shape s;
    s.rows = rows;
    s.cvecs = cvecs;
    s.grid = dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy), 1);
    s.block = dim3(tx, ty, 1);
    return s;
}

template <typename T, int VEC, template <typename> class F, int MODE>
static inline void launch2d(dh_ctx *ctx, T *res, size_t ld_res, const T *lhs, size_t ld_lhs, const T *rhs,
                            size_t ld_rhs, T sca, size_t rows, size_t cols, int *flag) {
    if (rows == 0 || cols == 0)
        return;
    Shape s = plan(ctx, rows, cols / VEC);
    hipLaunchKernelGGL((ew_kernel<T, VEC, F, MODE>), s.grid, s.block, 0, ctx->stream, res, ld_res, lhs, ld_lhs, rhs,
                       ld_rhs, sca, rows, cols / VEC, flag);
}

// Dispatch on layout: flat view for contiguous elementwise-only modes, vector width by alignment.
template <typename T, template <typename> class F, int MODE>
static inline void launch(dh_ctx *ctx, T *res, size_t ld_res, const T *lhs, size_t ld_lhs, const T *rhs,
                          size_t ld_rhs, T sca, size_t rows, size_t cols, int *flag) {
    constexpr int V = dh_vec<T>::N;
    if (rows == 0 || cols == 0)
        return;
    const bool flat_mode = (MODE == SAME || MODE == SCALAR || MODE == UNARY);
    const bool contiguous = (rows == 1) || (ld_res == cols && ld_lhs == cols && (MODE != SAME || ld_rhs == cols));
    if (flat_mode && contiguous) {
        const size_t n = rows * cols;
        const bool al = dh_aligned(res, 16) && dh_aligned(lhs, 16) && (MODE != SAME || dh_aligned(rhs, 16));
        const size_t width = static_cast<size_t>(EW_THREADS) * V; // elements per virtual row
        size_t body_rows = al ? n / width : 0;
        if (body_rows)
            launch2d<T, V, F, MODE>(ctx, res, width, lhs, width, rhs, width, sca, body_rows, width, flag);
        const size_t done = body_rows * width;
        if (done < n)
            launch2d<T, 1, F, MODE>(ctx, res + done, n - done, lhs + done, n - done,
                                    MODE == SAME ? rhs + done : rhs, n - done, sca, 1, n - done, flag);
        return;
    }
    bool vec_ok = (cols % V == 0) && (ld_res % V == 0) && (ld_lhs % V == 0) && dh_aligned(res, 16) &&
                  dh_aligned(lhs, 16);
    if (MODE == SAME)
        vec_ok = vec_ok && (ld_rhs % V == 0) && dh_aligned(rhs, 16);
    if (MODE == ROWVEC)
        vec_ok = vec_ok && dh_aligned(rhs, 16);
    if (vec_ok)
        launch2d<T, V, F, MODE>(ctx, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, sca, rows, cols, flag);
    else
        launch2d<T, 1, F, MODE>(ctx, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, sca, rows, cols, flag);
}

template <typename T, int MODE>
static inline dh_status dispatch_binary(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *lhs, size_t ld_lhs,
                                        const T *rhs, size_t ld_rhs, T sca, size_t rows, size_t cols) {
    // integer DIV and MOD report operands that have no integer result (see ew_ops.h) through the context's flag
    const bool checks = dh_is_int<T>::value && (op == DH_BIN_DIV || op == DH_BIN_MOD);
    if (checks)
        hipLaunchKernelGGL(set_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev, 0);
#define DH_CASE(CODE, FUN)                                                                         \
    case CODE:                                                                                     \
        launch<T, FUN, MODE>(ctx, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, sca, rows, cols, ctx->flag_dev); \
        break;
    switch (op) {
        DH_CASE(DH_BIN_ADD, BAdd)
        DH_CASE(DH_BIN_SUB, BSub)
        DH_CASE(DH_BIN_MUL, BMul)
        DH_CASE(DH_BIN_DIV, BDiv)
        DH_CASE(DH_BIN_POW, BPow)
        DH_CASE(DH_BIN_MOD, BMod)
        DH_CASE(DH_BIN_LOG, BLog)
        DH_CASE(DH_BIN_EQ, BEq)
        DH_CASE(DH_BIN_NEQ, BNeq)
        DH_CASE(DH_BIN_LT, BLt)
        DH_CASE(DH_BIN_LE, BLe)
        DH_CASE(DH_BIN_GT, BGt)
        DH_CASE(DH_BIN_GE, BGe)
        DH_CASE(DH_BIN_MIN, BMin)
        DH_CASE(DH_BIN_MAX, BMax)
        DH_CASE(DH_BIN_AND, BAnd)
        DH_CASE(DH_BIN_OR, BOr)
    case DH_BIN_BITWISE_AND:
    case DH_BIN_CONCAT:
        // EwBinarySca.h:75-77: the op exists but is not supported on these value types.
        return dh_fail(DH_ERR_RUNTIME, "the binary operation %s is not supported on the value types %s (res), %s (lhs), and %s (rhs)",
                       op == DH_BIN_CONCAT ? "CONCAT" : "BITWISE_AND", type_name<T>(), type_name<T>(), type_name<T>());
    default:
        // EwBinarySca.h:73
        return dh_fail(DH_ERR_RUNTIME, "unknown BinaryOpCode: %d", op);
    }
#undef DH_CASE
    DH_CHECK_LAUNCH();
    if (checks) {
        if (ctx->deferred_depth > 0) // the verdict waits for dh_check_deferred
            return dh_latch_deferred(ctx, 0, DH_DEFERRED_INT_DIVMOD, op, nullptr, 0, 0);
        DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        if (*ctx->flag_host != 0)
            return dh_fail_int_divmod(op);
    }
    return DH_OK;
}

template <typename T>
dh_status ew_binary(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs,
                    const T *rhs, size_t rr, size_t rc, size_t ld_rhs) {
    DH_REQUIRE_CTX(ctx);
    if (ld_res < lc || ld_lhs < lc || ld_rhs < rc)
        return dh_fail(DH_ERR_RUNTIME, "EwBinaryMat(Dense) - a leading dimension is smaller than its column count");
    // Case order and conditions of kernels/EwBinaryMat.h:72-106; the result always has lhs' shape.
    if (lr == rr && lc == rc)
        return dispatch_binary<T, SAME>(ctx, op, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, T(0), lr, lc);
    if (lc == rc && (rr == 1 || lr == 1))
        return dispatch_binary<T, ROWVEC>(ctx, op, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, T(0), lr, lc);
    if (lr == rr && (rc == 1 || lc == 1))
        return dispatch_binary<T, COLVEC>(ctx, op, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, T(0), lr, lc);
    return dh_fail(DH_ERR_RUNTIME,
                   "EwBinaryMat(Dense) - lhs and rhs must either have the same dimensions, or one of them must be a "
                   "row/column vector with the width/height of the other, but lhs has shape (%zu x %zu) and rhs has "
                   "shape (%zu x %zu)",
                   lr, lc, rr, rc);
}

template <typename T>
dh_status ew_binary_sca(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *lhs, size_t rows, size_t cols,
                        size_t ld_lhs, T rhs) {
    DH_REQUIRE_CTX(ctx);
    if (ld_res < cols || ld_lhs < cols)
        return dh_fail(DH_ERR_RUNTIME, "EwBinaryObjSca - a leading dimension is smaller than the column count");
    return dispatch_binary<T, SCALAR>(ctx, op, res, ld_res, lhs, ld_lhs, nullptr, 0, rhs, rows, cols);
}

template <typename T>
dh_status ew_unary(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,
                   size_t ld_arg) {
    DH_REQUIRE_CTX(ctx);
    if (ld_res < cols || ld_arg < cols)
        return dh_fail(DH_ERR_RUNTIME, "EwUnaryMat - a leading dimension is smaller than the column count");
    const bool checks = (op == DH_UN_SQRT || op == DH_UN_LN || op == DH_UN_ASIN || op == DH_UN_ACOS);
    const bool small_checked = checks && rows * cols <= EW_SMALL_CHECKED && rows * cols > 0;
    if (small_checked) {
#define DH_SMALL(FUN)                                                                                                   \
    hipLaunchKernelGGL((ew_unary_small_checked_kernel<T, FUN>), dim3(1), dim3(EW_THREADS), 0, ctx->stream, res, ld_res, arg, ld_arg, \
                       static_cast<unsigned>(rows), static_cast<unsigned>(cols), ctx->flag_dev)
        if (op == DH_UN_SQRT)
            DH_SMALL(USqrt);
        else if (op == DH_UN_LN)
            DH_SMALL(ULn);
        else if (op == DH_UN_ASIN)
            DH_SMALL(UAsin);
        else
            DH_SMALL(UAcos);
#undef DH_SMALL
    } else if (checks) {
        hipLaunchKernelGGL(set_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev, 0);
    }
#define DH_CASE(CODE, FUN)                                                                         \
    case CODE:                                                                                     \
        launch<T, FUN, UNARY>(ctx, res, ld_res, arg, ld_arg, nullptr, 0, T(0), rows, cols, ctx->flag_dev); \
        break;
    switch (small_checked ? -1 : op) {
    case -1: // done above
        break;
        DH_CASE(DH_UN_MINUS, UMinus)
        DH_CASE(DH_UN_ABS, UAbs)
        DH_CASE(DH_UN_SIGN, USign)
        DH_CASE(DH_UN_SQRT, USqrt)
        DH_CASE(DH_UN_EXP, UExp)
        DH_CASE(DH_UN_LN, ULn)
        DH_CASE(DH_UN_SIN, USin)
        DH_CASE(DH_UN_COS, UCos)
        DH_CASE(DH_UN_TAN, UTan)
        DH_CASE(DH_UN_ASIN, UAsin)
        DH_CASE(DH_UN_ACOS, UAcos)
        DH_CASE(DH_UN_ATAN, UAtan)
        DH_CASE(DH_UN_SINH, USinh)
        DH_CASE(DH_UN_COSH, UCosh)
        DH_CASE(DH_UN_TANH, UTanh)
        DH_CASE(DH_UN_FLOOR, UFloor)
        DH_CASE(DH_UN_CEIL, UCeil)
        DH_CASE(DH_UN_ROUND, URound)
        DH_CASE(DH_UN_ISNAN, UIsNan)
    case DH_UN_UPPER:
    case DH_UN_LOWER:
        // EwUnarySca.h:104-107
        return dh_fail(DH_ERR_RUNTIME, "the unary operation %s is not supported on the value types %s (res) and %s(arg)",
                       op == DH_UN_UPPER ? "UPPER" : "LOWER", type_name<T>(), type_name<T>());
    default:
        // EwUnarySca.h:102
        return dh_fail(DH_ERR_RUNTIME, "unknown UnaryOpCode: %d", op);
    }
#undef DH_CASE
    DH_CHECK_LAUNCH();
    if (checks) {
        if (ctx->deferred_depth > 0) // the verdict waits for dh_check_deferred
            return dh_latch_deferred(ctx, 0, DH_DEFERRED_UNARY_DOMAIN, op, nullptr, 0, 0);
        DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        if (*ctx->flag_host != 0)
            return dh_fail_unary_domain(op);
    }
    return DH_OK;
}

} // namespace dh_ew
