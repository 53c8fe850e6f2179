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
// column vectors of a row, TY rows are covered per block step, and each thread keeps UNROLL
// independent rows in flight so that a wavefront has several KiB of loads outstanding. A
// row-vector operand is loaded once per thread before the row loop; a column-vector operand is
// one scalar per row; no integer division or modulo is executed per element. Contiguous
// same-shape / scalar / unary inputs are viewed as a matrix that is one block-row (256 vectors)
// wide, which turns the flat array into the same 2-D walk.
#pragma once

#include "common.h"

#include <cmath>
#include <limits>

namespace dh_ew {

// ---------------------------------------------------------------------------------------
// scalar functors (op codes of BinaryOpCode.h:29-55 / UnaryOpCode.h:28-55)
// ---------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ T dh_pow(T a, T b);
template <> __device__ __forceinline__ float dh_pow<float>(float a, float b) { return powf(a, b); }
template <> __device__ __forceinline__ double dh_pow<double>(double a, double b) { return pow(a, b); }
template <typename T> __device__ __forceinline__ T dh_fmod(T a, T b);
template <> __device__ __forceinline__ float dh_fmod<float>(float a, float b) { return fmodf(a, b); }
template <> __device__ __forceinline__ double dh_fmod<double>(double a, double b) { return fmod(a, b); }
template <typename T> __device__ __forceinline__ T dh_log(T a);
template <> __device__ __forceinline__ float dh_log<float>(float a) { return logf(a); }
template <> __device__ __forceinline__ double dh_log<double>(double a) { return log(a); }

#define DH_BIN_FUNCTOR(NAME, EXPR)                                                                 \
    template <typename T> struct NAME {                                                            \
        static __device__ __forceinline__ T apply(T a, T b) { return EXPR; }                       \
    };
DH_BIN_FUNCTOR(BAdd, a + b)
DH_BIN_FUNCTOR(BSub, a - b)
DH_BIN_FUNCTOR(BMul, a *b)
DH_BIN_FUNCTOR(BDiv, a / b) // IEEE division, as the CPU kernel; the CUDA kernel multiplies by 1/b
DH_BIN_FUNCTOR(BPow, dh_pow<T>(a, b))
DH_BIN_FUNCTOR(BMod, dh_fmod<T>(a, b))
DH_BIN_FUNCTOR(BLog, dh_log<T>(a) / dh_log<T>(b))
DH_BIN_FUNCTOR(BEq, static_cast<T>(a == b))
DH_BIN_FUNCTOR(BNeq, static_cast<T>(a != b))
DH_BIN_FUNCTOR(BLt, static_cast<T>(a < b))
DH_BIN_FUNCTOR(BLe, static_cast<T>(a <= b))
DH_BIN_FUNCTOR(BGt, static_cast<T>(a > b))
DH_BIN_FUNCTOR(BGe, static_cast<T>(a >= b))
DH_BIN_FUNCTOR(BMin, (b < a) ? b : a) // std::min(a, b): NaN in b never wins, NaN in a stays
DH_BIN_FUNCTOR(BMax, (a < b) ? b : a) // std::max(a, b)
DH_BIN_FUNCTOR(BAnd, static_cast<T>((a != T(0)) && (b != T(0))))
DH_BIN_FUNCTOR(BOr, static_cast<T>((a != T(0)) || (b != T(0))))
#undef DH_BIN_FUNCTOR

// Unary functors also expose bad(a): true where the CPU kernel throws std::domain_error.
#define DH_UN_FUNCTOR(NAME, EXPR, BAD)                                                             \
    template <typename T> struct NAME {                                                            \
        static constexpr bool checks = !(#BAD[0] == 'f');                                          \
        static __device__ __forceinline__ T apply(T a, T) { return EXPR; }                         \
        static __device__ __forceinline__ bool bad(T a) { return BAD; }                            \
    };
template <typename T> __device__ __forceinline__ T dh_sign(T a) {
    return (a == T(0)) ? T(0) : ((a < T(0)) ? T(-1) : ((a > T(0)) ? T(1) : std::numeric_limits<T>::quiet_NaN()));
}
#define DH_MATH1(FN)                                                                               \
    template <typename T> __device__ __forceinline__ T dh_##FN(T a);                               \
    template <> __device__ __forceinline__ float dh_##FN<float>(float a) { return FN##f(a); }      \
    template <> __device__ __forceinline__ double dh_##FN<double>(double a) { return FN(a); }
DH_MATH1(sqrt)
DH_MATH1(exp)
DH_MATH1(sin)
DH_MATH1(cos)
DH_MATH1(tan)
DH_MATH1(asin)
DH_MATH1(acos)
DH_MATH1(atan)
DH_MATH1(sinh)
DH_MATH1(cosh)
DH_MATH1(tanh)
DH_MATH1(floor)
DH_MATH1(ceil)
DH_MATH1(round)
DH_MATH1(fabs)
#undef DH_MATH1

DH_UN_FUNCTOR(UMinus, -a, false)
DH_UN_FUNCTOR(UAbs, dh_fabs<T>(a), false)
DH_UN_FUNCTOR(USign, dh_sign<T>(a), false)
DH_UN_FUNCTOR(USqrt, dh_sqrt<T>(a), (T(-0.0) > a))
DH_UN_FUNCTOR(UExp, dh_exp<T>(a), false)
DH_UN_FUNCTOR(ULn, dh_log<T>(a), (T(-0.0) > a))
DH_UN_FUNCTOR(USin, dh_sin<T>(a), false)
DH_UN_FUNCTOR(UCos, dh_cos<T>(a), false)
DH_UN_FUNCTOR(UTan, dh_tan<T>(a), false)
DH_UN_FUNCTOR(UAsin, dh_asin<T>(a), (T(-1.0) > a || a > T(1.0)))
DH_UN_FUNCTOR(UAcos, dh_acos<T>(a), (T(-1.0) > a || a > T(1.0)))
DH_UN_FUNCTOR(UAtan, dh_atan<T>(a), false)
DH_UN_FUNCTOR(USinh, dh_sinh<T>(a), false)
DH_UN_FUNCTOR(UCosh, dh_cosh<T>(a), false)
DH_UN_FUNCTOR(UTanh, dh_tanh<T>(a), false)
DH_UN_FUNCTOR(UFloor, dh_floor<T>(a), false)
DH_UN_FUNCTOR(UCeil, dh_ceil<T>(a), false)
DH_UN_FUNCTOR(URound, dh_round<T>(a), false)
DH_UN_FUNCTOR(UIsNan, static_cast<T>(a != a), false)
#undef DH_UN_FUNCTOR

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
constexpr int EW_UNROLL = 4;

template <typename T, int VEC, template <typename> class F, int MODE>
__global__ __launch_bounds__(EW_THREADS) void ew_kernel(T *res, size_t ld_res, const T *lhs, size_t ld_lhs,
                                                        const T *rhs, size_t ld_rhs, T sca, size_t rows,
                                                        size_t cvecs, int *flag) {
    const size_t row_step = static_cast<size_t>(gridDim.x) * blockDim.y;
    bool any_bad = false;
    for (size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x; cv < cvecs;
         cv += static_cast<size_t>(gridDim.y) * blockDim.x) {
        const size_t c = cv * VEC;
        Pack<T, VEC> rv;
        if constexpr (MODE == ROWVEC)
            rv = load_pack<T, VEC>(rhs + c);
        if constexpr (MODE == SCALAR) {
#pragma unroll
            for (int i = 0; i < VEC; i++)
                rv.v[i] = sca;
        }
        for (size_t r0 = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y; r0 < rows;
             r0 += row_step * EW_UNROLL) {
            Pack<T, VEC> a[EW_UNROLL], b[EW_UNROLL];
#pragma unroll
            for (int u = 0; u < EW_UNROLL; u++) {
                const size_t r = r0 + u * row_step;
                if (r < rows) {
                    a[u] = load_pack<T, VEC>(lhs + r * ld_lhs + c);
                    if constexpr (MODE == SAME)
                        b[u] = load_pack<T, VEC>(rhs + r * ld_rhs + c);
                    if constexpr (MODE == COLVEC) {
                        const T s = rhs[r * ld_rhs];
#pragma unroll
                        for (int i = 0; i < VEC; i++)
                            b[u].v[i] = s;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < EW_UNROLL; u++) {
                const size_t r = r0 + u * row_step;
                if (r < rows) {
                    Pack<T, VEC> o;
#pragma unroll
                    for (int i = 0; i < VEC; i++) {
                        T bb;
                        if constexpr (MODE == SAME || MODE == COLVEC)
                            bb = b[u].v[i];
                        else if constexpr (MODE == UNARY)
                            bb = T(0);
                        else
                            bb = rv.v[i];
                        o.v[i] = F<T>::apply(a[u].v[i], bb);
                        if constexpr (MODE == UNARY) {
                            if constexpr (F<T>::checks)
                                any_bad |= F<T>::bad(a[u].v[i]);
                        }
                    }
                    store_pack<T, VEC>(res + r * ld_res + c, o);
                }
            }
        }
    }
    if constexpr (MODE == UNARY) {
        if constexpr (F<T>::checks) {
            if (any_bad)
                *flag = 1;
        }
    }
}

static __global__ void set_flag_kernel(int *flag, int v) { *flag = v; }

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
    if (gy > 1024)
        gy = 1024;
    const size_t max_blocks = static_cast<size_t>(ctx->num_cus) * 16;
    size_t gx = dh_ceil_div(rows, static_cast<size_t>(ty) * EW_UNROLL);
    size_t cap = max_blocks / gy;
    if (cap < 1)
        cap = 1;
    if (gx > cap)
        gx = cap;
    if (gx < 1)
        gx = 1;
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
#define DH_CASE(CODE, FUN)                                                                         \
    case CODE:                                                                                     \
        launch<T, FUN, MODE>(ctx, res, ld_res, lhs, ld_lhs, rhs, ld_rhs, sca, rows, cols, nullptr); \
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
                       op == DH_BIN_CONCAT ? "CONCAT" : "BITWISE_AND", sizeof(T) == 4 ? "float" : "double",
                       sizeof(T) == 4 ? "float" : "double", sizeof(T) == 4 ? "float" : "double");
    default:
        // EwBinarySca.h:73
        return dh_fail(DH_ERR_RUNTIME, "unknown BinaryOpCode: %d", op);
    }
#undef DH_CASE
    DH_CHECK_LAUNCH();
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
    if (checks) {
        hipLaunchKernelGGL(set_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev, 0);
    }
#define DH_CASE(CODE, FUN)                                                                         \
    case CODE:                                                                                     \
        launch<T, FUN, UNARY>(ctx, res, ld_res, arg, ld_arg, nullptr, 0, T(0), rows, cols, ctx->flag_dev); \
        break;
    switch (op) {
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
                       op == DH_UN_UPPER ? "UPPER" : "LOWER", sizeof(T) == 4 ? "float" : "double",
                       sizeof(T) == 4 ? "float" : "double");
    default:
        // EwUnarySca.h:102
        return dh_fail(DH_ERR_RUNTIME, "unknown UnaryOpCode: %d", op);
    }
#undef DH_CASE
    DH_CHECK_LAUNCH();
    if (checks) {
        DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        if (*ctx->flag_host != 0) {
            const char *dom = op == DH_UN_SQRT   ? "SQRT with domain [-0, inf]"
                              : op == DH_UN_LN   ? "LN with domain [-0, inf]"
                              : op == DH_UN_ASIN ? "ASIN with domain [-1, 1]"
                                                 : "ACOS with domain [-1, 1]";
            return dh_fail(DH_ERR_DOMAIN, "invalid argument passed to unary func %s", dom);
        }
    }
    return DH_OK;
}

} // namespace dh_ew
