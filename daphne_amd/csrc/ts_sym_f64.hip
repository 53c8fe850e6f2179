// Symmetric tall-skinny product and the normal equations, double instantiation. See ts_sym_impl.h for the design.
#include "ts_sym_impl.h"

template bool dh_gemm::ts_sym<double>(dh_ctx *, size_t, size_t, const double *, size_t, const double *, size_t, double *, size_t, double *, size_t,
                                  double, dh_status *);

namespace {
__global__ void add_diagonal_kernel(double *C, size_t ldc, unsigned m, double lambda) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m)
        C[static_cast<size_t>(i) * ldc + i] += lambda;
}
} // namespace

// A = t(X) X + lambda I, b = t(X) y: lmDS's normal equations (scripts/algorithms/lmDS_.daph:60-75:
// A = syrk(X) + diagMatrix(lambda), b = t(X) @ y). Fused where the shape fits, otherwise the operator sequence.
extern "C" dh_status dh_normal_equations_f64(dh_ctx *ctx, double *A, size_t lda, double *b, size_t ldb, const double *X, size_t rows,
                                              size_t cols, size_t ldx, const double *y, size_t ldy, double lambda) {
    DH_REQUIRE_CTX(ctx);
    if (ldx < cols || lda < cols || ldb < 1 || ldy < 1)
        return dh_fail(DH_ERR_RUNTIME, "normalEquations - a leading dimension is smaller than its column count");
    if (cols == 0)
        return DH_OK;
    dh_status st = DH_OK;
    if (rows > 0 && dh_gemm::ts_sym<double>(ctx, cols, rows, X, ldx, y, ldy, A, lda, b, ldb, lambda, &st)) {
        if (st == DH_OK)
            DH_CHECK_LAUNCH();
        return st;
    }
    st = dh_syrk_f64(ctx, A, lda, X, rows, cols, ldx, 1);
    if (st != DH_OK)
        return st;
    hipLaunchKernelGGL(add_diagonal_kernel, dim3(static_cast<unsigned>((cols + 255) / 256)), dim3(256), 0, ctx->stream, A, lda,
                       static_cast<unsigned>(cols), lambda);
    DH_CHECK_LAUNCH();
    return dh_gemv_f64(ctx, b, ldb, X, rows, cols, ldx, y, rows, ldy);
}
