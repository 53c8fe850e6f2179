// Symmetric tall-skinny product and the normal equations, float instantiation. See ts_sym_impl.h for the design.
#include "ts_sym_impl.h"

template bool dh_gemm::ts_sym<float>(dh_ctx *, size_t, size_t, const float *, size_t, const float *, size_t, float *, size_t, float *, size_t,
                                  float, dh_status *);

namespace {
__global__ void add_diagonal_kernel(float *C, size_t ldc, unsigned m, float lambda) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m)
        C[static_cast<size_t>(i) * ldc + i] += lambda;
}
} // namespace

// A = t(X) X + lambda I, b = t(X) y: lmDS's normal equations (scripts/algorithms/lmDS_.daph:60-75:
// A = syrk(X) + diagMatrix(lambda), b = t(X) @ y). Fused where the shape fits, otherwise the operator sequence.
extern "C" dh_status dh_normal_equations_f32(dh_ctx *ctx, float *A, size_t lda, float *b, size_t ldb, const float *X, size_t rows,
                                              size_t cols, size_t ldx, const float *y, size_t ldy, float lambda) {
    DH_REQUIRE_CTX(ctx);
    if (ldx < cols || lda < cols || ldb < 1 || ldy < 1)
        return dh_fail(DH_ERR_RUNTIME, "normalEquations - a leading dimension is smaller than its column count");
    if (cols == 0)
        return DH_OK;
    dh_status st = DH_OK;
    if (rows > 0 && dh_gemm::ts_sym<float>(ctx, cols, rows, X, ldx, y, ldy, A, lda, b, ldb, lambda, &st)) {
        if (st == DH_OK)
            DH_CHECK_LAUNCH();
        return st;
    }
    st = dh_syrk_f32(ctx, A, lda, X, rows, cols, ldx, 1);
    if (st != DH_OK)
        return st;
    hipLaunchKernelGGL(add_diagonal_kernel, dim3(static_cast<unsigned>((cols + 255) / 256)), dim3(256), 0, ctx->stream, A, lda,
                       static_cast<unsigned>(cols), lambda);
    DH_CHECK_LAUNCH();
    return dh_gemv_f32(ctx, b, ldb, X, rows, cols, ldx, y, rows, ldy);
}
