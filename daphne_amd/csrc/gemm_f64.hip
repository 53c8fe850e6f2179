// MatMul / Syrk / Affine, double instantiation. See gemm_impl.h for the design and reference citations.
#include "gemm_impl.h"

extern "C" dh_status dh_matmul_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *lhs, size_t lhs_rows,
                                  size_t lhs_cols, size_t ld_lhs, const double *rhs, size_t rhs_rows, size_t rhs_cols,
                                  size_t ld_rhs, int transa, int transb) {
    return dh_gemm::matmul<double>(ctx, res, ld_res, lhs, lhs_rows, lhs_cols, ld_lhs, rhs, rhs_rows, rhs_cols, ld_rhs,
                               transa, transb);
}

extern "C" dh_status dh_syrk_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows, size_t cols,
                                size_t ld, int trans_left) {
    return dh_gemm::syrk<double>(ctx, res, ld_res, arg, rows, cols, ld, trans_left);
}

extern "C" dh_status dh_affine_forward_f64(dh_ctx *ctx, double *res, const double *data, size_t data_rows, size_t data_cols,
                                          const double *weights, size_t w_rows, size_t w_cols, const double *bias,
                                          size_t bias_rows, size_t bias_cols) {
    return dh_gemm::affine<double>(ctx, res, data, data_rows, data_cols, weights, w_rows, w_cols, bias, bias_rows,
                               bias_cols);
}

extern "C" dh_status dh_affine_forward_fused_f64(dh_ctx *ctx, double *res, const double *data, size_t data_rows, size_t data_cols,
                                                const double *weights, size_t w_rows, size_t w_cols, const double *bias,
                                                size_t bias_rows, size_t bias_cols, unsigned epilogue) {
    return dh_gemm::affine<double>(ctx, res, data, data_rows, data_cols, weights, w_rows, w_cols, bias, bias_rows,
                               bias_cols, epilogue);
}

// Gemv<DenseMatrix<T>,...>::apply (kernels/Gemv.h:51-77, kernels/CUDA/Gemv.cpp:42-68): res = t(mat) vec.
extern "C" dh_status dh_gemv_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *mat, size_t rows, size_t cols, size_t ld_mat,
                                  const double *vec, size_t vec_rows, size_t ld_vec) {
    DH_REQUIRE_CTX(ctx);
    if (vec_rows != rows)
        return dh_fail(DH_ERR_RUNTIME, "Gemv - #rows of mat and #rows of vec must be the same, but got %zu and %zu", rows,
                       vec_rows);
    if (ld_mat < cols || ld_res < 1 || ld_vec < 1)
        return dh_fail(DH_ERR_RUNTIME, "Gemv - a leading dimension is smaller than its column count");
    return dh_gemm::gemv<double>(ctx, true, rows, cols, mat, ld_mat, vec, ld_vec, res, ld_res);
}
