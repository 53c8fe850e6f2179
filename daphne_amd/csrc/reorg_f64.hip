#include "reorg_impl.h"

extern "C" dh_status dh_fill_f64(dh_ctx *ctx, double *res, size_t ld_res, double value, size_t rows, size_t cols) {
    return dh_reorg::fill<double>(ctx, res, ld_res, value, rows, cols);
}
extern "C" dh_status dh_col_bind_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *lhs, size_t lhs_rows, size_t lhs_cols,
                                     size_t ld_lhs, const double *rhs, size_t rhs_rows, size_t rhs_cols, size_t ld_rhs) {
    return dh_reorg::col_bind<double>(ctx, res, ld_res, lhs, lhs_rows, lhs_cols, ld_lhs, rhs, rhs_rows, rhs_cols, ld_rhs);
}
extern "C" dh_status dh_extract_col_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows, size_t cols,
                                        size_t ld, const int64_t *sel, size_t sel_rows, size_t sel_cols, size_t ld_sel) {
    return dh_reorg::extract_col<double>(ctx, res, ld_res, arg, rows, cols, ld, reinterpret_cast<const long long *>(sel),
                                        sel_rows, sel_cols, ld_sel);
}
extern "C" dh_status dh_transpose_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows, size_t cols,
                                      size_t ld) {
    return dh_reorg::transpose<double>(ctx, res, ld_res, arg, rows, cols, ld);
}
