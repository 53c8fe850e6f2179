#include "reorg_impl.h"

extern "C" dh_status dh_fill_f32(dh_ctx *ctx, float *res, size_t ld_res, float value, size_t rows, size_t cols) {
    return dh_reorg::fill<float>(ctx, res, ld_res, value, rows, cols);
}
extern "C" dh_status dh_col_bind_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *lhs, size_t lhs_rows, size_t lhs_cols,
                                     size_t ld_lhs, const float *rhs, size_t rhs_rows, size_t rhs_cols, size_t ld_rhs) {
    return dh_reorg::col_bind<float>(ctx, res, ld_res, lhs, lhs_rows, lhs_cols, ld_lhs, rhs, rhs_rows, rhs_cols, ld_rhs);
}
extern "C" dh_status dh_extract_col_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows, size_t cols,
                                        size_t ld, const int64_t *sel, size_t sel_rows, size_t sel_cols, size_t ld_sel) {
    return dh_reorg::extract_col<float>(ctx, res, ld_res, arg, rows, cols, ld, reinterpret_cast<const long long *>(sel),
                                        sel_rows, sel_cols, ld_sel);
}
extern "C" dh_status dh_transpose_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows, size_t cols,
                                      size_t ld) {
    return dh_reorg::transpose<float>(ctx, res, ld_res, arg, rows, cols, ld);
}
