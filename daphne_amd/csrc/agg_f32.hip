// Aggregation kernels, float instantiation. See agg_impl.h for the design and reference citations.
#include "agg_impl.h"

extern "C" dh_status dh_agg_all_f32(dh_ctx *ctx, int op, const float *arg, size_t rows, size_t cols, size_t ld,
                                   float *result_host) {
    return dh_agg::agg_all<float>(ctx, op, arg, rows, cols, ld, result_host);
}
extern "C" dh_status dh_agg_all_dev_f32(dh_ctx *ctx, int op, const float *arg, size_t rows, size_t cols, size_t ld,
                                       float *result_dev) {
    return dh_agg::agg_all_dev<float>(ctx, op, arg, rows, cols, ld, result_dev);
}
extern "C" dh_status dh_agg_row_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *arg, size_t rows,
                                   size_t cols, size_t ld) {
    return dh_agg::agg_row<float>(ctx, op, res, ld_res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_row_idx_f32(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const float *arg,
                                       size_t rows, size_t cols, size_t ld) {
    return dh_agg::agg_row_idx<float>(ctx, op, res, ld_res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_col_f32(dh_ctx *ctx, int op, float *res, const float *arg, size_t rows, size_t cols,
                                   size_t ld) {
    return dh_agg::agg_col<float>(ctx, op, res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_col_idx_f32(dh_ctx *ctx, int op, uint64_t *res, const float *arg, size_t rows,
                                       size_t cols, size_t ld) {
    return dh_agg::agg_col_idx<float>(ctx, op, res, arg, rows, cols, ld);
}

extern "C" dh_status dh_agg_col_moments_f32(dh_ctx *ctx, float *res_mean, float *res_var, int stddev, const float *arg, size_t rows,
                                             size_t cols, size_t ld) {
    return dh_agg::agg_col_moments<float>(ctx, res_mean, res_var, stddev, arg, rows, cols, ld);
}
