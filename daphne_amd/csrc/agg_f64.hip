// Aggregation kernels, double instantiation. See agg_impl.h for the design and reference citations.
#include "agg_impl.h"

extern "C" dh_status dh_agg_all_f64(dh_ctx *ctx, int op, const double *arg, size_t rows, size_t cols, size_t ld,
                                   double *result_host) {
    return dh_agg::agg_all<double>(ctx, op, arg, rows, cols, ld, result_host);
}
extern "C" dh_status dh_agg_all_dev_f64(dh_ctx *ctx, int op, const double *arg, size_t rows, size_t cols, size_t ld,
                                       double *result_dev) {
    return dh_agg::agg_all_dev<double>(ctx, op, arg, rows, cols, ld, result_dev);
}
extern "C" dh_status dh_agg_row_f64(dh_ctx *ctx, int op, double *res, size_t ld_res, const double *arg, size_t rows,
                                   size_t cols, size_t ld) {
    return dh_agg::agg_row<double>(ctx, op, res, ld_res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_row_idx_f64(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const double *arg,
                                       size_t rows, size_t cols, size_t ld) {
    return dh_agg::agg_row_idx<double>(ctx, op, res, ld_res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_col_f64(dh_ctx *ctx, int op, double *res, const double *arg, size_t rows, size_t cols,
                                   size_t ld) {
    return dh_agg::agg_col<double>(ctx, op, res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_col_idx_f64(dh_ctx *ctx, int op, uint64_t *res, const double *arg, size_t rows,
                                       size_t cols, size_t ld) {
    return dh_agg::agg_col_idx<double>(ctx, op, res, arg, rows, cols, ld);
}

extern "C" dh_status dh_agg_col_moments_f64(dh_ctx *ctx, double *res_mean, double *res_var, int stddev, const double *arg, size_t rows,
                                             size_t cols, size_t ld) {
    return dh_agg::agg_col_moments<double>(ctx, res_mean, res_var, stddev, arg, rows, cols, ld);
}
