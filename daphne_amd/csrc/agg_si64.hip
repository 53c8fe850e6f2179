// Aggregation kernels, signed 64-bit integer instantiation (the reference: kernels/CUDA/AggAll.cu:155, AggRow.cu:146,
// AggCol.cu:89). SUM / PROD / MIN / MAX and the index aggregations; sums wrap like the host's two's-complement adds.
// See agg_impl.h for the design.
#include "agg_impl.h"

extern "C" dh_status dh_agg_all_si64(dh_ctx *ctx, int op, const int64_t *arg, size_t rows, size_t cols, size_t ld,
                                    int64_t *result_host) {
    return dh_agg::agg_all<int64_t>(ctx, op, arg, rows, cols, ld, result_host);
}
extern "C" dh_status dh_agg_row_si64(dh_ctx *ctx, int op, int64_t *res, size_t ld_res, const int64_t *arg, size_t rows,
                                    size_t cols, size_t ld) {
    return dh_agg::agg_row<int64_t>(ctx, op, res, ld_res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_row_idx_si64(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const int64_t *arg,
                                        size_t rows, size_t cols, size_t ld) {
    return dh_agg::agg_row_idx<int64_t>(ctx, op, res, ld_res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_col_si64(dh_ctx *ctx, int op, int64_t *res, const int64_t *arg, size_t rows, size_t cols,
                                    size_t ld) {
    return dh_agg::agg_col<int64_t>(ctx, op, res, arg, rows, cols, ld);
}
extern "C" dh_status dh_agg_col_idx_si64(dh_ctx *ctx, int op, uint64_t *res, const int64_t *arg, size_t rows,
                                        size_t cols, size_t ld) {
    return dh_agg::agg_col_idx<int64_t>(ctx, op, res, arg, rows, cols, ld);
}
