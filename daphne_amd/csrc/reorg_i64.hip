// Fill / ColBind / ExtractCol / Transpose for 64-bit integers (the reference: kernels/CUDA/Fill.cu:47,49,
// ColBind.cu:75, ExtractCol.cu:58). See reorg_impl.h.
#include "reorg_impl.h"

extern "C" dh_status dh_fill_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, int64_t value, size_t rows, size_t cols) {
    return dh_reorg::fill<int64_t>(ctx, res, ld_res, value, rows, cols);
}
extern "C" dh_status dh_fill_ui64(dh_ctx *ctx, uint64_t *res, size_t ld_res, uint64_t value, size_t rows, size_t cols) {
    return dh_reorg::fill<uint64_t>(ctx, res, ld_res, value, rows, cols);
}
extern "C" dh_status dh_col_bind_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, const int64_t *lhs, size_t lhs_rows,
                                      size_t lhs_cols, size_t ld_lhs, const int64_t *rhs, size_t rhs_rows, size_t rhs_cols,
                                      size_t ld_rhs) {
    return dh_reorg::col_bind<int64_t>(ctx, res, ld_res, lhs, lhs_rows, lhs_cols, ld_lhs, rhs, rhs_rows, rhs_cols, ld_rhs);
}
extern "C" dh_status dh_extract_col_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, const int64_t *arg, size_t rows, size_t cols,
                                         size_t ld, const int64_t *sel, size_t sel_rows, size_t sel_cols, size_t ld_sel) {
    return dh_reorg::extract_col<int64_t>(ctx, res, ld_res, arg, rows, cols, ld, reinterpret_cast<const long long *>(sel),
                                          sel_rows, sel_cols, ld_sel);
}
extern "C" dh_status dh_transpose_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, const int64_t *arg, size_t rows, size_t cols,
                                       size_t ld) {
    return dh_reorg::transpose<int64_t>(ctx, res, ld_res, arg, rows, cols, ld);
}
