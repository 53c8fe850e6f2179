// k-means assignment and update passes, double instantiation. See kmeans_impl.h for the design and reference citations.
#include "kmeans_impl.h"

extern "C" dh_status dh_kmeans_assign_f64(dh_ctx *ctx, uint64_t *idx, const double *X, size_t rows, size_t cols, size_t ldx, const double *C,
                                         size_t k, size_t ldc, const double *xx, const double *cc) {
    return dh_kmeans::assign<double>(ctx, reinterpret_cast<unsigned long long *>(idx), X, rows, cols, ldx, C, k, ldc, xx, cc);
}

extern "C" dh_status dh_kmeans_update_f64(dh_ctx *ctx, double *C_new, size_t ld_new, double *counts, const double *X, size_t rows, size_t cols,
                                         size_t ldx, const uint64_t *idx, size_t k) {
    return dh_kmeans::update<double>(ctx, C_new, ld_new, counts, X, rows, cols, ldx, reinterpret_cast<const unsigned long long *>(idx), k);
}

extern "C" dh_status dh_kmeans_step_f64(dh_ctx *ctx, uint64_t *idx, double *C_new, size_t ld_new, double *counts, const double *X, size_t rows,
                                       size_t cols, size_t ldx, const double *C, size_t k, size_t ldc, const double *xx, const double *cc) {
    return dh_kmeans::step<double>(ctx, reinterpret_cast<unsigned long long *>(idx), C_new, ld_new, counts, X, rows, cols, ldx, C, k, ldc, xx, cc);
}
