// k-means assignment and update passes, float instantiation. See kmeans_impl.h for the design and reference citations.
#include "kmeans_impl.h"

extern "C" dh_status dh_kmeans_assign_f32(dh_ctx *ctx, uint64_t *idx, const float *X, size_t rows, size_t cols, size_t ldx, const float *C,
                                         size_t k, size_t ldc, const float *xx, const float *cc) {
    return dh_kmeans::assign<float>(ctx, reinterpret_cast<unsigned long long *>(idx), X, rows, cols, ldx, C, k, ldc, xx, cc);
}

extern "C" dh_status dh_kmeans_update_f32(dh_ctx *ctx, float *C_new, size_t ld_new, float *counts, const float *X, size_t rows, size_t cols,
                                         size_t ldx, const uint64_t *idx, size_t k) {
    return dh_kmeans::update<float>(ctx, C_new, ld_new, counts, X, rows, cols, ldx, reinterpret_cast<const unsigned long long *>(idx), k);
}

extern "C" dh_status dh_kmeans_step_f32(dh_ctx *ctx, uint64_t *idx, float *C_new, size_t ld_new, float *counts, const float *X, size_t rows,
                                       size_t cols, size_t ldx, const float *C, size_t k, size_t ldc, const float *xx, const float *cc) {
    return dh_kmeans::step<float>(ctx, reinterpret_cast<unsigned long long *>(idx), C_new, ld_new, counts, X, rows, cols, ldx, C, k, ldc, xx, cc);
}
