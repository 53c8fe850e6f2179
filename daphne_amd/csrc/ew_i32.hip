// Elementwise kernels, 32-bit integer instantiations (the reference instantiates EwBinaryMat / EwBinaryObjSca
// for them: kernels/CUDA/EwBinaryMat.cu:268-269, EwBinaryObjSca.cu:92-93). See ew_impl.h and ew_ops.h.
#include "ew_impl.h"

#define DH_EW_INT(SUF, T)                                                                                               \
    extern "C" dh_status dh_ew_binary_##SUF(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *lhs, size_t lhs_rows,  \
                                            size_t lhs_cols, size_t ld_lhs, const T *rhs, size_t rhs_rows,              \
                                            size_t rhs_cols, size_t ld_rhs) {                                           \
        return dh_ew::ew_binary<T>(ctx, op, res, ld_res, lhs, lhs_rows, lhs_cols, ld_lhs, rhs, rhs_rows, rhs_cols,      \
                                   ld_rhs);                                                                             \
    }                                                                                                                   \
    extern "C" dh_status dh_ew_binary_sca_##SUF(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *lhs, size_t rows,  \
                                                size_t cols, size_t ld_lhs, T rhs) {                                    \
        return dh_ew::ew_binary_sca<T>(ctx, op, res, ld_res, lhs, rows, cols, ld_lhs, rhs);                             \
    }

DH_EW_INT(si32, int32_t)
DH_EW_INT(ui32, uint32_t)
