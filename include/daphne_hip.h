/*
 * daphne_hip.h - C ABI of libdaphne_hip.so: the gfx950 (MI355X) device kernel set for
 * DenseMatrix<float/double> that DAPHNE's run-time dispatches to an accelerator.
 *
 * Every entry point takes plain device pointers, element counts and leading dimensions
 * (the reference's DenseMatrix::getRowSkip(), in elements). All matrices are row-major.
 * No C++ or torch type crosses this boundary. Each entry point names the reference
 * interface it stands in for (paths relative to the reference checkout, src/ omitted
 * where unambiguous).
 *
 * Error model: every function returns a dh_status. On failure a thread-local message is
 * available from dh_last_error(). The status selects the C++ exception type the reference
 * would have thrown (see the enum), so a C++ caller can re-throw it unchanged.
 *
 * Threading: a dh_ctx may be used from several host threads. Every call holds the context's
 * lock from entry to return, so calls on one context take turns and their kernels run in the
 * order of the context's stream; the workspace, the domain flag and the scalar result slot
 * that a context owns once are therefore never shared between two calls in flight. Kernels
 * that return a value to the host (dh_agg_all_*, domain checks of dh_ew_unary_*) synchronise
 * that stream while they hold the lock. Threads that should not wait for each other use one
 * context each.
 */
#ifndef DAPHNE_HIP_H
#define DAPHNE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------ */
/* status codes                                                                          */
/* ------------------------------------------------------------------------------------ */
typedef enum dh_status {
    DH_OK = 0,
    DH_ERR_RUNTIME = 1,      /* std::runtime_error: bad shapes, unknown/unsupported op code  */
    DH_ERR_INVALID_ARG = 2,  /* std::invalid_argument: e.g. conv filter larger than image    */
    DH_ERR_DOMAIN = 3,       /* std::domain_error: sqrt/ln/asin/acos outside their domain    */
    DH_ERR_HIP = 4,          /* std::runtime_error carrying the HIP error string             */
    DH_ERR_OOM = 5,          /* std::runtime_error: device allocation beyond the budget      */
    DH_ERR_OUT_OF_RANGE = 6  /* std::out_of_range: ExtractCol position outside the matrix    */
} dh_status;

/* Thread-local text of the last failure on the calling thread ("" if none). */
const char *dh_last_error(void);

/* ------------------------------------------------------------------------------------ */
/* op codes - numeric values equal the reference enums, so they pass through unchanged   */
/* ------------------------------------------------------------------------------------ */
/* runtime/local/kernels/BinaryOpCode.h:29-55 */
typedef enum dh_binary_op {
    DH_BIN_ADD = 0, DH_BIN_SUB = 1, DH_BIN_MUL = 2, DH_BIN_DIV = 3, DH_BIN_POW = 4,
    DH_BIN_MOD = 5, DH_BIN_LOG = 6, DH_BIN_EQ = 7, DH_BIN_NEQ = 8, DH_BIN_LT = 9,
    DH_BIN_LE = 10, DH_BIN_GT = 11, DH_BIN_GE = 12, DH_BIN_MIN = 13, DH_BIN_MAX = 14,
    DH_BIN_AND = 15, DH_BIN_OR = 16,
    DH_BIN_BITWISE_AND = 17, /* integer only in the reference: rejected for float/double */
    DH_BIN_CONCAT = 18       /* strings only: rejected */
} dh_binary_op;

/* runtime/local/kernels/UnaryOpCode.h:28-55 */
typedef enum dh_unary_op {
    DH_UN_MINUS = 0, DH_UN_ABS = 1, DH_UN_SIGN = 2, DH_UN_SQRT = 3, DH_UN_EXP = 4,
    DH_UN_LN = 5, DH_UN_SIN = 6, DH_UN_COS = 7, DH_UN_TAN = 8, DH_UN_ASIN = 9,
    DH_UN_ACOS = 10, DH_UN_ATAN = 11, DH_UN_SINH = 12, DH_UN_COSH = 13, DH_UN_TANH = 14,
    DH_UN_FLOOR = 15, DH_UN_CEIL = 16, DH_UN_ROUND = 17, DH_UN_ISNAN = 18,
    DH_UN_UPPER = 19, DH_UN_LOWER = 20 /* strings only: rejected */
} dh_unary_op;

/* runtime/local/kernels/AggOpCode.h:25-35 */
typedef enum dh_agg_op {
    DH_AGG_SUM = 0, DH_AGG_PROD = 1, DH_AGG_MIN = 2, DH_AGG_MAX = 3, DH_AGG_IDXMIN = 4,
    DH_AGG_IDXMAX = 5, DH_AGG_MEAN = 6, DH_AGG_STDDEV = 7, DH_AGG_VAR = 8
} dh_agg_op;

/* ------------------------------------------------------------------------------------ */
/* device context and allocator                                                          */
/* replaces runtime/local/context/CUDAContext.h:29-114, CUDAContext.cpp:41-135 and       */
/* runtime/local/kernels/CUDA/CreateCUDAContext.cpp:5-10                                 */
/* ------------------------------------------------------------------------------------ */
typedef struct dh_ctx dh_ctx;

/* Select `device`, read its properties, set the memory budget to 90 % of total device
 * memory (CUDAContext.cpp:49-50) and create the reduction workspace. */
dh_status dh_ctx_create(int device, dh_ctx **out);
/* Frees every allocation still registered, the workspace and the context. */
dh_status dh_ctx_destroy(dh_ctx *ctx);
/* CUDAContext::getMemBudget() (CUDAContext.h:83). */
size_t dh_ctx_mem_budget(const dh_ctx *ctx);
/* Bytes currently handed out by dh_malloc on this context. */
size_t dh_ctx_mem_in_use(const dh_ctx *ctx);
int dh_ctx_device(const dh_ctx *ctx);
/* Number of compute units and the max engine clock in kHz (for roofline print-outs). */
dh_status dh_ctx_props(const dh_ctx *ctx, int *compute_units, int *clock_khz, size_t *total_mem,
                       char *name, size_t name_cap);
/* Free and total memory of a device, without a context: what the compiler's device-placement pass asks when it
 * decides whether an operation's operands fit (compiler/lowering/MarkCUDAOpsPass.cpp:37-41 calls cudaMemGetInfo).
 * DH_ERR_HIP when there is no such device. */
dh_status dh_device_memory(int device, size_t *free_bytes, size_t *total_bytes);
/* Enqueue kernels of this context on `hip_stream` (a hipStream_t; NULL = the default
 * stream, which is also the initial setting). The context never owns the stream. */
dh_status dh_ctx_set_stream(dh_ctx *ctx, void *hip_stream);
void *dh_ctx_get_stream(const dh_ctx *ctx);
/* Blocks until all work enqueued on the context's stream has finished. */
dh_status dh_sync(dh_ctx *ctx);
/* Deferred verdicts. Some kernels can only tell on the device whether their arguments were valid: integer DIV and MOD
 * (a zero divisor, EwBinarySca.h:114-127 through the host's arithmetic), SQRT / LN / ASIN / ACOS (EwUnarySca.h:130-170),
 * the column positions of ExtractCol (ExtractCol.h:98-108), checked unary functions inside a fused pipeline body, and
 * the singular factor of Solve (Solve.h:113-115).
 * By default such a call waits for its kernels and returns the failure itself, as the CPU kernel throws. A caller that
 * runs many of them back to back - the task of a vectorized pipeline walking its batches,
 * vectorized/TasksCUDA.cpp:61-100 has no counterpart because the CUDA kernels do not check - enters deferred mode:
 *   dh_defer_checks(ctx, 1)   from now on these calls return DH_OK without waiting; the first failure in the stream's
 *                             order is kept on the device (results computed from invalid arguments are unspecified,
 *                             but every access stays inside its matrix). Calls nest; each needs a matching
 *   dh_defer_checks(ctx, 0)   which leaves the mode (a pending failure stays pending).
 *   dh_check_deferred(ctx)    returns DH_OK at once if no such call was made since the last verdict; else waits
 *                             for the stream and returns DH_OK, or the pending failure with the status and
 *                             message the immediate form would have given, and clears it. Valid in either mode.
 * Neither call has a counterpart in the reference. */
dh_status dh_defer_checks(dh_ctx *ctx, int on);
dh_status dh_check_deferred(dh_ctx *ctx);

/* CUDAContext::malloc(size, zero, id) / free(id) (CUDAContext.cpp:120-135). The device
 * pointer itself is the registry key. Fails with DH_ERR_OOM past the budget.
 * Unlike cudaMalloc/cudaFree there, freed blocks are kept by the context and handed out again to
 * later requests of the same size class, without a device synchronisation: reuse is ordered by the
 * context's stream, so a caller that used a buffer on another stream waits for that work before
 * dh_free. Cached blocks are returned to the driver when the budget or the device runs short, by
 * dh_ctx_release_cached, and by dh_ctx_destroy. */
dh_status dh_malloc(dh_ctx *ctx, size_t bytes, int zero, void **out);
dh_status dh_free(dh_ctx *ctx, void *ptr);
/* Bytes held in freed blocks awaiting reuse / give them back to the driver (synchronises). */
size_t dh_ctx_mem_cached(const dh_ctx *ctx);
dh_status dh_ctx_release_cached(dh_ctx *ctx);
/* AllocationDescriptorCUDA::transferTo / transferFrom
 * (runtime/local/datastructures/AllocationDescriptorCUDA.h:56-68): synchronous copies. */
dh_status dh_h2d(dh_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
dh_status dh_d2h(dh_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
dh_status dh_d2d(dh_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);
/* `rows` rows of `width_bytes` bytes between two pitched device buffers, in the order of the context's stream:
 * how a vectorized-pipeline task puts a row share's result into its place in the whole result
 * (CompiledPipelineTaskCUDA::accumulateOutputs, runtime/local/vectorized/TasksCUDA.cpp:73-100, one cudaMemcpy
 * per share or per row there). */
dh_status dh_d2d_2d(dh_ctx *ctx, void *dst_dev, size_t dst_pitch, const void *src_dev, size_t src_pitch,
                    size_t width_bytes, size_t rows);
/* The same from a pitched device buffer into pitched host memory, synchronous like dh_d2h: how the device's share of
 * a pipeline's result is put into a result in host memory when CPU workers computed the other rows
 * (MTWrapper<DenseMatrix<VT>>::combineOutputs, runtime/local/vectorized/MTWrapper_dense.cpp:339-373: one cudaMemcpy
 * for a row share, one per row for a column share). */
dh_status dh_d2h_2d(dh_ctx *ctx, void *dst_host, size_t dst_pitch, const void *src_dev, size_t src_pitch,
                    size_t width_bytes, size_t rows);

/* Stream-ordered stopwatch on the context's stream (hipEvent pair). dh_timer_stop_ms
 * synchronises on the stop event and returns the elapsed milliseconds. */
dh_status dh_timer_start(dh_ctx *ctx);
dh_status dh_timer_stop_ms(dh_ctx *ctx, float *ms);
/* A stopwatch on single kernels (no counterpart in the reference; for measurement). While it is on, a call whose time
 * is one dominant kernel beside small ones - dh_vectorized_pipeline_*: the body kernel, without the kernels that fold
 * its partial results - records a pair of events around that kernel alone, on the context's stream, without waiting.
 * dh_kernel_timing_read waits for the last of them, returns the sum of the kernels' durations and their number since
 * the stopwatch was switched on or last read, and starts counting again. At most 4096 kernels are kept per reading. */
dh_status dh_kernel_timing(dh_ctx *ctx, int on);
dh_status dh_kernel_timing_read(dh_ctx *ctx, double *total_ms, size_t *launches);

/* ------------------------------------------------------------------------------------ */
/* elementwise                                                                           */
/* ------------------------------------------------------------------------------------ */
/* CUDA::EwBinaryMat<DenseMatrix<VT>,...>::apply (kernels/CUDA/EwBinaryMat.h:31-47,
 * EwBinaryMat.cu:97-263) with the CPU kernel's semantics (kernels/EwBinaryMat.h:54-108,
 * EwBinarySca.h:143-167): res has the shape of lhs; rhs is the same shape, a 1 x cols
 * row vector, or a rows x 1 column vector, else DH_ERR_RUNTIME. All 17 floating-point op
 * codes are supported. res may alias lhs (or rhs of the same shape). */
dh_status dh_ew_binary_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *lhs,
                           size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const float *rhs,
                           size_t rhs_rows, size_t rhs_cols, size_t ld_rhs);
dh_status dh_ew_binary_f64(dh_ctx *ctx, int op, double *res, size_t ld_res, const double *lhs,
                           size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const double *rhs,
                           size_t rhs_rows, size_t rhs_cols, size_t ld_rhs);

/* CUDA::EwBinaryObjSca<DenseMatrix<VT>,DenseMatrix<VT>,VT>::apply
 * (kernels/CUDA/EwBinaryObjSca.h:37-60, .cu:31-88; CPU kernels/EwBinaryObjSca.h:57-79). */
dh_status dh_ew_binary_sca_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *lhs,
                               size_t rows, size_t cols, size_t ld_lhs, float rhs);
dh_status dh_ew_binary_sca_f64(dh_ctx *ctx, int op, double *res, size_t ld_res, const double *lhs,
                               size_t rows, size_t cols, size_t ld_lhs, double rhs);

/* EwUnaryMat<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/EwUnaryMat.h:57-77,
 * EwUnarySca.h:182-206); no device version exists in the reference. SQRT/LN with an
 * argument below zero and ASIN/ACOS outside [-1,1] return DH_ERR_DOMAIN
 * (EwUnarySca.h:134-157); res then holds what libm produced (NaN at the offending items).
 * Only these four op codes synchronise the stream. */
dh_status dh_ew_unary_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *arg,
                          size_t rows, size_t cols, size_t ld_arg);
dh_status dh_ew_unary_f64(dh_ctx *ctx, int op, double *res, size_t ld_res, const double *arg,
                          size_t rows, size_t cols, size_t ld_arg);

/* ------------------------------------------------------------------------------------ */
/* aggregations                                                                          */
/* ------------------------------------------------------------------------------------ */
/* CUDA::AggAll<VT,DenseMatrix<VT>>::apply (kernels/CUDA/AggAll.h:28-50, .cu:109-151; CPU
 * kernels/AggAll.h:124-193): SUM PROD MIN MAX MEAN VAR STDDEV (population variance).
 * The scalar is written to *result_host after a stream synchronise. */
dh_status dh_agg_all_f32(dh_ctx *ctx, int op, const float *arg, size_t rows, size_t cols,
                         size_t ld, float *result_host);
dh_status dh_agg_all_f64(dh_ctx *ctx, int op, const double *arg, size_t rows, size_t cols,
                         size_t ld, double *result_host);
/* Same, but the scalar stays on the device (result_dev[0]); no synchronisation. */
dh_status dh_agg_all_dev_f32(dh_ctx *ctx, int op, const float *arg, size_t rows, size_t cols,
                             size_t ld, float *result_dev);
dh_status dh_agg_all_dev_f64(dh_ctx *ctx, int op, const double *arg, size_t rows, size_t cols,
                             size_t ld, double *result_dev);

/* CUDA::AggRow<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/CUDA/AggRow.h:30-52,
 * .cu:108-143; CPU kernels/AggRow.h:60-161): res is rows x 1 with leading dimension
 * ld_res. SUM PROD MIN MAX MEAN VAR STDDEV. */
dh_status dh_agg_row_f32(dh_ctx *ctx, int op, float *res, size_t ld_res, const float *arg,
                         size_t rows, size_t cols, size_t ld);
dh_status dh_agg_row_f64(dh_ctx *ctx, int op, double *res, size_t ld_res, const double *arg,
                         size_t rows, size_t cols, size_t ld);
/* RowIdxMin / RowIdxMax = AggRow<DenseMatrix<size_t>,DenseMatrix<VT>> with IDXMIN / IDXMAX
 * (kernels/AggRow.h:71-94; op idxminRow, ir/daphneir/DaphneOps.td:544): first index of the
 * strict extremum, 64-bit unsigned output. No device version exists in the reference. */
dh_status dh_agg_row_idx_f32(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const float *arg,
                             size_t rows, size_t cols, size_t ld);
dh_status dh_agg_row_idx_f64(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res,
                             const double *arg, size_t rows, size_t cols, size_t ld);

/* CUDA::AggCol<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/CUDA/AggCol.h:30-52,
 * .cu:45-86; CPU kernels/AggCol.h:58-178): res is 1 x cols. */
dh_status dh_agg_col_f32(dh_ctx *ctx, int op, float *res, const float *arg, size_t rows,
                         size_t cols, size_t ld);
dh_status dh_agg_col_f64(dh_ctx *ctx, int op, double *res, const double *arg, size_t rows,
                         size_t cols, size_t ld);
/* dh_agg_col_f32 for callers that cannot allocate (code under HIP stream capture, tight serving loops,
 * harnesses that forbid hipMalloc). It has no counterpart in the reference. Same arguments, op codes and
 * results as dh_agg_col_f32, bit for bit; the partial results of its two kernels go to a fixed 8 MiB array
 * in device memory that the library holds per GPU, so the call reaches no hipMalloc / hipFree. An input whose
 * partials (4 B x columns x row slabs; twice that for VAR / STDDEV) exceed the array fails with DH_ERR_RUNTIME
 * and leaves res untouched; the slab count shrinks as the matrix gets wider, so on a 256-CU device that only
 * happens beyond 2 Mi columns (1 Mi for VAR / STDDEV). All calls on one GPU share the array: calls that overlap on one GPU race, calls in stream order
 * do not. */
dh_status dh_agg_col_noalloc_f32(dh_ctx *ctx, int op, float *res, const float *arg, size_t rows,
                                 size_t cols, size_t ld);
/* Size of that array in bytes. */
size_t dh_agg_col_noalloc_scratch_bytes(void);
/* colMeans and colVars (or colStddevs when `stddev` != 0) of the same matrix in ONE pass: what
 * dh_agg_col with DH_AGG_MEAN and DH_AGG_VAR / DH_AGG_STDDEV (kernels/AggCol.h:143-170) return, for a
 * caller - a fused pipeline, or a rewrite of mean(X,1) + var(X,1) on one input - that needs both. The
 * reference has two separate kernel calls here; results agree with them within rounding. */
dh_status dh_agg_col_moments_f32(dh_ctx *ctx, float *res_mean, float *res_var, int stddev,
                                 const float *arg, size_t rows, size_t cols, size_t ld);
dh_status dh_agg_col_moments_f64(dh_ctx *ctx, double *res_mean, double *res_var, int stddev,
                                 const double *arg, size_t rows, size_t cols, size_t ld);
/* AggCol with IDXMIN / IDXMAX (kernels/AggCol.h:70-122): first row of the strict extremum
 * per column. */
dh_status dh_agg_col_idx_f32(dh_ctx *ctx, int op, uint64_t *res, const float *arg, size_t rows,
                             size_t cols, size_t ld);
dh_status dh_agg_col_idx_f64(dh_ctx *ctx, int op, uint64_t *res, const double *arg, size_t rows,
                             size_t cols, size_t ld);

/* ------------------------------------------------------------------------------------ */
/* contractions                                                                          */
/* ------------------------------------------------------------------------------------ */
/* CUDA::MatMul<DenseMatrix<T>,...>::apply (kernels/CUDA/MatMul.h:31-51, MatMul.cpp:45-91;
 * CPU kernels/MatMul.cpp:248-290): res = op(lhs) * op(rhs), alpha = 1, beta = 0. The shapes
 * are those of the stored matrices; the transposes are applied by the kernel. Returns
 * DH_ERR_RUNTIME if the inner dimensions differ (MatMul.cpp:256-259). Matrix-vector and
 * vector-vector shapes take streaming paths (MatMul.cpp:277-283). */
dh_status dh_matmul_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *lhs, size_t lhs_rows,
                        size_t lhs_cols, size_t ld_lhs, const float *rhs, size_t rhs_rows,
                        size_t rhs_cols, size_t ld_rhs, int transa, int transb);
dh_status dh_matmul_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *lhs,
                        size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const double *rhs,
                        size_t rhs_rows, size_t rhs_cols, size_t ld_rhs, int transa, int transb);

/* CUDA::Syrk<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/CUDA/Syrk.h:29-46,
 * Syrk.cu:54-87) with the CPU signature that carries transLeft (kernels/Syrk.h:51-93):
 * res = transLeft ? arg^T * arg : arg * arg^T, full symmetric n x n (both triangles). */
dh_status dh_syrk_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows,
                      size_t cols, size_t ld, int trans_left);
dh_status dh_syrk_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows,
                      size_t cols, size_t ld, int trans_left);

/* CUDA::Solve<DenseMatrix<VT>,...>::apply (kernels/CUDA/Solve.cpp:75-151, cuSOLVER getrf/getrs;
 * CPU kernels/Solve.h:86-116, LAPACKE_?gesv): solves A x = b for one right-hand side by LU with
 * partial pivoting. A is n x n with leading dimension lda and is left untouched; x and b hold n
 * values. DH_ERR_RUNTIME if a pivot is exactly zero (Solve.h:113-115). Synchronises the stream. */
dh_status dh_solve_f32(dh_ctx *ctx, float *x, const float *A, size_t n, size_t lda, const float *b);
dh_status dh_solve_f64(dh_ctx *ctx, double *x, const double *A, size_t n, size_t lda, const double *b);

/* One Lloyd iteration of k-means in two passes over X, without the rows x k matrices (distances, one-hot
 * membership) that the operator sequence of the script writes and reads back
 * (test/api/cli/algorithms/kmeans.daphne:14-21 with the row arg-min as membership). No single kernel of
 * the reference does this; the calls replace
 *   assign:  MatMul X @ t(C) (kernels/CUDA/MatMul.cpp), EwBinaryObjSca MUL -2, EwBinaryMat ADD of the column
 *            xx (rows x 1) and of the row cc (1 x k) (kernels/CUDA/EwBinaryMat.cpp:95-155), AggRow IDXMIN
 *            (kernels/AggRow.h:71-94): idx[i] = first position of the minimum of
 *            ((X t(C))[i][c] * -2 + xx[i]) + cc[c]. The distances are rounded as in that sequence, so idx
 *            equals its result wherever dh_matmul takes its streaming kernel for X t(C) (65536 rows or
 *            more); elsewhere the product's last bits, and with them near-ties, may differ.
 *   update:  the one-hot comparison, MatMul t(P) @ X, AggCol SUM, EwBinaryMat DIV:
 *            C_new[c][:] = (sum of the rows with idx = c) / (their number); counts (k values, may be
 *            NULL) receives the numbers. An empty cluster comes out as 0 / 0.
 * X is rows x cols with leading dimension ldx, C is k x cols (ldc), idx holds rows values. Limits
 * (DH_ERR_INVALID_ARG beyond them): k <= 32; cols <= 512 for assign and <= 256 (float) / 128 (double)
 * for update; rows of X and C 16-byte aligned and a whole number of 16-byte vectors long. */
dh_status dh_kmeans_assign_f32(dh_ctx *ctx, uint64_t *idx, const float *X, size_t rows, size_t cols,
                               size_t ldx, const float *C, size_t k, size_t ldc, const float *xx,
                               const float *cc);
dh_status dh_kmeans_assign_f64(dh_ctx *ctx, uint64_t *idx, const double *X, size_t rows, size_t cols,
                               size_t ldx, const double *C, size_t k, size_t ldc, const double *xx,
                               const double *cc);
dh_status dh_kmeans_update_f32(dh_ctx *ctx, float *C_new, size_t ld_new, float *counts, const float *X,
                               size_t rows, size_t cols, size_t ldx, const uint64_t *idx, size_t k);
dh_status dh_kmeans_update_f64(dh_ctx *ctx, double *C_new, size_t ld_new, double *counts,
                               const double *X, size_t rows, size_t cols, size_t ldx,
                               const uint64_t *idx, size_t k);

/* dh_kmeans_assign followed by dh_kmeans_update, in one pass over X where the library has a kernel for
 * it (up to 64 features, in double up to 16 centroids: a row, once loaded, serves the distances and then the sums), as the two
 * calls one after the other elsewhere. idx as dh_kmeans_assign gives it; C_new and counts as
 * dh_kmeans_update gives them (C_new to rounding: the rows are added in another order). Arguments,
 * limits and errors of the two calls. */
dh_status dh_kmeans_step_f32(dh_ctx *ctx, uint64_t *idx, float *C_new, size_t ld_new, float *counts,
                             const float *X, size_t rows, size_t cols, size_t ldx, const float *C,
                             size_t k, size_t ldc, const float *xx, const float *cc);
dh_status dh_kmeans_step_f64(dh_ctx *ctx, uint64_t *idx, double *C_new, size_t ld_new, double *counts,
                             const double *X, size_t rows, size_t cols, size_t ldx, const double *C,
                             size_t k, size_t ldc, const double *xx, const double *cc);

/* ------------------------------------------------------------------------------------ */
/* DNN inference ops (NCHW images flattened to rows: one image per matrix row)           */
/* ------------------------------------------------------------------------------------ */
/* CUDA::Convolution::Forward<...>::apply (kernels/CUDA/Convolution.h:33-38, .cpp:21-135;
 * CPU kernels/Conv2DForward.h:77-140): cross-correlation, data N x (C*H*W), filter
 * filter_rows x filter_cols = F x (C*Hf*Wf), res N x (F*P*Q) with
 * P = (H + 2*pad_h - Hf)/stride_h + 1. bias is F values or NULL (no bias, as the CUDA kernel
 * allows). *res_h / *res_w receive P / Q. DH_ERR_INVALID_ARG if the filter does not hold
 * F*C*Hf*Wf items (Convolution.cpp:32-39) or exceeds the padded image. */
dh_status dh_conv2d_forward_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w,
                                const float *data, const float *filter, size_t filter_rows,
                                size_t filter_cols, const float *bias, size_t batch,
                                size_t channels, size_t img_h, size_t img_w, size_t filter_h,
                                size_t filter_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                size_t pad_w);
dh_status dh_conv2d_forward_f64(dh_ctx *ctx, double *res, size_t *res_h, size_t *res_w,
                                const double *data, const double *filter, size_t filter_rows,
                                size_t filter_cols, const double *bias, size_t batch,
                                size_t channels, size_t img_h, size_t img_w, size_t filter_h,
                                size_t filter_w, size_t stride_h, size_t stride_w, size_t pad_h,
                                size_t pad_w);

/* Convolution with the operators that follow it in a network folded into its epilogue, so that the
 * activations are written once. No single kernel of the reference does this; a call replaces the
 * kernel sequence that a script's conv2d(...), relu(...), max_pool2d(...) compile to
 * (src/parser/daphnedsl/DaphneDSLBuiltins.cpp:883-896):
 *   DH_EPILOGUE_RELU:         CUDA::Convolution::Forward (kernels/CUDA/Convolution.cpp:21-135), then
 *                             CUDA::NN::Activation::Forward<ReLU> (kernels/CUDA/Activation.cpp:21-47);
 *   DH_EPILOGUE_MAXPOOL_2X2:  then CUDA::NN::Pooling::Forward<MAX> with a 2 x 2 window, stride 2,
 *                             no padding (kernels/CUDA/Pooling.cpp:22-65);
 * and the result equals that of dh_conv2d_forward, dh_relu_forward and dh_maxpool_forward applied
 * one after the other bit for bit. With pooling, res is N x (F * (P / 2) * (Q / 2)) and *res_h /
 * *res_w receive the pooled extents; P or Q below 2 is DH_ERR_INVALID_ARG as in
 * dh_maxpool_forward. Other arguments and errors as dh_conv2d_forward. */
enum dh_epilogue { DH_EPILOGUE_NONE = 0, DH_EPILOGUE_RELU = 1, DH_EPILOGUE_MAXPOOL_2X2 = 2 };
dh_status dh_conv2d_forward_fused_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w,
                                      const float *data, const float *filter, size_t filter_rows,
                                      size_t filter_cols, const float *bias, size_t batch,
                                      size_t channels, size_t img_h, size_t img_w, size_t filter_h,
                                      size_t filter_w, size_t stride_h, size_t stride_w,
                                      size_t pad_h, size_t pad_w, unsigned epilogue);
dh_status dh_conv2d_forward_fused_f64(dh_ctx *ctx, double *res, size_t *res_h, size_t *res_w,
                                      const double *data, const double *filter, size_t filter_rows,
                                      size_t filter_cols, const double *bias, size_t batch,
                                      size_t channels, size_t img_h, size_t img_w, size_t filter_h,
                                      size_t filter_w, size_t stride_h, size_t stride_w,
                                      size_t pad_h, size_t pad_w, unsigned epilogue);

/* CUDA::NN::Pooling::Forward<MAX,...>::apply (kernels/CUDA/Pooling.h:31-35, .cpp:22-65) with
 * the CPU kernel's arithmetic (kernels/Pooling.cpp:28-107, Pooling.h:46-54,
 * MaxPoolForward.h:35-44): the result is max(0, window) because the CPU kernel folds the
 * window into a zero-initialised output; P is derived with stride_w and Q with stride_h
 * (Pooling.cpp:38-39); windows are clipped at the image border. */
dh_status dh_maxpool_forward_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w,
                                 const float *data, size_t batch, size_t channels, size_t img_h,
                                 size_t img_w, size_t pool_h, size_t pool_w, size_t stride_h,
                                 size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_maxpool_forward_f64(dh_ctx *ctx, double *res, size_t *res_h, size_t *res_w,
                                 const double *data, size_t batch, size_t channels, size_t img_h,
                                 size_t img_w, size_t pool_h, size_t pool_w, size_t stride_h,
                                 size_t stride_w, size_t pad_h, size_t pad_w);

/* CUDA::NN::Affine::Forward<...>::apply (kernels/CUDA/Affine.h:24-26, Affine.cpp:42-83):
 * res = data * weights (+ bias broadcast over rows). bias may be NULL. DH_ERR_RUNTIME if
 * data_cols != w_rows or bias is not 1 x w_cols (Affine.cpp:50-60). */
dh_status dh_affine_forward_f32(dh_ctx *ctx, float *res, const float *data, size_t data_rows,
                                size_t data_cols, const float *weights, size_t w_rows,
                                size_t w_cols, const float *bias, size_t bias_rows,
                                size_t bias_cols);
dh_status dh_affine_forward_f64(dh_ctx *ctx, double *res, const double *data, size_t data_rows,
                                size_t data_cols, const double *weights, size_t w_rows,
                                size_t w_cols, const double *bias, size_t bias_rows,
                                size_t bias_cols);

/* dh_affine_forward with DH_EPILOGUE_RELU folded into the store: the kernel sequence of affine(...)
 * and relu(...) (CUDA::NN::Affine::Forward, kernels/CUDA/Affine.cpp:42-83, then
 * CUDA::NN::Activation::Forward<ReLU>, kernels/CUDA/Activation.cpp:21-47), same result bit for bit.
 * epilogue is DH_EPILOGUE_NONE or DH_EPILOGUE_RELU. */
dh_status dh_affine_forward_fused_f32(dh_ctx *ctx, float *res, const float *data, size_t data_rows,
                                      size_t data_cols, const float *weights, size_t w_rows,
                                      size_t w_cols, const float *bias, size_t bias_rows,
                                      size_t bias_cols, unsigned epilogue);
dh_status dh_affine_forward_fused_f64(dh_ctx *ctx, double *res, const double *data, size_t data_rows,
                                      size_t data_cols, const double *weights, size_t w_rows,
                                      size_t w_cols, const double *bias, size_t bias_rows,
                                      size_t bias_cols, unsigned epilogue);

/* CUDA::BiasAdd<...>::apply (kernels/CUDA/BiasAdd.h:26-28, BiasAdd.cpp:20-55; CPU
 * kernels/BiasAdd.h:34-52): res[i, c*HW + j] = data[i, c*HW + j] + bias[c], HW = cols /
 * num_bias. num_bias is the bias item count (rows for the CPU test's C x 1 bias, cols for
 * the CUDA test's 1 x C bias). */
dh_status dh_bias_add_f32(dh_ctx *ctx, float *res, const float *data, size_t rows, size_t cols,
                          const float *bias, size_t num_bias);
dh_status dh_bias_add_f64(dh_ctx *ctx, double *res, const double *data, size_t rows, size_t cols,
                          const double *bias, size_t num_bias);

/* CUDA::BatchNormInferenceForward<...>::apply (kernels/CUDA/BatchNorm.h:26-29, .cpp:21-55;
 * CPU kernels/BatchNorm2DTestForward.h:77-101):
 *   res = gamma_s * (x - mean_s) / sqrt(var_s + eps) + beta_s.
 * stat_index = 0: s is the channel of the element, channels = rows of gamma (the cuDNN
 * spatial mode of the CUDA kernel); stat_index = 1: s is the row (image) index, which is
 * what the CPU kernel does (BatchNorm2DTestForward.h:96-97). */
dh_status dh_batchnorm_inference_f32(dh_ctx *ctx, float *res, const float *data, size_t rows,
                                     size_t cols, const float *gamma, const float *beta,
                                     const float *ema_mean, const float *ema_var,
                                     size_t channels, float eps, int stat_index);
dh_status dh_batchnorm_inference_f64(dh_ctx *ctx, double *res, const double *data, size_t rows,
                                     size_t cols, const double *gamma, const double *beta,
                                     const double *ema_mean, const double *ema_var,
                                     size_t channels, double eps, int stat_index);

/* CUDA::Softmax<...>::apply (kernels/CUDA/Softmax.h:32-34, Softmax.cpp:22-48; CPU
 * kernels/Softmax.h:22-58): row-wise exp(x - max) / sum. */
dh_status dh_softmax_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows,
                         size_t cols, size_t ld);
dh_status dh_softmax_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows,
                         size_t cols, size_t ld);

/* CUDA::NN::Pooling::Forward<AVG,...>::apply (kernels/CUDA/Pooling.h:31-35) with the CPU kernel's
 * arithmetic (kernels/Pooling.cpp:28-107, Pooling.h:33-44, AvgPoolForward.h): every window row is
 * summed left to right, scaled by 1 / (pool_h * pool_w) - the full window, zero padding included -
 * and added to the running result. Output extents as for MAX. */
dh_status dh_avgpool_forward_f32(dh_ctx *ctx, float *res, size_t *res_h, size_t *res_w,
                                 const float *data, size_t batch, size_t channels, size_t img_h,
                                 size_t img_w, size_t pool_h, size_t pool_w, size_t stride_h,
                                 size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_avgpool_forward_f64(dh_ctx *ctx, double *res, size_t *res_h, size_t *res_w,
                                 const double *data, size_t batch, size_t channels, size_t img_h,
                                 size_t img_w, size_t pool_h, size_t pool_w, size_t stride_h,
                                 size_t stride_w, size_t pad_h, size_t pad_w);

/* CUDA::NN::Activation::Forward<ReLU,DTRes,DTArg>::apply (kernels/CUDA/Activation.h:24-33,
 * Activation.cpp:21-47: cudnnActivationForward, RELU, NaN propagated): res = max(0, data). */
dh_status dh_relu_forward_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *data, size_t rows,
                              size_t cols, size_t ld_data);
dh_status dh_relu_forward_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *data,
                              size_t rows, size_t cols, size_t ld_data);

/* ------------------------------------------------------------------------------------ */
/* data reorganisation                                                                   */
/* ------------------------------------------------------------------------------------ */
/* CUDA::Fill<DenseMatrix<VT>,VT>::apply (kernels/CUDA/Fill.h:30-47, Fill.cu:27-49): every element
 * of the rows x cols result becomes `value`. */
dh_status dh_fill_f32(dh_ctx *ctx, float *res, size_t ld_res, float value, size_t rows, size_t cols);
dh_status dh_fill_f64(dh_ctx *ctx, double *res, size_t ld_res, double value, size_t rows, size_t cols);

/* CUDA::ColBind<...>::apply (kernels/CUDA/ColBind.h:26-34, ColBind.cu:47-70): res = [lhs | rhs],
 * lhs_rows x (lhs_cols + rhs_cols). DH_ERR_RUNTIME if the row counts differ (kernels/ColBind.h:62-67). */
dh_status dh_col_bind_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *lhs, size_t lhs_rows,
                          size_t lhs_cols, size_t ld_lhs, const float *rhs, size_t rhs_rows,
                          size_t rhs_cols, size_t ld_rhs);
dh_status dh_col_bind_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *lhs, size_t lhs_rows,
                          size_t lhs_cols, size_t ld_lhs, const double *rhs, size_t rhs_rows,
                          size_t rhs_cols, size_t ld_rhs);

/* CUDA::ExtractCol<DenseMatrix<VT>,DenseMatrix<VT>,DenseMatrix<int64_t>>::apply
 * (kernels/CUDA/ExtractCol.h:26-35, ExtractCol.cu:21-56): res[r][k] = arg[r][sel[k]] with sel a
 * sel_rows x 1 matrix of positions in device memory. As in the CPU kernel
 * (kernels/ExtractCol.h:57-64,96-108) a negative position counts from the last column,
 * DH_ERR_RUNTIME if sel has more than one column, DH_ERR_OUT_OF_RANGE for a position outside
 * [0, cols). Synchronises (the positions are validated before the copy). */
dh_status dh_extract_col_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows,
                             size_t cols, size_t ld, const int64_t *sel, size_t sel_rows,
                             size_t sel_cols, size_t ld_sel);
dh_status dh_extract_col_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows,
                             size_t cols, size_t ld, const int64_t *sel, size_t sel_rows,
                             size_t sel_cols, size_t ld_sel);

/* CUDA::Transpose<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/CUDA/Transpose.h:33-39,
 * Transpose.cpp: cublas geam): res (cols x rows) = t(arg). */
dh_status dh_transpose_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *arg, size_t rows,
                           size_t cols, size_t ld);
dh_status dh_transpose_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *arg, size_t rows,
                           size_t cols, size_t ld);

/* CUDA::Gemv<DenseMatrix<T>,...>::apply (kernels/CUDA/Gemv.h:34-40, Gemv.cpp:42-68; CPU
 * kernels/Gemv.h:51-77, cblas_?gemv with CblasTrans): res (cols x 1) = t(mat) * vec, vec a
 * rows x 1 column with row stride ld_vec. */
dh_status dh_gemv_f32(dh_ctx *ctx, float *res, size_t ld_res, const float *mat, size_t rows, size_t cols,
                      size_t ld_mat, const float *vec, size_t vec_rows, size_t ld_vec);
dh_status dh_gemv_f64(dh_ctx *ctx, double *res, size_t ld_res, const double *mat, size_t rows,
                      size_t cols, size_t ld_mat, const double *vec, size_t vec_rows, size_t ld_vec);


/* ------------------------------------------------------------------------------------ */
/* integer value types                                                                   */
/* ------------------------------------------------------------------------------------ */
/* The reference instantiates its device kernels for integers as well:
 * EwBinaryMat for si64 / si32 / ui32 / ui64 (kernels/CUDA/EwBinaryMat.cu:267-270), EwBinaryObjSca for
 * the same four (EwBinaryObjSca.cu:91-94), AggAll / AggRow / AggCol for si64 (AggAll.cu:155,
 * AggRow.cu:146, AggCol.cu:89), Fill for si64 / ui64 (Fill.cu:47,49), ColBind and ExtractCol for si64
 * (ColBind.cu:75, ExtractCol.cu:58). Arguments as for the floating-point entry points above.
 *
 * Elementwise semantics are those of the CPU kernel's expressions evaluated on integers
 * (kernels/EwBinarySca.h:143-167): + - * / wrap and truncate as C++ integer arithmetic does,
 * POW / MOD / LOG go through double (pow, fmod, log(l)/log(r)) and are truncated back, comparisons and
 * AND / OR give 0 or 1. Where the host process would trap - division or remainder by zero, and the most
 * negative value divided by -1 - the call returns DH_ERR_DOMAIN (res then holds 0 at those items);
 * only DIV and MOD synchronise the stream for that check.
 *
 * Aggregations: SUM PROD MIN MAX and (dh_agg_row_idx / dh_agg_col_idx) IDXMIN IDXMAX; sums wrap.
 * MEAN VAR STDDEV return DH_ERR_RUNTIME for integers (the reference's device library has none
 * either; its CPU kernel divides in integer arithmetic, kernels/AggAll.h:163-191). */
dh_status dh_ew_binary_si64(dh_ctx *ctx, int op, int64_t *res, size_t ld_res, const int64_t *lhs,
                            size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const int64_t *rhs,
                            size_t rhs_rows, size_t rhs_cols, size_t ld_rhs);
dh_status dh_ew_binary_sca_si64(dh_ctx *ctx, int op, int64_t *res, size_t ld_res, const int64_t *lhs,
                                size_t rows, size_t cols, size_t ld_lhs, int64_t rhs);
dh_status dh_ew_binary_ui64(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const uint64_t *lhs,
                            size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const uint64_t *rhs,
                            size_t rhs_rows, size_t rhs_cols, size_t ld_rhs);
dh_status dh_ew_binary_sca_ui64(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const uint64_t *lhs,
                                size_t rows, size_t cols, size_t ld_lhs, uint64_t rhs);
dh_status dh_ew_binary_si32(dh_ctx *ctx, int op, int32_t *res, size_t ld_res, const int32_t *lhs,
                            size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const int32_t *rhs,
                            size_t rhs_rows, size_t rhs_cols, size_t ld_rhs);
dh_status dh_ew_binary_sca_si32(dh_ctx *ctx, int op, int32_t *res, size_t ld_res, const int32_t *lhs,
                                size_t rows, size_t cols, size_t ld_lhs, int32_t rhs);
dh_status dh_ew_binary_ui32(dh_ctx *ctx, int op, uint32_t *res, size_t ld_res, const uint32_t *lhs,
                            size_t lhs_rows, size_t lhs_cols, size_t ld_lhs, const uint32_t *rhs,
                            size_t rhs_rows, size_t rhs_cols, size_t ld_rhs);
dh_status dh_ew_binary_sca_ui32(dh_ctx *ctx, int op, uint32_t *res, size_t ld_res, const uint32_t *lhs,
                                size_t rows, size_t cols, size_t ld_lhs, uint32_t rhs);

dh_status dh_agg_all_si64(dh_ctx *ctx, int op, const int64_t *arg, size_t rows, size_t cols, size_t ld,
                          int64_t *result_host);
dh_status dh_agg_row_si64(dh_ctx *ctx, int op, int64_t *res, size_t ld_res, const int64_t *arg,
                          size_t rows, size_t cols, size_t ld);
dh_status dh_agg_row_idx_si64(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const int64_t *arg,
                              size_t rows, size_t cols, size_t ld);
dh_status dh_agg_col_si64(dh_ctx *ctx, int op, int64_t *res, const int64_t *arg, size_t rows,
                          size_t cols, size_t ld);
dh_status dh_agg_col_idx_si64(dh_ctx *ctx, int op, uint64_t *res, const int64_t *arg, size_t rows,
                              size_t cols, size_t ld);

dh_status dh_fill_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, int64_t value, size_t rows, size_t cols);
dh_status dh_fill_ui64(dh_ctx *ctx, uint64_t *res, size_t ld_res, uint64_t value, size_t rows, size_t cols);
dh_status dh_col_bind_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, const int64_t *lhs, size_t lhs_rows,
                           size_t lhs_cols, size_t ld_lhs, const int64_t *rhs, size_t rhs_rows,
                           size_t rhs_cols, size_t ld_rhs);
dh_status dh_extract_col_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, const int64_t *arg, size_t rows,
                              size_t cols, size_t ld, const int64_t *sel, size_t sel_rows,
                              size_t sel_cols, size_t ld_sel);
/* Transpose has no integer instantiation in the reference (cublas geam); provided for completeness. */
dh_status dh_transpose_si64(dh_ctx *ctx, int64_t *res, size_t ld_res, const int64_t *arg, size_t rows,
                            size_t cols, size_t ld);


/* ------------------------------------------------------------------------------------ */
/* DNN training kernels                                                                  */
/* ------------------------------------------------------------------------------------ */
/* Device counterparts of kernels the reference has on the CPU only. Images are rows: data is
 * N x (C*H*W), per-channel parameters are vectors of `channels` values in device memory.
 *
 * BatchNorm2DTrainForward<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/BatchNorm2DTrainForward.h:66-118):
 * per channel mean and (population) variance over all images and pixels; mean[c], inv_var[c] =
 * 1 / sqrt(var + eps), new_ema_x[c] = (1 - mu) * ema_x[c] + mu * x, res = gamma * (in - mean) /
 * sqrt(var + eps) + beta. (The reference allocates its four statistics results as C x C matrices and fills
 * the first C values; here they are C values.) */
dh_status dh_batchnorm_train_forward_f32(dh_ctx *ctx, float *res, float *new_ema_mean, float *new_ema_var,
                                         float *mean, float *inv_var, const float *in, size_t rows, size_t cols,
                                         const float *gamma, const float *beta, const float *ema_mean,
                                         const float *ema_var, size_t channels, float eps, float mu);
dh_status dh_batchnorm_train_forward_f64(dh_ctx *ctx, double *res, double *new_ema_mean, double *new_ema_var,
                                         double *mean, double *inv_var, const double *in, size_t rows, size_t cols,
                                         const double *gamma, const double *beta, const double *ema_mean,
                                         const double *ema_var, size_t channels, double eps, double mu);

/* BatchNorm2DBackward<...>::apply (kernels/BatchNorm2DBackward.h:63-120): dBeta = sum dout, dGamma =
 * sum dout * (in - mean) * inv_var, dX as derived there; `mean` and `inv_var` are the results of the
 * training forward pass. eps is accepted and unused, as in the reference. */
dh_status dh_batchnorm_backward_f32(dh_ctx *ctx, float *dX, float *dGamma, float *dBeta, const float *mean,
                                    const float *inv_var, const float *in, const float *dout, size_t rows,
                                    size_t cols, const float *gamma, size_t channels, float eps);
dh_status dh_batchnorm_backward_f64(dh_ctx *ctx, double *dX, double *dGamma, double *dBeta, const double *mean,
                                    const double *inv_var, const double *in, const double *dout, size_t rows,
                                    size_t cols, const double *gamma, size_t channels, double eps);

/* MaxPoolBackward / AvgPoolBackward<...>::apply (kernels/MaxPoolBackward.h:35-82, AvgPoolBackward.h:35-77):
 * res (N x C*H*W) = gradient w.r.t. the pooling input, dOut is N x (C*P*Q) with P and Q as in the forward
 * kernels (P from stride_w, Q from stride_h). MAX sends a window's gradient to its first maximum in
 * row-major order over the zero-padded image (what lands on the padding is dropped); AVG spreads
 * dOut / (pool_h * pool_w) over the window. */
dh_status dh_maxpool_backward_f32(dh_ctx *ctx, float *res, const float *input, const float *dOut, size_t N,
                                  size_t C, size_t H, size_t W, size_t pool_h, size_t pool_w, size_t stride_h,
                                  size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_maxpool_backward_f64(dh_ctx *ctx, double *res, const double *input, const double *dOut, size_t N,
                                  size_t C, size_t H, size_t W, size_t pool_h, size_t pool_w, size_t stride_h,
                                  size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_avgpool_backward_f32(dh_ctx *ctx, float *res, const float *input, const float *dOut, size_t N,
                                  size_t C, size_t H, size_t W, size_t pool_h, size_t pool_w, size_t stride_h,
                                  size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_avgpool_backward_f64(dh_ctx *ctx, double *res, const double *input, const double *dOut, size_t N,
                                  size_t C, size_t H, size_t W, size_t pool_h, size_t pool_w, size_t stride_h,
                                  size_t stride_w, size_t pad_h, size_t pad_w);

/* Conv2DBackwardData<...>::apply (kernels/Conv2DBackwardData.h:88-158): dX (N x C*H*W) from the filter
 * (F x C*Hf*Wf) and the output gradient dY (N x F*P*Q) - the adjoint of dh_conv2d_forward in its data
 * argument. The reference's kernel is consistent only where the output extent equals the filter extent
 * and pad_h == pad_w (its loops use the filter's extent for dY, :72-82,142); results coincide there.
 * Conv2DBackwardFilter<...>::apply (kernels/Conv2DBackwardFilter.h:68-152): dW (F x C*Hf*Wf) from the
 * input and dY - the adjoint in the filter argument. */
dh_status dh_conv2d_backward_data_f32(dh_ctx *ctx, float *dX, const float *filter, const float *dY, size_t N,
                                         size_t C, size_t H, size_t W, size_t F, size_t Hf, size_t Wf,
                                         size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_conv2d_backward_data_f64(dh_ctx *ctx, double *dX, const double *filter, const double *dY, size_t N,
                                         size_t C, size_t H, size_t W, size_t F, size_t Hf, size_t Wf,
                                         size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_conv2d_backward_filter_f32(dh_ctx *ctx, float *dW, const float *input, const float *dY, size_t N,
                                         size_t C, size_t H, size_t W, size_t F, size_t Hf, size_t Wf,
                                         size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w);
dh_status dh_conv2d_backward_filter_f64(dh_ctx *ctx, double *dW, const double *input, const double *dY, size_t N,
                                         size_t C, size_t H, size_t W, size_t F, size_t Hf, size_t Wf,
                                         size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w);



/* ------------------------------------------------------------------------------------ */
/* normal equations                                                                      */
/* ------------------------------------------------------------------------------------ */
/* A (cols x cols) = t(X) X + lambda I and b (cols x 1, stride ldb) = t(X) y from ONE pass over X (rows x cols):
 * what scripts/algorithms/lmDS_.daph:60-75 computes as `A = syrk(X) + diagMatrix(lambda)` and `b = t(X) @ y`, i.e.
 * the operator sequence Syrk (kernels/Syrk.h:51-93) + EwBinaryObjSca MUL + EwBinaryMat ADD + MatMul with transa
 * (kernels/MatMul.h) - two reads of X and five launches there. For 65..128 columns and at least 4096 rows only the
 * upper triangle of the product is computed on the matrix cores and t(X) y rides along on the ordinary ALUs; other
 * shapes run the sequence dh_syrk, a diagonal add, dh_gemv. Results equal the operator sequence's within the
 * tolerances of the tests (sums in another order). y is rows x 1 with stride ldy. */
dh_status dh_normal_equations_f32(dh_ctx *ctx, float *A, size_t lda, float *b, size_t ldb, const float *X, size_t rows,
                                  size_t cols, size_t ldx, const float *y, size_t ldy, float lambda);
dh_status dh_normal_equations_f64(dh_ctx *ctx, double *A, size_t lda, double *b, size_t ldb, const double *X, size_t rows,
                                  size_t cols, size_t ldx, const double *y, size_t ldy, double lambda);

/* ------------------------------------------------------------------------------------ */
/* fused vectorized pipeline                                                             */
/* ------------------------------------------------------------------------------------ */
/* Device side of VectorizedPipeline<DenseMatrix<VT>>::apply
 * (runtime/local/kernels/VectorizedPipeline.h:35-69) and of the device worker that runs a
 * pipeline body operator by operator on row chunks (runtime/local/vectorized/TasksCUDA.cpp:21-63,
 * MTWrapper_dense.cpp:203-336). Here the body is given as a short instruction list and runs as
 * one kernel over all rows: inputs split by ROWS, outputs combined by ROWS (tile / row
 * stores) or ADD / MIN / MAX (REDUCE_ALL), the split/combine kinds of
 * ir/daphneir/DaphneVectorizableOpInterface.td:23-34.
 *
 * Two implicit values per row: t, the row tile (cols values) which starts as the row of the
 * primary input x, and r, the row scalar set by ROW_AGG. `domain` selects which of them an
 * elementwise instruction works on (0 = t, 1 = r). */
#define DH_PIPE_MAX_INSTR 16
#define DH_PIPE_MAX_OPERANDS 4

typedef enum dh_pipe_kind {
    DH_PIPE_EW_BINARY = 0,     /* t|r = op(t|r, operand); swap != 0: op(operand, t|r); op: dh_binary_op */
    DH_PIPE_EW_UNARY = 1,      /* t|r = op(t|r); op: dh_unary_op                                        */
    DH_PIPE_ROW_AGG = 2,       /* r = agg(t); op: dh_agg_op (IDXMIN / IDXMAX give the index as a value)   */
    DH_PIPE_STORE_TILE = 3,    /* out_tile[index] row = t                                                 */
    DH_PIPE_STORE_ROW = 4,     /* out_row[index][row] = r (value type)                                    */
    DH_PIPE_STORE_ROW_IDX = 5, /* out_row[index][row] = (uint64_t) r                                      */
    DH_PIPE_REDUCE_ALL = 6     /* out_all[index] = combine over all rows of r (domain 1) or of every item
                                  of t (domain 0); op: DH_AGG_SUM / MIN / MAX; index 0 or 1               */
} dh_pipe_kind;

typedef enum dh_pipe_operand {
    DH_OPD_SCALAR = 0, /* the immediate `scalar`                                  */
    DH_OPD_SELF = 1,   /* t (or r) itself, e.g. t * t                             */
    DH_OPD_ROWVEC = 2, /* rowvec[index], 1 x cols, broadcast over rows (domain 0) */
    DH_OPD_COLVEC = 3, /* colvec[index], rows x 1, broadcast over columns         */
    DH_OPD_MATRIX = 4, /* matrix[index], rows x cols (domain 0)                   */
    DH_OPD_ROWREG = 5  /* r broadcast over the row (domain 0)                     */
} dh_pipe_operand;

typedef struct dh_pipe_instr {
    int32_t kind;    /* dh_pipe_kind */
    int32_t op;      /* op code of the kind's enum */
    int32_t domain;  /* 0: row tile t, 1: row scalar r */
    int32_t operand; /* dh_pipe_operand (EW_BINARY only) */
    int32_t index;   /* operand / output slot */
    int32_t swap;    /* EW_BINARY: operand on the left-hand side */
    double scalar;   /* DH_OPD_SCALAR immediate */
} dh_pipe_instr;

#define DH_PIPE_IO(SUF, T)                                                                         \
    typedef struct dh_pipe_io_##SUF {                                                              \
        const T *x;                 /* primary input, rows x cols */                               \
        size_t ld_x;                                                                               \
        const T *matrix[DH_PIPE_MAX_OPERANDS];                                                     \
        size_t ld_matrix[DH_PIPE_MAX_OPERANDS];                                                    \
        const T *rowvec[DH_PIPE_MAX_OPERANDS];                                                     \
        const T *colvec[DH_PIPE_MAX_OPERANDS];                                                     \
        size_t ld_colvec[DH_PIPE_MAX_OPERANDS];                                                    \
        T *out_tile[DH_PIPE_MAX_OPERANDS];                                                         \
        size_t ld_out_tile[DH_PIPE_MAX_OPERANDS];                                                  \
        void *out_row[DH_PIPE_MAX_OPERANDS]; /* T or uint64_t per row */                           \
        size_t ld_out_row[DH_PIPE_MAX_OPERANDS];                                                   \
        T *out_all[2];              /* device scalars */                                           \
    } dh_pipe_io_##SUF;
DH_PIPE_IO(f32, float)
DH_PIPE_IO(f64, double)
#undef DH_PIPE_IO

/* Runs `num_instr` instructions over every row. Unbound slots are NULL. Rows wider than
 * 1024 floats / 512 doubles do not fit the register tile: DH_ERR_RUNTIME, and the caller runs
 * the operators one by one. Unary domain errors are reported as for dh_ew_unary_*. */
dh_status dh_vectorized_pipeline_f32(dh_ctx *ctx, const dh_pipe_instr *program, int num_instr,
                                     const dh_pipe_io_f32 *io, size_t rows, size_t cols);
dh_status dh_vectorized_pipeline_f64(dh_ctx *ctx, const dh_pipe_instr *program, int num_instr,
                                     const dh_pipe_io_f64 *io, size_t rows, size_t cols);

/* A pipeline body is specialised at run time: the kernel source is compiled once per distinct
 * instruction list (hiprtc) and cached, the counterpart of the reference JIT-compiling every
 * VectorizedPipelineOp body (compiler/lowering/LowerToLLVMPass.cpp:654-726). If that is
 * switched off (environment DH_PIPELINE_JIT=0) or fails, a generic kernel interprets the list.
 * Returns how the calling thread's last pipeline ran: 1 specialised, 0 interpreted. */
int dh_vectorized_pipeline_last_mode(void);
/* How bodies run on this context: 1 specialised at run time, 0 interpreted by the generic kernel, -1 (the
 * initial setting) as the environment says. A specialisation that fails does not fail the call: the body is
 * interpreted, dh_vectorized_pipeline_last_mode() returns 0 and dh_last_error() holds the compiler's output. */
dh_status dh_ctx_set_pipeline_mode(dh_ctx *ctx, int mode);
int dh_ctx_get_pipeline_mode(const dh_ctx *ctx);
/* Number of specialised bodies this process holds. A body is keyed by its instruction kinds, op codes,
 * operand slots, value type and row width; its immediates are kernel arguments, so a scalar that changes
 * from call to call (a threshold, a learning rate) reuses the compiled kernel. At most 128 bodies stay
 * loaded by default, the least recently used one is unloaded beyond that. Compiled code is also kept on disk
 * between processes ($DH_PIPELINE_JIT_CACHE, "0" / "off": nowhere; else $XDG_CACHE_HOME/daphne_hip, else
 * $HOME/.cache/daphne_hip), named by and checked against the compiler's version, the options and the source. */
size_t dh_vectorized_pipeline_cache_size(void);
/* Sets how many specialised bodies stay loaded (at least 1) and returns the previous limit. A body that leaves the
 * cache is unloaded once no caller is about to launch it and its device has drained. */
size_t dh_vectorized_pipeline_set_cache_limit(size_t bodies);
/* Compiles the specialised kernel of a body for rows of `cols` values without loading or running
 * it (no device needed). value_type 0 = float, 1 = double; vectorised != 0: rows are read as
 * 16-byte vectors (cols a multiple of 4 / 2), as the launch does for aligned operands. */
dh_status dh_vectorized_pipeline_compile_check(int value_type, size_t cols, int vectorised,
                                               const dh_pipe_instr *program, int num_instr);

#ifdef __cplusplus
}
#endif
#endif /* DAPHNE_HIP_H */
