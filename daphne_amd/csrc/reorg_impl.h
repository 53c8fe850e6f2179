// Data reorganisation kernels for DenseMatrix<float|double>: Fill, ColBind, ExtractCol, Transpose.
// They stand in for kernels/CUDA/{Fill.cu,ColBind.cu,ExtractCol.cu,Transpose.cpp} of the reference
// (paths relative to src/runtime/local/) with the argument checks of the CPU kernels
// (kernels/ColBind.h:58-91, kernels/ExtractCol.h:57-114, kernels/Transpose.h:51-76), and all take
// leading dimensions so that views work. Instantiated per value type by reorg_f32.hip / reorg_f64.hip.
//
// All four are pure HBM traffic; each thread moves one 16-byte vector where pointers and leading
// dimensions allow it, a scalar otherwise, in one-shot grids (no grid-stride loops).
#pragma once

#include "common.h"

#include <cmath>

namespace dh_reorg {

// dst[r][c] = src ? src[r][c] : value, for a cols-wide block (cols counted in vectors of VEC)
template <typename T, int VEC, bool FILL>
__global__ __launch_bounds__(256) void block2d_kernel(T *dst, size_t ld_dst, const T *src, size_t ld_src, size_t rows,
                                                      size_t cvecs, T value) {
    const size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y; // rows on grid.x: no 65535 limit
    if (cv >= cvecs || r >= rows)
        return;
    T v[VEC];
    if constexpr (FILL) {
#pragma unroll
        for (int i = 0; i < VEC; i++)
            v[i] = value;
    } else {
        dh_load_vec_stream<T, VEC>(src + r * ld_src + cv * VEC, v);
    }
    dh_store_vec<T, VEC>(dst + r * ld_dst + cv * VEC, v);
}

template <typename T, bool FILL>
static inline dh_status block2d(dh_ctx *ctx, T *dst, size_t ld_dst, const T *src, size_t ld_src, size_t rows, size_t cols,
                                T value) {
    if (rows == 0 || cols == 0)
        return DH_OK;
    constexpr int V = 16 / sizeof(T);
    // a contiguous block is one long row: keeps narrow matrices on full-width vectors
    if (ld_dst == cols && (FILL || ld_src == cols)) {
        const size_t total = rows * cols;
        size_t w = 256 * V;
        while (w > 1 && total % w)
            w >>= 1;
        if (w >= static_cast<size_t>(V)) {
            cols = w;
            rows = total / w;
            ld_dst = w;
            ld_src = w;
        }
    }
    const bool vec = cols % V == 0 && ld_dst % V == 0 && dh_aligned(dst, 16) && (FILL || (ld_src % V == 0 && dh_aligned(src, 16)));
    const size_t cvecs = vec ? cols / V : cols;
    unsigned tx = 1;
    while (tx < 256 && tx < cvecs)
        tx <<= 1;
    const unsigned ty = 256 / tx;
    const size_t gcols = dh_ceil_div(cvecs, tx), grows = dh_ceil_div(rows, ty);
    if (gcols >= 65536 || grows >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "matrix extents exceed one launch (%zu x %zu)", rows, cols);
    const dim3 grid(static_cast<unsigned>(grows), static_cast<unsigned>(gcols)), block(tx, ty);
    if (vec)
        hipLaunchKernelGGL((block2d_kernel<T, V, FILL>), grid, block, 0, ctx->stream, dst, ld_dst, src, ld_src, rows, cvecs,
                           value);
    else
        hipLaunchKernelGGL((block2d_kernel<T, 1, FILL>), grid, block, 0, ctx->stream, dst, ld_dst, src, ld_src, rows, cvecs,
                           value);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// Fill<DenseMatrix<VT>,VT>::apply (kernels/CUDA/Fill.cu:27-49)
template <typename T> dh_status fill(dh_ctx *ctx, T *res, size_t ld_res, T value, size_t rows, size_t cols) {
    DH_REQUIRE_CTX(ctx);
    if (ld_res < cols)
        return dh_fail(DH_ERR_RUNTIME, "Fill - leading dimension smaller than the column count");
    return block2d<T, true>(ctx, res, ld_res, nullptr, 0, rows, cols, value);
}

// One thread per 16-byte vector of the result row: whole result rows leave as contiguous runs.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void col_bind_kernel(T *res, size_t ld_res, const T *lhs, size_t ld_lhs, size_t lvecs,
                                                       const T *rhs, size_t ld_rhs, size_t rvecs, size_t rows) {
    const size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y; // rows on grid.x: no 65535 limit
    if (cv >= lvecs + rvecs || r >= rows)
        return;
    T v[VEC];
    if (cv < lvecs)
        dh_load_vec_stream<T, VEC>(lhs + r * ld_lhs + cv * VEC, v);
    else
        dh_load_vec_stream<T, VEC>(rhs + r * ld_rhs + (cv - lvecs) * VEC, v);
    dh_store_vec<T, VEC>(res + r * ld_res + cv * VEC, v);
}

// The same with the threads numbered through rows x vectors, for row widths that are not a power of two (a thread
// tile of TX lanes per row would leave lanes idle): one division per thread, 32-bit where the count allows.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void col_bind_flat_kernel(T *res, size_t ld_res, const T *lhs, size_t ld_lhs, size_t lvecs,
                                                            const T *rhs, size_t ld_rhs, size_t rvecs, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total)
        return;
    const size_t cvecs = lvecs + rvecs;
    size_t r, cv;
    if (total <= 0xffffffffull) {
        r = static_cast<unsigned>(i) / static_cast<unsigned>(cvecs);
        cv = static_cast<unsigned>(i) % static_cast<unsigned>(cvecs);
    } else {
        r = i / cvecs;
        cv = i % cvecs;
    }
    T v[VEC];
    if (cv < lvecs)
        dh_load_vec_stream<T, VEC>(lhs + r * ld_lhs + cv * VEC, v);
    else
        dh_load_vec_stream<T, VEC>(rhs + r * ld_rhs + (cv - lvecs) * VEC, v);
    dh_store_vec<T, VEC>(res + r * ld_res + cv * VEC, v);
}

// ColBind<DenseMatrix<VT>,...>::apply (kernels/ColBind.h:58-91, kernels/CUDA/ColBind.cu:47-70)
template <typename T>
dh_status col_bind(dh_ctx *ctx, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs, const T *rhs,
                   size_t rr, size_t rc, size_t ld_rhs) {
    DH_REQUIRE_CTX(ctx);
    if (lr != rr)
        return dh_fail(DH_ERR_RUNTIME,
                       "ColBind - the two operands must have the same number of rows, but lhs has %zu and rhs has %zu rows",
                       lr, rr);
    if (ld_res < lc + rc || ld_lhs < lc || ld_rhs < rc)
        return dh_fail(DH_ERR_RUNTIME, "ColBind - a leading dimension is smaller than its column count");
    constexpr int V = 16 / sizeof(T);
    const bool vec = lc % V == 0 && rc % V == 0 && ld_res % V == 0 && ld_lhs % V == 0 && ld_rhs % V == 0 &&
                     dh_aligned(res, 16) && dh_aligned(lhs, 16) && dh_aligned(rhs, 16);
    if (vec && lr > 0 && lc + rc > 0) {
        const size_t cvecs = (lc + rc) / V;
        if ((cvecs & (cvecs - 1)) != 0 && cvecs % 256 != 0 && dh_ceil_div(lr * cvecs, static_cast<size_t>(256)) < (size_t(1) << 31)) {
            const size_t total = lr * cvecs;
            hipLaunchKernelGGL((col_bind_flat_kernel<T, V>), dim3(static_cast<unsigned>(dh_ceil_div(total, static_cast<size_t>(256)))),
                               dim3(256), 0, ctx->stream, res, ld_res, lhs, ld_lhs, lc / V, rhs, ld_rhs, rc / V, total);
            DH_CHECK_LAUNCH();
            return DH_OK;
        }
        unsigned tx = 1;
        while (tx < 256 && tx < cvecs)
            tx <<= 1;
        const unsigned ty = 256 / tx;
        const size_t gcols = dh_ceil_div(cvecs, tx), grows = dh_ceil_div(lr, ty);
        if (gcols < 65536 && grows < (size_t(1) << 31)) {
            hipLaunchKernelGGL((col_bind_kernel<T, V>), dim3(static_cast<unsigned>(grows), static_cast<unsigned>(gcols)),
                               dim3(tx, ty), 0, ctx->stream, res, ld_res, lhs, ld_lhs, lc / V, rhs, ld_rhs, rc / V, lr);
            DH_CHECK_LAUNCH();
            return DH_OK;
        }
    }
    dh_status st = block2d<T, false>(ctx, res, ld_res, lhs, ld_lhs, lr, lc, T(0));
    if (st != DH_OK)
        return st;
    return block2d<T, false>(ctx, res + lc, ld_res, rhs, ld_rhs, lr, rc, T(0));
}

// Column positions: negative ones count from the end (kernels/ExtractCol.h:98-101); the first position
// that is still out of range is reported through the flag as index + 1.
static __global__ void check_sel_kernel(const long long *sel, size_t nsel, size_t ld_sel, size_t cols, int *flag) {
    for (size_t k = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; k < nsel;
         k += static_cast<size_t>(gridDim.x) * blockDim.x) {
        long long v = sel[k * ld_sel];
        if (v < 0)
            v += static_cast<long long>(cols);
        if (v < 0 || static_cast<unsigned long long>(v) >= cols)
            atomicMin(flag, static_cast<int>(k < 0x7ffffffe ? k + 1 : 0x7fffffff));
    }
}

template <typename T>
__global__ __launch_bounds__(256) void extract_col_kernel(T *res, size_t ld_res, const T *arg, size_t ld, size_t rows,
                                                          size_t cols, const long long *sel, size_t nsel, size_t ld_sel) {
    const size_t k = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r = static_cast<size_t>(blockIdx.x) * blockDim.y + threadIdx.y;
    if (k >= nsel || r >= rows)
        return;
    long long c = sel[k * ld_sel];
    if (c < 0)
        c += static_cast<long long>(cols);
    // a position that is out of range (reported by check_sel_kernel) reads column 0
    c = (c < 0 || static_cast<unsigned long long>(c) >= cols) ? 0 : c;
    res[r * ld_res + k] = arg[r * ld + static_cast<size_t>(c)];
}

// The same for selections that touch most of a row's 64-byte segments anyway (eight random columns of 64 floats reach
// 3.6 of the 4): the rows are streamed whole - a wavefront loads 4 KB of consecutive rows with four 16-byte vectors a
// lane, parks them in a piece of LDS of its own (no barrier: its LDS instructions execute in order) and picks the
// selected values from there, so that the results of its rows leave as one contiguous run.
// LPR: lanes (16-byte vectors) per row, a power of two up to 64.
template <typename T>
__global__ __launch_bounds__(256) void extract_col_rows_kernel(T *res, size_t ld_res, const T *arg, size_t ld, size_t rows,
                                                               unsigned cols, const long long *sel, unsigned nsel, size_t ld_sel,
                                                               unsigned lpr) {
    constexpr int VEC = 16 / sizeof(T), UN = 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char extract_lds[];
    unsigned *selc = reinterpret_cast<unsigned *>(extract_lds);                    // nsel positions, as given or counted from the end
    T *park = reinterpret_cast<T *>(extract_lds + ((nsel * 4u + 15u) & ~15u));     // 4 waves x UN KB
    const unsigned tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const unsigned rps = 64 / lpr, rpw = rps * UN;                                 // rows per load, rows per wavefront
    const size_t row0 = (static_cast<size_t>(blockIdx.x) * 4 + wave) * rpw;
    T v[UN][VEC];
#pragma unroll
    for (int u = 0; u < UN; u++) {
        size_t r = row0 + u * rps + lane / lpr;
        r = r < rows ? r : rows - 1; // beyond the end: the last row again, never stored
        dh_load_vec_stream<T, VEC>(arg + r * ld + (lane % lpr) * VEC, v[u]);
    }
    for (unsigned k = tid; k < nsel; k += 256) {
        long long c = sel[k * ld_sel];
        c = c < 0 ? c + static_cast<long long>(cols) : c;
        // a position that is out of range (reported by check_sel_kernel) reads column 0
        selc[k] = (c < 0 || c >= static_cast<long long>(cols)) ? 0u : static_cast<unsigned>(c);
    }
    T *mine = park + wave * (UN * 64 * VEC);
#pragma unroll
    for (int u = 0; u < UN; u++)
        dh_store_vec<T, VEC>(mine + (u * 64 + lane) * VEC, v[u]); // row u rps + lane / lpr at (that row) * cols: cols = lpr VEC
    __syncthreads(); // the positions
    if (row0 >= rows)
        return;
    const unsigned live = rows - row0 < rpw ? static_cast<unsigned>(rows - row0) : rpw;
    const unsigned nout = live * nsel;
    for (unsigned o = lane; o < nout; o += 64) {
        const unsigned r = o / nsel, k = o - r * nsel;
        dh_store_stream(res + (row0 + r) * ld_res + k, mine[r * cols + selc[k]]);
    }
}

// ExtractCol<DenseMatrix<VT>,DenseMatrix<VT>,DenseMatrix<int64_t>>::apply
// (kernels/ExtractCol.h:74-114, kernels/CUDA/ExtractCol.cu:21-56)
template <typename T>
dh_status extract_col(dh_ctx *ctx, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld,
                      const long long *sel, size_t sel_rows, size_t sel_cols, size_t ld_sel) {
    DH_REQUIRE_CTX(ctx);
    if (sel_cols != 1)
        return dh_fail(DH_ERR_RUNTIME,
                       "invalid argument passed to ExtractCol: column selection must be given as column matrix but has "
                       "'%zu' columns instead of one",
                       sel_cols);
    if (ld < cols || ld_res < sel_rows || ld_sel < 1)
        return dh_fail(DH_ERR_RUNTIME, "ExtractCol - a leading dimension is smaller than its column count");
    if (sel_rows == 0 || rows == 0)
        return DH_OK;
    // validate the positions first: the CPU kernel throws before anything is usable
    *ctx->flag_host = 0x7fffffff;
    DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_dev, ctx->flag_host, sizeof(int), hipMemcpyHostToDevice, ctx->stream));
    size_t cg = dh_ceil_div(sel_rows, 256);
    if (cg > 1024)
        cg = 1024;
    hipLaunchKernelGGL(check_sel_kernel, dim3(static_cast<unsigned>(cg)), dim3(256), 0, ctx->stream, sel, sel_rows, ld_sel,
                       cols, ctx->flag_dev);
    DH_CHECK_LAUNCH();
    if (ctx->deferred_depth > 0) {
        // the verdict waits for dh_check_deferred; the kernels below keep a bad position inside the row, and what
        // they then extract is never used
        if (dh_status st = dh_latch_deferred(ctx, 0x7fffffff, DH_DEFERRED_EXTRACT_COL, 0, sel, ld_sel, static_cast<long long>(cols));
            st != DH_OK)
            return st;
    } else {
        DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        if (*ctx->flag_host != 0x7fffffff) {
            const size_t bad = static_cast<size_t>(*ctx->flag_host) - 1;
            long long v = 0;
            DH_CHECK_HIP(hipMemcpy(&v, sel + bad * ld_sel, sizeof(v), hipMemcpyDeviceToHost));
            return dh_fail_extract_col(v, cols);
        }
    }
    {
        // whole rows where a gather would fetch most of them anyway: rows of a power-of-two number of 16-byte vectors
        // (up to 1 KB), an expected share of at least 60 % of a row's 64-byte segments hit by the selection
        constexpr size_t V = 16 / sizeof(T);
        const size_t row_bytes = cols * sizeof(T), lpr = cols / V;
        const double segments = row_bytes < 64 ? 1.0 : static_cast<double>(row_bytes) / 64.0;
        const double coverage = 1.0 - pow(1.0 - 1.0 / segments, static_cast<double>(sel_rows));
        const size_t rpw = lpr ? (64 / lpr) * 4 : 0;
        if (cols % V == 0 && lpr >= 1 && lpr <= 64 && (lpr & (lpr - 1)) == 0 && ld % V == 0 && dh_aligned(arg, 16) &&
            sel_rows <= 1024 && coverage >= 0.6 && rows >= 4096 && dh_ceil_div(rows, rpw * 4) < (size_t(1) << 31)) {
            const size_t lds = ((sel_rows * 4 + 15) & ~size_t(15)) + 4 * 4 * 1024;
            hipLaunchKernelGGL((extract_col_rows_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(rows, rpw * 4))), dim3(256), lds,
                               ctx->stream, res, ld_res, arg, ld, rows, static_cast<unsigned>(cols), sel,
                               static_cast<unsigned>(sel_rows), ld_sel, static_cast<unsigned>(lpr));
            DH_CHECK_LAUNCH();
            return DH_OK;
        }
    }
    unsigned tx = 1;
    while (tx < 256 && tx < sel_rows)
        tx <<= 1;
    const unsigned ty = 256 / tx;
    const size_t gcols = dh_ceil_div(sel_rows, tx), grows = dh_ceil_div(rows, ty);
    if (gcols >= 65536 || grows >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "ExtractCol - extents exceed one launch");
    hipLaunchKernelGGL((extract_col_kernel<T>), dim3(static_cast<unsigned>(grows), static_cast<unsigned>(gcols)), dim3(tx, ty),
                       0, ctx->stream, res, ld_res, arg, ld, rows, cols, sel, sel_rows, ld_sel);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// 64 x 64 tile through LDS: rows are read along columns of the source and written along columns of the
// result, both as contiguous 256-byte runs per wavefront; the odd LDS stride keeps the transposed read
// free of bank conflicts.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(T *res, size_t ld_res, const T *arg, size_t ld, size_t rows,
                                                        size_t cols) {
    constexpr int TS = 64;
    __shared__ T tile[TS][TS + 1];
    const int tx = threadIdx.x % TS, ty = threadIdx.x / TS; // 64 x 4
    const size_t r0 = static_cast<size_t>(blockIdx.x) * TS, c0 = static_cast<size_t>(blockIdx.y) * TS;
    // all sixteen loads of a thread are issued before the first LDS store (a guard around each load would make the
    // compiler wait for every one in turn): positions past the matrix read its last element, which is never stored
    T v[TS / 4];
#pragma unroll
    for (int k = 0; k < TS / 4; k++) {
        const size_t r = r0 + ty + 4 * k, c = c0 + tx;
        v[k] = arg[(r < rows ? r : rows - 1) * ld + (c < cols ? c : cols - 1)];
    }
#pragma unroll
    for (int k = 0; k < TS / 4; k++)
        tile[ty + 4 * k][tx] = v[k];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TS; i += 4) {
        const size_t orow = c0 + ty + i, ocol = r0 + tx; // result is cols x rows
        if (orow < cols && ocol < rows)
            res[orow * ld_res + ocol] = tile[tx][ty + i];
    }
}

// The same tile with 16-byte global accesses on both sides: a lane loads VEC consecutive source columns and
// later stores VEC consecutive result columns (= source rows). LDS is written and read with scalars (the odd
// stride that makes both directions conflict free rules out vector LDS accesses). Needs rows, cols and both
// leading dimensions to be multiples of VEC and 16-byte aligned pointers.
template <typename T>
__global__ __launch_bounds__(256) void transpose_vec_kernel(T *res, size_t ld_res, const T *arg, size_t ld, size_t rows,
                                                            size_t cols) {
    constexpr int TS = 64, VEC = 16 / sizeof(T);
    constexpr int LPR = TS / VEC;        // lanes per tile row
    constexpr int RPS = 256 / LPR;       // tile rows per step of the workgroup
    __shared__ T tile[TS][TS + 1];
    const int m = threadIdx.x % LPR, q = threadIdx.x / LPR;
    const size_t r0 = static_cast<size_t>(blockIdx.x) * TS, c0 = static_cast<size_t>(blockIdx.y) * TS;
    T v[TS / RPS][VEC];
#pragma unroll
    for (int s_ = 0; s_ < TS / RPS; s_++) {
        const size_t r = r0 + q + s_ * RPS, c = c0 + m * VEC;
        if (r < rows && c < cols)
            dh_load_vec_stream<T, VEC>(arg + r * ld + c, v[s_]);
    }
#pragma unroll
    for (int s_ = 0; s_ < TS / RPS; s_++)
#pragma unroll
        for (int e = 0; e < VEC; e++)
            tile[q + s_ * RPS][m * VEC + e] = v[s_][e];
    __syncthreads();
#pragma unroll
    for (int s_ = 0; s_ < TS / RPS; s_++) {
        const int cq = q + s_ * RPS; // source column inside the tile = result row
        const size_t orow = c0 + cq, ocol = r0 + m * VEC;
        T o[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++)
            o[e] = tile[m * VEC + e][cq];
        if (orow < cols && ocol < rows)
            dh_store_vec_stream<T, VEC>(res + orow * ld_res + ocol, o);
    }
}

// Transpose<DenseMatrix<VT>,DenseMatrix<VT>>::apply (kernels/Transpose.h:51-76, kernels/CUDA/Transpose.cpp)
template <typename T> dh_status transpose(dh_ctx *ctx, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols || ld_res < rows)
        return dh_fail(DH_ERR_RUNTIME, "Transpose - a leading dimension is smaller than its column count");
    if (rows == 0 || cols == 0)
        return DH_OK;
    const size_t gcols = dh_ceil_div(cols, 64), grows = dh_ceil_div(rows, 64);
    if (gcols >= 65536 || grows >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "Transpose - extents exceed one launch (%zu x %zu)", rows, cols);
    constexpr int V = 16 / sizeof(T);
    const bool vec = rows % V == 0 && cols % V == 0 && ld % V == 0 && ld_res % V == 0 && dh_aligned(arg, 16) &&
                     dh_aligned(res, 16);
    const dim3 grid(static_cast<unsigned>(grows), static_cast<unsigned>(gcols));
    if (vec)
        hipLaunchKernelGGL((transpose_vec_kernel<T>), grid, dim3(256), 0, ctx->stream, res, ld_res, arg, ld, rows, cols);
    else
        hipLaunchKernelGGL((transpose_kernel<T>), grid, dim3(256), 0, ctx->stream, res, ld_res, arg, ld, rows, cols);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

} // namespace dh_reorg
