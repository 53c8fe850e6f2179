// Aggregation kernels (full, per row, per column, index of row/column extremum) for
// DenseMatrix<float|double>; instantiated per value type by agg_f32.hip / agg_f64.hip.
//
// Semantics follow the reference's CPU kernels:
//   AggAll  runtime/local/kernels/AggAll.h:64-96,124-193   (SUM PROD MIN MAX MEAN VAR STDDEV)
//   AggRow  runtime/local/kernels/AggRow.h:60-161          (+ IDXMIN / IDXMAX at :71-94)
//   AggCol  runtime/local/kernels/AggCol.h:58-178          (+ IDXMIN / IDXMAX at :70-122)
// What is kept from them: population variance (divide by N); MIN/MAX built on std::min /
// std::max, so a NaN never replaces the running value, and the running value of AggRow / AggCol
// starts at the first element (a NaN there is the result) while AggAll starts at +-inf (NaNs are
// ignored); IDXMIN / IDXMAX return the first position of the strict extremum and position 0 if
// the first element is NaN. What differs is only the summation order (trees instead of one
// sequential chain), which is why floating-point results are compared with a tolerance.
//
// Mapping to the hardware: every kernel streams its input once with 16-byte loads, with the
// lanes of a wavefront on consecutive addresses. Row aggregations give each row to a group of
// G = 1..64 lanes (a 64-wide f32 row is 16 lanes x float4, four rows per wavefront) and finish
// with cross-lane shuffles, so a tall-skinny matrix needs neither one block per row nor LDS.
// Column aggregations give each block a contiguous slab of rows, keep per-column partials in
// registers, fold the TY row-lanes of the block through LDS and leave one partial row per block
// for a small second kernel; no atomics, so results are deterministic. Variance per column is
// computed in the same single pass as (count, mean, M2) triples merged with Chan's formula.
#pragma once

#include "common.h"

#include <cmath>
#include <limits>

namespace dh_agg {

constexpr int THREADS = 256;
constexpr int UNROLL = 4;

template <typename T> struct RSum {
    static __device__ __forceinline__ T id() { return T(0); }
    static __device__ __forceinline__ T comb(T a, T b) { return a + b; }
};
template <typename T> struct RProd {
    static __device__ __forceinline__ T id() { return T(1); }
    static __device__ __forceinline__ T comb(T a, T b) { return a * b; }
};
// identity of MIN (largest) / MAX (smallest): the infinities, or the extreme values of an integer type
template <typename T> __device__ __forceinline__ constexpr T agg_largest() {
    return std::numeric_limits<T>::is_integer ? std::numeric_limits<T>::max() : std::numeric_limits<T>::infinity();
}
template <typename T> __device__ __forceinline__ constexpr T agg_smallest() {
    return std::numeric_limits<T>::is_integer ? std::numeric_limits<T>::lowest() : -std::numeric_limits<T>::infinity();
}
template <typename T> constexpr bool agg_is_int = std::numeric_limits<T>::is_integer;
template <typename T> struct RMin {
    static __device__ __forceinline__ T id() { return agg_largest<T>(); }
    static __device__ __forceinline__ T comb(T a, T b) { return (b < a) ? b : a; }
};
template <typename T> struct RMax {
    static __device__ __forceinline__ T id() { return agg_smallest<T>(); }
    static __device__ __forceinline__ T comb(T a, T b) { return (a < b) ? b : a; }
};

template <typename T> __device__ __forceinline__ T dev_sqrt(T a);
template <> __device__ __forceinline__ float dev_sqrt<float>(float a) { return sqrtf(a); }
template <> __device__ __forceinline__ double dev_sqrt<double>(double a) { return sqrt(a); }
template <> __device__ __forceinline__ long dev_sqrt<long>(long a) { return static_cast<long>(sqrt(static_cast<double>(a))); }
template <typename T> __device__ __forceinline__ bool dev_isnan(T a) { return a != a; }

template <typename T, int VEC> __device__ __forceinline__ void load_vec(const T *p, T (&v)[VEC]) {
    if constexpr (VEC == 1) {
        v[0] = *p;
    } else {
        using V = typename dh_vec<T>::type;
        V t = *reinterpret_cast<const V *>(p);
        const T *tp = reinterpret_cast<const T *>(&t);
#pragma unroll
        for (int i = 0; i < VEC; i++)
            v[i] = tp[i];
    }
}

template <typename T, class R> __device__ __forceinline__ T wave_reduce(T v) {
    dh_butterfly(DH_WAVE, [&](auto peer) { v = R::comb(v, peer(v)); });
    return v;
}

// Reduces over the whole block; the result is valid in thread 0.
template <typename T, class R> __device__ __forceinline__ T block_reduce(T v) {
    __shared__ T lds[THREADS / DH_WAVE];
    const int tid = threadIdx.y * blockDim.x + threadIdx.x;
    v = wave_reduce<T, R>(v);
    if ((tid % DH_WAVE) == 0)
        lds[tid / DH_WAVE] = v;
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int w = 1; w < THREADS / DH_WAVE; w++)
            v = R::comb(v, lds[w]);
    }
    __syncthreads();
    return v;
}

// =======================================================================================
// AggAll
// =======================================================================================
// Stage 1: block b owns the contiguous rows [b*slab, (b+1)*slab) and walks them with (TX, TY) threads over
// rows x cvecs vectors; one partial per block.
template <typename T, int VEC, class R, bool SQDEV>
__global__ __launch_bounds__(THREADS) void all_stage1(const T *arg, size_t rows, size_t cvecs, size_t ld, size_t slab,
                                                      const T *mean_dev, T *partials) {
    T m = T(0);
    if constexpr (SQDEV)
        m = *mean_dev;
    T acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++)
        acc[i] = R::id();
    const size_t row_step = blockDim.y;
    const size_t r_begin = static_cast<size_t>(blockIdx.x) * slab;
    const size_t r_end = (r_begin + slab < rows) ? r_begin + slab : rows;
    for (size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x; cv < cvecs;
         cv += static_cast<size_t>(gridDim.y) * blockDim.x) {
        // main loop: UNROLL independent, unguarded loads in flight; then a guarded tail
        size_t r0 = r_begin + threadIdx.y;
        for (; r0 + (UNROLL - 1) * row_step < r_end; r0 += row_step * UNROLL) {
            T x[UNROLL][VEC];
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
                dh_load_vec_stream<T, VEC>(arg + (r0 + u * row_step) * ld + cv * VEC, x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                for (int i = 0; i < VEC; i++) {
                    T v = x[u][i];
                    if constexpr (SQDEV)
                        v = (v - m) * (v - m);
                    acc[i] = R::comb(acc[i], v);
                }
            }
        }
        for (; r0 < r_end; r0 += row_step) {
            T x[VEC];
            dh_load_vec_stream<T, VEC>(arg + r0 * ld + cv * VEC, x);
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                T v = x[i];
                if constexpr (SQDEV)
                    v = (v - m) * (v - m);
                acc[i] = R::comb(acc[i], v);
            }
        }
    }
    T a = acc[0];
#pragma unroll
    for (int i = 1; i < VEC; i++)
        a = R::comb(a, acc[i]);
    a = block_reduce<T, R>(a);
    if (threadIdx.x == 0 && threadIdx.y == 0)
        partials[static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x] = a;
}

// Stage 2: one block folds the partials. FINAL: 0 as is, 1 divide by count, 2 divide then sqrt.
template <typename T, class R, int FINAL>
__global__ __launch_bounds__(THREADS) void all_stage2(const T *partials, size_t np, T *out, T count) {
    T a = R::id();
    for (size_t i = threadIdx.x; i < np; i += THREADS)
        a = R::comb(a, partials[i]);
    a = block_reduce<T, R>(a);
    if (threadIdx.x == 0) {
        if constexpr (FINAL >= 1)
            a = a / count;
        if constexpr (FINAL == 2)
            a = dev_sqrt<T>(a);
        out[0] = a;
    }
}

struct Plan2D {
    dim3 grid, block;
    size_t nblocks, slab;
};
static inline Plan2D plan2d(const dh_ctx *ctx, size_t rows, size_t cvecs) {
    unsigned tx = 1;
    while (tx < THREADS && tx < cvecs)
        tx <<= 1;
    unsigned ty = THREADS / tx;
    size_t gy = dh_ceil_div(cvecs, tx);
    if (gy > 512)
        gy = 512;
    const size_t max_blocks = static_cast<size_t>(ctx->num_cus) * 8;
    const size_t min_slab = static_cast<size_t>(ty) * UNROLL;
    size_t gx = dh_ceil_div(rows, min_slab);
    size_t cap = max_blocks / gy;
    if (cap < 1)
        cap = 1;
    if (gx > cap)
        gx = cap;
    if (gx < 1)
        gx = 1;
    size_t slab = dh_ceil_div(dh_ceil_div(rows, gx), min_slab) * min_slab;
    gx = dh_ceil_div(rows, slab);
    if (gx < 1)
        gx = 1;
    Plan2D p;
    p.slab = slab;
    p.grid = dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy), 1);
    p.block = dim3(tx, ty, 1);
    p.nblocks = gx * gy;
    return p;
}

// Runs stage 1 over (rows, cols, ld) - flat if contiguous - and returns the number of partials.
template <typename T, class R, bool SQDEV>
static inline size_t all_stage1_launch(dh_ctx *ctx, const T *arg, size_t rows, size_t cols, size_t ld,
                                       const T *mean_dev, T *partials) {
    constexpr int V = dh_vec<T>::N;
    size_t np = 0;
    if (ld == cols || rows == 1) {
        const size_t n = rows * cols;
        const size_t width = static_cast<size_t>(THREADS) * V;
        const size_t body_rows = dh_aligned(arg, 16) ? n / width : 0;
        if (body_rows) {
            Plan2D p = plan2d(ctx, body_rows, THREADS);
            hipLaunchKernelGGL((all_stage1<T, V, R, SQDEV>), p.grid, p.block, 0, ctx->stream, arg, body_rows,
                               size_t(THREADS), width, p.slab, mean_dev, partials);
            np += p.nblocks;
        }
        const size_t done = body_rows * width;
        if (done < n) {
            Plan2D p = plan2d(ctx, 1, n - done);
            hipLaunchKernelGGL((all_stage1<T, 1, R, SQDEV>), p.grid, p.block, 0, ctx->stream, arg + done, size_t(1),
                               n - done, n - done, p.slab, mean_dev, partials + np);
            np += p.nblocks;
        }
        return np;
    }
    const bool vec_ok = (cols % V == 0) && (ld % V == 0) && dh_aligned(arg, 16);
    if (vec_ok) {
        Plan2D p = plan2d(ctx, rows, cols / V);
        hipLaunchKernelGGL((all_stage1<T, V, R, SQDEV>), p.grid, p.block, 0, ctx->stream, arg, rows, cols / V, ld,
                           p.slab, mean_dev, partials);
        np = p.nblocks;
    } else {
        Plan2D p = plan2d(ctx, rows, cols);
        hipLaunchKernelGGL((all_stage1<T, 1, R, SQDEV>), p.grid, p.block, 0, ctx->stream, arg, rows, cols, ld,
                           p.slab, mean_dev, partials);
        np = p.nblocks;
    }
    return np;
}

template <typename T> dh_status agg_all_dev(dh_ctx *ctx, int op, const T *arg, size_t rows, size_t cols, size_t ld, T *out) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols)
        return dh_fail(DH_ERR_RUNTIME, "AggAll - leading dimension smaller than the column count");
    if (op == DH_AGG_IDXMIN || op == DH_AGG_IDXMAX || op < 0 || op > DH_AGG_VAR)
        return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode"); // AggAll.h:147,161
    if constexpr (agg_is_int<T>) {
        // The reference's integer MEAN / VAR / STDDEV divide and subtract in integer arithmetic (AggAll.h:163-191);
        // its device library has SUM / MIN / MAX for si64 only (CUDA/AggAll.cu:155, AggRow.cu:146, AggCol.cu:89).
        if (op == DH_AGG_MEAN || op == DH_AGG_VAR || op == DH_AGG_STDDEV)
            return dh_fail(DH_ERR_RUNTIME, "%s: MEAN, VAR and STDDEV of integer value types are not supported on the device", __func__);
    }
    void *wsv = nullptr;
    const size_t max_partials = static_cast<size_t>(ctx->num_cus) * 8 * 2 + 1024 + 16;
    dh_status st = dh_workspace(ctx, (max_partials + 64) * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    T *mean_slot = static_cast<T *>(wsv); // first 256 bytes: the mean for the variance pass
    T *partials = reinterpret_cast<T *>(static_cast<char *>(wsv) + 256);
    const T count = static_cast<T>(rows * cols);
    size_t np;
    switch (op) {
    case DH_AGG_SUM:
        np = all_stage1_launch<T, RSum<T>, false>(ctx, arg, rows, cols, ld, nullptr, partials);
        hipLaunchKernelGGL((all_stage2<T, RSum<T>, 0>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        break;
    case DH_AGG_PROD:
        np = all_stage1_launch<T, RProd<T>, false>(ctx, arg, rows, cols, ld, nullptr, partials);
        hipLaunchKernelGGL((all_stage2<T, RProd<T>, 0>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        break;
    case DH_AGG_MIN:
        np = all_stage1_launch<T, RMin<T>, false>(ctx, arg, rows, cols, ld, nullptr, partials);
        hipLaunchKernelGGL((all_stage2<T, RMin<T>, 0>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        break;
    case DH_AGG_MAX:
        np = all_stage1_launch<T, RMax<T>, false>(ctx, arg, rows, cols, ld, nullptr, partials);
        hipLaunchKernelGGL((all_stage2<T, RMax<T>, 0>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        break;
    case DH_AGG_MEAN:
        np = all_stage1_launch<T, RSum<T>, false>(ctx, arg, rows, cols, ld, nullptr, partials);
        hipLaunchKernelGGL((all_stage2<T, RSum<T>, 1>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        break;
    case DH_AGG_VAR:
    case DH_AGG_STDDEV:
        // Two passes like AggAll.h:165-191: the mean, then the mean squared deviation from it.
        np = all_stage1_launch<T, RSum<T>, false>(ctx, arg, rows, cols, ld, nullptr, partials);
        hipLaunchKernelGGL((all_stage2<T, RSum<T>, 1>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, mean_slot, count);
        np = all_stage1_launch<T, RSum<T>, true>(ctx, arg, rows, cols, ld, mean_slot, partials);
        if (op == DH_AGG_VAR)
            hipLaunchKernelGGL((all_stage2<T, RSum<T>, 1>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        else
            hipLaunchKernelGGL((all_stage2<T, RSum<T>, 2>), dim3(1), dim3(THREADS), 0, ctx->stream, partials, np, out, count);
        break;
    default:
        return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode");
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T> dh_status agg_all(dh_ctx *ctx, int op, const T *arg, size_t rows, size_t cols, size_t ld, T *result_host) {
    DH_REQUIRE_CTX(ctx);
    if (result_host == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "AggAll - result pointer is null");
    T *slot = reinterpret_cast<T *>(reinterpret_cast<char *>(ctx->flag_dev) + 64);
    dh_status st = agg_all_dev<T>(ctx, op, arg, rows, cols, ld, slot);
    if (st != DH_OK)
        return st;
    T *host_slot = reinterpret_cast<T *>(reinterpret_cast<char *>(ctx->flag_host) + 64);
    DH_CHECK_HIP(hipMemcpyAsync(host_slot, slot, sizeof(T), hipMemcpyDeviceToHost, ctx->stream));
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    *result_host = *host_slot;
    return DH_OK;
}

// =======================================================================================
// AggRow
// =======================================================================================
// n / b for a divisor b that stays the same over many divisions, r = 1 / b computed once: the product n * r
// corrected by its exactly computed residual (one fused multiply-add for the residual, one for the correction),
// which yields the correctly rounded quotient of normal operands in three instructions instead of a full
// division sequence. Infinite and NaN numerators keep the product (their residual is NaN).
template <typename T> __device__ __forceinline__ T div_by_constant(T n, T b, T r) {
    const T q0 = n * r;
    const T e = __builtin_fma(-b, q0, n);
    const T q1 = __builtin_fma(e, r, q0);
    return (e == e) ? q1 : q0;
}

constexpr int ROW_UR = 4; // rows per lane group and step of the row kernels

// FINAL: 0 plain reduction, 1 mean, 2 var, 3 stddev. G lanes share a row (G a power of two
// <= 64, G divides 64). NANFIRST: MIN/MAX take a NaN in column 0 as the result (AggRow.h:108).
template <typename T, int VEC, class R, int FINAL, bool NANFIRST, int KV>
__global__ __launch_bounds__(THREADS) void row_kernel(T *res, size_t ld_res, const T *arg, size_t rows,
                                                      size_t cols, size_t ld, int G) {
    // UR rows per lane group are processed together so that UR independent loads are in flight;
    // rows past the end are clamped to the last row for loading and dropped at the store.
    // Per step a wavefront owns GPW * UR consecutive rows (row (u, g) = base + u * GPW + g for
    // lane group g): load u covers GPW whole rows back to back, and the step's results are one
    // contiguous run stored by the first GPW * UR lanes. A lane takes KV vectors of a row per pass, G lanes
    // apart: fewer lanes per row mean fewer exchange levels, which is what 8-byte values (two moves per level
    // and value) are short of.
    constexpr int UR = ROW_UR;
    const int tid = threadIdx.x;
    const int lane = tid % G;
    const int wlane = tid % DH_WAVE;
    const int GPW = DH_WAVE / G;
    const int g_in_wave = wlane / G;
    const size_t cvecs = cols / VEC;
    const size_t rows_per_step = static_cast<size_t>(GPW) * UR;
    const size_t wave_id = static_cast<size_t>(blockIdx.x) * (THREADS / DH_WAVE) + tid / DH_WAVE;
    const size_t wave_stride = static_cast<size_t>(gridDim.x) * (THREADS / DH_WAVE) * rows_per_step;
    const T ncols = static_cast<T>(cols), rcols = T(1) / ncols;
    const size_t pass = static_cast<size_t>(G) * KV; // vectors of a row per pass of its lane group
    for (size_t base = wave_id * rows_per_step; base < rows; base += wave_stride) {
        const T *row[UR];
#pragma unroll
        for (int u = 0; u < UR; u++) {
            const size_t r = base + static_cast<size_t>(u * GPW + g_in_wave);
            row[u] = arg + (r < rows ? r : rows - 1) * ld;
        }
        T acc[UR];
        T first[UR];      // element 0 of the row, known to the lane that loads it (NANFIRST)
        T xk[UR][KV][VEC]; // the lane's values when the row fits one pass (second pass of VAR / STDDEV)
        const bool in_regs = cvecs <= pass;
#pragma unroll
        for (int u = 0; u < UR; u++) {
            acc[u] = R::id();
            first[u] = T(0);
        }
        for (size_t cv = lane; cv < cvecs; cv += pass) {
            T x[UR][KV][VEC];
            // vectors past the row's end re-read the lane's first one and are left out below
#pragma unroll
            for (int k = 0; k < KV; k++)
#pragma unroll
                for (int u = 0; u < UR; u++) {
                    const size_t c = cv + static_cast<size_t>(k) * G;
                    dh_load_vec_stream<T, VEC>(row[u] + (c < cvecs ? c : cv) * VEC, x[u][k]);
                }
#pragma unroll
            for (int k = 0; k < KV; k++) {
                const bool valid = k == 0 || cv + static_cast<size_t>(k) * G < cvecs;
#pragma unroll
                for (int u = 0; u < UR; u++) {
                    if constexpr (NANFIRST) {
                        if (k == 0 && cv == 0)
                            first[u] = x[u][0][0];
                    }
#pragma unroll
                    for (int i = 0; i < VEC; i++) {
                        const T next = R::comb(acc[u], x[u][k][i]);
                        acc[u] = valid ? next : acc[u];
                        if constexpr (FINAL >= 2)
                            xk[u][k][i] = x[u][k][i];
                    }
                }
            }
        }
        dh_butterfly(G, [&](auto peer) {
#pragma unroll
            for (int u = 0; u < UR; u++)
                acc[u] = R::comb(acc[u], peer(acc[u]));
        });
        if constexpr (FINAL >= 1) {
#pragma unroll
            for (int u = 0; u < UR; u++) {
                if constexpr (agg_is_int<T>)
                    acc[u] = acc[u] / ncols;
                else
                    acc[u] = div_by_constant<T>(acc[u], ncols, rcols);
            }
        }
        if constexpr (FINAL >= 2) {
            T s[UR];
#pragma unroll
            for (int u = 0; u < UR; u++)
                s[u] = T(0);
            if (in_regs) {
#pragma unroll
                for (int k = 0; k < KV; k++) {
                    const bool valid = static_cast<size_t>(lane) + static_cast<size_t>(k) * G < cvecs;
#pragma unroll
                    for (int u = 0; u < UR; u++)
#pragma unroll
                        for (int i = 0; i < VEC; i++) {
                            const T d = xk[u][k][i] - acc[u];
                            const T next = s[u] + d * d;
                            s[u] = valid ? next : s[u];
                        }
                }
            } else {
                for (size_t cv = lane; cv < cvecs; cv += pass) {
                    T x[UR][KV][VEC];
#pragma unroll
                    for (int k = 0; k < KV; k++)
#pragma unroll
                        for (int u = 0; u < UR; u++) {
                            const size_t c = cv + static_cast<size_t>(k) * G;
                            load_vec<T, VEC>(row[u] + (c < cvecs ? c : cv) * VEC, x[u][k]);
                        }
#pragma unroll
                    for (int k = 0; k < KV; k++) {
                        const bool valid = k == 0 || cv + static_cast<size_t>(k) * G < cvecs;
#pragma unroll
                        for (int u = 0; u < UR; u++)
#pragma unroll
                            for (int i = 0; i < VEC; i++) {
                                const T d = x[u][k][i] - acc[u];
                                const T next = s[u] + d * d;
                                s[u] = valid ? next : s[u];
                            }
                    }
                }
            }
            dh_butterfly(G, [&](auto peer) {
#pragma unroll
                for (int u = 0; u < UR; u++)
                    s[u] = s[u] + peer(s[u]);
            });
#pragma unroll
            for (int u = 0; u < UR; u++) {
                if constexpr (agg_is_int<T>)
                    s[u] = s[u] / ncols;
                else
                    s[u] = div_by_constant<T>(s[u], ncols, rcols);
                acc[u] = (FINAL == 3) ? dev_sqrt<T>(s[u]) : s[u];
            }
        }
#pragma unroll
        for (int u = 0; u < UR; u++) {
            if constexpr (NANFIRST) {
                // only the group's lane 0 holds the row's element 0; the results are taken from that lane below
                if (dev_isnan(first[u]))
                    acc[u] = first[u];
            }
        }
        if (GPW * UR <= DH_WAVE) {
            // lane j takes the result of row base + j: it sits in group j % GPW as acc[j / GPW]
            T mine = T(0);
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const T v = __shfl(acc[u], (wlane % GPW) * G, DH_WAVE);
                if (wlane / GPW == u)
                    mine = v;
            }
            const size_t orow = base + static_cast<size_t>(wlane);
            if (wlane < GPW * UR && orow < rows)
                dh_store_stream(res + orow * ld_res, mine);
        } else {
            // fewer than 4 lanes per row: more rows per step than lanes, every group stores its own
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const size_t r = base + static_cast<size_t>(u * GPW + g_in_wave);
                if (lane == 0 && r < rows)
                    res[r * ld_res] = acc[u];
            }
        }
    }
}

// IDXMIN / IDXMAX per row: (value, index) pairs; on equal values the lower index wins. Same row
// mapping as row_kernel (a wavefront owns GPW * UR consecutive rows per step, results stored as one
// contiguous run). I is the index type carried through the reduction: 32 bits unless a row has 2^32
// or more columns.
template <typename T, int VEC, bool IS_MIN, typename I, int KV>
__global__ __launch_bounds__(THREADS) void row_idx_kernel(uint64_t *res, size_t ld_res, const T *arg, size_t rows,
                                                          size_t cols, size_t ld, int G) {
    constexpr int UR = ROW_UR;
    constexpr I NONE = ~static_cast<I>(0);
    const int tid = threadIdx.x;
    const int lane = tid % G;
    const int wlane = tid % DH_WAVE;
    const int GPW = DH_WAVE / G;
    const int g_in_wave = wlane / G;
    const size_t cvecs = cols / VEC;
    const size_t rows_per_step = static_cast<size_t>(GPW) * UR;
    const size_t wave_id = static_cast<size_t>(blockIdx.x) * (THREADS / DH_WAVE) + tid / DH_WAVE;
    const size_t wave_stride = static_cast<size_t>(gridDim.x) * (THREADS / DH_WAVE) * rows_per_step;
    const T worst = IS_MIN ? agg_largest<T>() : agg_smallest<T>();
    for (size_t base = wave_id * rows_per_step; base < rows; base += wave_stride) {
        const T *row[UR];
        T best[UR];
        I bi[UR];
        bool nan0[UR]; // element 0 of the row is NaN (known to the lane that loads it)
#pragma unroll
        for (int u = 0; u < UR; u++) {
            const size_t r = base + static_cast<size_t>(u * GPW + g_in_wave);
            row[u] = arg + (r < rows ? r : rows - 1) * ld;
            best[u] = worst;
            bi[u] = NONE;
            nan0[u] = false;
        }
        const size_t pass = static_cast<size_t>(G) * KV; // vectors of a row per pass: KV per lane, G lanes apart
        for (size_t cv = lane; cv < cvecs; cv += pass) {
            T x[UR][KV][VEC];
            // vectors past the row's end re-read the lane's first one and are left out below
#pragma unroll
            for (int k = 0; k < KV; k++)
#pragma unroll
                for (int u = 0; u < UR; u++) {
                    const size_t c = cv + static_cast<size_t>(k) * G;
                    dh_load_vec_stream<T, VEC>(row[u] + (c < cvecs ? c : cv) * VEC, x[u][k]);
                }
#pragma unroll
            for (int k = 0; k < KV; k++) {
                const size_t c = cv + static_cast<size_t>(k) * G;
                const bool valid = k == 0 || c < cvecs;
#pragma unroll
                for (int u = 0; u < UR; u++) {
                    if (k == 0 && cv == 0)
                        nan0[u] = dev_isnan(x[u][0][0]);
#pragma unroll
                    for (int i = 0; i < VEC; i++) {
                        const I idx = static_cast<I>(c * VEC + i);
                        const bool better = IS_MIN ? (x[u][k][i] < best[u]) : (x[u][k][i] > best[u]);
                        // within a lane indices only grow, so a tie keeps the earlier one, except
                        // against the sentinel (an actual +-inf value must beat "nothing seen yet")
                        const bool first_seen = (bi[u] == NONE) && (x[u][k][i] == best[u]);
                        if (valid && (better || first_seen)) {
                            best[u] = x[u][k][i];
                            bi[u] = idx;
                        }
                    }
                }
            }
        }
        dh_butterfly(G, [&](auto peer) {
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const T ov = peer(best[u]);
                const I oi = peer(bi[u]);
                const bool better = IS_MIN ? (ov < best[u]) : (ov > best[u]);
                if (better || (ov == best[u] && oi < bi[u])) {
                    best[u] = ov;
                    bi[u] = oi;
                }
            }
        });
#pragma unroll
        for (int u = 0; u < UR; u++) {
            // AggRow.h:73-80: the scan starts from element 0; if that is NaN no later element
            // compares below/above it, so 0 is returned. A row of NaNs only leaves bi untouched.
            // (after the exchange every lane of the group holds the group's result; lane 0 knows nan0)
            if (nan0[u] || bi[u] == NONE)
                bi[u] = 0;
        }
        if (GPW * UR <= DH_WAVE) {
            // lane j takes the result of row base + j: group j % GPW, slot j / GPW, from that group's lane 0
            I mine = 0;
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const I v = __shfl(bi[u], (wlane % GPW) * G, DH_WAVE);
                if (wlane / GPW == u)
                    mine = v;
            }
            const size_t orow = base + static_cast<size_t>(wlane);
            if (wlane < GPW * UR && orow < rows)
                dh_store_stream(res + orow * ld_res, static_cast<uint64_t>(mine));
        } else {
#pragma unroll
            for (int u = 0; u < UR; u++) {
                const size_t r = base + static_cast<size_t>(u * GPW + g_in_wave);
                if (lane == 0 && r < rows)
                    res[r * ld_res] = bi[u];
            }
        }
    }
}

static inline int pick_group(size_t cvecs, int kv = 1) {
    int g = 1;
    while (g < DH_WAVE && static_cast<size_t>(g) * kv < cvecs)
        g <<= 1;
    return g;
}
// Vectors per lane and pass of the row kernels. Two where the exchanges dominate: 8-byte values in the two-butterfly
// reductions and in the (value, index) reductions. Measured on 10M x 64 doubles: VAR 963 -> 842 us, IDXMIN 943 -> 793 us;
// the one-butterfly reductions and all 4-byte cases lose 3-5 % with two.
template <typename T> constexpr int row_kv(bool two_exchanges_or_index) { return sizeof(T) == 8 && two_exchanges_or_index ? 2 : 1; }

static inline unsigned row_grid(const dh_ctx *ctx, size_t rows, int G) {
    const size_t rpb = static_cast<size_t>(THREADS / G) * 4; // rows per block and step (4 per lane group)
    size_t g = dh_ceil_div(rows, rpb);
    // one step per wavefront wherever the grid can express it: measured faster than a capped grid with a
    // grid-stride loop (20M x 64 floats, SUM: 812 against 855 us)
    const size_t cap = 0x7fffffffull;
    if (g > cap)
        g = cap;
    if (g < 1)
        g = 1;
    return static_cast<unsigned>(g);
}

template <typename T, class R, int FINAL, bool NANFIRST>
static inline void row_launch(dh_ctx *ctx, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    constexpr int V = dh_vec<T>::N;
    const bool vec_ok = (cols % V == 0) && (ld % V == 0) && dh_aligned(arg, 16);
    if (vec_ok) {
        constexpr int KV = row_kv<T>(FINAL >= 2);
        const int G = pick_group(cols / V, KV);
        hipLaunchKernelGGL((row_kernel<T, V, R, FINAL, NANFIRST, KV>), dim3(row_grid(ctx, rows, G)), dim3(THREADS), 0,
                           ctx->stream, res, ld_res, arg, rows, cols, ld, G);
    } else {
        const int G = pick_group(cols);
        hipLaunchKernelGGL((row_kernel<T, 1, R, FINAL, NANFIRST, 1>), dim3(row_grid(ctx, rows, G)), dim3(THREADS), 0,
                           ctx->stream, res, ld_res, arg, rows, cols, ld, G);
    }
}

template <typename T> dh_status agg_row(dh_ctx *ctx, int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols || ld_res < 1)
        return dh_fail(DH_ERR_RUNTIME, "AggRow - leading dimension smaller than the column count");
    if (rows == 0)
        return DH_OK;
    if (cols == 0)
        return dh_fail(DH_ERR_RUNTIME, "AggRow - the argument has no columns");
    if constexpr (agg_is_int<T>) {
        // The reference's integer MEAN / VAR / STDDEV divide and subtract in integer arithmetic (AggAll.h:163-191);
        // its device library has SUM / MIN / MAX for si64 only (CUDA/AggAll.cu:155, AggRow.cu:146, AggCol.cu:89).
        if (op == DH_AGG_MEAN || op == DH_AGG_VAR || op == DH_AGG_STDDEV)
            return dh_fail(DH_ERR_RUNTIME, "%s: MEAN, VAR and STDDEV of integer value types are not supported on the device", __func__);
    }
    // A few very wide rows (a 1 x N vector is the common case) would occupy one wavefront each in the row kernel:
    // every such row goes through the whole-matrix reduction instead, which spreads it over the device. SUM, PROD and
    // the moments only: they do not depend on the order of NaNs, MIN / MAX follow AggRow's own NaN rule.
    if (rows <= 16 && cols >= (size_t(1) << 16) &&
        (op == DH_AGG_SUM || op == DH_AGG_PROD || op == DH_AGG_MEAN || op == DH_AGG_VAR || op == DH_AGG_STDDEV)) {
        for (size_t r = 0; r < rows; r++) {
            const dh_status st = agg_all_dev<T>(ctx, op, arg + r * ld, 1, cols, ld, res + r * ld_res);
            if (st != DH_OK)
                return st;
        }
        return DH_OK;
    }
    switch (op) {
    case DH_AGG_SUM:
        row_launch<T, RSum<T>, 0, false>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    case DH_AGG_PROD:
        row_launch<T, RProd<T>, 0, false>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    case DH_AGG_MIN:
        row_launch<T, RMin<T>, 0, true>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    case DH_AGG_MAX:
        row_launch<T, RMax<T>, 0, true>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    case DH_AGG_MEAN:
        row_launch<T, RSum<T>, 1, false>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    case DH_AGG_VAR:
        row_launch<T, RSum<T>, 2, false>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    case DH_AGG_STDDEV:
        row_launch<T, RSum<T>, 3, false>(ctx, res, ld_res, arg, rows, cols, ld);
        break;
    default:
        return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode"); // AggOpCode.h:48
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T>
dh_status agg_row_idx(dh_ctx *ctx, int op, uint64_t *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols || ld_res < 1)
        return dh_fail(DH_ERR_RUNTIME, "AggRow - leading dimension smaller than the column count");
    if (op != DH_AGG_IDXMIN && op != DH_AGG_IDXMAX)
        return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode");
    if (rows == 0)
        return DH_OK;
    if (cols == 0)
        return dh_fail(DH_ERR_RUNTIME, "AggRow - the argument has no columns");
    constexpr int V = dh_vec<T>::N;
    const bool vec_ok = (cols % V == 0) && (ld % V == 0) && dh_aligned(arg, 16);
    constexpr int KV = row_kv<T>(true);
    const int G = vec_ok ? pick_group(cols / V, KV) : pick_group(cols);
    const dim3 grid(row_grid(ctx, rows, G)), block(THREADS);
    const bool wide = cols >= 0xffffffffull; // index does not fit 32 bits next to the sentinel
#define DH_ROW_IDX(VEC_, MIN_)                                                                                          \
    do {                                                                                                                \
        if (wide)                                                                                                       \
            hipLaunchKernelGGL((row_idx_kernel<T, VEC_, MIN_, unsigned long long, 1>), grid, block, 0, ctx->stream,     \
                               res, ld_res, arg, rows, cols, ld, G);                                                    \
        else                                                                                                            \
            hipLaunchKernelGGL((row_idx_kernel<T, VEC_, MIN_, unsigned, (VEC_) == 1 ? 1 : KV>), grid, block, 0,         \
                               ctx->stream, res, ld_res, arg, rows, cols, ld, G);                                       \
    } while (0)
    if (vec_ok) {
        if (op == DH_AGG_IDXMIN)
            DH_ROW_IDX(V, true);
        else
            DH_ROW_IDX(V, false);
    } else {
        if (op == DH_AGG_IDXMIN)
            DH_ROW_IDX(1, true);
        else
            DH_ROW_IDX(1, false);
    }
#undef DH_ROW_IDX
    DH_CHECK_LAUNCH();
    return DH_OK;
}

constexpr int S2_TX = 16, S2_TY = 16; // second-stage block: columns x partial lanes
constexpr int V2_TX = 4, V2_TY = 64;   // variance second stage: small blocks, few columns each. It is a chain of two
                                       // passes over ~1000 partials and three barriers, i.e. latency: 16 x 64 threads in
                                       // 4 blocks took 32 us on 64 columns, 4 x 256 in 16 blocks 24 us, 4 x 64 9 us

// =======================================================================================
// AggCol
// =======================================================================================
// Block b owns rows [b*slab, (b+1)*slab). Threads (tx, ty): tx walks column vectors (grid.y
// covers wider matrices), ty interleaves the slab's rows.
template <typename T, int VEC, class R>
__global__ __launch_bounds__(THREADS) void col_stage1(const T *arg, size_t rows, size_t cvecs, size_t ld, size_t slab,
                                                      T *partials /* [gridDim.x][cvecs*VEC] */) {
    extern __shared__ unsigned char lds_raw[];
    T *lds = reinterpret_cast<T *>(lds_raw); // [blockDim.y][blockDim.x * VEC]
    const size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r_begin = static_cast<size_t>(blockIdx.x) * slab;
    const size_t r_end = (r_begin + slab < rows) ? r_begin + slab : rows;
    T acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++)
        acc[i] = R::id();
    if (cv < cvecs) {
        const size_t step = blockDim.y;
        size_t r0 = r_begin + threadIdx.y;
        for (; r0 + (UNROLL - 1) * step < r_end; r0 += step * UNROLL) {
            T x[UNROLL][VEC];
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
                dh_load_vec_stream<T, VEC>(arg + (r0 + u * step) * ld + cv * VEC, x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
#pragma unroll
                for (int i = 0; i < VEC; i++)
                    acc[i] = R::comb(acc[i], x[u][i]);
        }
        for (; r0 < r_end; r0 += step) {
            T x[VEC];
            dh_load_vec_stream<T, VEC>(arg + r0 * ld + cv * VEC, x);
#pragma unroll
            for (int i = 0; i < VEC; i++)
                acc[i] = R::comb(acc[i], x[i]);
        }
    }
    const int w = blockDim.x * VEC;
#pragma unroll
    for (int i = 0; i < VEC; i++)
        lds[threadIdx.y * w + threadIdx.x * VEC + i] = acc[i];
    __syncthreads();
    if (threadIdx.y == 0 && cv < cvecs) {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            T a = acc[i];
            for (unsigned y = 1; y < blockDim.y; y++)
                a = R::comb(a, lds[y * w + threadIdx.x * VEC + i]);
            partials[static_cast<size_t>(blockIdx.x) * cvecs * VEC + cv * VEC + i] = a;
        }
    }
}

// FINAL: 0 as is, 1 mean. NANFIRST as for rows (AggCol.h:135-141: row 0 seeds the result).
template <typename T, class R, int FINAL, bool NANFIRST>
__global__ __launch_bounds__(THREADS) void col_stage2(const T *partials, size_t nparts, size_t cols, T *res,
                                                      const T *arg, T count) {
    // block = (S2_TX columns, S2_TY partial lanes): the partial rows are split over the TY lanes
    // (4 independent loads in flight each) and folded through LDS in a fixed order.
    __shared__ T lds[S2_TY][S2_TX];
    const size_t c = static_cast<size_t>(blockIdx.x) * S2_TX + threadIdx.x;
    T a0 = R::id(), a1 = R::id(), a2 = R::id(), a3 = R::id();
    if (c < cols) {
        size_t p = threadIdx.y;
        for (; p + 3 * S2_TY < nparts; p += 4 * S2_TY) {
            a0 = R::comb(a0, partials[p * cols + c]);
            a1 = R::comb(a1, partials[(p + S2_TY) * cols + c]);
            a2 = R::comb(a2, partials[(p + 2 * S2_TY) * cols + c]);
            a3 = R::comb(a3, partials[(p + 3 * S2_TY) * cols + c]);
        }
        for (; p < nparts; p += S2_TY)
            a0 = R::comb(a0, partials[p * cols + c]);
    }
    lds[threadIdx.y][threadIdx.x] = R::comb(R::comb(a0, a1), R::comb(a2, a3));
    __syncthreads();
    if (threadIdx.y != 0 || c >= cols)
        return;
    T a = lds[0][threadIdx.x];
    for (int y = 1; y < S2_TY; y++)
        a = R::comb(a, lds[y][threadIdx.x]);
    if constexpr (FINAL == 1)
        a = a / count;
    if constexpr (NANFIRST) {
        const T first = arg[c];
        if (dev_isnan(first))
            a = first;
    }
    res[c] = a;
}

// Single-pass variance: per thread shifted sums around the first value it sees, converted to
// (n, mean, M2); the TY row-lanes are merged through LDS, blocks are merged in stage 2.
template <typename T, int VEC>
__global__ __launch_bounds__(THREADS) void col_var_stage1(const T *arg, size_t rows, size_t cvecs, size_t ld,
                                                          size_t slab, T *part_mean, T *part_m2) {
    extern __shared__ unsigned char lds_raw[];
    T *lds_mean = reinterpret_cast<T *>(lds_raw);             // [TY][TX*VEC]
    T *lds_m2 = lds_mean + blockDim.y * blockDim.x * VEC;     // [TY][TX*VEC]
    const size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r_begin = static_cast<size_t>(blockIdx.x) * slab;
    const size_t r_end = (r_begin + slab < rows) ? r_begin + slab : rows;
    const size_t step = blockDim.y;
    T shift[VEC], s1[VEC], s2[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) {
        shift[i] = T(0);
        s1[i] = T(0);
        s2[i] = T(0);
    }
    size_t n = 0;
    if (cv < cvecs && r_begin + threadIdx.y < r_end) {
        load_vec<T, VEC>(arg + (r_begin + threadIdx.y) * ld + cv * VEC, shift);
        n = (r_end - r_begin - threadIdx.y + step - 1) / step;
        size_t r0 = r_begin + threadIdx.y;
        for (; r0 + (UNROLL - 1) * step < r_end; r0 += step * UNROLL) {
            T x[UNROLL][VEC];
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
                dh_load_vec_stream<T, VEC>(arg + (r0 + u * step) * ld + cv * VEC, x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
#pragma unroll
                for (int i = 0; i < VEC; i++) {
                    const T d = x[u][i] - shift[i];
                    s1[i] += d;
                    s2[i] += d * d;
                }
        }
        for (; r0 < r_end; r0 += step) {
            T x[VEC];
            dh_load_vec_stream<T, VEC>(arg + r0 * ld + cv * VEC, x);
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const T d = x[i] - shift[i];
                s1[i] += d;
                s2[i] += d * d;
            }
        }
    }
    const int w = blockDim.x * VEC;
#pragma unroll
    for (int i = 0; i < VEC; i++) {
        T mean = T(0), m2 = T(0);
        if (n) {
            const T nn = static_cast<T>(n);
            mean = shift[i] + s1[i] / nn;
            m2 = s2[i] - s1[i] * s1[i] / nn;
            if (m2 < T(0))
                m2 = T(0);
        }
        lds_mean[threadIdx.y * w + threadIdx.x * VEC + i] = mean;
        lds_m2[threadIdx.y * w + threadIdx.x * VEC + i] = m2;
    }
    __syncthreads();
    if (threadIdx.y == 0 && cv < cvecs) {
        const size_t total = (r_end > r_begin) ? r_end - r_begin : 0;
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            double cn = 0.0, cmean = 0.0, cm2 = 0.0;
            for (unsigned y = 0; y < blockDim.y; y++) {
                if (y >= total)
                    break;
                const double ny = static_cast<double>((total - y + step - 1) / step);
                const double my = static_cast<double>(lds_mean[y * w + threadIdx.x * VEC + i]);
                const double qy = static_cast<double>(lds_m2[y * w + threadIdx.x * VEC + i]);
                const double delta = my - cmean;
                const double nt = cn + ny;
                cmean += delta * ny / nt;
                cm2 += qy + delta * delta * cn * ny / nt;
                cn = nt;
            }
            part_mean[static_cast<size_t>(blockIdx.x) * cvecs * VEC + cv * VEC + i] = static_cast<T>(cmean);
            part_m2[static_cast<size_t>(blockIdx.x) * cvecs * VEC + cv * VEC + i] = static_cast<T>(cm2);
        }
    }
}

// OUT: 0 variance, 1 stddev, 2 mean (unused by the public API but kept for pipelines).
template <typename T, int OUT>
__global__ __launch_bounds__(V2_TX * V2_TY) void col_var_stage2(const T *part_mean, const T *part_m2, size_t nparts,
                                                          size_t cols, size_t rows, size_t slab, T *res,
                                                          T *res_mean = nullptr) {
    // (V2_TX columns, V2_TY partial lanes: 1024 threads). Pooled moments of the per-block (count, mean, M2) triples in double:
    //     mean = sum n_p mean_p / N,   M2 = sum M2_p + sum n_p (mean_p - mean)^2
    // - the closed form of merging them pairwise with Chan's formula, without a division per partial.
    __shared__ double lds_a[V2_TY][V2_TX], lds_b[V2_TY][V2_TX];
    const size_t c = static_cast<size_t>(blockIdx.x) * V2_TX + threadIdx.x;
    auto count = [&](size_t p) {
        const size_t r_begin = p * slab;
        if (r_begin >= rows)
            return 0.0;
        return static_cast<double>(((r_begin + slab < rows) ? r_begin + slab : rows) - r_begin);
    };
    // eight partials per thread are loaded together (indices past the end are clamped; their count is zero)
    constexpr int UN2 = 8;
    double s1 = 0.0, s2 = 0.0;
    if (c < cols)
        for (size_t p0 = threadIdx.y; p0 < nparts; p0 += V2_TY * UN2) {
            T pm[UN2], pq[UN2];
#pragma unroll
            for (int k = 0; k < UN2; k++) {
                const size_t p = p0 + static_cast<size_t>(k) * V2_TY;
                const size_t pc = p < nparts ? p : nparts - 1;
                pm[k] = part_mean[pc * cols + c];
                pq[k] = part_m2[pc * cols + c];
            }
            __builtin_amdgcn_sched_barrier(0); // all sixteen loads are issued before the first value is used
#pragma unroll
            for (int k = 0; k < UN2; k++) {
                const size_t p = p0 + static_cast<size_t>(k) * V2_TY;
                s1 += count(p) * static_cast<double>(pm[k]);
                s2 += p < nparts ? static_cast<double>(pq[k]) : 0.0;
            }
        }
    lds_a[threadIdx.y][threadIdx.x] = s1;
    lds_b[threadIdx.y][threadIdx.x] = s2;
    __syncthreads();
    double tot1 = 0.0, tot2 = 0.0;
    for (int y = 0; y < V2_TY; y++) {
        tot1 += lds_a[y][threadIdx.x];
        tot2 += lds_b[y][threadIdx.x];
    }
    const double cmean = tot1 / static_cast<double>(rows);
    __syncthreads();
    double s3 = 0.0;
    if (c < cols)
        for (size_t p0 = threadIdx.y; p0 < nparts; p0 += V2_TY * UN2) {
            T pm[UN2];
#pragma unroll
            for (int k = 0; k < UN2; k++) {
                const size_t p = p0 + static_cast<size_t>(k) * V2_TY;
                pm[k] = part_mean[(p < nparts ? p : nparts - 1) * cols + c];
            }
#pragma unroll
            for (int k = 0; k < UN2; k++) {
                const double d = static_cast<double>(pm[k]) - cmean;
                s3 += count(p0 + static_cast<size_t>(k) * V2_TY) * d * d;
            }
        }
    lds_a[threadIdx.y][threadIdx.x] = s3;
    __syncthreads();
    if (threadIdx.y != 0 || c >= cols)
        return;
    double cm2 = tot2;
    for (int y = 0; y < V2_TY; y++)
        cm2 += lds_a[y][threadIdx.x];
    double v = cm2 / static_cast<double>(rows);
    if constexpr (OUT == 1)
        v = sqrt(v);
    if constexpr (OUT == 2)
        v = cmean;
    res[c] = static_cast<T>(v);
    if (res_mean)
        res_mean[c] = static_cast<T>(cmean);
}

// IDXMIN / IDXMAX per column.
template <typename T, int VEC, bool IS_MIN>
__global__ __launch_bounds__(THREADS) void col_idx_stage1(const T *arg, size_t rows, size_t cvecs, size_t ld, size_t slab,
                                                          T *part_val, unsigned long long *part_idx) {
    extern __shared__ unsigned char lds_raw[];
    unsigned long long *lds_idx = reinterpret_cast<unsigned long long *>(lds_raw);        // [TY][TX*VEC]
    T *lds_val = reinterpret_cast<T *>(lds_idx + blockDim.y * blockDim.x * VEC);          // [TY][TX*VEC]
    const T worst = IS_MIN ? agg_largest<T>() : agg_smallest<T>();
    const size_t cv = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r_begin = static_cast<size_t>(blockIdx.x) * slab;
    const size_t r_end = (r_begin + slab < rows) ? r_begin + slab : rows;
    // the running index is kept relative to the slab, in 32 bits (the launch checks that a slab is shorter than 2^32 rows)
    constexpr unsigned NONE = ~0u;
    T best[VEC];
    unsigned bk[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) {
        best[i] = worst;
        bk[i] = NONE;
    }
    if (cv < cvecs) {
        const size_t step = blockDim.y;
        const T *col = arg + cv * VEC;
        size_t r0 = r_begin + threadIdx.y;
        // rows are visited in ascending order by every thread, so that on equal values the first one stays
        for (; r0 + (UNROLL - 1) * step < r_end; r0 += step * UNROLL) {
            T x[UNROLL][VEC];
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
                dh_load_vec_stream<T, VEC>(col + (r0 + u * step) * ld, x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const unsigned k = static_cast<unsigned>(r0 - r_begin) + static_cast<unsigned>(u * step);
#pragma unroll
                for (int i = 0; i < VEC; i++) {
                    const bool better = IS_MIN ? (x[u][i] < best[i]) : (x[u][i] > best[i]);
                    const bool first_seen = (bk[i] == NONE) && !dev_isnan(x[u][i]);
                    if (better || first_seen) {
                        best[i] = x[u][i];
                        bk[i] = k;
                    }
                }
            }
        }
        for (; r0 < r_end; r0 += step) {
            T x[VEC];
            dh_load_vec_stream<T, VEC>(col + r0 * ld, x);
            const unsigned k = static_cast<unsigned>(r0 - r_begin);
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const bool better = IS_MIN ? (x[i] < best[i]) : (x[i] > best[i]);
                const bool first_seen = (bk[i] == NONE) && !dev_isnan(x[i]);
                if (better || first_seen) {
                    best[i] = x[i];
                    bk[i] = k;
                }
            }
        }
    }
    unsigned long long bi[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++)
        bi[i] = bk[i] == NONE ? ~0ull : static_cast<unsigned long long>(r_begin) + bk[i];
    const int w = blockDim.x * VEC;
#pragma unroll
    for (int i = 0; i < VEC; i++) {
        lds_val[threadIdx.y * w + threadIdx.x * VEC + i] = best[i];
        lds_idx[threadIdx.y * w + threadIdx.x * VEC + i] = bi[i];
    }
    __syncthreads();
    if (threadIdx.y == 0 && cv < cvecs) {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            T b = best[i];
            unsigned long long k = bi[i];
            for (unsigned y = 1; y < blockDim.y; y++) {
                const T ov = lds_val[y * w + threadIdx.x * VEC + i];
                const unsigned long long oi = lds_idx[y * w + threadIdx.x * VEC + i];
                const bool better = IS_MIN ? (ov < b) : (ov > b);
                if (better || (ov == b && oi < k)) {
                    b = ov;
                    k = oi;
                }
            }
            part_val[static_cast<size_t>(blockIdx.x) * cvecs * VEC + cv * VEC + i] = b;
            part_idx[static_cast<size_t>(blockIdx.x) * cvecs * VEC + cv * VEC + i] = k;
        }
    }
}

template <typename T, bool IS_MIN>
__global__ __launch_bounds__(THREADS) void col_idx_stage2(const T *part_val, const unsigned long long *part_idx,
                                                          size_t nparts, size_t cols, const T *arg, uint64_t *res) {
    // block = (S2_TX columns, S2_TY partial lanes) like col_stage2: each lane merges every S2_TY-th partial with four
    // loads in flight, the lanes are merged through LDS. The merge (better value, or equal value and lower index) is
    // associative and commutative, so the result does not depend on the split.
    __shared__ T lds_v[S2_TY][S2_TX];
    __shared__ unsigned long long lds_k[S2_TY][S2_TX];
    const size_t c = static_cast<size_t>(blockIdx.x) * S2_TX + threadIdx.x;
    T b = IS_MIN ? agg_largest<T>() : agg_smallest<T>();
    unsigned long long k = ~0ull;
    auto merge = [&](T ov, unsigned long long oi) {
        const bool better = IS_MIN ? (ov < b) : (ov > b);
        if (better || (ov == b && oi < k)) {
            b = ov;
            k = oi;
        }
    };
    if (c < cols) {
        size_t p = threadIdx.y;
        for (; p + 3 * S2_TY < nparts; p += 4 * S2_TY) {
            T v[4];
            unsigned long long id[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                v[u] = part_val[(p + u * S2_TY) * cols + c];
                id[u] = part_idx[(p + u * S2_TY) * cols + c];
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
                merge(v[u], id[u]);
        }
        for (; p < nparts; p += S2_TY)
            merge(part_val[p * cols + c], part_idx[p * cols + c]);
    }
    lds_v[threadIdx.y][threadIdx.x] = b;
    lds_k[threadIdx.y][threadIdx.x] = k;
    __syncthreads();
    if (threadIdx.y != 0 || c >= cols)
        return;
    for (int y = 1; y < S2_TY; y++)
        merge(lds_v[y][threadIdx.x], lds_k[y][threadIdx.x]);
    // AggCol.h:75-91: row 0 seeds the running extremum; a NaN there is never displaced.
    if (dev_isnan(arg[c]) || k == ~0ull)
        k = 0;
    res[c] = k;
}

struct ColPlan {
    dim3 grid, block;
    size_t slab, nparts, cvecs;
    int vec;
};
template <typename T> static inline ColPlan col_plan(const dh_ctx *ctx, const T *arg, size_t rows, size_t cols, size_t ld) {
    constexpr int V = dh_vec<T>::N;
    ColPlan p;
    const bool vec_ok = (cols % V == 0) && (ld % V == 0) && dh_aligned(arg, 16);
    p.vec = vec_ok ? V : 1;
    p.cvecs = cols / p.vec;
    unsigned tx = 1;
    while (tx < THREADS && tx < p.cvecs)
        tx <<= 1;
    unsigned ty = THREADS / tx;
    size_t gy = dh_ceil_div(p.cvecs, tx);
    size_t max_blocks = static_cast<size_t>(ctx->num_cus) * 4; // few, fat blocks: short second stage
    size_t gx = max_blocks / gy;
    if (gx < 1)
        gx = 1;
    const size_t min_slab = static_cast<size_t>(ty) * UNROLL;
    size_t slab = dh_ceil_div(rows, gx);
    slab = dh_ceil_div(slab, min_slab) * min_slab;
    gx = dh_ceil_div(rows, slab);
    if (gx < 1)
        gx = 1;
    p.grid = dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy), 1);
    p.block = dim3(tx, ty, 1);
    p.slab = slab;
    p.nparts = gx;
    return p;
}

// Where the per-block partials of a column aggregation live: the context's workspace (grown on demand), or a
// buffer the caller of agg_col brings along, which is then never grown - a request beyond it is an error.
struct ColScratch {
    void *buf = nullptr;
    size_t bytes = 0;
};
static inline dh_status col_partials(dh_ctx *ctx, const ColScratch &sc, size_t need, void **out) {
    if (sc.buf == nullptr)
        return dh_workspace(ctx, need, out);
    if (need > sc.bytes)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - %zu bytes of partial results do not fit the fixed scratch buffer of %zu bytes",
                       need, sc.bytes);
    *out = sc.buf;
    return DH_OK;
}

template <typename T, class R, int FINAL, bool NANFIRST>
static inline dh_status col_launch(dh_ctx *ctx, T *res, const T *arg, size_t rows, size_t cols, size_t ld, const ColScratch &sc) {
    constexpr int V = dh_vec<T>::N;
    ColPlan p = col_plan<T>(ctx, arg, rows, cols, ld);
    void *wsv = nullptr;
    dh_status st = col_partials(ctx, sc, p.nparts * cols * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    T *partials = static_cast<T *>(wsv);
    const size_t lds = static_cast<size_t>(THREADS) * p.vec * sizeof(T);
    if (p.vec == V)
        hipLaunchKernelGGL((col_stage1<T, V, R>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, partials);
    else
        hipLaunchKernelGGL((col_stage1<T, 1, R>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, partials);
    hipLaunchKernelGGL((col_stage2<T, R, FINAL, NANFIRST>), dim3(static_cast<unsigned>(dh_ceil_div(cols, S2_TX))),
                       dim3(S2_TX, S2_TY), 0, ctx->stream, partials, p.nparts, cols, res, arg, static_cast<T>(rows));
    return DH_OK;
}

template <typename T>
dh_status agg_col(dh_ctx *ctx, int op, T *res, const T *arg, size_t rows, size_t cols, size_t ld, const ColScratch &sc = ColScratch()) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - leading dimension smaller than the column count");
    if (cols == 0)
        return DH_OK;
    if (rows == 0)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - the argument has no rows");
    if constexpr (agg_is_int<T>) {
        // The reference's integer MEAN / VAR / STDDEV divide and subtract in integer arithmetic (AggAll.h:163-191);
        // its device library has SUM / MIN / MAX for si64 only (CUDA/AggAll.cu:155, AggRow.cu:146, AggCol.cu:89).
        if (op == DH_AGG_MEAN || op == DH_AGG_VAR || op == DH_AGG_STDDEV)
            return dh_fail(DH_ERR_RUNTIME, "%s: MEAN, VAR and STDDEV of integer value types are not supported on the device", __func__);
    }
    dh_status st = DH_OK;
    switch (op) {
    case DH_AGG_SUM:
        st = col_launch<T, RSum<T>, 0, false>(ctx, res, arg, rows, cols, ld, sc);
        break;
    case DH_AGG_PROD:
        st = col_launch<T, RProd<T>, 0, false>(ctx, res, arg, rows, cols, ld, sc);
        break;
    case DH_AGG_MIN:
        st = col_launch<T, RMin<T>, 0, true>(ctx, res, arg, rows, cols, ld, sc);
        break;
    case DH_AGG_MAX:
        st = col_launch<T, RMax<T>, 0, true>(ctx, res, arg, rows, cols, ld, sc);
        break;
    case DH_AGG_MEAN:
        st = col_launch<T, RSum<T>, 1, false>(ctx, res, arg, rows, cols, ld, sc);
        break;
    case DH_AGG_VAR:
    case DH_AGG_STDDEV: {
        constexpr int V = dh_vec<T>::N;
        ColPlan p = col_plan<T>(ctx, arg, rows, cols, ld);
        void *wsv = nullptr;
        st = col_partials(ctx, sc, 2 * p.nparts * cols * sizeof(T), &wsv);
        if (st != DH_OK)
            return st;
        T *pm = static_cast<T *>(wsv);
        T *pq = pm + p.nparts * cols;
        const size_t lds = 2 * static_cast<size_t>(THREADS) * p.vec * sizeof(T);
        if (p.vec == V)
            hipLaunchKernelGGL((col_var_stage1<T, V>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pm, pq);
        else
            hipLaunchKernelGGL((col_var_stage1<T, 1>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pm, pq);
        const dim3 g2(static_cast<unsigned>(dh_ceil_div(cols, V2_TX)));
        if (op == DH_AGG_VAR)
            hipLaunchKernelGGL((col_var_stage2<T, 0>), g2, dim3(V2_TX, V2_TY), 0, ctx->stream, pm, pq, p.nparts, cols, rows, p.slab, res);
        else
            hipLaunchKernelGGL((col_var_stage2<T, 1>), g2, dim3(V2_TX, V2_TY), 0, ctx->stream, pm, pq, p.nparts, cols, rows, p.slab, res);
        break;
    }
    default:
        return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode");
    }
    if (st != DH_OK)
        return st;
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// Column means and variances (or standard deviations) from ONE pass over the matrix: the per-block
// (count, mean, M2) triples that the variance needs carry the mean anyway. Same results as agg_col with
// MEAN and VAR / STDDEV within rounding (the mean comes out of the Chan merge in double instead of sum / rows).
template <typename T>
dh_status agg_col_moments(dh_ctx *ctx, T *res_mean, T *res_var, int stddev, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - leading dimension smaller than the column count");
    if (res_mean == nullptr || res_var == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - result pointer is null");
    if (cols == 0)
        return DH_OK;
    if (rows == 0)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - the argument has no rows");
    constexpr int V = dh_vec<T>::N;
    ColPlan p = col_plan<T>(ctx, arg, rows, cols, ld);
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, 2 * p.nparts * cols * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    T *pm = static_cast<T *>(wsv);
    T *pq = pm + p.nparts * cols;
    const size_t lds = 2 * static_cast<size_t>(THREADS) * p.vec * sizeof(T);
    if (p.vec == V)
        hipLaunchKernelGGL((col_var_stage1<T, V>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pm, pq);
    else
        hipLaunchKernelGGL((col_var_stage1<T, 1>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pm, pq);
    const dim3 g2(static_cast<unsigned>(dh_ceil_div(cols, V2_TX)));
    if (stddev)
        hipLaunchKernelGGL((col_var_stage2<T, 1>), g2, dim3(V2_TX, V2_TY), 0, ctx->stream, pm, pq, p.nparts, cols, rows, p.slab,
                           res_var, res_mean);
    else
        hipLaunchKernelGGL((col_var_stage2<T, 0>), g2, dim3(V2_TX, V2_TY), 0, ctx->stream, pm, pq, p.nparts, cols, rows, p.slab,
                           res_var, res_mean);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

template <typename T> dh_status agg_col_idx(dh_ctx *ctx, int op, uint64_t *res, const T *arg, size_t rows, size_t cols, size_t ld) {
    DH_REQUIRE_CTX(ctx);
    if (ld < cols)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - leading dimension smaller than the column count");
    if (op != DH_AGG_IDXMIN && op != DH_AGG_IDXMAX)
        return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode");
    if (cols == 0)
        return DH_OK;
    if (rows == 0)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - the argument has no rows");
    constexpr int V = dh_vec<T>::N;
    ColPlan p = col_plan<T>(ctx, arg, rows, cols, ld);
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, p.nparts * cols * (sizeof(T) + sizeof(unsigned long long)) + 256, &wsv);
    if (st != DH_OK)
        return st;
    unsigned long long *pidx = static_cast<unsigned long long *>(wsv);
    T *pval = reinterpret_cast<T *>(pidx + p.nparts * cols);
    const size_t lds = static_cast<size_t>(THREADS) * p.vec * (sizeof(T) + sizeof(unsigned long long));
    if (p.slab >= 0xffffffffull)
        return dh_fail(DH_ERR_RUNTIME, "AggCol - more than 2^32 rows per workgroup are not supported");
    const dim3 g2(static_cast<unsigned>(dh_ceil_div(cols, S2_TX)));
    if (op == DH_AGG_IDXMIN) {
        if (p.vec == V)
            hipLaunchKernelGGL((col_idx_stage1<T, V, true>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pval, pidx);
        else
            hipLaunchKernelGGL((col_idx_stage1<T, 1, true>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pval, pidx);
        hipLaunchKernelGGL((col_idx_stage2<T, true>), g2, dim3(S2_TX, S2_TY), 0, ctx->stream, pval, pidx, p.nparts, cols, arg, res);
    } else {
        if (p.vec == V)
            hipLaunchKernelGGL((col_idx_stage1<T, V, false>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pval, pidx);
        else
            hipLaunchKernelGGL((col_idx_stage1<T, 1, false>), p.grid, p.block, lds, ctx->stream, arg, rows, p.cvecs, ld, p.slab, pval, pidx);
        hipLaunchKernelGGL((col_idx_stage2<T, false>), g2, dim3(S2_TX, S2_TY), 0, ctx->stream, pval, pidx, p.nparts, cols, arg, res);
    }
    DH_CHECK_LAUNCH();
    return DH_OK;
}

} // namespace dh_agg
