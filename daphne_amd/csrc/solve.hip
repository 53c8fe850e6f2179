// Dense linear solve A x = b for one right-hand side: LU with partial pivoting in a single
// workgroup, then forward elimination of b (done alongside) and back substitution.
//
// Stands in for CUDA::Solve (src/runtime/local/kernels/CUDA/Solve.cpp:75-151, cuSOLVER
// getrf + getrs) with the result of the CPU kernel (src/runtime/local/kernels/Solve.h:86-116,
// LAPACKE_?gesv): same pivot choice (first row of maximal magnitude), multipliers formed with
// the reciprocal of the pivot. The systems on this path are small (100 x 100 normal equations),
// so the work is latency-bound: a system that fits in LDS (up to about 135 doubles / 190 floats a
// side) is factored there with two barriers per column; larger ones work in a global scratch copy.
#include "common.h"

#include <type_traits>

namespace {

constexpr int SOLVE_THREADS = 1024;

template <typename T> __device__ __forceinline__ T dev_abs(T a) { return a < T(0) ? -a : a; }

template <typename T>
__global__ __launch_bounds__(SOLVE_THREADS) void lu_solve_kernel(T *lu, T *x, const T *A, size_t lda, const T *b,
                                                                 unsigned n, int *flag) {
    __shared__ T s_val[SOLVE_THREADS];
    __shared__ unsigned s_idx[SOLVE_THREADS];
    __shared__ int s_stop;
    const unsigned tid = threadIdx.x, nt = blockDim.x;
    for (size_t i = tid; i < static_cast<size_t>(n) * n; i += nt)
        lu[i] = A[(i / n) * lda + (i % n)];
    for (unsigned i = tid; i < n; i += nt)
        x[i] = b[i];
    if (tid == 0)
        s_stop = 0;
    __syncthreads();
    for (unsigned j = 0; j < n; j++) {
        // pivot: first row i >= j with the largest |lu[i][j]|
        T best = T(-1);
        unsigned bi = j;
        for (unsigned i = j + tid; i < n; i += nt) {
            const T v = dev_abs(lu[static_cast<size_t>(i) * n + j]);
            if (v > best) {
                best = v;
                bi = i;
            }
        }
        s_val[tid] = best;
        s_idx[tid] = bi;
        __syncthreads();
        for (unsigned s = nt / 2; s >= 1; s >>= 1) {
            if (tid < s) {
                const T ov = s_val[tid + s];
                const unsigned oi = s_idx[tid + s];
                if (ov > s_val[tid] || (ov == s_val[tid] && oi < s_idx[tid])) {
                    s_val[tid] = ov;
                    s_idx[tid] = oi;
                }
            }
            __syncthreads();
        }
        const unsigned p = s_idx[0];
        if (tid == 0 && lu[static_cast<size_t>(p) * n + j] == T(0)) {
            *flag = static_cast<int>(j) + 1; // info > 0 of ?gesv
            s_stop = 1;
        }
        __syncthreads();
        if (s_stop)
            return;
        if (p != j) {
            for (unsigned c = tid; c < n; c += nt) {
                const T t = lu[static_cast<size_t>(j) * n + c];
                lu[static_cast<size_t>(j) * n + c] = lu[static_cast<size_t>(p) * n + c];
                lu[static_cast<size_t>(p) * n + c] = t;
            }
            if (tid == 0) {
                const T t = x[j];
                x[j] = x[p];
                x[p] = t;
            }
        }
        __syncthreads();
        const T inv = T(1) / lu[static_cast<size_t>(j) * n + j];
        for (unsigned i = j + 1 + tid; i < n; i += nt) {
            const T l = lu[static_cast<size_t>(i) * n + j] * inv;
            lu[static_cast<size_t>(i) * n + j] = l;
            x[i] -= l * x[j];
        }
        __syncthreads();
        const unsigned rem = n - j - 1;
        for (size_t e = tid; e < static_cast<size_t>(rem) * rem; e += nt) {
            const unsigned i = j + 1 + static_cast<unsigned>(e / rem), c = j + 1 + static_cast<unsigned>(e % rem);
            lu[static_cast<size_t>(i) * n + c] -= lu[static_cast<size_t>(i) * n + j] * lu[static_cast<size_t>(j) * n + c];
        }
        __syncthreads();
    }
    // back substitution
    for (unsigned ii = n; ii-- > 0;) {
        T s = T(0);
        for (unsigned c = ii + 1 + tid; c < n; c += nt)
            s += lu[static_cast<size_t>(ii) * n + c] * x[c];
        s_val[tid] = s;
        __syncthreads();
        for (unsigned st = nt / 2; st >= 1; st >>= 1) {
            if (tid < st)
                s_val[tid] += s_val[tid + st];
            __syncthreads();
        }
        if (tid == 0)
            x[ii] = (x[ii] - s_val[0]) / lu[static_cast<size_t>(ii) * n + ii];
        __syncthreads();
    }
}

// The whole system in LDS, the right-hand side as column n of the matrix. Per column: wave 0 finds the pivot
// (register-move reduction), swaps the rows and publishes the pivot row; after one barrier all 1024 threads apply
// the rank-1 update (32 x 32 thread grid, multipliers recomputed per row instead of stored: only U and the
// eliminated right-hand side are needed afterwards); a second barrier closes the column. Back substitution runs
// in wave 0 alone, right-hand side in registers, one shuffle per unknown. The kernel clears the singularity flag
// itself.
constexpr int LDS_SOLVE_MAX_SLOTS = 3; // rows per lane in the back substitution: n <= 192
constexpr unsigned LDS_SOLVE_TG = 32;  // the update runs on a TG x TG grid of threads (1024: four waves per SIMD)

template <typename T>
__global__ __launch_bounds__(LDS_SOLVE_TG * LDS_SOLVE_TG) void lu_solve_lds_kernel(T *x_out, const T *A, size_t lda, const T *b, unsigned n,
                                                           int *flag) {
    extern __shared__ __attribute__((aligned(16))) unsigned char solve_lds[];
    __shared__ int s_stop;
    const unsigned ld = (n + 1) | 1u; // n + 1 columns; odd stride: column walks spread over the banks
    T *a = reinterpret_cast<T *>(solve_lds);
    T *prow = a + static_cast<size_t>(n) * ld; // n + 1 entries
    const unsigned tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    constexpr unsigned TG = LDS_SOLVE_TG;
    const unsigned tx = tid % TG, ty = tid / TG;
    // copy-in: TG x TG threads over (row, column); a thread's loads go out in batches of eight before the first
    // LDS store (positions past the matrix read its last element and are not stored)
    for (unsigned r0 = ty; r0 < n; r0 += TG * 8) {
        for (unsigned c = tx; c < n; c += TG) {
            T v[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const unsigned r = r0 + TG * k;
                v[k] = A[static_cast<size_t>(r < n ? r : n - 1) * lda + c];
            }
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const unsigned r = r0 + TG * k;
                if (r < n)
                    a[r * ld + c] = v[k];
            }
        }
    }
    for (unsigned i = tid; i < n; i += TG * TG)
        a[i * ld + n] = b[i];
    if (tid == 0) {
        s_stop = 0;
        *flag = 0;
    }
    __syncthreads();
    for (unsigned j = 0; j < n; j++) {
        if (wave == 0) {
            // pivot: first row i >= j with the largest |a[i][j]|
            T best = T(-1);
            unsigned bi = j;
            for (unsigned i = j + lane; i < n; i += 64) {
                const T v = dev_abs(a[i * ld + j]);
                if (v > best) {
                    best = v;
                    bi = i;
                }
            }
            // the largest value first (one instruction per level), then the lowest row among the lanes that hold it
            T top = best;
            dh_butterfly(64, [&](auto peer) {
                const T ov = peer(top);
                top = ov > top ? ov : top;
            });
            if (best != top)
                bi = 0xffffffffu;
            dh_butterfly(64, [&](auto peer) {
                const unsigned oi = peer(bi);
                bi = oi < bi ? oi : bi;
            });
            const unsigned p = bi;
            if (a[p * ld + j] == T(0)) {
                if (lane == 0) {
                    *flag = static_cast<int>(j) + 1; // info > 0 of ?gesv
                    s_stop = 1;
                }
            } else {
                for (unsigned c = j + lane; c <= n; c += 64) {
                    const T pv = a[p * ld + c];
                    prow[c] = pv;
                    if (p != j) {
                        a[p * ld + c] = a[j * ld + c];
                        a[j * ld + c] = pv;
                    }
                }
            }
        }
        __syncthreads();
        if (s_stop)
            return;
        const T inv = T(1) / prow[j];
        // Rank-1 update of the rows and columns past j, KM rows x (KM + 1) columns per thread. All operands are read
        // before the first result is written (the compiler must assume that the stores alias the loads, which
        // would make every element wait for its predecessor): positions past the end read element (n - 1, n).
        auto update = [&](auto km_tag) {
            constexpr int KM = decltype(km_tag)::value;
            T l[KM], pc[KM + 1], v[KM][KM + 1];
#pragma unroll
            for (int k = 0; k < KM; k++) {
                const unsigned i = j + 1 + ty + TG * k;
                l[k] = a[(i < n ? i : n - 1) * ld + j];
            }
#pragma unroll
            for (int m = 0; m <= KM; m++) {
                const unsigned c = j + 1 + tx + TG * m;
                pc[m] = prow[c <= n ? c : n];
            }
#pragma unroll
            for (int k = 0; k < KM; k++)
#pragma unroll
                for (int m = 0; m <= KM; m++) {
                    const unsigned i = j + 1 + ty + TG * k, c = j + 1 + tx + TG * m;
                    v[k][m] = a[(i < n ? i : n - 1) * ld + (c <= n ? c : n)];
                }
#pragma unroll
            for (int k = 0; k < KM; k++) {
                const unsigned i = j + 1 + ty + TG * k;
                const T lk = l[k] * inv;
#pragma unroll
                for (int m = 0; m <= KM; m++) {
                    const unsigned c = j + 1 + tx + TG * m;
                    if (i < n && c <= n)
                        a[i * ld + c] = v[k][m] - lk * pc[m];
                }
            }
        };
        switch ((n - j - 1 + TG - 1) / TG) { // blocks of TG rows left; the columns (one more: the right-hand side) need at most one block more
        case 0:
            break;
        case 1:
            update(std::integral_constant<int, 1>{});
            break;
        case 2:
            update(std::integral_constant<int, 2>{});
            break;
        case 3:
            update(std::integral_constant<int, 3>{});
            break;
        case 4:
            update(std::integral_constant<int, 4>{});
            break;
        case 5:
            update(std::integral_constant<int, 5>{});
            break;
        case 6:
            update(std::integral_constant<int, 6>{});
            break;
        default:
            for (unsigned i = j + 1 + ty; i < n; i += TG) {
                const T l = a[i * ld + j] * inv;
                for (unsigned c = j + 1 + tx; c <= n; c += TG)
                    a[i * ld + c] -= l * prow[c];
            }
        }
        __syncthreads();
    }
    if (wave != 0)
        return;
    // back substitution, column oriented: x[j] = rhs[j] / U[j][j]; rhs[r] -= U[r][j] x[j] for r < j
    T rhs[LDS_SOLVE_MAX_SLOTS], res[LDS_SOLVE_MAX_SLOTS];
#pragma unroll
    for (int s_ = 0; s_ < LDS_SOLVE_MAX_SLOTS; s_++) {
        const unsigned r = lane + 64 * s_;
        rhs[s_] = r < n ? a[r * ld + n] : T(0);
        res[s_] = T(0);
    }
    for (unsigned jj = n; jj-- > 0;) {
        const unsigned slot = jj / 64, owner = jj % 64;
        const T mine = slot == 0 ? rhs[0] : (slot == 1 ? rhs[1] : rhs[2]);
        const T xj = __shfl(mine, owner) / a[jj * ld + jj];
#pragma unroll
        for (int s_ = 0; s_ < LDS_SOLVE_MAX_SLOTS; s_++) {
            const unsigned r = lane + 64 * s_;
            if (r < jj)
                rhs[s_] -= a[r * ld + jj] * xj;
            else if (r == jj)
                res[s_] = xj;
        }
    }
#pragma unroll
    for (int s_ = 0; s_ < LDS_SOLVE_MAX_SLOTS; s_++) {
        const unsigned r = lane + 64 * s_;
        if (r < n)
            x_out[r] = res[s_];
    }
}

__global__ void clear_flag_kernel(int *flag) { *flag = 0; }

template <typename T> dh_status solve(dh_ctx *ctx, T *x, const T *A, size_t n, size_t lda, const T *b) {
    DH_REQUIRE_CTX(ctx);
    if (n == 0)
        return DH_OK;
    if (lda < n)
        return dh_fail(DH_ERR_RUNTIME, "#cols of lhs must match row skip");
    if (n >= (size_t(1) << 15))
        return dh_fail(DH_ERR_RUNTIME, "Solve: systems beyond 32767 unknowns are not supported by this kernel");
    const size_t lds_bytes = (n * ((n + 1) | 1) + n + 1) * sizeof(T);
    if (n <= 64 * LDS_SOLVE_MAX_SLOTS && lds_bytes <= (size_t(150) << 10)) {
        if (lds_bytes > (size_t(64) << 10)) {
            static std::mutex attr_lock;
            static bool attr_set[16] = {};
            std::lock_guard<std::mutex> guard(attr_lock);
            if (ctx->device < 16 && !attr_set[ctx->device]) {
                DH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&lu_solve_lds_kernel<T>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 150 << 10));
                attr_set[ctx->device] = true;
            }
        }
        hipLaunchKernelGGL((lu_solve_lds_kernel<T>), dim3(1), dim3(LDS_SOLVE_TG * LDS_SOLVE_TG), lds_bytes, ctx->stream, x, A, lda, b,
                           static_cast<unsigned>(n), ctx->flag_dev);
    } else {
        hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev);
        void *wsv = nullptr;
        dh_status st = dh_workspace(ctx, n * n * sizeof(T), &wsv);
        if (st != DH_OK)
            return st;
        hipLaunchKernelGGL((lu_solve_kernel<T>), dim3(1), dim3(SOLVE_THREADS), 0, ctx->stream, static_cast<T *>(wsv), x,
                           A, lda, b, static_cast<unsigned>(n), ctx->flag_dev);
    }
    DH_CHECK_LAUNCH();
    DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (*ctx->flag_host != 0)
        // Solve.h:113-115
        return dh_fail(DH_ERR_RUNTIME, "A factor Ui is exactly singular, so the solution could not be computed");
    return DH_OK;
}

} // namespace

extern "C" dh_status dh_solve_f32(dh_ctx *ctx, float *x, const float *A, size_t n, size_t lda, const float *b) {
    return solve<float>(ctx, x, A, n, lda, b);
}
extern "C" dh_status dh_solve_f64(dh_ctx *ctx, double *x, const double *A, size_t n, size_t lda, const double *b) {
    return solve<double>(ctx, x, A, n, lda, b);
}
