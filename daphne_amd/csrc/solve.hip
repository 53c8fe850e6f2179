// Dense linear solve A x = b for one right-hand side: LU with partial pivoting in a single
// workgroup, then forward elimination of b (done alongside) and back substitution.
//
// Stands in for CUDA::Solve (src/runtime/local/kernels/CUDA/Solve.cpp:75-151, cuSOLVER
// getrf + getrs) with the result of the CPU kernel (src/runtime/local/kernels/Solve.h:86-116,
// LAPACKE_?gesv): same pivot choice (first row of maximal magnitude), multipliers formed with
// the reciprocal of the pivot. The systems on this path are small (100 x 100 normal equations),
// so one workgroup working in a global scratch copy of A is latency-, not throughput-bound.
#include "common.h"

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

__global__ void clear_flag_kernel(int *flag) { *flag = 0; }

template <typename T> dh_status solve(dh_ctx *ctx, T *x, const T *A, size_t n, size_t lda, const T *b) {
    DH_REQUIRE_CTX(ctx);
    if (n == 0)
        return DH_OK;
    if (lda < n)
        return dh_fail(DH_ERR_RUNTIME, "#cols of lhs must match row skip");
    if (n >= (size_t(1) << 15))
        return dh_fail(DH_ERR_RUNTIME, "Solve: systems beyond 32767 unknowns are not supported by this kernel");
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, n * n * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev);
    hipLaunchKernelGGL((lu_solve_kernel<T>), dim3(1), dim3(SOLVE_THREADS), 0, ctx->stream, static_cast<T *>(wsv), x, A,
                       lda, b, static_cast<unsigned>(n), ctx->flag_dev);
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
