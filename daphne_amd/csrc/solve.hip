// Dense linear solve A x = b for one right-hand side: LU with partial pivoting in a single
// workgroup, then forward elimination of b (done alongside) and back substitution.
//
// Stands in for CUDA::Solve (src/runtime/local/kernels/CUDA/Solve.cpp:75-151, cuSOLVER
// getrf + getrs) with the result of the CPU kernel (src/runtime/local/kernels/Solve.h:86-116,
// LAPACKE_?gesv): same pivot choice (first row of maximal magnitude), multipliers formed with
// the reciprocal of the pivot. The systems on this path are small (100 x 100 normal equations),
// so the work is latency-bound: a system that fits in LDS (up to about 135 doubles / 190 floats a
// side) is factored there in panels of eight columns; larger ones work in a global scratch copy.
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

// The whole system in LDS, the right-hand side as column n of the matrix, factored in panels of NB columns
// (right-looking LU with partial pivoting; U and the eliminated right-hand side are all that is needed afterwards).
// The work is a chain of latencies, not of arithmetic, so the kernel is built around the number of workgroup
// barriers: three per panel instead of two per column.
//   P   wave 0 alone factors the panel in registers: a lane holds the panel's NB values of rows lane, lane + 64, ...;
//       per column one wave-wide arg-max (register moves), the pivot row broadcast with readlane, the row exchange
//       and the elimination inside the registers. The panel and the NB pivot rows go back to LDS.
//   S1  one thread per column right of the panel: applies the NB row exchanges to its column and solves the NB x NB
//       unit-lower triangle for the column's part of U (forward substitution in registers).
//   S2  all threads: rank-NB update of the trailing matrix, thread (column, row group) keeping the column's NB values
//       of U in registers.
// Same pivot choice as ?gesv (first row of the largest magnitude), multipliers formed with the reciprocal of the
// pivot. Back substitution runs in wave 0 alone, right-hand side in registers, one register exchange per unknown.
// The kernel clears the singularity flag itself.
constexpr int LDS_SOLVE_MAX_SLOTS = 3;   // rows per lane of wave 0: n <= 192
constexpr int LDS_SOLVE_NB = 8;          // panel width
constexpr unsigned LDS_SOLVE_THREADS = 512;
constexpr unsigned LDS_SOLVE_TX = 128;   // column threads of the update; LDS_SOLVE_THREADS / TX row groups

#ifdef DH_SOLVE_PROFILE
__device__ long long g_solve_prof[8];
#define DH_PROF_DECL long long prof_t = __builtin_amdgcn_s_memtime(), prof_acc[6] = {0, 0, 0, 0, 0, 0}
#define DH_PROF(slot)                                                                                                      \
    do {                                                                                                                   \
        const long long now__ = __builtin_amdgcn_s_memtime();                                                              \
        prof_acc[slot] += now__ - prof_t;                                                                                  \
        prof_t = now__;                                                                                                    \
    } while (0)
#define DH_PROF_FLUSH                                                                                                      \
    do {                                                                                                                   \
        if (threadIdx.x == 0)                                                                                              \
            for (int q__ = 0; q__ < 6; q__++)                                                                              \
                g_solve_prof[q__] = prof_acc[q__];                                                                         \
    } while (0)
#else
#define DH_PROF_DECL
#define DH_PROF(slot)
#define DH_PROF_FLUSH
#endif

template <typename T> __device__ __forceinline__ T read_lane(T v, int src) { // src is the same in all lanes
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src));
    } else {
        const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(u & 0xffffffffu), src));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(u >> 32), src));
        return __builtin_bit_cast(T, (static_cast<unsigned long long>(hi) << 32) | lo);
    }
}

template <typename T, int SLOTS>
__global__ __launch_bounds__(LDS_SOLVE_THREADS) void lu_solve_lds_kernel(T *x_out, const T *A, size_t lda, const T *b, unsigned n,
                                                                         int *flag) {
    constexpr int NB = LDS_SOLVE_NB;
    constexpr unsigned TX = LDS_SOLVE_TX, TY = LDS_SOLVE_THREADS / LDS_SOLVE_TX;
    extern __shared__ __attribute__((aligned(16))) unsigned char solve_lds[];
    __shared__ int s_stop;
    __shared__ unsigned s_piv[NB];
    const unsigned ld = (n + 1) | 1u; // n + 1 columns; odd stride: column walks spread over the banks
    T *a = reinterpret_cast<T *>(solve_lds);
    const unsigned tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const unsigned tx = tid % TX, ty = tid / TX;
    // copy-in: a thread's loads go out in batches of eight before the first LDS store (positions past the matrix
    // read its last row and are not stored)
    for (unsigned r0 = ty; r0 < n; r0 += TY * 8) {
        for (unsigned c = tx; c < n; c += TX) {
            T v[8];
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const unsigned r = r0 + TY * q;
                v[q] = A[static_cast<size_t>(r < n ? r : n - 1) * lda + c];
            }
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const unsigned r = r0 + TY * q;
                if (r < n)
                    a[r * ld + c] = v[q];
            }
        }
    }
    for (unsigned i = tid; i < n; i += LDS_SOLVE_THREADS)
        a[i * ld + n] = b[i];
    if (tid == 0) {
        s_stop = 0;
        *flag = 0;
    }
    DH_PROF_DECL;
    __syncthreads();
    DH_PROF(0); // copy-in

    for (unsigned k0 = 0; k0 < n; k0 += NB) {
        const unsigned nb = n - k0 < NB ? n - k0 : NB;
        if (wave == 0) {
            // ---- P: the panel, rows k0 .. n - 1, in registers
            T pv[SLOTS][NB];
#pragma unroll
            for (int s = 0; s < SLOTS; s++) {
                const unsigned r = lane + 64 * s;
#pragma unroll
                for (int c = 0; c < NB; c++)
                    pv[s][c] = (r >= k0 && r < n && static_cast<unsigned>(c) < nb) ? a[r * ld + k0 + c] : T(0);
            }
            bool singular = false;
#pragma unroll
            for (int jj = 0; jj < NB; jj++) {
                if (static_cast<unsigned>(jj) < nb && !singular) {
                    const unsigned j = k0 + jj;
                    // pivot: first row r >= j with the largest |value| in column jj
                    T best = T(-1);
                    unsigned bi = 0xffffffffu;
#pragma unroll
                    for (int s = 0; s < SLOTS; s++) {
                        const unsigned r = lane + 64 * s;
                        const T v = dev_abs(pv[s][jj]);
                        if (r >= j && r < n && v > best) {
                            best = v;
                            bi = r;
                        }
                    }
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
                    unsigned p = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(bi)));
                    if (p == 0xffffffffu) // nothing compares larger (a column of NaNs): stay on the diagonal
                        p = j;
                    {
                        if (lane == 0)
                            s_piv[jj] = p;
                        const int lp = static_cast<int>(p % 64), sp = static_cast<int>(p / 64);
                        const int lj = static_cast<int>(j % 64), sj = static_cast<int>(j / 64);
                        T prow[NB];
#pragma unroll
                        for (int c = 0; c < NB; c++) {
                            T mine_p = pv[0][c], mine_j = pv[0][c];
#pragma unroll
                            for (int s = 1; s < SLOTS; s++) {
                                mine_p = sp == s ? pv[s][c] : mine_p;
                                mine_j = sj == s ? pv[s][c] : mine_j;
                            }
                            const T vp = read_lane(mine_p, lp), vj = read_lane(mine_j, lj);
                            prow[c] = vp;
                            if (p != j) { // exchange rows p and j inside the panel
#pragma unroll
                                for (int s = 0; s < SLOTS; s++) {
                                    if (sp == s && static_cast<int>(lane) == lp)
                                        pv[s][c] = vj;
                                    if (sj == s && static_cast<int>(lane) == lj)
                                        pv[s][c] = vp;
                                }
                            }
                        }
                        if (prow[jj] == T(0)) { // info > 0 of ?gesv
                            singular = true;
                            if (lane == 0) {
                                *flag = static_cast<int>(j) + 1;
                                s_stop = 1;
                            }
                        }
                        const T inv = T(1) / prow[jj];
#pragma unroll
                        for (int s = 0; s < SLOTS; s++) {
                            const unsigned r = lane + 64 * s;
                            if (r > j && r < n && !singular) {
                                const T l = pv[s][jj] * inv;
                                pv[s][jj] = l;
#pragma unroll
                                for (int c = jj + 1; c < NB; c++)
                                    pv[s][c] -= l * prow[c];
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < SLOTS; s++) {
                const unsigned r = lane + 64 * s;
                if (r >= k0 && r < n) {
#pragma unroll
                    for (int c = 0; c < NB; c++)
                        if (static_cast<unsigned>(c) < nb)
                            a[r * ld + k0 + c] = pv[s][c];
                }
            }
        }
        __syncthreads();
        DH_PROF(1); // panel
        if (s_stop)
            return;
        const unsigned cfirst = k0 + nb; // first column right of the panel; column n is the right-hand side
        // ---- S1: row exchanges and the panel's rows of U, one thread per column
        for (unsigned c = cfirst + tid; c <= n; c += LDS_SOLVE_THREADS) {
            for (unsigned jj = 0; jj < nb; jj++) {
                const unsigned p = s_piv[jj], j = k0 + jj;
                if (p != j) {
                    const T t = a[j * ld + c];
                    a[j * ld + c] = a[p * ld + c];
                    a[p * ld + c] = t;
                }
            }
            T u[NB];
#pragma unroll
            for (int jj = 0; jj < NB; jj++)
                u[jj] = static_cast<unsigned>(jj) < nb ? a[(k0 + jj) * ld + c] : T(0);
#pragma unroll
            for (int jj = 1; jj < NB; jj++) {
                if (static_cast<unsigned>(jj) < nb) {
#pragma unroll
                    for (int m = 0; m < jj; m++)
                        u[jj] -= a[(k0 + jj) * ld + k0 + m] * u[m];
                    a[(k0 + jj) * ld + c] = u[jj];
                }
            }
        }
        __syncthreads();
        DH_PROF(2); // exchanges and the panel's rows of U
        // ---- S2: trailing update, thread (column, row group)
        if (cfirst < n) {
            for (unsigned c = cfirst + tx; c <= n; c += TX) {
                T u[NB];
#pragma unroll
                for (int m = 0; m < NB; m++)
                    u[m] = static_cast<unsigned>(m) < nb ? a[(k0 + m) * ld + c] : T(0);
                for (unsigned i = cfirst + ty; i < n; i += TY) {
                    T v = a[i * ld + c];
#pragma unroll
                    for (int m = 0; m < NB; m++)
                        v -= (static_cast<unsigned>(m) < nb ? a[i * ld + k0 + m] : T(0)) * u[m];
                    a[i * ld + c] = v;
                }
            }
        }
        __syncthreads();
        DH_PROF(3); // trailing update
    }
    if (wave != 0)
        return;
    // back substitution, column oriented: x[j] = rhs[j] / U[j][j]; rhs[r] -= U[r][j] x[j] for r < j
    T rhs[SLOTS], res[SLOTS];
#pragma unroll
    for (int s_ = 0; s_ < SLOTS; s_++) {
        const unsigned r = lane + 64 * s_;
        rhs[s_] = r < n ? a[r * ld + n] : T(0);
        res[s_] = T(0);
    }
    for (unsigned jj = n; jj-- > 0;) {
        const int slot = static_cast<int>(jj / 64), owner = static_cast<int>(jj % 64);
        T mine = rhs[0];
#pragma unroll
        for (int s_ = 1; s_ < SLOTS; s_++)
            mine = slot == s_ ? rhs[s_] : mine;
        const T xj = read_lane(mine, owner) / a[jj * ld + jj];
#pragma unroll
        for (int s_ = 0; s_ < SLOTS; s_++) {
            const unsigned r = lane + 64 * s_;
            if (r < jj)
                rhs[s_] -= a[r * ld + jj] * xj;
            else if (r == jj)
                res[s_] = xj;
        }
    }
#pragma unroll
    for (int s_ = 0; s_ < SLOTS; s_++) {
        const unsigned r = lane + 64 * s_;
        if (r < n)
            x_out[r] = res[s_];
    }
    DH_PROF(4); // back substitution
    DH_PROF_FLUSH;
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
    const size_t lds_bytes = n * ((n + 1) | 1) * sizeof(T);
    if (n <= 64 * LDS_SOLVE_MAX_SLOTS && lds_bytes <= (size_t(150) << 10)) {
        auto launch = [&](auto kernel) -> dh_status {
            if (lds_bytes > (size_t(64) << 10)) {
                static std::mutex attr_lock;
                static bool attr_set[16] = {};
                std::lock_guard<std::mutex> guard(attr_lock);
                if (ctx->device < 16 && !attr_set[ctx->device]) {
                    DH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                     150 << 10));
                    attr_set[ctx->device] = true;
                }
            }
            hipLaunchKernelGGL(kernel, dim3(1), dim3(LDS_SOLVE_THREADS), lds_bytes, ctx->stream, x, A, lda, b,
                               static_cast<unsigned>(n), ctx->flag_dev);
            return DH_OK;
        };
        dh_status lst;
        if (n <= 64)
            lst = launch(&lu_solve_lds_kernel<T, 1>);
        else if (n <= 128)
            lst = launch(&lu_solve_lds_kernel<T, 2>);
        else
            lst = launch(&lu_solve_lds_kernel<T, 3>);
        if (lst != DH_OK)
            return lst;
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
