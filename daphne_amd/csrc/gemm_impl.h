// MFMA GEMM for gfx950, the engine under MatMul, Syrk, Affine (and the 1x1 / fully connected
// ends of the DNN path). Instantiated per value type by gemm_f32.hip / gemm_f64.hip.
//
//   C[m x n] = op(A) * op(B)     row-major, op = identity or transpose (the reference's
//                                 transa / transb flags, kernels/CUDA/MatMul.h:31-51)
//
// Matrix instructions: v_mfma_f64_16x16x4_f64 for double, v_mfma_f32_32x32x2_f32 for float
// (gfx950 has no xf32 variant). A workgroup of WM x WN wavefronts owns a BM x BN tile of C; each
// wavefront owns (BM/WM) x (BN/WN) of it as FM x FN MFMA tiles whose accumulators stay in
// registers for the whole K loop.
//
// Operand tiles travel global -> registers -> LDS with 16-byte loads along whatever dimension
// is contiguous in memory, and are stored in LDS *as loaded* (no transposition on the write
// side): an operand whose K index is contiguous lands as [row][k] ("RK"), the other way round as
// [k][row] ("KR"). The MFMA fragment reads adapt to the layout, and the inner LDS stride is
// padded so that the 16 (f64) / 32 (f32) lanes of a fragment row group and the K groups next to
// them fall into different banks. LDS is double buffered: the global loads of K tile t+1 are
// issued before the MFMAs of tile t and written to the other buffer after them, so one barrier
// per K tile suffices.
//
// Workgroup -> tile mapping is XCD aware: consecutive workgroup ids are dealt round-robin to the
// 8 XCDs (each with a private L2), so ids are first regrouped per XCD and then walked in
// column-major order over panels of 8 tile rows, which keeps the A panel and the current B tile
// column hot in that XCD's L2.
//
// Split-K (grid.z) writes one partial slab per K slice into a workspace; a second kernel adds
// the slabs in a fixed order (deterministic), optionally mirrors the upper triangle (Syrk) or
// adds a bias row (Affine).
#pragma once

#include "common.h"

namespace dh_gemm {

typedef double mfma_f64x4 __attribute__((ext_vector_type(4)));
typedef float mfma_f32x16 __attribute__((ext_vector_type(16)));

template <typename T> struct Mfma;
template <> struct Mfma<double> {
    static constexpr int MT = 16, NT = 16, KT = 4, ACC = 4, ROWS = 16; // lanes per K group = 16
    using acc_t = mfma_f64x4;
    static __device__ __forceinline__ acc_t zero() { return acc_t{0, 0, 0, 0}; }
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    // accumulator register v of lane l holds C[row(l, v)][col(l)]
    static __device__ __forceinline__ int row(int lane, int v) { return 4 * v + (lane / 16); }
    static __device__ __forceinline__ int col(int lane) { return lane % 16; }
};
template <> struct Mfma<float> {
    static constexpr int MT = 32, NT = 32, KT = 2, ACC = 16, ROWS = 32;
    using acc_t = mfma_f32x16;
    static __device__ __forceinline__ acc_t zero() {
        return acc_t{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    }
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int lane, int v) { return 8 * (v / 4) + 4 * (lane / 32) + (v % 4); }
    static __device__ __forceinline__ int col(int lane) { return lane % 32; }
};

// LDS layout of one operand tile of R rows (M or N side) by BK.
//   KCONTIG: memory contiguous along K  -> [R][BK + PAD]  ("RK")
//   else:    memory contiguous along R  -> [BK][R + PAD]  ("KR")
template <typename T, int R, int BK, bool KCONTIG> struct TileLayout {
    static constexpr int VEC = 16 / sizeof(T);
    static constexpr int OUTER = KCONTIG ? R : BK;
    static constexpr int INNER = KCONTIG ? BK : R;
    // pads chosen so that fragment reads spread over the banks (see file comment)
    static constexpr int PAD = KCONTIG ? (sizeof(T) == 8 ? 2 : 4) : (sizeof(T) == 8 ? 16 : 32);
    static constexpr int STRIDE = INNER + PAD;
    static constexpr int ELEMS = OUTER * STRIDE;
    static __device__ __forceinline__ int at(int row, int k) { return KCONTIG ? row * STRIDE + k : k * STRIDE + row; }
};

// Loads this thread's share of a tile from global memory into registers (zero filled outside
// the matrix) and stores it to LDS. `outer0` / `inner0` are the tile origin along the
// non-contiguous / contiguous dimension of the stored matrix, `outer_n` / `inner_n` its extents.
template <typename T, int R, int BK, bool KCONTIG, int THREADS> struct TileMover {
    using L = TileLayout<T, R, BK, KCONTIG>;
    static constexpr int VEC = L::VEC;
    static constexpr int VPR = L::INNER / VEC;               // vectors per tile row
    static constexpr int NVEC = L::OUTER * VPR;              // vectors per tile
    static constexpr int PER_THREAD = (NVEC + THREADS - 1) / THREADS;
    T regs[PER_THREAD][VEC];

    __device__ __forceinline__ void load(const T *__restrict__ base, size_t ld, size_t outer0, size_t inner0,
                                         size_t outer_n, size_t inner_n, bool aligned, int tid) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int v = tid + i * THREADS;
            const int o = v / VPR, iv = v % VPR;
            const size_t go = outer0 + o, gi = inner0 + static_cast<size_t>(iv) * VEC;
            const bool in_tile = (NVEC % THREADS == 0) || (v < NVEC);
            if (in_tile && go < outer_n && aligned && gi + VEC <= inner_n) {
                using V = typename dh_vec<T>::type;
                const V t = *reinterpret_cast<const V *>(base + go * ld + gi);
                const T *tp = reinterpret_cast<const T *>(&t);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    regs[i][e] = tp[e];
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    regs[i][e] = (in_tile && go < outer_n && gi + e < inner_n) ? base[go * ld + gi + e] : T(0);
            }
        }
    }
    // Interior tile of an aligned matrix: plain 16-byte loads, no bounds logic.
    __device__ __forceinline__ void load_full(const T *__restrict__ base, size_t ld, size_t outer0, size_t inner0,
                                              int tid) {
        static_assert(NVEC % THREADS == 0, "full tiles only for tile shapes that divide evenly");
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int v = tid + i * THREADS;
            const int o = v / VPR, iv = v % VPR;
            dh_load_vec<T, VEC>(base + (outer0 + o) * ld + inner0 + static_cast<size_t>(iv) * VEC, regs[i]);
        }
    }
    __device__ __forceinline__ void store(T *lds, int tid) const {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int v = tid + i * THREADS;
            if ((NVEC % THREADS == 0) || (v < NVEC)) {
                const int o = v / VPR, iv = v % VPR;
                using V = typename dh_vec<T>::type;
                V t;
                T *tp = reinterpret_cast<T *>(&t);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    tp[e] = regs[i][e];
                *reinterpret_cast<V *>(lds + o * L::STRIDE + iv * VEC) = t;
            }
        }
    }
};

enum Epilogue { EPI_STORE = 0, EPI_BIAS = 1 };

struct GemmArgs {
    const void *A;
    const void *B;
    void *C;
    const void *bias; // EPI_BIAS: added to every row, bias[c * bias_stride]
    size_t bias_stride; // 1: one value per column; 0: a single value broadcast (1 x 1 bias)
    size_t m, n, k;
    size_t lda, ldb, ldc;
    size_t k_chunk;     // K range per grid.z slice (multiple of BK)
    size_t slab_stride; // elements between the C slabs of consecutive K slices (0 if grid.z == 1)
    int tiles_m, tiles_n;
    int triangular;     // 1: only tiles with tile_n >= tile_m exist (Syrk)
    int aligned_a, aligned_b;
    int tile_offset;    // added to the workgroup's tile id (the launch that finishes the tiles a first launch left)
    int compact;        // 1: C holds one dense BM x BN block per (K slice, workgroup) instead of the result matrix
    int relu;           // 1: max(0, .) on the finished values (with the bias, where the bias is added)
};

// max(x, 0) with the comparison of the elementwise MAX operator ((x < 0) ? 0 : x: NaN and -0 pass through).
template <typename T> __device__ __forceinline__ T relu_of(T x) { return (x < T(0)) ? T(0) : x; }

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs: regroup them so that each XCD walks a
// contiguous range of tile ids.
__device__ __forceinline__ int regroup_for_xcds(int id, int nb) {
    constexpr int XCDS = 8;
    return (nb % XCDS == 0) ? (id % XCDS) * (nb / XCDS) + id / XCDS : id;
}

// Maps a tile id to a tile. Rectangular results: panels of 8 tile rows, walked down the rows first, so that
// 64 consecutive ids share 8 row panels of A and 8 column panels of B. Triangular results: the same 8 x 8
// groups over the tiles on and above the diagonal (the groups on the diagonal hold their upper triangle).
__device__ __forceinline__ void tile_of_id(const GemmArgs &g, int id, int &tm, int &tn) {
    constexpr int PANEL = 8;
    if (g.triangular) {
        const int nt = g.tiles_n;
        int first = 0, rem = id, h = 0, diag = 0;
        for (;; first += PANEL) {
            h = (nt - first < PANEL) ? nt - first : PANEL; // tile rows in this panel
            diag = h * (h + 1) / 2;
            const int right = (nt - first - PANEL > 0) ? nt - first - PANEL : 0; // tile columns right of the diagonal group
            const int here = diag + h * right;
            if (rem < here || first + PANEL >= nt)
                break;
            rem -= here;
        }
        if (rem < diag) {
            int i = 0;
            while (rem >= h - i) {
                rem -= h - i;
                i++;
            }
            tm = first + i;
            tn = first + i + rem;
        } else {
            rem -= diag;
            tm = first + rem % h;
            tn = first + PANEL + rem / h;
        }
        return;
    }
    const int per_panel = PANEL * g.tiles_n;
    const int panel = id / per_panel;
    const int first_m = panel * PANEL;
    const int rows_here = (g.tiles_m - first_m < PANEL) ? g.tiles_m - first_m : PANEL;
    const int in_panel = id % per_panel;
    tm = first_m + in_panel % rows_here;
    tn = in_panel / rows_here;
}

// FULL: every tile is interior and both operands are 16-byte aligned (checked on the host): no
// bounds logic in the loads and stores, and the register budget is held to two workgroups per CU
// so that a second wavefront per SIMD covers the global-load latency of the first.
template <typename T, int BM, int BN, int BK, int WM, int WN, bool TA, bool TB, int EPI, bool FULL = false>
__global__ __launch_bounds__(64 * WM * WN, FULL ? 2 : 1) void gemm_kernel(GemmArgs g) {
    using M = Mfma<T>;
    constexpr int THREADS = 64 * WM * WN;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / M::MT, FN = TN / M::NT;
    static_assert(TM % M::MT == 0 && TN % M::NT == 0 && BK % M::KT == 0, "tile shape");
    // A: stored m x k (K contiguous) unless TA, then stored k x m. B: stored k x n (N contiguous)
    // unless TB, then stored n x k (K contiguous).
    constexpr bool A_KC = !TA, B_KC = TB;
    using LA = TileLayout<T, BM, BK, A_KC>;
    using LB = TileLayout<T, BN, BK, B_KC>;
    __shared__ __attribute__((aligned(16))) T lds_a[2][LA::ELEMS];
    __shared__ __attribute__((aligned(16))) T lds_b[2][LB::ELEMS];

    int tile_m, tile_n;
    tile_of_id(g, regroup_for_xcds(blockIdx.x, gridDim.x) + g.tile_offset, tile_m, tile_n);
    const size_t m0 = static_cast<size_t>(tile_m) * BM, n0 = static_cast<size_t>(tile_n) * BN;
    const size_t k_begin = static_cast<size_t>(blockIdx.z) * g.k_chunk;
    const size_t k_end = (k_begin + g.k_chunk < g.k) ? k_begin + g.k_chunk : g.k;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wave = tid / 64;
    const int wave_m = wave / WN, wave_n = wave % WN;
    const T *A = static_cast<const T *>(g.A);
    const T *B = static_cast<const T *>(g.B);

    typename M::acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
            acc[i][j] = M::zero();

    TileMover<T, BM, BK, A_KC, THREADS> mv_a;
    TileMover<T, BN, BK, B_KC, THREADS> mv_b;
    auto fetch = [&](size_t k0) {
        if constexpr (FULL) {
            if constexpr (A_KC)
                mv_a.load_full(A, g.lda, m0, k0, tid);
            else
                mv_a.load_full(A, g.lda, k0, m0, tid);
            if constexpr (B_KC)
                mv_b.load_full(B, g.ldb, n0, k0, tid);
            else
                mv_b.load_full(B, g.ldb, k0, n0, tid);
            return;
        }
        if constexpr (A_KC)
            mv_a.load(A, g.lda, m0, k0, g.m, k_end, g.aligned_a, tid);
        else
            mv_a.load(A, g.lda, k0, m0, k_end, g.m, g.aligned_a, tid);
        if constexpr (B_KC)
            mv_b.load(B, g.ldb, n0, k0, g.n, k_end, g.aligned_b, tid);
        else
            mv_b.load(B, g.ldb, k0, n0, k_end, g.n, g.aligned_b, tid);
    };

    const int frag_row = lane % M::ROWS; // row (A) / column (B) inside an MFMA tile
    const int frag_k = lane / M::ROWS;   // K group of this lane

    if (k_begin < k_end) {
        fetch(k_begin);
        mv_a.store(lds_a[0], tid);
        mv_b.store(lds_b[0], tid);
    }
    __syncthreads();
    int buf = 0;
    for (size_t k0 = k_begin; k0 < k_end; k0 += BK) {
        const bool more = k0 + BK < k_end;
        if (more)
            fetch(k0 + BK);
        const T *la = lds_a[buf];
        const T *lb = lds_b[buf];
#pragma unroll
        for (int kk = 0; kk < BK; kk += M::KT) {
            T fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; i++)
                fa[i] = la[LA::at(wave_m * TM + i * M::MT + frag_row, kk + frag_k)];
#pragma unroll
            for (int j = 0; j < FN; j++)
                fb[j] = lb[LB::at(wave_n * TN + j * M::NT + frag_row, kk + frag_k)];
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++)
                    acc[i][j] = M::mma(fa[i], fb[j], acc[i][j]);
        }
        if (more) {
            mv_a.store(lds_a[buf ^ 1], tid);
            mv_b.store(lds_b[buf ^ 1], tid);
        }
        __syncthreads();
        buf ^= 1;
    }

    // epilogue
    T *C = static_cast<T *>(g.C) + static_cast<size_t>(blockIdx.z) * g.slab_stride;
    size_t ldc = g.ldc, row_off = 0, col_off = 0;
    if (g.compact) {
        C = static_cast<T *>(g.C) + (static_cast<size_t>(blockIdx.z) * gridDim.x + blockIdx.x) * (BM * BN);
        ldc = BN;
        row_off = m0;
        col_off = n0;
    }
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++) {
            const size_t c = n0 + wave_n * TN + j * M::NT + M::col(lane);
            if (FULL || c < g.n) {
                T b = T(0);
                if constexpr (EPI == EPI_BIAS)
                    b = static_cast<const T *>(g.bias)[c * g.bias_stride];
#pragma unroll
                for (int v = 0; v < M::ACC; v++) {
                    const size_t r = m0 + wave_m * TM + i * M::MT + M::row(lane, v);
                    if (FULL || r < g.m) {
                        const T o = acc[i][j][v] + b;
                        C[(r - row_off) * ldc + (c - col_off)] = (EPI == EPI_BIAS && g.relu) ? relu_of(o) : o;
                    }
                }
            }
        }
}

// Adds `nslabs` partial results in slab order. MIRROR: only c >= r is read and the sum is written
// to both (r, c) and (c, r). bias may be null.
template <typename T, bool MIRROR>
__global__ __launch_bounds__(256) void slab_reduce_kernel(T *C, size_t ldc, const T *slabs, size_t slab_stride,
                                                          size_t ld_slab, int nslabs, size_t m, size_t n,
                                                          const T *bias, size_t bias_stride, int relu) {
    const size_t c = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t r = static_cast<size_t>(blockIdx.y) * blockDim.y + threadIdx.y;
    if (r >= m || c >= n)
        return;
    if (MIRROR && c < r)
        return;
    T s = T(0);
    for (int z = 0; z < nslabs; z++)
        s += slabs[static_cast<size_t>(z) * slab_stride + r * ld_slab + c];
    if (bias)
        s += bias[c * bias_stride];
    if (relu)
        s = relu_of(s);
    C[r * ldc + c] = s;
    if (MIRROR && c != r)
        C[c * ldc + r] = s;
}

// Folds the dense BM x BN blocks that a compact launch of `ntail` workgroups and `nslabs` K slices left
// (block of slice z, workgroup b at slabs[(z * ntail + b) * BM * BN]) into the result, in slice order.
template <typename T, int BM, int BN>
__global__ __launch_bounds__(256) void tail_reduce_kernel(GemmArgs g, const T *slabs, int nslabs, int ntail) {
    int tm, tn;
    tile_of_id(g, regroup_for_xcds(blockIdx.x, ntail) + g.tile_offset, tm, tn);
    T *C = static_cast<T *>(g.C);
    const T *bias = static_cast<const T *>(g.bias);
    const int e = blockIdx.y * 256 + threadIdx.x; // grid.y = BM * BN / 256: one element of the tile per thread
    const size_t r = static_cast<size_t>(tm) * BM + e / BN, c = static_cast<size_t>(tn) * BN + e % BN;
    if (r >= g.m || c >= g.n)
        return;
    const T *p = slabs + static_cast<size_t>(blockIdx.x) * (BM * BN) + e;
    const size_t step = static_cast<size_t>(ntail) * (BM * BN);
    T sum = T(0);
    int z = 0;
    for (; z + 4 <= nslabs; z += 4) {
        const T a0 = p[z * step], a1 = p[(z + 1) * step], a2 = p[(z + 2) * step], a3 = p[(z + 3) * step];
        sum = (((sum + a0) + a1) + a2) + a3;
    }
    for (; z < nslabs; z++)
        sum += p[z * step];
    if (bias)
        sum += bias[c * g.bias_stride];
    if (g.relu)
        sum = relu_of(sum);
    C[r * g.ldc + c] = sum;
}

// Upper -> lower mirror for a Syrk that ran without split-K: workgroup (bx, by), by >= bx, copies the 64 x 64
// tile (bx, by) above the diagonal through LDS into tile (by, bx) below it, both sides along rows.
template <typename T> __global__ __launch_bounds__(256) void mirror_kernel(T *C, size_t ldc, size_t n) {
    __shared__ T tile[64][65];
    if (blockIdx.y < blockIdx.x)
        return;
    const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    const size_t up = static_cast<size_t>(blockIdx.x) * 64, low = static_cast<size_t>(blockIdx.y) * 64;
    // sixteen loads per thread, all issued before the first LDS store (a guard around each load would make the
    // compiler wait for every one in turn): positions past the matrix read its last element, which is never stored
#pragma unroll
    for (int h = 0; h < 2; h++) {
        T v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const size_t r = up + ty + 4 * (h * 8 + k), c = low + tx;
            v[k] = C[(r < n ? r : n - 1) * ldc + (c < n ? c : n - 1)];
        }
#pragma unroll
        for (int k = 0; k < 8; k++)
            tile[ty + 4 * (h * 8 + k)][tx] = v[k];
    }
    __syncthreads();
#pragma unroll 4
    for (int i = ty; i < 64; i += 4) {
        const size_t r = low + i, c = up + tx;
        if (r < n && c < r)
            C[r * ldc + c] = tile[tx][i];
    }
}

// ---------------------------------------------------------------------------------------
// streaming paths for vector shapes (MatMul.cpp:277-283 of the reference's CPU kernel)
// ---------------------------------------------------------------------------------------
// y[i] = sum_k A[i][k] * x[k*incx]   (A stored m x k): G lanes per row, shuffle reduction.
template <typename T>
__global__ __launch_bounds__(256) void gemv_n_kernel(T *y, size_t incy, const T *A, size_t lda, const T *x,
                                                     size_t incx, size_t m, size_t k, int G) {
    const int lane = threadIdx.x % G;
    const size_t rpb = 256 / G;
    for (size_t r = static_cast<size_t>(blockIdx.x) * rpb + threadIdx.x / G; r < m;
         r += static_cast<size_t>(gridDim.x) * rpb) {
        T s = T(0);
        for (size_t c = lane; c < k; c += G)
            s += A[r * lda + c] * x[c * incx];
        dh_butterfly(G, [&](auto peer) { s += peer(s); });
        if (lane == 0)
            y[r * incy] = s;
    }
}

// partial[b][j] = sum_{r in slab b} A[r][j] * x[r*incx]   (A stored k x n, result n values):
// tx walks columns, ty interleaves the slab's rows, LDS folds ty.
template <typename T>
__global__ __launch_bounds__(256) void gemv_t_stage1(const T *A, size_t lda, const T *x, size_t incx, size_t rows,
                                                     size_t cols, size_t slab, T *partials) {
    extern __shared__ unsigned char lds_raw[];
    T *lds = reinterpret_cast<T *>(lds_raw);
    const size_t c = static_cast<size_t>(blockIdx.y) * blockDim.x + threadIdx.x;
    const size_t r_begin = static_cast<size_t>(blockIdx.x) * slab;
    const size_t r_end = (r_begin + slab < rows) ? r_begin + slab : rows;
    T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
    if (c < cols) {
        const size_t st = blockDim.y;
        size_t r = r_begin + threadIdx.y;
        for (; r + 3 * st < r_end; r += 4 * st) {
            s0 += A[r * lda + c] * x[r * incx];
            s1 += A[(r + st) * lda + c] * x[(r + st) * incx];
            s2 += A[(r + 2 * st) * lda + c] * x[(r + 2 * st) * incx];
            s3 += A[(r + 3 * st) * lda + c] * x[(r + 3 * st) * incx];
        }
        for (; r < r_end; r += st)
            s0 += A[r * lda + c] * x[r * incx];
    }
    lds[threadIdx.y * blockDim.x + threadIdx.x] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (threadIdx.y == 0 && c < cols) {
        T s = T(0);
        for (unsigned y = 0; y < blockDim.y; y++)
            s += lds[y * blockDim.x + threadIdx.x];
        partials[static_cast<size_t>(blockIdx.x) * cols + c] = s;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void gemv_t_stage2(const T *partials, size_t nparts, size_t cols, T *y, size_t incy) {
    const size_t c = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (c >= cols)
        return;
    T s = T(0);
    for (size_t p = 0; p < nparts; p++)
        s += partials[p * cols + c];
    y[c * incy] = s;
}

} // namespace dh_gemm

#include "ts_impl.h"

namespace dh_gemm {

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WM, int WN, int EPI, bool FULL = false>
static inline void launch_cfg(dh_ctx *ctx, const GemmArgs &g, bool ta, bool tb, dim3 grid) {
    const dim3 block(64 * WM * WN);
    if (!ta && !tb)
        hipLaunchKernelGGL((gemm_kernel<T, BM, BN, BK, WM, WN, false, false, EPI, FULL>), grid, block, 0, ctx->stream, g);
    else if (!ta && tb)
        hipLaunchKernelGGL((gemm_kernel<T, BM, BN, BK, WM, WN, false, true, EPI, FULL>), grid, block, 0, ctx->stream, g);
    else if (ta && !tb)
        hipLaunchKernelGGL((gemm_kernel<T, BM, BN, BK, WM, WN, true, false, EPI, FULL>), grid, block, 0, ctx->stream, g);
    else
        hipLaunchKernelGGL((gemm_kernel<T, BM, BN, BK, WM, WN, true, true, EPI, FULL>), grid, block, 0, ctx->stream, g);
}

// K depth of an LDS tile: 16 floats or 8 doubles (64 bytes per row either way), which keeps the
// double-buffered tiles of every shape below under 64 KiB of LDS.
template <typename T> struct GemmBK {
    static constexpr int value = sizeof(T) == 8 ? 8 : 16;
};

// C = op(A) op(B) (+ bias row). `triangular`: Syrk, compute tiles on/above the diagonal and mirror.
// A, B are the stored matrices; m, n, k are the GEMM dimensions after applying the transposes.
template <typename T>
dh_status gemm(dh_ctx *ctx, bool ta, bool tb, size_t m, size_t n, size_t k, const T *A, size_t lda, const T *B,
               size_t ldb, T *C, size_t ldc, const T *bias, bool triangular, size_t bias_stride = 1, bool relu = false) {
    // relu: only together with a bias (the stage that adds the bias applies it)
    if (m == 0 || n == 0)
        return DH_OK;
    // tall-and-skinny shapes stream straight from HBM into the matrix cores
    if (bias == nullptr) {
        dh_status st = DH_OK;
        if (ta && !tb && ts_tn<T>(ctx, m, n, k, A, lda, B, ldb, C, ldc, &st)) {
            if (st == DH_OK)
                DH_CHECK_LAUNCH();
            return st;
        }
        if (!ta && tb && !triangular && ts_nt<T>(ctx, m, n, k, A, lda, B, ldb, C, ldc, &st)) {
            if (st == DH_OK)
                DH_CHECK_LAUNCH();
            return st;
        }
    }
    constexpr int V = 16 / sizeof(T);
    GemmArgs g{};
    g.A = A;
    g.B = B;
    g.bias = bias;
    g.bias_stride = bias_stride;
    g.relu = (relu && bias != nullptr) ? 1 : 0;
    g.m = m;
    g.n = n;
    g.k = k;
    g.lda = lda;
    g.ldb = ldb;
    g.aligned_a = dh_aligned(A, 16) && (lda % V == 0);
    g.aligned_b = dh_aligned(B, 16) && (ldb % V == 0);
    g.triangular = triangular ? 1 : 0;

    // tile shape: square tiles by default, tall or wide ones when the other side is narrow
    constexpr int GEMM_BK = GemmBK<T>::value;
    int bm = 128, bn = 128;
    if (!triangular) {
        if (n <= 32 && m >= 256) {
            bm = 256;
            bn = 32;
        } else if (m <= 32 && n >= 256) {
            bm = 32;
            bn = 256;
        } else if (m <= 32 && n <= 64) {
            bm = 32;
            bn = 64;
        } else if (m <= 64 && n >= 512) {
            bm = 64;
            bn = 256;
        } else if (n <= 64 && m >= 512) {
            bm = 256;
            bn = 64;
        }
    }
    g.tiles_m = static_cast<int>(dh_ceil_div(m, bm));
    g.tiles_n = static_cast<int>(dh_ceil_div(n, bn));
    const size_t tiles = triangular ? static_cast<size_t>(g.tiles_n) * (g.tiles_n + 1) / 2
                                    : static_cast<size_t>(g.tiles_m) * g.tiles_n;
    // split K when the tile grid alone cannot fill the device and K is long
    const size_t slots = static_cast<size_t>(ctx->num_cus) * 2;
    size_t ksplit = 1;
    const size_t k_tiles = dh_ceil_div(k, GEMM_BK);
    if (tiles < slots && k_tiles >= 16) {
        ksplit = slots / tiles;
        const size_t max_split = k_tiles / 8; // keep at least 8 K tiles per slice
        if (ksplit > max_split)
            ksplit = max_split;
        if (ksplit < 1)
            ksplit = 1;
    }
    size_t k_chunk = dh_ceil_div(k_tiles, ksplit) * GEMM_BK;
    if (k_chunk == 0)
        k_chunk = GEMM_BK;
    ksplit = k ? dh_ceil_div(k, k_chunk) : 1;
    g.k_chunk = k_chunk;

    const bool direct = (ksplit == 1);
    T *slabs = nullptr;
    if (direct) {
        g.C = C;
        g.ldc = ldc;
        g.slab_stride = 0;
    } else {
        void *wsv = nullptr;
        dh_status st = dh_workspace(ctx, ksplit * m * n * sizeof(T), &wsv);
        if (st != DH_OK)
            return st;
        slabs = static_cast<T *>(wsv);
        g.C = slabs;
        g.ldc = n;
        g.slab_stride = m * n;
    }
    // A tile count a little above a multiple of the resident workgroups would leave most of the device idle while
    // the last few tiles run: those tiles go to a second launch that also splits K, into dense per-tile blocks
    // that a small kernel folds into the result in slice order.
    size_t tail = 0, tail_split = 1;
    if (direct && bm == 128 && bn == 128 && tiles > slots && k_tiles >= 32) {
        const size_t excess = tiles % slots;
        if (excess > 0 && excess * 4 <= slots) {
            tail = excess;
            tail_split = slots / excess;
            if (tail_split > k_tiles / 8)
                tail_split = k_tiles / 8;
        }
    }
    T *tail_slabs = nullptr;
    if (tail) {
        void *wsv = nullptr;
        dh_status st = dh_workspace(ctx, tail_split * tail * bm * bn * sizeof(T), &wsv);
        if (st != DH_OK)
            return st;
        tail_slabs = static_cast<T *>(wsv);
    }
    const dim3 grid(static_cast<unsigned>(tiles - tail), 1, static_cast<unsigned>(ksplit));
    const bool fuse_bias = direct && bias != nullptr;
#define DH_LAUNCH(BM_, BN_, WM_, WN_)                                                              \
    do {                                                                                           \
        if (fuse_bias)                                                                             \
            launch_cfg<T, BM_, BN_, GEMM_BK, WM_, WN_, EPI_BIAS>(ctx, g, ta, tb, grid);            \
        else                                                                                       \
            launch_cfg<T, BM_, BN_, GEMM_BK, WM_, WN_, EPI_STORE>(ctx, g, ta, tb, grid);           \
    } while (0)
    const bool interior = bm == 128 && bn == 128 && m % 128 == 0 && n % 128 == 0 && k % GEMM_BK == 0 &&
                          g.aligned_a && g.aligned_b && k > 0;
    const bool full = interior && !fuse_bias;
    if (full)
        launch_cfg<T, 128, 128, GEMM_BK, 2, 2, EPI_STORE, true>(ctx, g, ta, tb, grid);
    else if (bm == 128 && bn == 128)
        DH_LAUNCH(128, 128, 2, 2);
    else if (bm == 256 && bn == 64)
        DH_LAUNCH(256, 64, 4, 1);
    else if (bm == 64 && bn == 256)
        DH_LAUNCH(64, 256, 1, 4);
    else if (bm == 256)
        DH_LAUNCH(256, 32, 4, 1);
    else if (bn == 256)
        DH_LAUNCH(32, 256, 1, 4);
    else
        DH_LAUNCH(32, 64, 1, 2);
#undef DH_LAUNCH
    DH_CHECK_LAUNCH();
    if (tail) {
        GemmArgs t = g;
        t.C = tail_slabs;
        t.bias = nullptr;
        t.tile_offset = static_cast<int>(tiles - tail);
        t.compact = 1;
        t.k_chunk = dh_ceil_div(k_tiles, tail_split) * GEMM_BK;
        const size_t slices = dh_ceil_div(k, t.k_chunk);
        const dim3 tgrid(static_cast<unsigned>(tail), 1, static_cast<unsigned>(slices));
        if (interior)
            launch_cfg<T, 128, 128, GEMM_BK, 2, 2, EPI_STORE, true>(ctx, t, ta, tb, tgrid);
        else
            launch_cfg<T, 128, 128, GEMM_BK, 2, 2, EPI_STORE>(ctx, t, ta, tb, tgrid);
        DH_CHECK_LAUNCH();
        GemmArgs r = g;
        r.tile_offset = t.tile_offset;
        hipLaunchKernelGGL((tail_reduce_kernel<T, 128, 128>), dim3(static_cast<unsigned>(tail), 128 * 128 / 256), dim3(256), 0, ctx->stream, r,
                           tail_slabs, static_cast<int>(slices), static_cast<int>(tail));
        DH_CHECK_LAUNCH();
    }
    const dim3 eb(64, 4), eg(static_cast<unsigned>(dh_ceil_div(n, 64)), static_cast<unsigned>(dh_ceil_div(m, 4)));
    if (!direct) {
        if (triangular)
            hipLaunchKernelGGL((slab_reduce_kernel<T, true>), eg, eb, 0, ctx->stream, C, ldc, slabs, m * n, n,
                               static_cast<int>(ksplit), m, n, bias, bias_stride, g.relu);
        else
            hipLaunchKernelGGL((slab_reduce_kernel<T, false>), eg, eb, 0, ctx->stream, C, ldc, slabs, m * n, n,
                               static_cast<int>(ksplit), m, n, bias, bias_stride, g.relu);
        DH_CHECK_LAUNCH();
    } else if (triangular) {
        const unsigned mt = static_cast<unsigned>(dh_ceil_div(n, 64));
        hipLaunchKernelGGL((mirror_kernel<T>), dim3(mt, mt), dim3(256), 0, ctx->stream, C, ldc, n);
        DH_CHECK_LAUNCH();
    }
    return DH_OK;
}

template <typename T>
dh_status gemv(dh_ctx *ctx, bool trans, size_t rows, size_t cols, const T *A, size_t lda, const T *x, size_t incx,
               T *y, size_t incy) {
    // A stored rows x cols. !trans: y[rows] = A x[cols]; trans: y[cols] = A^T x[rows].
    if (!trans) {
        if (rows == 0)
            return DH_OK;
        int G = 1;
        while (G < 64 && static_cast<size_t>(G) < cols)
            G <<= 1;
        size_t grid = dh_ceil_div(rows, 256 / G);
        const size_t cap = static_cast<size_t>(ctx->num_cus) * 16;
        if (grid > cap)
            grid = cap;
        hipLaunchKernelGGL((gemv_n_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, y, incy,
                           A, lda, x, incx, rows, cols, G);
        DH_CHECK_LAUNCH();
        return DH_OK;
    }
    if (cols == 0)
        return DH_OK;
    {
        // y = t(A) x as a one-column case of the streaming contraction
        dh_status st = DH_OK;
        if (ts_tn<T>(ctx, cols, 1, rows, A, lda, x, incx, y, incy, &st)) {
            if (st == DH_OK)
                DH_CHECK_LAUNCH();
            return st;
        }
    }
    unsigned tx = 1;
    while (tx < 256 && tx < cols)
        tx <<= 1;
    const unsigned ty = 256 / tx;
    const size_t gy = dh_ceil_div(cols, tx);
    size_t gx = static_cast<size_t>(ctx->num_cus) * 8 / gy;
    if (gx < 1)
        gx = 1;
    size_t slab = dh_ceil_div(rows ? rows : 1, gx);
    slab = dh_ceil_div(slab, static_cast<size_t>(ty) * 4) * ty * 4;
    gx = dh_ceil_div(rows ? rows : 1, slab);
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, gx * cols * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    T *partials = static_cast<T *>(wsv);
    hipLaunchKernelGGL((gemv_t_stage1<T>), dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), dim3(tx, ty),
                       256 * sizeof(T), ctx->stream, A, lda, x, incx, rows, cols, slab, partials);
    hipLaunchKernelGGL((gemv_t_stage2<T>), dim3(static_cast<unsigned>(dh_ceil_div(cols, 256))), dim3(256), 0,
                       ctx->stream, partials, gx, cols, y, incy);
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// MatMul<DenseMatrix<T>,...>::apply: shape check and dispatch of kernels/MatMul.cpp:248-290.
template <typename T>
dh_status matmul(dh_ctx *ctx, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs, const T *rhs,
                 size_t rr, size_t rc, size_t ld_rhs, int transa, int transb) {
    DH_REQUIRE_CTX(ctx);
    const size_t nr1 = transa ? lc : lr, nc1 = transa ? lr : lc;
    const size_t nr2 = transb ? rc : rr, nc2 = transb ? rr : rc;
    if (nc1 != nr2)
        return dh_fail(DH_ERR_RUNTIME, "MatMul - #cols of lhs and #rows of rhs must be the same, but got%zuand%zu",
                       nc1, nr2);
    if (ld_lhs < lc || ld_rhs < rc || ld_res < nc2)
        return dh_fail(DH_ERR_RUNTIME, "MatMul - a leading dimension is smaller than its column count");
    if (nc2 == 1) {
        // matrix-vector (and vector-vector): x is rhs as a column (stride ld_rhs) or, transposed, as a row
        return gemv<T>(ctx, transa != 0, lr, lc, lhs, ld_lhs, rhs, transb ? 1 : ld_rhs, res, ld_res);
    }
    return gemm<T>(ctx, transa != 0, transb != 0, nr1, nc2, nc1, lhs, ld_lhs, rhs, ld_rhs, res, ld_res, nullptr, false);
}

// ts_sym_impl.h, instantiated in ts_sym_f32.hip / ts_sym_f64.hip
template <typename T>
bool ts_sym(dh_ctx *ctx, size_t m, size_t K, const T *X, size_t ldx, const T *y, size_t ldy, T *C, size_t ldc, T *b, size_t ldb,
            T lambda, dh_status *status);

// Syrk<DenseMatrix<T>,DenseMatrix<T>>::apply of kernels/Syrk.h:51-93.
template <typename T>
dh_status syrk(dh_ctx *ctx, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld, int trans_left) {
    DH_REQUIRE_CTX(ctx);
    const size_t n = trans_left ? cols : rows;
    const size_t k = trans_left ? rows : cols;
    if (ld < cols || ld_res < n)
        return dh_fail(DH_ERR_RUNTIME, "Syrk - a leading dimension is smaller than its column count");
    // t(X) X of a tall matrix with 65..128 columns: the triangle only, all four waves of a workgroup splitting the rows
    if (trans_left) {
        dh_status st = DH_OK;
        if (ts_sym<T>(ctx, n, k, arg, ld, nullptr, 0, res, ld_res, nullptr, 0, T(0), &st)) {
            if (st == DH_OK)
                DH_CHECK_LAUNCH();
            return st;
        }
    }
    // transLeft: C = X^T X -> A = X transposed, B = X; else C = X X^T -> A = X, B = X transposed
    return gemm<T>(ctx, trans_left != 0, trans_left == 0, n, n, k, arg, ld, arg, ld, res, ld_res, nullptr, true);
}

template <typename T> __global__ __launch_bounds__(256) void relu_inplace_kernel(T *p, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256)
        p[i] = relu_of(p[i]);
}

// CUDA::NN::Affine::Forward::apply of kernels/CUDA/Affine.cpp:42-83; epilogue DH_EPILOGUE_RELU: followed by
// CUDA::NN::Activation::Forward<ReLU> (kernels/CUDA/Activation.cpp:21-47), in the same pass where a bias is added.
template <typename T>
dh_status affine(dh_ctx *ctx, T *res, const T *data, size_t dr, size_t dc, const T *w, size_t wr, size_t wc,
                 const T *bias, size_t br, size_t bc, unsigned epilogue = 0) {
    DH_REQUIRE_CTX(ctx);
    if (epilogue & ~static_cast<unsigned>(DH_EPILOGUE_RELU))
        return dh_fail(DH_ERR_INVALID_ARG, "Affine: unknown epilogue flags %#x", epilogue);
    const bool relu = epilogue != 0;
    if (dc != wr)
        return dh_fail(DH_ERR_RUNTIME, "CUDA::NN::Affine: #cols of lhs and #rows of rhs must be the same (%zu != %zu)",
                       dc, wr);
    if (bias) {
        if (br != 1)
            return dh_fail(DH_ERR_RUNTIME,
                           "Affine (CUDA): bias dimensions not matching up with weights matrix (W[MxN] -> b[1xN]");
        // cudnnAddTensor, which the reference uses here, broadcasts a 1 x 1 bias over all columns
        // (its own test passes one: test/runtime/local/kernels/CUDA/DNNAffineTest.cpp:36)
        if (bc != wc && bc != 1)
            return dh_fail(DH_ERR_RUNTIME, "Affine: bias has %zu columns but the weights have %zu", bc, wc);
    }
    dh_status st = gemm<T>(ctx, false, false, dr, wc, dc, data, dc, w, wc, res, wc, bias, false,
                           (bias && bc == 1 && wc != 1) ? 0 : 1, relu);
    if (st == DH_OK && relu && !bias && dr * wc > 0) {
        size_t grid = dh_ceil_div(dr * wc, 256);
        if (grid > 65536)
            grid = 65536;
        hipLaunchKernelGGL((relu_inplace_kernel<T>), dim3(static_cast<unsigned>(grid)), dim3(256), 0, ctx->stream, res, dr * wc);
        DH_CHECK_LAUNCH();
    }
    return st;
}

} // namespace dh_gemm
