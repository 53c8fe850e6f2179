// One Lloyd iteration of k-means in two passes over X, for DenseMatrix<float|double>:
//   assign:  idx[i] = IDXMIN_c( (X t(C))[i][c] * -2 + xx[i] + cc[c] )      - X read once, nothing else of size rows x k
//   update:  C'[c][:] = (sum of the rows i with idx[i] = c) / (their number)  - X read once more, with idx
// They stand for the operator sequence of the k-means script (test/api/cli/algorithms/kmeans.daphne:14-21, with the
// row arg-min in place of `D <= minD`): MatMul (X @ t(C)), EwBinaryObjSca MUL, two EwBinaryMat ADD and AggRow IDXMIN
// for the first, the one-hot comparison, MatMul (t(P) @ X), AggCol SUM and EwBinaryMat DIV for the second. Neither
// the distances nor the one-hot matrix exist in memory.
// assign is the streaming product of ts_impl.h with another epilogue, so its distances are, bit for bit, those that
// the operator sequence computes from the stored product of the same kernel.
#pragma once

#include "ts_impl.h"

namespace dh_kmeans {

using dh_gemm::Mfma16;
using dh_gemm::ts_load;
using dh_gemm::ts_load_nt;
using dh_gemm::TsNtArgs;

template <typename T>
dh_status assign(dh_ctx *ctx, unsigned long long *idx, const T *X, size_t rows, size_t cols, size_t ldx, const T *C, size_t k,
                 size_t ldc, const T *xx, const T *cc) {
    DH_REQUIRE_CTX(ctx);
    constexpr int V = 16 / sizeof(T), KC = 4 * V;
    if (rows == 0)
        return DH_OK;
    // the kernel reads and writes all of these unconditionally: a null pointer is an error of the caller, not a fault
    if (idx == nullptr || X == nullptr || C == nullptr || xx == nullptr || cc == nullptr)
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans assign: idx, X, C, xx and cc must not be null");
    if (k == 0 || k > 32 || cols == 0 || cols > 512)
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans assign: 1..32 centroids of 1..512 features are supported (got %zu of %zu)", k, cols);
    if (!dh_aligned(X, 16) || !dh_aligned(C, 16) || ldx % V || ldc % V || cols % V || ldx < cols || ldc < cols)
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans assign: rows of X and C must start on 16-byte boundaries and hold whole 16-byte vectors");
    if (ldx * sizeof(T) >= (size_t(1) << 24))
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans assign: rows of X are more than 16 MiB apart");
    const int nb = k <= 16 ? 1 : 2;
    TsNtArgs g{};
    g.A = X;
    g.B = C;
    g.C = nullptr;
    g.lda = ldx;
    g.ldb = ldc;
    g.ldc = 0;
    g.M = rows;
    g.n = static_cast<unsigned>(k);
    g.K = static_cast<unsigned>(cols);
    g.kpad = static_cast<unsigned>(dh_ceil_div(cols, KC) * KC);
    g.row_add = xx;
    g.col_add = cc;
    g.idx = idx;
    const dh_status st = nb == 1 ? dh_gemm::ts_nt_launch<T, 1, true>(ctx, g) : dh_gemm::ts_nt_launch<T, 2, true>(ctx, g);
    if (st != DH_OK)
        return st;
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// ---------------------------------------------------------------------------------------
// update: S = t(P) X with P = one-hot(idx) made on the fly, and the cluster sizes.
// The 16x16x4 matrix instruction with the four lane groups on four consecutive rows of X: lane (i, h) supplies
// P[row h][centroid i] - a comparison - and a 16-byte vector of row h of X, whose element e feeds instruction e (that
// one computes the columns {V i + e}). A wave load covers whole contiguous rows of X. The four waves of a workgroup
// split its rows; workgroups write partial sums into slabs that a second kernel adds in a fixed order, divides and
// stores. Cluster sizes are counted beside the matrix instructions (exact in T up to 2^24 / 2^53 rows).
// ---------------------------------------------------------------------------------------
struct UpdateArgs {
    const void *X;
    const unsigned long long *idx;
    void *slabs;   // [blocks][KB*16][ncols] sums, then [blocks][KB*16] sizes
    size_t ldx, rows, k_chunk;
    unsigned k, cols, blocks;
};

template <typename T, int KB, int CB>
__global__ __launch_bounds__(256) void kmeans_update_kernel(UpdateArgs g) {
    using M = Mfma16<T>;
    constexpr int V = 16 / sizeof(T);
    constexpr int U = 4; // quads (four rows) per register set
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, h = lane / 16;
    const T *X = static_cast<const T *>(g.X);
    // first column of each vector this lane loads; vectors that start beyond the matrix read column 0 and are not stored
    unsigned col[CB], col_ld[CB];
#pragma unroll
    for (int c = 0; c < CB; c++) {
        col[c] = (c * 16 + i) * V;
        col_ld[c] = col[c] < g.cols ? col[c] : 0;
    }
    typename M::acc_t acc[KB][CB][V];
    T cnt[KB];
#pragma unroll
    for (int a = 0; a < KB; a++) {
        cnt[a] = T(0);
#pragma unroll
        for (int c = 0; c < CB; c++)
#pragma unroll
            for (int e = 0; e < V; e++)
                acc[a][c][e] = typename M::acc_t{0, 0, 0, 0};
    }
    const size_t kb = static_cast<size_t>(blockIdx.x) * g.k_chunk;
    const size_t ke = kb + g.k_chunk < g.rows ? kb + g.k_chunk : g.rows;
    struct Frag {
        unsigned long long id[U];
        T x[U][CB][V];
    };
    // loads are unconditional (rows beyond the end read the last row and count for nothing)
    auto load_quad = [&](Frag &fr, int u, size_t r) {
        const size_t rl = r < ke ? r : ke - 1;
        fr.id[u] = g.idx[rl];
#pragma unroll
        for (int c = 0; c < CB; c++)
            ts_load_nt<T, V>(X + rl * g.ldx + col_ld[c], fr.x[u][c]);
    };
    auto mma_quad = [&](const Frag &fr, int u, bool live) {
#pragma unroll
        for (int a = 0; a < KB; a++) {
            const T p = (live && fr.id[u] == static_cast<unsigned long long>(a * 16 + i)) ? T(1) : T(0);
            cnt[a] += p;
#pragma unroll
            for (int c = 0; c < CB; c++)
#pragma unroll
                for (int e = 0; e < V; e++)
                    acc[a][c][e] = M::mma(p, live ? fr.x[u][c][e] : T(0), acc[a][c][e]);
        }
    };
    // quad q of this wave covers rows kb + (4 q + wave) * 4 .. + 3; lane group h takes row + h
    size_t r = kb + static_cast<size_t>(wave) * 4 + h;
    constexpr size_t STEP = 16;
    Frag f0, f1;
    auto load_group = [&](Frag &fr) {
#pragma unroll
        for (int u = 0; u < U; u++)
            load_quad(fr, u, r + u * STEP);
        r += U * STEP;
    };
    auto mma_group = [&](const Frag &fr) {
#pragma unroll
        for (int u = 0; u < U; u++)
            mma_quad(fr, u, true);
    };
    // full groups in a counted loop of one basic block, two register sets (the next group's loads in flight under
    // the matrix instructions of the current one); what is left is finished quad by quad with a guard
    const size_t r0 = kb + static_cast<size_t>(wave) * 4;
    const size_t need = (U - 1) * STEP + 4;
    const unsigned n_full = ke >= r0 + need ? static_cast<unsigned>((ke - r0 - need) / (U * STEP)) + 1 : 0;
    if (n_full > 0) {
        load_group(f0);
        const unsigned pairs = (n_full - 1) / 2;
        for (unsigned p = 0; p < pairs; p++) {
            load_group(f1);
            __builtin_amdgcn_sched_barrier(0);
            mma_group(f0);
            __builtin_amdgcn_sched_barrier(0);
            load_group(f0);
            __builtin_amdgcn_sched_barrier(0);
            mma_group(f1);
            __builtin_amdgcn_sched_barrier(0);
        }
        if ((n_full - 1) % 2) {
            load_group(f1);
            __builtin_amdgcn_sched_barrier(0);
            mma_group(f0);
            mma_group(f1);
        } else {
            mma_group(f0);
        }
    }
    while (r - h < ke) {
        load_quad(f0, 0, r);
        mma_quad(f0, 0, r < ke);
        r += STEP;
    }
    // sizes: the four lane groups of a wave counted different rows
#pragma unroll
    for (int a = 0; a < KB; a++) {
        cnt[a] += dh_peer_swap<16>{}(cnt[a]);
        cnt[a] += dh_peer_swap<32>{}(cnt[a]);
    }
    // the four waves, added in wave order by wave 0
    constexpr int NV = KB * CB * V * 4 + KB;
    __shared__ __attribute__((aligned(16))) T red[NV][64];
    for (int w = 1; w < 4; w++) {
        if (wave == w) {
            int q = 0;
#pragma unroll
            for (int a = 0; a < KB; a++) {
#pragma unroll
                for (int c = 0; c < CB; c++)
#pragma unroll
                    for (int e = 0; e < V; e++)
#pragma unroll
                        for (int v = 0; v < 4; v++)
                            red[q++][lane] = acc[a][c][e][v];
                red[q++][lane] = cnt[a];
            }
        }
        __syncthreads();
        if (wave == 0) {
            int q = 0;
#pragma unroll
            for (int a = 0; a < KB; a++) {
#pragma unroll
                for (int c = 0; c < CB; c++)
#pragma unroll
                    for (int e = 0; e < V; e++)
#pragma unroll
                        for (int v = 0; v < 4; v++)
                            acc[a][c][e][v] += red[q++][lane];
                cnt[a] += red[q++][lane];
            }
        }
        __syncthreads();
    }
    if (wave != 0)
        return;
    T *slab = static_cast<T *>(g.slabs) + static_cast<size_t>(blockIdx.x) * (KB * 16) * g.cols;
    T *sizes = static_cast<T *>(g.slabs) + static_cast<size_t>(g.blocks) * (KB * 16) * g.cols + static_cast<size_t>(blockIdx.x) * (KB * 16);
#pragma unroll
    for (int a = 0; a < KB; a++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const unsigned cen = a * 16 + M::row(lane, v);
#pragma unroll
            for (int c = 0; c < CB; c++)
#pragma unroll
                for (int e = 0; e < V; e++)
                    if (col[c] + e < g.cols)
                        slab[static_cast<size_t>(cen) * g.cols + col[c] + e] = acc[a][c][e][v];
        }
        if (h == 0)
            sizes[a * 16 + i] = cnt[a];
    }
}

// C'[c][j] = (sum of the slabs' S[c][j]) / (sum of the slabs' sizes[c]), slabs added in index order inside each of GY
// interleaved groups and the groups in order after that; the sizes go to `counts` (1 x k) if that is given.
template <typename T>
__global__ __launch_bounds__(256) void kmeans_finish_kernel(T *Cn, size_t ldc, T *counts, const T *slabs, unsigned nslabs, unsigned kpad,
                                                            unsigned k, unsigned cols) {
    constexpr int EX = 8, GY = 32;
    __shared__ T part[GY][EX], psize[GY][EX];
    const int ex = threadIdx.x % EX, gy = threadIdx.x / EX;
    const size_t elems = static_cast<size_t>(k) * cols, slab_elems = static_cast<size_t>(kpad) * cols;
    const size_t e = static_cast<size_t>(blockIdx.x) * EX + ex;
    const T *sizes = slabs + static_cast<size_t>(nslabs) * slab_elems;
    const unsigned cen = e < elems ? static_cast<unsigned>(e / cols) : 0;
    const size_t el = e < elems ? e : 0;
    // four loads of each kind in flight at a time; a slab index past the end reads slab 0 and adds nothing
    T s = T(0), n = T(0);
    for (unsigned z0 = gy; z0 < nslabs; z0 += 4 * GY) {
        T sv[4], nv[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const unsigned z = z0 + q * GY;
            sv[q] = slabs[static_cast<size_t>(z < nslabs ? z : 0) * slab_elems + el];
            nv[q] = sizes[static_cast<size_t>(z < nslabs ? z : 0) * kpad + cen];
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const bool in = z0 + q * GY < nslabs;
            s += in ? sv[q] : T(0);
            n += in ? nv[q] : T(0);
        }
    }
    part[gy][ex] = s;
    psize[gy][ex] = n;
    __syncthreads();
    if (gy == 0 && e < elems) {
        T st = part[0][ex], nt = psize[0][ex];
#pragma unroll
        for (int q = 1; q < GY; q++) {
            st += part[q][ex];
            nt += psize[q][ex];
        }
        Cn[static_cast<size_t>(cen) * ldc + e % cols] = st / nt;
        if (counts && e % cols == 0)
            counts[cen] = nt;
    }
}

template <typename T>
dh_status update(dh_ctx *ctx, T *Cn, size_t ldc, T *counts, const T *X, size_t rows, size_t cols, size_t ldx,
                 const unsigned long long *idx, size_t k) {
    DH_REQUIRE_CTX(ctx);
    constexpr int V = 16 / sizeof(T);
    constexpr size_t COLS_PER_BLOCK = 16 * V;
    if (Cn == nullptr || (rows > 0 && (X == nullptr || idx == nullptr))) // `counts` alone may be null
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans update: C_new, X and idx must not be null");
    if (k == 0 || k > 32 || cols == 0 || cols > 4 * COLS_PER_BLOCK)
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans update: 1..32 centroids of 1..%zu features are supported (got %zu of %zu)",
                       4 * COLS_PER_BLOCK, k, cols);
    if (!dh_aligned(X, 16) || ldx % V || cols % V || ldx < cols || ldc < cols)
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans update: rows of X must start on 16-byte boundaries and hold whole 16-byte vectors");
    const int kbn = k <= 16 ? 1 : 2;
    const int cbn = static_cast<int>(dh_ceil_div(cols, COLS_PER_BLOCK));
    const size_t kpad = static_cast<size_t>(kbn) * 16;
    // rows per workgroup: a multiple of what its four waves take per register set; two workgroups per CU
    const size_t gran = 4 * 4 * 4;
    size_t blocks = static_cast<size_t>(ctx->num_cus) * 2;
    size_t k_chunk = dh_ceil_div(dh_ceil_div(rows > 0 ? rows : 1, blocks), gran) * gran;
    if (k_chunk < 8 * gran)
        k_chunk = 8 * gran;
    blocks = rows > 0 ? dh_ceil_div(rows, k_chunk) : 1;
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, blocks * (kpad * cols + kpad) * sizeof(T), &wsv);
    if (st != DH_OK)
        return st;
    UpdateArgs g{};
    g.X = X;
    g.idx = idx;
    g.slabs = wsv;
    g.ldx = ldx;
    g.rows = rows;
    g.k_chunk = k_chunk;
    g.k = static_cast<unsigned>(k);
    g.cols = static_cast<unsigned>(cols);
    g.blocks = static_cast<unsigned>(blocks);
    const dim3 grid(static_cast<unsigned>(blocks));
    if (rows == 0)
        g.blocks = 0; // nothing to add up: every centroid comes out as 0 / 0
#define DH_KM_UPDATE(KB_, CB_) hipLaunchKernelGGL((kmeans_update_kernel<T, KB_, CB_>), grid, dim3(256), 0, ctx->stream, g)
#define DH_KM_COLS(KB_)                                                                            \
    do {                                                                                           \
        if (cbn == 1)                                                                              \
            DH_KM_UPDATE(KB_, 1);                                                                  \
        else if (cbn == 2)                                                                         \
            DH_KM_UPDATE(KB_, 2);                                                                  \
        else if (cbn == 3)                                                                         \
            DH_KM_UPDATE(KB_, 3);                                                                  \
        else                                                                                       \
            DH_KM_UPDATE(KB_, 4);                                                                  \
    } while (0)
    if (rows == 0)
        ;
    else if (kbn == 1)
        DH_KM_COLS(1);
    else
        DH_KM_COLS(2);
#undef DH_KM_COLS
#undef DH_KM_UPDATE
    DH_CHECK_LAUNCH();
    hipLaunchKernelGGL((kmeans_finish_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(k * cols, 8))), dim3(256), 0, ctx->stream, Cn,
                       ldc, counts, static_cast<const T *>(wsv), g.blocks, static_cast<unsigned>(kpad),
                       static_cast<unsigned>(k), static_cast<unsigned>(cols));
    DH_CHECK_LAUNCH();
    return DH_OK;
}

// assign and update in one pass over X where the one-pass kernel exists (float, up to 64 features, 16-byte rows), else
// one after the other; idx, C_new and counts as those two give them (C_new to rounding: other order of addition)
template <typename T>
dh_status step(dh_ctx *ctx, unsigned long long *idx, T *Cn, size_t ldcn, T *counts, const T *X, size_t rows, size_t cols, size_t ldx,
               const T *C, size_t k, size_t ldc, const T *xx, const T *cc) {
    DH_REQUIRE_CTX(ctx);
    if (Cn == nullptr || (rows > 0 && (idx == nullptr || X == nullptr || C == nullptr || xx == nullptr || cc == nullptr)))
        return dh_fail(DH_ERR_INVALID_ARG, "kmeans step: idx, C_new, X, C, xx and cc must not be null");
    {
        // One pass: up to 64 columns (a lane per column when the rows are added up). Float: the columns are one step
        // of 1 .. 4 chunks of 16. Double: chunks of 8 - up to four of them one step, five to eight two steps of four
        // (the rows of both stay staged until the pair's assignment is known).
        constexpr int V = 16 / sizeof(T), KC = 4 * V;
        size_t kpad = dh_ceil_div(cols, KC) * KC;
        if (sizeof(T) == 8 && kpad > 4 * KC && kpad <= 64)
            kpad = 64;
        const size_t chunks_per_step = kpad / KC <= 4 ? kpad / KC : 4;
        // (32 sums of doubles per lane do not fit the registers of two waves per SIMD: up to 16 centroids in double)
        constexpr size_t max_k = sizeof(T) == 4 ? 32 : 16;
        if (rows > 0 && k >= 1 && k <= max_k && kpad <= 64 && dh_aligned(X, 16) && dh_aligned(C, 16) && ldx % V == 0 && ldc % V == 0 &&
            cols % V == 0 && ldx >= cols && ldc >= cols && ldcn >= cols && ldx * sizeof(T) < (size_t(1) << 24)) {
            const int nb = k <= 16 ? 1 : 2;
            TsNtArgs g{};
            g.A = X;
            g.B = C;
            g.lda = ldx;
            g.ldb = ldc;
            g.M = rows;
            g.n = static_cast<unsigned>(k);
            g.K = static_cast<unsigned>(cols);
            g.kpad = static_cast<unsigned>(kpad);
            g.row_add = xx;
            g.col_add = cc;
            g.idx = idx;
            size_t blocks = 0;
            // with g.slabs == nullptr: how many partial results; then the launch
            constexpr int NB2 = sizeof(T) == 4 ? 2 : 1; // double: nb is always 1
            auto launch = [&]() -> dh_status {
                if (chunks_per_step == 4)
                    return nb == 1 ? dh_gemm::ts_nt_update_launch<T, 1, 4>(ctx, g, &blocks) : dh_gemm::ts_nt_update_launch<T, NB2, 4>(ctx, g, &blocks);
                if (chunks_per_step == 3)
                    return nb == 1 ? dh_gemm::ts_nt_update_launch<T, 1, 3>(ctx, g, &blocks) : dh_gemm::ts_nt_update_launch<T, NB2, 3>(ctx, g, &blocks);
                if (chunks_per_step == 2)
                    return nb == 1 ? dh_gemm::ts_nt_update_launch<T, 1, 2>(ctx, g, &blocks) : dh_gemm::ts_nt_update_launch<T, NB2, 2>(ctx, g, &blocks);
                return nb == 1 ? dh_gemm::ts_nt_update_launch<T, 1, 1>(ctx, g, &blocks) : dh_gemm::ts_nt_update_launch<T, NB2, 1>(ctx, g, &blocks);
            };
            dh_status st = launch();
            if (st != DH_OK)
                return st;
            const size_t kp = static_cast<size_t>(nb) * 16;
            void *wsv = nullptr;
            st = dh_workspace(ctx, blocks * (kp * cols + kp) * sizeof(T), &wsv);
            if (st != DH_OK)
                return st;
            g.slabs = wsv;
            st = launch();
            if (st != DH_OK)
                return st;
            DH_CHECK_LAUNCH();
            hipLaunchKernelGGL((kmeans_finish_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(k * cols, 8))), dim3(256), 0, ctx->stream, Cn,
                               ldcn, counts, static_cast<const T *>(wsv), static_cast<unsigned>(blocks), static_cast<unsigned>(kp),
                               static_cast<unsigned>(k), static_cast<unsigned>(cols));
            DH_CHECK_LAUNCH();
            return DH_OK;
        }
    }
    dh_status st = assign<T>(ctx, idx, X, rows, cols, ldx, C, k, ldc, xx, cc);
    if (st != DH_OK)
        return st;
    return update<T>(ctx, Cn, ldcn, counts, X, rows, cols, ldx, idx, k);
}

} // namespace dh_kmeans
