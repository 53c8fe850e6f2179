// t(X) X for a tall matrix with 65..128 columns, upper triangle only, optionally with t(X) y from the same pass:
// the normal equations of a linear regression (A = t(X) X + lambda I, b = t(X) y) from ONE read of X.
//
// The work is bound by the matrix cores, not by memory (f64: 2 m^2 flop per row of X against 8 m bytes), so the
// point is to issue as few matrix instructions as possible: the columns are cut into NT tiles of 16 and only the
// NT (NT + 1) / 2 tile pairs on or above the diagonal are computed (100 columns: 28 instead of the 64 of a padded
// full product). All four waves of a workgroup hold the whole triangle in registers and split the rows of X between
// them, as the workgroups do; a workgroup adds its four triangles through LDS and writes one partial ("slab"), and
// a second kernel adds the slabs in a fixed order, mirrors the triangle, and adds lambda on the diagonal.
//
// Fragments, as in ts_impl.h: the matrix instruction 16x16x4 takes A[i = lane % 16][k = lane / 16] and
// B[k][j = lane % 16]; here both are the same row k of X, so one set of loads feeds both sides. Lane group
// h = lane / 16 takes row k0 + h of a quad of rows. The first NV * V tiles come from NV vector loads of V values
// (value e of vector a belongs to tile a * V + e, which therefore stands for the columns 16 V a + V i + e), the
// last NS tiles from scalar loads of 16 consecutive columns each. That way 100 doubles are 3 vectors + 1 scalar =
// 7 tiles, not 8. t(X) y costs no matrix instruction: every lane multiplies the values it has loaded by y[k] on
// the ordinary ALUs, which are idle otherwise.
#pragma once

#include "ts_impl.h"

namespace dh_gemm {

struct TsSymArgs {
    const void *X, *y;
    void *slabs;     // [gridDim.x][m * m + m]: the triangle in matrix layout (row <= col), then the m values of t(X) y
    size_t ldx, ldy, K;
    size_t k_chunk;  // rows per workgroup, a multiple of 16 * U
    unsigned m;
};

template <typename T, int NV, int NS> struct TsSymShape {
    static constexpr int V = 16 / sizeof(T);
    static constexpr int NT = NV * V + NS;                  // tiles of 16 columns
    static constexpr int NP = NT * (NT + 1) / 2;            // tile pairs on or above the diagonal
    static constexpr int U = 2;                             // quads per register set
    // first column of tile t for lane column i
    static __device__ __forceinline__ unsigned col(int t, int i) {
        return t < NV * V ? static_cast<unsigned>(16 * V * (t / V) + V * i + (t % V))
                          : static_cast<unsigned>(NV * 16 * V + (t - NV * V) * 16 + i);
    }
    static constexpr size_t lds_bytes() { return static_cast<size_t>(NP) * 4 * 64 * sizeof(T) + (WITH_Y_SLOTS) * sizeof(T); }
    static constexpr int WITH_Y_SLOTS = NT * 16;
};

template <typename T, int NV, int NS, bool WITH_Y>
__global__ __launch_bounds__(256) void ts_sym_kernel(TsSymArgs g) {
    using M = Mfma16<T>;
    using S = TsSymShape<T, NV, NS>;
    constexpr int V = S::V, NT = S::NT, U = S::U;
    extern __shared__ __attribute__((aligned(16))) unsigned char ts_sym_lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, h = lane / 16;
    const T *X = static_cast<const T *>(g.X);
    const T *Y = static_cast<const T *>(g.y);

    // columns this lane loads; a vector or scalar that starts beyond the matrix reads column 0 instead (it only
    // feeds rows / columns of the result beyond m, which are never stored)
    unsigned cv[NV > 0 ? NV : 1], cs[NS > 0 ? NS : 1];
#pragma unroll
    for (int a = 0; a < NV; a++) {
        const unsigned c = 16 * V * a + V * i;
        cv[a] = c < g.m ? c : 0;
    }
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const unsigned c = NV * 16 * V + s * 16 + i;
        cs[s] = c < g.m ? c : 0;
    }

    typename M::acc_t acc[S::NP];
#pragma unroll
    for (int p = 0; p < S::NP; p++)
        acc[p] = typename M::acc_t{0, 0, 0, 0};
    T bacc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
        bacc[t] = T(0);

    const size_t kb = static_cast<size_t>(blockIdx.x) * g.k_chunk;
    const size_t ke = kb + g.k_chunk < g.K ? kb + g.k_chunk : g.K;

    struct Frag {
        T f[U][NT];
        T y[U];
    };
    // Unconditional loads (a branch around a load makes the compiler wait for all outstanding loads there). Rows
    // beyond the chunk, possible in the tail loop only, read its last row and are zeroed.
    auto load_quad = [&](Frag &fr, int u, size_t k, bool guard) {
        const bool row_ok = !guard || k < ke;
        const size_t kl = row_ok ? k : ke - 1;
        const T *row = X + kl * g.ldx;
#pragma unroll
        for (int a = 0; a < NV; a++) {
            T v[V];
            ts_load<T, V>(row + cv[a], v, true);
#pragma unroll
            for (int e = 0; e < V; e++)
                fr.f[u][a * V + e] = v[e];
        }
#pragma unroll
        for (int s = 0; s < NS; s++)
            fr.f[u][NV * V + s] = __builtin_nontemporal_load(row + cs[s]);
        if constexpr (WITH_Y)
            fr.y[u] = Y[kl * g.ldy];
        if (guard) {
#pragma unroll
            for (int t = 0; t < NT; t++)
                fr.f[u][t] = row_ok ? fr.f[u][t] : T(0);
        }
    };
    auto mma_quad = [&](const Frag &fr, int u) {
        int p = 0;
#pragma unroll
        for (int ta = 0; ta < NT; ta++)
#pragma unroll
            for (int tb = ta; tb < NT; tb++)
                acc[p] = M::mma(fr.f[u][ta], fr.f[u][tb], acc[p]), p++;
        if constexpr (WITH_Y) {
#pragma unroll
            for (int t = 0; t < NT; t++)
                bacc[t] = __builtin_fma(fr.f[u][t], fr.y[u], bacc[t]);
        }
    };

    // quad q of this wave covers rows kb + (4 q + wave) * 4 .. + 3; lane group h takes row + h
    size_t k = kb + static_cast<size_t>(wave) * 4 + h;
    constexpr size_t STEP = 16;
    auto load_group = [&](Frag &fr) {
#pragma unroll
        for (int u = 0; u < U; u++)
            load_quad(fr, u, k + u * STEP, false);
        k += U * STEP;
    };
    auto mma_group = [&](const Frag &fr) {
#pragma unroll
        for (int u = 0; u < U; u++)
            mma_quad(fr, u);
    };
    Frag f0, f1;
    const size_t k0 = kb + static_cast<size_t>(wave) * 4;
    const size_t need = (U - 1) * STEP + 4;
    const unsigned n_full = ke >= k0 + need ? static_cast<unsigned>((ke - k0 - need) / (U * STEP)) + 1 : 0;
    if (n_full > 0) {
        load_group(f0);
        const unsigned pairs = (n_full - 1) / 2;
        for (unsigned q = 0; q < pairs; q++) {
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
    while (k - h < ke) {
        load_quad(f0, 0, k, true);
        mma_quad(f0, 0);
        k += STEP;
    }

    // t(X) y: add the four rows of a quad (lane groups), leaving the sum for column col(t, i) in every lane group
    if constexpr (WITH_Y) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            bacc[t] += __shfl_xor(bacc[t], 16, 64);
            bacc[t] += __shfl_xor(bacc[t], 32, 64);
        }
    }

    // add up the four waves, one at a time into wave 0 (fixed order)
    T *red = reinterpret_cast<T *>(ts_sym_lds);            // [NP * 4][64]
    T *redb = red + static_cast<size_t>(S::NP) * 4 * 64;   // [NT][16]
    for (int w = 1; w < 4; w++) {
        if (wave == w) {
#pragma unroll
            for (int p = 0; p < S::NP; p++)
#pragma unroll
                for (int v = 0; v < 4; v++)
                    red[(p * 4 + v) * 64 + lane] = acc[p][v];
            if constexpr (WITH_Y) {
                if (h == 0) {
#pragma unroll
                    for (int t = 0; t < NT; t++)
                        redb[t * 16 + i] = bacc[t];
                }
            }
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int p = 0; p < S::NP; p++)
#pragma unroll
                for (int v = 0; v < 4; v++)
                    acc[p][v] += red[(p * 4 + v) * 64 + lane];
            if constexpr (WITH_Y) {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    bacc[t] += redb[t * 16 + i];
            }
        }
        __syncthreads();
    }
    if (wave != 0)
        return;

    T *slab = static_cast<T *>(g.slabs) + static_cast<size_t>(blockIdx.x) * (static_cast<size_t>(g.m) * g.m + g.m);
    int p = 0;
#pragma unroll
    for (int ta = 0; ta < NT; ta++)
#pragma unroll
        for (int tb = ta; tb < NT; tb++) {
            const unsigned col = S::col(tb, i);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const unsigned row = S::col(ta, M::row(lane, v));
                // inside a diagonal tile both halves were computed; the lower one is dropped
                if (row < g.m && col < g.m && row <= col)
                    slab[static_cast<size_t>(row) * g.m + col] = acc[p][v];
            }
            p++;
        }
    if constexpr (WITH_Y) {
        if (h == 0) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const unsigned c = S::col(t, i);
                if (c < g.m)
                    slab[static_cast<size_t>(g.m) * g.m + c] = bacc[t];
            }
        }
    }
}

// C[r][c] = C[c][r] = sum over slabs of slab[r][c] (r <= c), + lambda on the diagonal; b[c] = sum of the slabs' tails.
// Slabs are added in index order inside each of GY interleaved groups and the groups in order after that.
template <typename T>
__global__ __launch_bounds__(256) void ts_sym_reduce_kernel(T *C, size_t ldc, T *b, size_t ldb, const T *slabs, unsigned nslabs,
                                                            unsigned m, T lambda) {
    constexpr int EX = 32, GY = 8;
    __shared__ T part[GY][EX];
    const int ex = threadIdx.x % EX, gy = threadIdx.x / EX;
    const size_t stride = static_cast<size_t>(m) * m + m;
    const size_t elems = b ? stride : static_cast<size_t>(m) * m;
    const size_t e = static_cast<size_t>(blockIdx.x) * EX + ex;
    const unsigned r = static_cast<unsigned>(e / m), c = static_cast<unsigned>(e % m);
    const bool live = e < elems && (r >= m || r <= c); // the triangle, and the tail
    T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
    if (live) {
        unsigned z = gy;
        for (; z + 3 * GY < nslabs; z += 4 * GY) {
            s0 += slabs[static_cast<size_t>(z) * stride + e];
            s1 += slabs[static_cast<size_t>(z + GY) * stride + e];
            s2 += slabs[static_cast<size_t>(z + 2 * GY) * stride + e];
            s3 += slabs[static_cast<size_t>(z + 3 * GY) * stride + e];
        }
        for (; z < nslabs; z += GY)
            s0 += slabs[static_cast<size_t>(z) * stride + e];
    }
    part[gy][ex] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (gy == 0 && live) {
        T s = part[0][ex];
#pragma unroll
        for (int q = 1; q < GY; q++)
            s += part[q][ex];
        if (r >= m) {
            b[static_cast<size_t>(c) * ldb] = s;
        } else {
            if (r == c)
                s += lambda;
            C[static_cast<size_t>(r) * ldc + c] = s;
            if (r != c)
                C[static_cast<size_t>(c) * ldc + r] = s;
        }
    }
}

template <typename T, int NV, int NS>
static inline dh_status ts_sym_launch(dh_ctx *ctx, const TsSymArgs &g, unsigned blocks, bool with_y) {
    using S = TsSymShape<T, NV, NS>;
    const size_t lds = S::lds_bytes();
    auto k0 = &ts_sym_kernel<T, NV, NS, false>;
    auto k1 = &ts_sym_kernel<T, NV, NS, true>;
    if (lds > (size_t(64) << 10)) {
        static std::mutex attr_lock;
        static bool attr_set[16][2] = {};
        std::lock_guard<std::mutex> guard(attr_lock);
        if (ctx->device < 16 && !attr_set[ctx->device][with_y]) {
            DH_CHECK_HIP(hipFuncSetAttribute(with_y ? reinterpret_cast<const void *>(k1) : reinterpret_cast<const void *>(k0),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            attr_set[ctx->device][with_y] = true;
        }
    }
    if (with_y)
        hipLaunchKernelGGL(k1, dim3(blocks), dim3(256), lds, ctx->stream, g);
    else
        hipLaunchKernelGGL(k0, dim3(blocks), dim3(256), lds, ctx->stream, g);
    return DH_OK;
}

// C (m x m) = t(X) X + lambda I and, when y is given, b (m x 1, stride ldb) = t(X) y, for X of K rows and m columns,
// 64 < m <= 128. Returns false when the shape or the alignment does not fit; the caller then takes other kernels.
template <typename T>
bool ts_sym(dh_ctx *ctx, size_t m, size_t K, const T *X, size_t ldx, const T *y, size_t ldy, T *C, size_t ldc, T *b, size_t ldb,
            T lambda, dh_status *status) {
    constexpr int V = 16 / sizeof(T);
    if (m <= 64 || m > 128 || K < 4096)
        return false;
    if (!dh_aligned(X, 16) || ldx % V != 0 || !(m % V == 0 || ldx >= (m + V - 1) / V * V))
        return false;
    const size_t gran = 16 * 2; // rows per group of a workgroup's four waves
    size_t blocks = static_cast<size_t>(ctx->num_cus);
    size_t k_chunk = dh_ceil_div(dh_ceil_div(K, blocks), gran) * gran;
    if (k_chunk < gran * 4)
        k_chunk = gran * 4;
    blocks = dh_ceil_div(K, k_chunk);
    const size_t stride = m * m + m;
    void *wsv = nullptr;
    *status = dh_workspace(ctx, blocks * stride * sizeof(T), &wsv);
    if (*status != DH_OK)
        return true;
    TsSymArgs g{};
    g.X = X;
    g.y = y;
    g.slabs = wsv;
    g.ldx = ldx;
    g.ldy = ldy;
    g.K = K;
    g.k_chunk = k_chunk;
    g.m = static_cast<unsigned>(m);
    const unsigned nb = static_cast<unsigned>(blocks);
    const bool with_y = y != nullptr;
    // tiles: as many whole vectors (16 V columns each) as fit, the rest in scalar tiles of 16 columns, unless a
    // further vector covers it with no more tiles
    const size_t nt = dh_ceil_div(m, 16);
    dh_status st;
    if constexpr (sizeof(T) == 8) { // V = 2: a vector is two tiles
        switch (nt) {
        case 5:
            st = ts_sym_launch<T, 2, 1>(ctx, g, nb, with_y);
            break;
        case 6:
            st = ts_sym_launch<T, 3, 0>(ctx, g, nb, with_y);
            break;
        case 7:
            st = ts_sym_launch<T, 3, 1>(ctx, g, nb, with_y);
            break;
        default:
            st = ts_sym_launch<T, 4, 0>(ctx, g, nb, with_y);
        }
    } else { // V = 4: a vector is four tiles
        switch (nt) {
        case 5:
            st = ts_sym_launch<T, 1, 1>(ctx, g, nb, with_y);
            break;
        case 6:
            st = ts_sym_launch<T, 1, 2>(ctx, g, nb, with_y);
            break;
        case 7:
            st = ts_sym_launch<T, 1, 3>(ctx, g, nb, with_y);
            break;
        default:
            st = ts_sym_launch<T, 2, 0>(ctx, g, nb, with_y);
        }
    }
    if (st != DH_OK) {
        *status = st;
        return true;
    }
    const size_t elems = with_y ? stride : m * m;
    hipLaunchKernelGGL((ts_sym_reduce_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(elems, 32))), dim3(256), 0, ctx->stream, C,
                       ldc, with_y ? b : nullptr, ldb, static_cast<const T *>(wsv), nb, g.m, lambda);
    *status = DH_OK;
    return true;
}

} // namespace dh_gemm
