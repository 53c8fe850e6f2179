// t(X) X for a tall matrix with 65..128 columns, upper triangle only, optionally with t(X) y from the same pass:
// the normal equations of a linear regression (A = t(X) X + lambda I, b = t(X) y) from ONE read of X.
//
// The work is bound by the matrix cores, not by memory (f64: 2 m^2 flop per row of X against 8 m bytes), so the
// point is to issue as few matrix instructions as possible: the columns are cut into NT tiles of 16 and only the
// NT (NT + 1) / 2 tile pairs on or above the diagonal are computed (100 columns: 28 instead of the 64 of a padded
// full product). The rows of X are cut over the workgroups; the four waves of a workgroup take a quarter of the
// tile pairs each, over all rows of the workgroup. A workgroup writes one partial ("slab"), and a second kernel adds
// the slabs in a fixed order, mirrors the triangle, and adds lambda on the diagonal.
//
// Fragments, as in ts_impl.h: the matrix instruction 16x16x4 takes A[i = lane % 16][k = lane / 16] and
// B[k][j = lane % 16]; here both are the same row k of X, so one set of loads feeds both sides. Lane group
// h = lane / 16 takes row k0 + h of a quad of rows. The first NV * V tiles come from NV vector loads of V values
// (value e of vector a belongs to tile a * V + e, which therefore stands for the columns 16 V a + V i + e), the
// last NS tiles from scalar loads of 16 consecutive columns each. That way 100 doubles are 3 vectors + 1 scalar =
// 7 tiles, not 8. t(X) y costs no matrix instruction: the wave that owns the diagonal pair of a tile multiplies the
// values it has loaded by y[k] on the ordinary ALUs, which are idle otherwise.
#pragma once

#include "ts_impl.h"

namespace dh_gemm {
#ifndef TS_SYM_BLOCKS_PER_CU
#define TS_SYM_BLOCKS_PER_CU 1
#endif
#ifndef TS_SYM_DEPTH
#define TS_SYM_DEPTH 4
#endif

#ifdef DH_TS_SYM_PROFILE
__device__ long long g_ts_sym_prof[2][8][4];
#define TS_PROF(slot)                                                                                                     \
    do {                                                                                                                   \
        if (threadIdx.x % 64 == 0 && (blockIdx.x == 0 || blockIdx.x + 1 == gridDim.x))                                     \
            g_ts_sym_prof[blockIdx.x == 0 ? 0 : 1][threadIdx.x / 64][slot] = __builtin_amdgcn_s_memtime();                 \
    } while (0)
#else
#define TS_PROF(slot)
#endif

struct TsSymArgs {
    const void *X, *y;
    void *slabs;     // [gridDim.x][m * m + m]: the triangle in matrix layout (row <= col), then the m values of t(X) y
    size_t ldx, ldy, K;
    size_t k_chunk;  // rows per workgroup, a multiple of 4 TS_SYM_DEPTH
    unsigned m;
};

template <typename T, int NV, int NS> struct TsSymShape {
    static constexpr int V = 16 / sizeof(T);
    static constexpr int NT = NV * V + NS;                  // tiles of 16 columns
    static constexpr int NP = NT * (NT + 1) / 2;            // tile pairs on or above the diagonal
    static constexpr int PPW = (NP + 3) / 4;                // pairs per wave, dealt in row-major order
    // first column of tile t for lane column i
    static __device__ __forceinline__ unsigned col(int t, int i) {
        return t < NV * V ? static_cast<unsigned>(16 * V * (t / V) + V * i + (t % V))
                          : static_cast<unsigned>(NV * 16 * V + (t - NV * V) * 16 + i);
    }
    // pair p (row-major over ta <= tb) -> ta, tb
    struct Pairs {
        int a[NP], b[NP];
    };
    static constexpr Pairs pairs() {
        Pairs r{};
        int p = 0;
        for (int ta = 0; ta < NT; ta++)
            for (int tb = ta; tb < NT; tb++) {
                r.a[p] = ta;
                r.b[p] = tb;
                p++;
            }
        return r;
    }
    // bit t: wave w needs tile t (as either side of one of its pairs) / owns the diagonal pair (t, t)
    static constexpr unsigned need_mask(int w) {
        const Pairs pr = pairs();
        unsigned m = 0;
        for (int p = w * PPW; p < (w + 1) * PPW && p < NP; p++)
            m |= (1u << pr.a[p]) | (1u << pr.b[p]);
        return m;
    }
    static constexpr unsigned diag_mask(int w) {
        const Pairs pr = pairs();
        unsigned m = 0;
        for (int p = w * PPW; p < (w + 1) * PPW && p < NP; p++)
            if (pr.a[p] == pr.b[p])
                m |= 1u << pr.a[p];
        return m;
    }
};

// The work of wave W: its quarter of the tile pairs over all rows of the workgroup's chunk.
//
// A wave issues its instructions in order, and the waves of a SIMD are served oldest first (measured: a second wave on
// a SIMD gets the matrix core only when the first has nothing for it), so what counts is how few instructions a wave
// issues beside its matrix instructions: one wave per SIMD, the row address in scalar registers (advanced by scalar
// adds), every load addressed as that scalar base plus a lane offset that never changes, and no work at all on the
// loaded values.
template <typename T, int NV, int NS, bool WITH_Y, int W> __device__ __forceinline__ void ts_sym_wave(const TsSymArgs g) {
    using M = Mfma16<T>;
    using S = TsSymShape<T, NV, NS>;
    constexpr int V = S::V, NT = S::NT;
    constexpr int P0 = W * S::PPW, P1 = (W + 1) * S::PPW < S::NP ? (W + 1) * S::PPW : S::NP;
    constexpr int NPW = P1 > P0 ? P1 - P0 : 0;
    constexpr unsigned NEED = S::need_mask(W), DIAG = S::diag_mask(W);
    constexpr typename S::Pairs PR = S::pairs();
    if constexpr (NPW == 0) {
        return;
    } else {
        const int lane = threadIdx.x % 64;
        const int i = lane % 16, h = lane / 16;
        const char *X = static_cast<const char *>(g.X);
        const char *Y = static_cast<const char *>(g.y);
        TS_PROF(0);

        // byte offsets of this lane's loads from the first row of a quad: lane group h reads row + h; a vector or
        // scalar that starts beyond the matrix reads column 0 instead (it only feeds rows / columns of the result
        // beyond m, which are never stored)
        unsigned ov[NV > 0 ? NV : 1], os[NS > 0 ? NS : 1];
        const unsigned rowoff = static_cast<unsigned>(h) * static_cast<unsigned>(g.ldx);
#pragma unroll
        for (int a = 0; a < NV; a++) {
            const unsigned c = 16 * V * a + V * i;
            ov[a] = (rowoff + (c < g.m ? c : 0)) * static_cast<unsigned>(sizeof(T));
        }
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const unsigned c = NV * 16 * V + s * 16 + i;
            os[s] = (rowoff + (c < g.m ? c : 0)) * static_cast<unsigned>(sizeof(T));
        }
        unsigned oy = static_cast<unsigned>(h) * static_cast<unsigned>(g.ldy) * static_cast<unsigned>(sizeof(T));

        typename M::acc_t acc[NPW];
#pragma unroll
        for (int p = 0; p < NPW; p++)
            acc[p] = typename M::acc_t{0, 0, 0, 0};
        T bacc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++)
            bacc[t] = T(0);

        const size_t kb = static_cast<size_t>(blockIdx.x) * g.k_chunk;
        const size_t ke = kb + g.k_chunk < g.K ? kb + g.k_chunk : g.K;

        struct Frag {
            T f[NT];
            T y;
        };
        // the quad whose first row `row` points at into a register set, only the tiles this wave multiplies; `row`
        // is the same in all lanes and lives in scalar registers
        auto load_quad = [&](Frag &fr, const char *row, const char *yrow) {
            // (the empty statements keep the widening of a 32-bit lane offset beside its load, where it becomes part
            // of the load's addressing - scalar base plus 32-bit lane offset - instead of a 64-bit addition)
            if constexpr (WITH_Y) {
                asm volatile("" : "+v"(oy));
                fr.y = *reinterpret_cast<const T *>(yrow + oy);
            }
#pragma unroll
            for (int a = 0; a < NV; a++)
                asm volatile("" : "+v"(ov[a]));
#pragma unroll
            for (int sc = 0; sc < NS; sc++)
                asm volatile("" : "+v"(os[sc]));
#pragma unroll
            for (int a = 0; a < NV; a++) {
                bool all = true;
#pragma unroll
                for (int e = 0; e < V; e++)
                    all = all && ((NEED >> (a * V + e)) & 1u);
                if (all) {
                    T v[V];
                    ts_load<T, V>(reinterpret_cast<const T *>(row + ov[a]), v);
#pragma unroll
                    for (int e = 0; e < V; e++)
                        fr.f[a * V + e] = v[e];
                } else {
                    // a vector of which this wave uses only some values: those alone (a load whose other half goes
                    // nowhere gets its registers shared with other loads, and the waits that protects cost more)
#pragma unroll
                    for (int e = 0; e < V; e++)
                        if ((NEED >> (a * V + e)) & 1u)
                            fr.f[a * V + e] = *reinterpret_cast<const T *>(row + ov[a] + e * sizeof(T));
                }
            }
#pragma unroll
            for (int s = 0; s < NS; s++)
                if ((NEED >> (NV * V + s)) & 1u)
                    fr.f[NV * V + s] = *reinterpret_cast<const T *>(row + os[s]);
        };
        auto mma_quad = [&](const Frag &fr) {
            const T(&f)[NT] = fr.f;
#pragma unroll
            for (int p = 0; p < NPW; p++)
                acc[p] = M::mma(f[PR.a[P0 + p]], f[PR.b[P0 + p]], acc[p]);
            if constexpr (WITH_Y) {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    if ((DIAG >> t) & 1u)
                        bacc[t] = __builtin_fma(f[t], fr.y, bacc[t]);
            }
        };

        // D register sets: the loads of D - 1 quads are in flight while one is being multiplied. The pointer of the
        // next quad to load advances on the scalar unit.
        constexpr int D = TS_SYM_DEPTH;
        const unsigned nfull = static_cast<unsigned>((ke - kb) / (4 * D)) * D; // quads in whole groups of D
        Frag fr[D];
        if (nfull > 0) {
            const size_t sx = 4 * g.ldx * sizeof(T), sy = 4 * g.ldy * sizeof(T);
            const char *px = X + kb * g.ldx * sizeof(T), *py = WITH_Y ? Y + kb * g.ldy * sizeof(T) : nullptr;
            auto advance = [&]() {
                px += sx;
                if constexpr (WITH_Y)
                    py += sy;
            };
            // the matrix instructions of a quad with its other instructions dealt out between them
            auto spread = [&]() {
#pragma unroll
                for (int n = 0; n < NPW; n++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one matrix instruction
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // one load
                    __builtin_amdgcn_sched_group_barrier(0x002, 2, 0); // two vector instructions
                    __builtin_amdgcn_sched_group_barrier(0x004, 3, 0); // three scalar instructions
                }
                __builtin_amdgcn_sched_barrier(0); // a quad's loads stay in its own step
            };
#pragma unroll
            for (int d = 0; d < D - 1; d++) {
                load_quad(fr[d], px, py);
                advance();
            }
            // All groups of D quads but the last: every step loads the quad D - 1 ahead, which exists, so nothing
            // is clamped or tested. Measured with the wave's clock around this loop (100 000 x 100 doubles, 100 quads
            // per workgroup): what an instruction of the same wave costs beside the matrix instructions (64 cycles
            // each) does not depend on where it stands - some 7 cycles each, dealt out between them or all behind
            // them -, so their number is what matters.
            for (unsigned q = D; q < nfull; q += D) {
#pragma unroll
                for (int d = 0; d < D; d++) {
                    load_quad(fr[(d + D - 1) % D], px, py);
                    advance();
                    mma_quad(fr[d]);
                    spread();
                }
            }
            // the last group: one quad is still to load
            load_quad(fr[D - 1], px, py);
#pragma unroll
            for (int d = 0; d < D; d++) {
                mma_quad(fr[d]);
                spread();
            }
        }
        // The rows after the last whole group of quads (fewer than 4 D, in the last workgroup only: the other
        // workgroups' chunks are whole groups), a quad at a time without the pipeline: every lane addresses its own row
        // here; lane groups without a row read the last one and contribute zeros
#pragma unroll
        for (int j = 0; j < D; j++) {
            const size_t r0 = kb + 4 * static_cast<size_t>(nfull + j);
            if (r0 >= ke)
                break;
            const size_t r = r0 + h;
            const bool ok = r < ke;
            const size_t rl = ok ? r : ke - 1;
            const char *row = X + (rl * g.ldx - rowoff) * sizeof(T); // the lane offsets include h * ldx
            Frag ft;
#pragma unroll
            for (int a = 0; a < NV; a++) {
                T v[V];
                ts_load<T, V>(reinterpret_cast<const T *>(row + ov[a]), v);
#pragma unroll
                for (int e = 0; e < V; e++)
                    ft.f[a * V + e] = ok ? v[e] : T(0);
            }
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const T v = *reinterpret_cast<const T *>(row + os[s]);
                ft.f[NV * V + s] = ok ? v : T(0);
            }
            if constexpr (WITH_Y)
                ft.y = *reinterpret_cast<const T *>(Y + rl * g.ldy * sizeof(T));
            mma_quad(ft);
        }
        TS_PROF(1);

        T *slab = static_cast<T *>(g.slabs) + static_cast<size_t>(blockIdx.x) * (static_cast<size_t>(g.m) * g.m + g.m);
#pragma unroll
        for (int p = 0; p < NPW; p++) {
            const int ta = PR.a[P0 + p], tb = PR.b[P0 + p];
            const unsigned col = S::col(tb, i);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const unsigned row = S::col(ta, M::row(lane, v));
                // A tile pair (ta, tb > ta) is the only one that holds the products of its columns, and with
                // interleaved columns some of them lie below the diagonal of the matrix: those go to their mirror
                // position. A diagonal pair computed both halves; the lower one is dropped.
                if (row < g.m && col < g.m && (ta != tb || row <= col)) {
                    const unsigned lo = row < col ? row : col, hi = row < col ? col : row;
                    slab[static_cast<size_t>(lo) * g.m + hi] = acc[p][v];
                }
            }
        }
        // t(X) y: add the four rows of a quad (lane groups); lane group 0 stores
        if constexpr (WITH_Y) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if ((DIAG >> t) & 1u) {
                    T s = bacc[t];
                    s += __shfl_xor(s, 16, 64);
                    s += __shfl_xor(s, 32, 64);
                    const unsigned c = S::col(t, i);
                    if (h == 0 && c < g.m)
                        slab[static_cast<size_t>(g.m) * g.m + c] = s;
                }
            }
        }
        TS_PROF(3);
    }
}

// Four waves per workgroup, one per SIMD, one workgroup per CU. A workgroup takes k_chunk rows of X and each of its
// waves a quarter of the tile pairs over all of those rows. The waves read the same rows at nearly the same time (all
// but the first read are served by the cache), share nothing else and never wait for each other: no LDS, no barrier.
template <typename T, int NV, int NS, bool WITH_Y>
__global__ __launch_bounds__(256) void ts_sym_kernel(TsSymArgs g) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    switch (wave) {
    case 0:
        ts_sym_wave<T, NV, NS, WITH_Y, 0>(g);
        break;
    case 1:
        ts_sym_wave<T, NV, NS, WITH_Y, 1>(g);
        break;
    case 2:
        ts_sym_wave<T, NV, NS, WITH_Y, 2>(g);
        break;
    default:
        ts_sym_wave<T, NV, NS, WITH_Y, 3>(g);
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
    if (with_y)
        hipLaunchKernelGGL((ts_sym_kernel<T, NV, NS, true>), dim3(blocks), dim3(256), 0, ctx->stream, g);
    else
        hipLaunchKernelGGL((ts_sym_kernel<T, NV, NS, false>), dim3(blocks), dim3(256), 0, ctx->stream, g);
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
    const size_t gran = 4 * TS_SYM_DEPTH; // rows per turn of a wave's register sets
    size_t blocks = static_cast<size_t>(ctx->num_cus) * TS_SYM_BLOCKS_PER_CU;
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
