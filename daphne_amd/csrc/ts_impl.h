// Streaming contractions for tall-and-skinny operands, the shapes of the reference's ML scripts
// (t(X) %*% X, t(X) %*% y, t(P) %*% X, X %*% t(C) with X of millions of rows and tens of columns).
// They are bound by HBM, not by the matrix cores, so nothing is staged through LDS: every
// wavefront loads its operands from global memory directly in MFMA fragment layout and keeps going
// without barriers.
//
// Both use the 16x16x4 matrix instruction (v_mfma_f32_16x16x4_f32 / v_mfma_f64_16x16x4_f64):
// lane l supplies A[i = l%16][k = l/16] and B[k = l/16][j = l%16]. Which row of C a lane's "i"
// stands for, and which k its "k" stands for, is free as long as both operands agree - that is what
// lets a lane use whole 16-byte vectors:
//
//   ts_tn:  C[m x n] = t(A) B,  A: K x m, B: K x n, K huge, m, n <= 128.
//           The four lane groups take four consecutive rows k; a lane loads a vector of V consecutive
//           columns of that row, and element e of the vector feeds MFMA number e, which therefore
//           computes the C rows {V*i + e}. A wave load covers whole contiguous rows. The K range is
//           cut over workgroups (and over the waves of a workgroup when the output is small); each
//           workgroup writes one partial slab, and a second kernel adds the slabs in a fixed order.
//   ts_nt:  C[M x n] = A t(B),  A: M x K, B: n x K, M huge, n <= 32, K small.
//           Lane group h takes the k values [c*4V + h*V, +V) of chunk c: one vector load per lane and
//           chunk, V MFMAs. B sits in LDS (a few KB, loaded once per workgroup).
#pragma once

#include "common.h"

#include <type_traits>

namespace dh_gemm {
#ifndef TS_NT_PAIRS
#define TS_NT_PAIRS 4 // pairs of 16-row blocks per wavefront of ts_nt_kernel
#endif
#ifndef TS_SYM_U
#define TS_SYM_U 4 // quads per register set of the symmetric one-wave form (measured: 2 1.00 ms, 4 0.90, 8 0.92, 12 0.95)
#endif

typedef float ts_f32x4 __attribute__((ext_vector_type(4)));
typedef double ts_f64x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma16;
template <> struct Mfma16<float> {
    using acc_t = ts_f32x4;
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    // accumulator register v of lane l holds C[row(l, v)][l % 16]
    static __device__ __forceinline__ int row(int lane, int v) { return 4 * (lane / 16) + v; }
};
template <> struct Mfma16<double> {
    using acc_t = ts_f64x4;
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int lane, int v) { return 4 * v + (lane / 16); }
};

// V consecutive values
template <typename T, int V> __device__ __forceinline__ void ts_load(const T *p, T (&v)[V]) {
    if constexpr (V == 1) {
        v[0] = *p;
    } else {
        typedef T vec_t __attribute__((ext_vector_type(V)));
        const vec_t t = *reinterpret_cast<const vec_t *>(p);
#pragma unroll
        for (int e = 0; e < V; e++)
            v[e] = t[e];
    }
}

// The same for data that no other wave will ask for again. (A separate function: a hint chosen by a flag, even a
// literal one, is lost when the compiler merges the hinted and the plain load of one address.)
template <typename T, int V> __device__ __forceinline__ void ts_load_nt(const T *p, T (&v)[V]) {
    if constexpr (V == 1) {
        v[0] = __builtin_nontemporal_load(p);
    } else {
        typedef T vec_t __attribute__((ext_vector_type(V)));
        const vec_t t = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(p));
#pragma unroll
        for (int e = 0; e < V; e++)
            v[e] = t[e];
    }
}

struct TsTnArgs {
    const void *A, *B;
    void *slabs;       // [gridDim.x][m][n]
    size_t lda, ldb, K;
    size_t k_chunk;    // rows per workgroup, a multiple of 4 * waves-along-K * unroll
    unsigned m, n;
    int stream;        // operands are read once (no reuse between waves or operands)
};

// Wave tile: TM = 16*VA*RA rows by TN = 16*VB*RB columns of C; WM x WN wave tiles per workgroup,
// the remaining 4/(WM*WN) waves split K.
// SYM: A and B are the same matrix (t(X) X). Only MFMA tiles on or above the diagonal are computed and the
// slab is filled by mirroring; waves whose tile lies below the diagonal have nothing to do.
// STREAM: the operands are read once, by one wave (loads carry the streaming hint).
template <typename T, int VA, int RA, int VB, int RB, int WM, int WN, bool SYM = false, bool STREAM = false>
__global__ __launch_bounds__(256) void ts_tn_kernel(TsTnArgs g) {
    using M = Mfma16<T>;
    static_assert(!SYM || (VA == VB && RA == RB && WM == WN), "the symmetric form needs the same tiling on both sides");
    constexpr int KW = 4 / (WM * WN);
    constexpr int TM = 16 * VA * RA, TN = 16 * VB * RB;
    constexpr int NACC = RA * VA * RB * VB;         // MFMA tiles per wave
    // quads (4 rows of K) per register set: with 16 accumulator tiles only two fit beside them, except in the symmetric
    // one-wave form, where the B fragments are the A fragments and 10 of the 16 tiles exist
    constexpr int U = NACC >= 16 ? ((SYM && WM == 1) ? TS_SYM_U : 2) : 4;
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave % WM, wn = (wave / WM) % WN, wk = wave / (WM * WN);
    const int i = lane % 16, h = lane / 16;
    const T *A = static_cast<const T *>(g.A);
    const T *B = static_cast<const T *>(g.B);
    // diagonal wave tile of a symmetric product: B fragments are the A fragments, lower MFMA tiles are skipped
    const bool diag = SYM && wm == wn;
    if (SYM && wm > wn)
        return; // only with WM = WN = 2, where no wave splits K and there is no barrier below

    // first column of each vector this lane loads; vectors that start beyond the matrix are skipped
    unsigned ca[RA], cb[RB];
    bool oka[RA], okb[RB];
#pragma unroll
    for (int a = 0; a < RA; a++) {
        ca[a] = wm * TM + a * 16 * VA + i * VA;
        oka[a] = ca[a] < g.m;
    }
#pragma unroll
    for (int b = 0; b < RB; b++) {
        cb[b] = wn * TN + b * 16 * VB + i * VB;
        okb[b] = cb[b] < g.n;
    }

    typename M::acc_t acc[RA][VA][RB][VB];
#pragma unroll
    for (int a = 0; a < RA; a++)
#pragma unroll
        for (int e = 0; e < VA; e++)
#pragma unroll
            for (int b = 0; b < RB; b++)
#pragma unroll
                for (int f = 0; f < VB; f++)
                    acc[a][e][b][f] = typename M::acc_t{0, 0, 0, 0};

    const size_t kb = static_cast<size_t>(blockIdx.x) * g.k_chunk;
    const size_t ke = kb + g.k_chunk < g.K ? kb + g.k_chunk : g.K;

    // one group = U quads; two register sets so that the loads of the next group are in flight while
    // the matrix cores work on the current one
    struct Frag {
        T a[U][RA][VA], b[U][RB][VB];
    };
    // Every load is issued unconditionally, and nothing touches the loaded registers before the matrix instructions
    // do: a branch around a load (or a fix-up right after it) makes the compiler wait for ALL outstanding loads at
    // that point, which would serialise the two register sets. Vectors that start beyond the matrix read column 0
    // instead - they only feed rows / columns of C beyond m / n, which are never stored. Rows beyond the chunk
    // (possible in the tail loop only) read its last row and are zeroed, since a row of K reaches every output.
    unsigned ca_ld[RA], cb_ld[RB];
#pragma unroll
    for (int a = 0; a < RA; a++)
        ca_ld[a] = oka[a] ? ca[a] : 0;
#pragma unroll
    for (int b = 0; b < RB; b++)
        cb_ld[b] = okb[b] ? cb[b] : 0;
    auto load_quad = [&](Frag &fr, int u, size_t k, bool guard) {
        const bool row_ok = !guard || k < ke;
        const size_t kl = row_ok ? k : ke - 1;
#pragma unroll
        for (int a = 0; a < RA; a++) {
            if constexpr (STREAM)
                ts_load_nt<T, VA>(A + kl * g.lda + ca_ld[a], fr.a[u][a]);
            else
                ts_load<T, VA>(A + kl * g.lda + ca_ld[a], fr.a[u][a]);
            if (guard) {
#pragma unroll
                for (int e = 0; e < VA; e++)
                    fr.a[u][a][e] = row_ok ? fr.a[u][a][e] : T(0);
            }
        }
        if (diag) {
            if constexpr (SYM) {
#pragma unroll
                for (int b = 0; b < RB; b++)
#pragma unroll
                    for (int f = 0; f < VB; f++)
                        fr.b[u][b][f] = fr.a[u][b][f];
            }
            return;
        }
#pragma unroll
        for (int b = 0; b < RB; b++) {
            if constexpr (STREAM)
                ts_load_nt<T, VB>(B + kl * g.ldb + cb_ld[b], fr.b[u][b]);
            else
                ts_load<T, VB>(B + kl * g.ldb + cb_ld[b], fr.b[u][b]);
            if (guard) {
#pragma unroll
                for (int f = 0; f < VB; f++)
                    fr.b[u][b][f] = row_ok ? fr.b[u][b][f] : T(0);
            }
        }
    };
    auto mma_quad = [&](const Frag &fr, int u) {
        if (diag) {
#pragma unroll
            for (int a = 0; a < RA; a++)
#pragma unroll
                for (int e = 0; e < VA; e++)
#pragma unroll
                    for (int b = 0; b < RB; b++)
#pragma unroll
                        for (int f = 0; f < VB; f++)
                            if (a * VA + e <= b * VB + f)
                                acc[a][e][b][f] = M::mma(fr.a[u][a][e], fr.b[u][b][f], acc[a][e][b][f]);
            return;
        }
#pragma unroll
        for (int a = 0; a < RA; a++)
#pragma unroll
            for (int e = 0; e < VA; e++)
#pragma unroll
                for (int b = 0; b < RB; b++)
#pragma unroll
                    for (int f = 0; f < VB; f++)
                        acc[a][e][b][f] = M::mma(fr.a[u][a][e], fr.b[u][b][f], acc[a][e][b][f]);
    };

    // quad q of this wave covers rows kb + (q*KW + wk)*4 .. +3; lane group h takes row +h
    size_t k = kb + static_cast<size_t>(wk) * 4 + h;
    constexpr size_t STEP = static_cast<size_t>(KW) * 4;
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
    // The number of full groups of this wavefront is known up front, so the steady state is a counted loop whose
    // body is one basic block: loads into one register set, matrix instructions on the other, twice. That lets the
    // compiler's wait counts leave the new loads in flight (a load inside a conditional would make the wait at
    // the join cover it). The odd group left over is finished after the loop.
    const size_t k0 = kb + static_cast<size_t>(wk) * 4; // first row of this wavefront's first quad
    const size_t need = (U - 1) * STEP + 4;             // rows from the start of a group to the end of its last quad
    const unsigned n_full = ke >= k0 + need ? static_cast<unsigned>((ke - k0 - need) / (U * STEP)) + 1 : 0;
    if (n_full > 0) {
        load_group(f0);
        const unsigned pairs = (n_full - 1) / 2;
        // (the scheduling barriers keep the compiler from sinking the loads below the matrix instructions that
        // they are meant to overlap with)
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
    while (k - h < ke) {
        load_quad(f0, 0, k, true);
        mma_quad(f0, 0);
        k += STEP;
    }

    // add up the waves that split K: wave 0 of each tile collects the others one at a time (fixed order)
    if constexpr (KW > 1) {
        __shared__ __attribute__((aligned(16))) T red[WM * WN][NACC * 4][64];
        const int tile = wave % (WM * WN);
        for (int w = 1; w < KW; w++) {
            if (wk == w) {
                int r = 0;
#pragma unroll
                for (int a = 0; a < RA; a++)
#pragma unroll
                    for (int e = 0; e < VA; e++)
#pragma unroll
                        for (int b = 0; b < RB; b++)
#pragma unroll
                            for (int f = 0; f < VB; f++)
#pragma unroll
                                for (int v = 0; v < 4; v++)
                                    red[tile][r++][lane] = acc[a][e][b][f][v];
            }
            __syncthreads();
            if (wk == 0) {
                int r = 0;
#pragma unroll
                for (int a = 0; a < RA; a++)
#pragma unroll
                    for (int e = 0; e < VA; e++)
#pragma unroll
                        for (int b = 0; b < RB; b++)
#pragma unroll
                            for (int f = 0; f < VB; f++)
#pragma unroll
                                for (int v = 0; v < 4; v++)
                                    acc[a][e][b][f][v] += red[tile][r++][lane];
            }
            __syncthreads();
        }
    }
    if (wk != 0)
        return;

    // slab[row][col], row = wm*TM + a*16*VA + VA*i' + e with i' = the accumulator's row inside its MFMA
    // tile, col = cb[b] + f: the VB values f of one (a, e, b, v) are neighbours in memory
    T *slab = static_cast<T *>(g.slabs) + static_cast<size_t>(blockIdx.x) * g.m * g.n;
#pragma unroll
    for (int a = 0; a < RA; a++)
#pragma unroll
        for (int e = 0; e < VA; e++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const unsigned row = wm * TM + a * 16 * VA + VA * M::row(lane, v) + e;
                if (row < g.m) {
#pragma unroll
                    for (int b = 0; b < RB; b++)
#pragma unroll
                        for (int f = 0; f < VB; f++) {
                            if (diag && a * VA + e > b * VB + f)
                                continue; // not computed: arrives as the mirror image of its transpose
                            const unsigned col = cb[b] + f;
                            if (col < g.n) {
                                slab[static_cast<size_t>(row) * g.n + col] = acc[a][e][b][f][v];
                                if (SYM && (!diag || a * VA + e < b * VB + f))
                                    slab[static_cast<size_t>(col) * g.n + row] = acc[a][e][b][f][v];
                            }
                        }
                }
            }
}

// C[e] = sum over slabs, slabs added in index order inside each of GY interleaved groups and the groups in
// order after that: the same association for the same shapes, whatever the timing.
template <typename T>
__global__ __launch_bounds__(256) void ts_slab_reduce_kernel(T *C, size_t ldc, const T *slabs, unsigned nslabs, unsigned m,
                                                             unsigned n) {
    constexpr int EX = 32, GY = 8;
    __shared__ T part[GY][EX];
    const int ex = threadIdx.x % EX, gy = threadIdx.x / EX;
    const size_t elems = static_cast<size_t>(m) * n;
    const size_t e = static_cast<size_t>(blockIdx.x) * EX + ex;
    T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
    if (e < elems) {
        unsigned z = gy;
        for (; z + 3 * GY < nslabs; z += 4 * GY) {
            s0 += slabs[static_cast<size_t>(z) * elems + e];
            s1 += slabs[static_cast<size_t>(z + GY) * elems + e];
            s2 += slabs[static_cast<size_t>(z + 2 * GY) * elems + e];
            s3 += slabs[static_cast<size_t>(z + 3 * GY) * elems + e];
        }
        for (; z < nslabs; z += GY)
            s0 += slabs[static_cast<size_t>(z) * elems + e];
    }
    part[gy][ex] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (gy == 0 && e < elems) {
        T s = part[0][ex];
#pragma unroll
        for (int q = 1; q < GY; q++)
            s += part[q][ex];
        C[(e / n) * ldc + e % n] = s;
    }
}

// ---------------------------------------------------------------------------------------
// ts_nt
// ---------------------------------------------------------------------------------------
struct TsNtArgs {
    const void *A, *B;
    void *C;
    size_t lda, ldb, ldc, M;
    unsigned n, K;
    unsigned kpad;   // K rounded up to whole chunks
    int vec_store;   // C rows are 16-byte aligned
    // ASSIGN: instead of C, the first position of the row minimum of (C * -2 + row_add[row]) + col_add[col]
    const void *row_add, *col_add;
    unsigned long long *idx;
    // UPDATE: besides, the sums of the rows of each position (the rows of t(one-hot(idx)) A) and their numbers, one
    // partial result per workgroup: slabs[block][16 NB][K], then sizes[block][16 NB]
    void *slabs;
};

// NB column blocks of 16; each wave walks over row blocks of 16, two at a time, CPG chunks of k at a time (1, 2 or 4:
// a count that divides the number of chunks, so that a step's body has no branch in it).
// ASSIGN: the product is not stored; it goes on, rounded exactly as the stored one would be, into the distance
// (C * -2 + row_add[row]) + col_add[col] (three separately rounded operations) and the row's IDXMIN over it: the first
// position of the strict minimum, NaN never better, position 0 if the first value is NaN or all are.
// UPDATE (with ASSIGN; float, one step per pair of row blocks, i.e. K of exactly CPG chunks, CPG = 1 .. 4: up to 64 columns): the rows, read
// back from the wave's staging piece one at a time - lane j on column j -, are added to the sum of the position just
// found for them. A lane keeps its column's 16 NB sums in registers, and the position, the same for all lanes, picks
// the register (register-relative moves): four ordinary instructions and an LDS read per row, where the one-hot
// product t(P) X on the matrix cores costs as many matrix instructions again as the distances - sixteen times the
// flops of these additions - plus the one-hot itself. One pass over A then gives the assignment, the per-position
// sums and the counts. The grid is what the device holds at once (one partial result per workgroup) and deals the
// pairs round-robin.
template <typename T, int NB, bool ASSIGN, int CPG, bool UPDATE = false>
__global__ __launch_bounds__(256, UPDATE ? ((NB == 1 && sizeof(T) == 4) ? 3 : 2) : 1) void ts_nt_kernel(TsNtArgs g) {
    static_assert(!UPDATE || ASSIGN, "the one-pass form goes on from the assignment");
    using M = Mfma16<T>;
    constexpr int V = 16 / sizeof(T);
    constexpr int KC = 4 * V;     // k values per chunk
    // float: the operands of the matrix instruction are exchanged, which transposes the result tile in the
    // registers (row = 4 * (lane / 16) + v becomes the column) and turns four 4-byte stores per lane into one of
    // 16 bytes; the double layout (row = 4 * v + lane / 16) already stores whole 128-byte rows
    // ASSIGN in double exchanges them as well: nothing is stored there, and a row whose 16 values sit in four lanes
    // (column 4 v + h in register v) finds its minimum with two exchanges between lanes where the sixteen lanes of
    // the plain layout need four - for each of the lane's four rows
    constexpr bool SWAP = sizeof(T) == 4 || ASSIGN;
    // the column, within a block of 16, of register v in lane group h of the exchanged layout
    auto swapped_col = [](int hh, int vv) { return sizeof(T) == 4 ? 4 * hh + vv : 4 * vv + hh; };
    extern __shared__ __attribute__((aligned(16))) unsigned char ts_nt_lds[];
    T *lb = reinterpret_cast<T *>(ts_nt_lds); // [NB*16][kpad + V], zero padded
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64); // the same in all lanes: addresses built on it stay scalar
    const int i = lane % 16, h = lane / 16;
    const T *A = static_cast<const T *>(g.A);
    const T *B = static_cast<const T *>(g.B);
    T *C = static_cast<T *>(g.C);
    const unsigned ldl = g.kpad + V;
    // ASSIGN: this lane's columns' addends (float: columns 16 b + 4 h + v; double: column 16 b + i)
    constexpr int CPL = SWAP ? 4 : 1;
    T col_add[NB][CPL];
    if constexpr (ASSIGN) {
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < CPL; v++) {
                const unsigned col = SWAP ? b * 16 + swapped_col(h, v) : b * 16 + i;
                col_add[b][v] = col < g.n ? static_cast<const T *>(g.col_add)[col] : dh_inf<T>(); // beyond n: never the minimum
            }
    }

    // The work of a wavefront is a sequence of steps (pair of 16-row blocks, group of four k chunks), walked with two
    // register sets: the eight vector loads of step s + 1 are in flight while the matrix cores work on step s, and
    // the first step's loads are issued before B is staged into LDS, so that they overlap the staging and its barrier.
    // All loads are unconditional (a branch around a load makes the compiler wait for every outstanding load at
    // its first use): rows beyond M read the last row - they only produce rows of C that are not stored -, k
    // beyond K reads k = 0 and is zeroed when it is used (the padded part of B is zero, but 0 * NaN would still
    // be NaN), and steps beyond the last repeat the last one.
    // A wavefront takes TS_NT_PAIRS consecutive pairs of row blocks (short-lived workgroups, thousands of them: measured
    // against a grid of resident workgroups that deal the pairs round-robin, this is as fast at 2M rows and 7 % faster
    // at 20M).
    const unsigned chunks = g.kpad / KC;
    // chunk groups per row-block pair (CPG divides chunks); the one-pass form keeps the staged rows of all of a pair's
    // groups (at most 64 columns, a lane per column)
    const unsigned cg = chunks / CPG;
    const size_t total_pairs = (g.M + 31) / 32;
    const size_t first_pair = (static_cast<size_t>(blockIdx.x) * 4 + wave) * (UPDATE ? 1 : TS_NT_PAIRS);
    const size_t pair_stride = UPDATE ? static_cast<size_t>(gridDim.x) * 4 : 1;
    unsigned my_pairs = 0;
    if (first_pair < total_pairs) {
        if constexpr (UPDATE)
            my_pairs = static_cast<unsigned>((total_pairs - 1 - first_pair) / pair_stride) + 1;
        else
            my_pairs = static_cast<unsigned>(total_pairs - first_pair < TS_NT_PAIRS ? total_pairs - first_pair : TS_NT_PAIRS);
    }
    const unsigned nsteps = my_pairs * cg;
    constexpr int RPL = SWAP ? 1 : 4; // ASSIGN: rows per lane and row block in the result layout
    struct Frag {
        T a[2][CPG][V];
        T ra[2][RPL]; // ASSIGN: the row addends, fetched with the step so that the epilogue waits for nothing new
    };
    // A step's part of X - 32 rows by CPG chunks - is loaded the way memory likes it, whole runs of consecutive
    // vectors (vector number 64 c + lane of load c, counted along the rows of the 16 x VPR block), and turned into
    // the fragment layout (lane (i, h): row i, vector h of chunk c) through a piece of LDS that belongs to the wave:
    // no barrier, the wave's own LDS instructions execute in order. Row stride SX = CPG KC + V: free of bank conflicts.
    constexpr unsigned VPR = CPG * 4;      // vectors of a row in one step
    constexpr unsigned SX = CPG * KC + V;
    // one row block at a time; UPDATE: both row blocks of the pair for each of its chunk groups ([group][block][row]),
    // which stay there until the pair is finished
    T *stage = lb + NB * 16 * ldl + wave * (UPDATE ? cg * 2 * 16 * SX : 16 * SX);
    // Addresses are a base that is the same for the whole wave - the pair's first row - plus a 32-bit byte offset per
    // lane (32 rows of at most 2^24 bytes): one 24-bit multiplication and an addition per load, rows beyond M cut
    // back to the last row by a minimum on the row number.
    const unsigned row_bytes = static_cast<unsigned>(g.lda * sizeof(T));
    auto load_step = [&](Frag &fr, unsigned pair, unsigned grp) {
        const size_t prow = (first_pair + static_cast<size_t>(pair) * pair_stride) * 32; // < M for every pair of this wave
        const char *pair_base = reinterpret_cast<const char *>(A + prow * g.lda);
        const unsigned last_local = g.M - 1 - prow < 31 ? static_cast<unsigned>(g.M - 1 - prow) : 31u;
#pragma unroll
        for (int c = 0; c < CPG; c++) {
            const unsigned id = c * 64 + lane;
            const unsigned kv = grp * CPG * KC + (id % VPR) * V;
            const unsigned kb = (kv < g.K ? kv : 0) * static_cast<unsigned>(sizeof(T));
            const unsigned r0 = id / VPR, r1 = r0 + 16;
            const unsigned l0 = r0 < last_local ? r0 : last_local, l1 = r1 < last_local ? r1 : last_local;
            // measured at 20M x 64 floats: the streaming hint takes the stored product from 1163 to 1047 us and the
            // one-pass form from 115 to 109 us (2M rows), and costs the arg-min form 8 % (944 -> 1017 us)
            if constexpr (ASSIGN && !UPDATE) {
                ts_load<T, V>(reinterpret_cast<const T *>(pair_base + (__umul24(l0, row_bytes) + kb)), fr.a[0][c]);
                ts_load<T, V>(reinterpret_cast<const T *>(pair_base + (__umul24(l1, row_bytes) + kb)), fr.a[1][c]);
            } else {
                ts_load_nt<T, V>(reinterpret_cast<const T *>(pair_base + (__umul24(l0, row_bytes) + kb)), fr.a[0][c]);
                ts_load_nt<T, V>(reinterpret_cast<const T *>(pair_base + (__umul24(l1, row_bytes) + kb)), fr.a[1][c]);
            }
        }
        if constexpr (ASSIGN) {
            const T *ra_base = static_cast<const T *>(g.row_add) + prow;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int v = 0; v < RPL; v++) {
                    const unsigned r = t * 16 + (SWAP ? i : M::row(lane, v));
                    fr.ra[t][v] = ra_base[r < last_local ? r : last_local];
                }
        }
    };
    // Two sets of accumulators: with a single step per pair of row blocks (K of at most CPG chunks) the result of one
    // pair is finished - distances and arg-min, or the store - beside the matrix instructions of the next.
    using AccSet = typename M::acc_t[2][NB];
    AccSet accA, accB;
    const bool whole_chunks = g.K == g.kpad; // no k beyond K anywhere: nothing to zero
    auto mma_step_k = [&](AccSet &acc, const Frag &fr, unsigned grp, auto full_k) {
        constexpr bool FULLK = decltype(full_k)::value;
        if (grp == 0) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                acc[0][b] = typename M::acc_t{0, 0, 0, 0};
                acc[1][b] = typename M::acc_t{0, 0, 0, 0};
            }
        }
        T xa[2][CPG][V];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            T *st = stage + (UPDATE ? (grp * 2 + t) * 16 * SX : 0);
#pragma unroll
            for (int c = 0; c < CPG; c++) {
                // vector 64 c + lane of the block: row (64 c + lane) / VPR; with 16 vectors a row that is row 4 c + h,
                // vector i, spelled out so that the four stores share one address register
                const unsigned id = c * 64 + lane;
                if constexpr (VPR == 16)
                    dh_store_vec<T, V>(st + (4 * c + h) * SX + i * V, fr.a[t][c]);
                else
                    dh_store_vec<T, V>(st + (id / VPR) * SX + (id % VPR) * V, fr.a[t][c]);
            }
#pragma unroll
            for (int c = 0; c < CPG; c++)
                dh_load_vec<T, V>(st + i * SX + c * KC + h * V, xa[t][c]);
        }
#pragma unroll
        for (int c = 0; c < CPG; c++) {
            const unsigned ch = grp * CPG + c;
            {
                const bool kok = FULLK || ch * KC + h * V < g.K;
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    T fb[V];
                    dh_load_vec<T, V>(lb + (b * 16 + i) * ldl + ch * KC + h * V, fb);
#pragma unroll
                    for (int e = 0; e < V; e++) {
                        const T x0 = kok ? xa[0][c][e] : T(0), x1 = kok ? xa[1][c][e] : T(0);
                        if constexpr (SWAP) {
                            acc[0][b] = M::mma(fb[e], x0, acc[0][b]);
                            acc[1][b] = M::mma(fb[e], x1, acc[1][b]);
                        } else {
                            acc[0][b] = M::mma(x0, fb[e], acc[0][b]);
                            acc[1][b] = M::mma(x1, fb[e], acc[1][b]);
                        }
                    }
                }
            }
        }
    };
    auto mma_step = [&](AccSet &acc, const Frag &fr, unsigned grp) {
        if (whole_chunks)
            mma_step_k(acc, fr, grp, std::true_type{});
        else
            mma_step_k(acc, fr, grp, std::false_type{});
    };
    // UPDATE: lane j holds the sums of column j for the 16 NB positions, the counts are integers in LDS (one set per wave)
    constexpr unsigned NPOS = NB * 16;
    typedef T sums_t __attribute__((ext_vector_type(UPDATE ? NB * 16 : 2)));
    sums_t sums;
    __shared__ unsigned cnts[UPDATE ? 4 * NPOS : 4];
    // UPDATE: where this lane's column lies in a staged row block (lanes beyond the columns repeat column 0; their
    // sums are never stored)
    const unsigned ucol = static_cast<unsigned>(lane) < g.kpad ? lane : 0;
    const unsigned colbase = (ucol / (CPG * KC)) * (2 * 16 * SX) + ucol % (CPG * KC);
    if constexpr (UPDATE) {
#pragma unroll
        for (unsigned p = 0; p < NPOS; p++)
            sums[p] = T(0);
        if (lane < NPOS)
            cnts[wave * NPOS + lane] = 0u; // the wave's own entries: its LDS instructions execute in order
    }
    auto finish_pair = [&](AccSet &acc, unsigned pair, const T (&radd)[2][RPL]) {
        const size_t rbase = (first_pair + static_cast<size_t>(pair) * pair_stride) * 32;
        if constexpr (ASSIGN) {
#pragma clang fp contract(off)
            constexpr unsigned NONE = ~0u;
            auto take = [](T &best, unsigned &bi, T ov, unsigned oi) { // selects, no branches
                const bool better = (ov < best) | ((ov == best) & (oi < bi));
                best = better ? ov : best;
                bi = better ? oi : bi;
            };
            static_assert(SWAP, "the arg-min epilogue reads the exchanged layout");
            {
                // register v of lane (i, h) is C[row i][column 16 b + 4 h + v] (double: 4 v + h): a row's values sit in the four lanes i + 16 h
                T d[2][NB][4];
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int b = 0; b < NB; b++)
#pragma unroll
                        for (int v = 0; v < 4; v++)
                            d[t][b][v] = (acc[t][b][v] * T(-2) + radd[t][0]) + col_add[b][v];
                // IDXMIN (AggRow.h:71-83: a running minimum from the row's first value, strict comparisons) for a row
                // whose values lie in four lanes: the first position of the least value that is below +inf - a NaN is
                // below nothing, so it is never taken, and columns beyond n carry +inf - and position 0 if there is
                // none or if the row's first value is a NaN (nothing is below a NaN either). No second path for rows
                // with NaNs: an empty cluster makes its centroid, and with it a whole column of distances, NaN.
                unsigned bi[2];
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    T best = dh_inf<T>();
                    unsigned at = NONE;
#pragma unroll
                    for (int b = 0; b < NB; b++)
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            const bool lt = d[t][b][v] < best;
                            best = lt ? d[t][b][v] : best;
                            at = lt ? static_cast<unsigned>(b * 16 + swapped_col(h, v)) : at;
                        }
                    take(best, at, dh_peer_swap<16>{}(best), dh_peer_swap<16>{}(at));
                    take(best, at, dh_peer_swap<32>{}(best), dh_peer_swap<32>{}(at));
                    const T first = d[t][0][0]; // column 0 in the lanes h = 0, the ones that store
                    bi[t] = ((first != first) || at == NONE) ? 0u : at;
                }
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const size_t row = rbase + static_cast<size_t>(t) * 16 + i;
                    if (h == 0 && row < g.M)
                        g.idx[row] = bi[t];
                }
                if constexpr (UPDATE) {
                    // after the exchanges every lane group holds the positions of its rows: lane r that of row r
                    auto add_rows = [&](auto whole_tag) {
                        constexpr bool WHOLE = decltype(whole_tag)::value; // no row of the pair lies beyond M
#pragma unroll
                        for (int t = 0; t < 2; t++) {
                            if (h == 0 && (WHOLE || rbase + t * 16 + i < g.M))
                                atomicAdd(cnts + wave * NPOS + bi[t], 1u); // integers: the order does not matter
#pragma unroll
                            for (int r = 0; r < 16; r++) {
                                const unsigned pos = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(bi[t]), r));
                                // the row as a row: lane j on column j
                                T x = stage[(t * 16 + r) * SX + colbase];
                                if constexpr (!WHOLE)
                                    x = rbase + t * 16 + r < g.M ? x : T(0); // rows beyond M repeat the last row
                                sums[pos] += x;
                            }
                        }
                    };
                    if (rbase + 32 <= g.M) // the same in all lanes
                        add_rows(std::true_type{});
                    else
                        add_rows(std::false_type{});
                }
            }
        } else if constexpr (SWAP) {
            // the tile was computed transposed: register v of lane (i, h) is C[row i][column 4h + v], so a lane
            // stores four neighbouring columns at once and a wavefront 16 whole rows
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const size_t row = rbase + static_cast<size_t>(t) * 16 + i;
                if (row < g.M) {
#pragma unroll
                    for (int b = 0; b < NB; b++) {
                        const int col = b * 16 + 4 * h;
                        T *dst = C + row * g.ldc + col;
                        if (g.vec_store && col + 3 < static_cast<int>(g.n)) {
                            T o[4] = {acc[t][b][0], acc[t][b][1], acc[t][b][2], acc[t][b][3]};
                            dh_store_vec_stream<T, 4>(dst, o);
                        } else {
#pragma unroll
                            for (int v = 0; v < 4; v++)
                                if (col + v < static_cast<int>(g.n))
                                    dst[v] = acc[t][b][v];
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const size_t row = rbase + static_cast<size_t>(t) * 16 + M::row(lane, v);
                    if (row < g.M) {
#pragma unroll
                        for (int b = 0; b < NB; b++)
                            if (b * 16 + i < static_cast<int>(g.n))
                                dh_store_stream(C + row * g.ldc + b * 16 + i, acc[t][b][v]);
                    }
                }
        }
    };
    auto compute_step = [&](const Frag &fr, unsigned pair, unsigned grp) {
        mma_step(accA, fr, grp);
        if (grp + 1 == cg)
            finish_pair(accA, pair, fr.ra);
    };
    // (pair, grp) of a step and of the one after it, stepped without divisions
    auto advance = [&](unsigned &pair, unsigned &grp) {
        if (++grp == cg) {
            grp = 0;
            if (pair + 1 < my_pairs)
                pair++;
            else
                grp = cg - 1; // beyond the last step: stay on it (loaded again, never computed)
        }
    };
    Frag f0, f1;
    unsigned lp = 0, lg = 0; // step being loaded
    unsigned cp = 0, cgp = 0; // step being computed
    if (nsteps > 0)
        load_step(f0, lp, lg);
    __builtin_amdgcn_sched_barrier(0);

    for (unsigned idx = tid; idx < NB * 16 * (g.kpad / V); idx += 256) {
        const unsigned j = idx / (g.kpad / V), kv = (idx % (g.kpad / V)) * V;
        T t[V];
        if (j < g.n && kv < g.K) {
            ts_load<T, V>(B + static_cast<size_t>(j) * g.ldb + kv, t);
        } else {
#pragma unroll
            for (int e = 0; e < V; e++)
                t[e] = T(0);
        }
        dh_store_vec<T, V>(lb + j * ldl + kv, t);
    }
    __syncthreads();

    if (cg == 1 && !ASSIGN) {
        // (Measured: this helps the store of the product, 119 -> 113 us at 2M rows and 1163 -> 1101 us at 20M, and
        // costs the arg-min epilogue, 103 -> 112 us and 941 -> 978 us, whose wavefronts have four steps in all.)
        // One step per pair: step s is pair s. Steady state = loads of step s + 1, matrix instructions of step s and
        // the finish of step s - 1 in one stretch of code, so that the three overlap inside the wavefront too.
        if (nsteps == 0)
            return;
        T ra0[2][RPL], ra1[2][RPL];
        auto keep = [&](T (&dst)[2][RPL], const Frag &fr) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int v = 0; v < RPL; v++)
                    dst[t][v] = fr.ra[t][v];
        };
        load_step(f1, nsteps > 1 ? 1 : 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        mma_step(accA, f0, 0);
        keep(ra0, f0);
        unsigned sdone = 1; // steps whose matrix instructions are done; the last of them is not finished yet
        for (; sdone + 1 < nsteps; sdone += 2) {
            load_step(f0, sdone + 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(accB, f1, 0);
            finish_pair(accA, sdone - 1, ra0);
            keep(ra1, f1);
            __builtin_amdgcn_sched_barrier(0);
            load_step(f1, sdone + 2 < nsteps ? sdone + 2 : nsteps - 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            mma_step(accA, f0, 0);
            finish_pair(accB, sdone, ra1);
            keep(ra0, f0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (sdone < nsteps) {
            mma_step(accB, f1, 0);
            finish_pair(accA, sdone - 1, ra0);
            finish_pair(accB, sdone, f1.ra);
        } else {
            finish_pair(accA, sdone - 1, ra0);
        }
        return;
    }
    for (unsigned s2 = 0; s2 < nsteps; s2 += 2) {
        advance(lp, lg);
        load_step(f1, lp, lg);
        __builtin_amdgcn_sched_barrier(0);
        compute_step(f0, cp, cgp);
        __builtin_amdgcn_sched_barrier(0);
        advance(cp, cgp);
        advance(lp, lg);
        load_step(f0, lp, lg);
        __builtin_amdgcn_sched_barrier(0);
        if (s2 + 1 < nsteps)
            compute_step(f1, cp, cgp);
        __builtin_amdgcn_sched_barrier(0);
        advance(cp, cgp);
    }
    if constexpr (UPDATE) {
        // the workgroup's partial result: the four waves' sums and counts, added in wave order
        __syncthreads(); // every wave is done with its staging piece: the exchange between the waves takes their place
                         // (the launch sizes the dynamic LDS for the larger of the two)
        T *red = lb + NB * 16 * ldl; // [wave][position][column]
#pragma unroll
        for (unsigned p = 0; p < NPOS; p++)
            red[(wave * NPOS + p) * 64 + lane] = sums[p];
        __syncthreads();
        T *slab = static_cast<T *>(g.slabs) + static_cast<size_t>(blockIdx.x) * NPOS * g.K;
        T *sizes = static_cast<T *>(g.slabs) + static_cast<size_t>(gridDim.x) * NPOS * g.K + static_cast<size_t>(blockIdx.x) * NPOS;
        for (unsigned e = tid; e < NPOS * 64; e += 256) {
            const unsigned cen = e / 64, col = e % 64;
            T t = red[e];
#pragma unroll
            for (unsigned w = 1; w < 4; w++)
                t += red[w * NPOS * 64 + e];
            if (col < g.K)
                slab[static_cast<size_t>(cen) * g.K + col] = t;
        }
        if (tid < NPOS)
            sizes[tid] = static_cast<T>((cnts[tid] + cnts[NPOS + tid]) + (cnts[2 * NPOS + tid] + cnts[3 * NPOS + tid]));
    }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
// side classes of ts_tn: up to 16 columns (scalar loads), up to 64 (one wave), up to 128 (two waves)
template <typename T> struct TsSide {
    static constexpr int V = 16 / sizeof(T);          // f32 4, f64 2
    static constexpr int R64 = 64 / (16 * V);         // loads per lane for a 64-wide wave tile: f32 1, f64 2
};

template <typename T, int VA, int RA, int WM, int VB, int RB, int WN>
static inline void ts_tn_launch(dh_ctx *ctx, const TsTnArgs &g, unsigned blocks) {
    if constexpr (WM * WN == 1) {
        if (g.stream) {
            hipLaunchKernelGGL((ts_tn_kernel<T, VA, RA, VB, RB, WM, WN, false, true>), dim3(blocks), dim3(256), 0, ctx->stream, g);
            return;
        }
    }
    hipLaunchKernelGGL((ts_tn_kernel<T, VA, RA, VB, RB, WM, WN>), dim3(blocks), dim3(256), 0, ctx->stream, g);
}
template <typename T, int V_, int R_, int W_> static inline void ts_tn_launch_sym(dh_ctx *ctx, const TsTnArgs &g, unsigned blocks) {
    hipLaunchKernelGGL((ts_tn_kernel<T, V_, R_, V_, R_, W_, W_, true>), dim3(blocks), dim3(256), 0, ctx->stream, g);
}

// Returns false when the shape or the alignment does not fit (the caller then takes the tiled GEMM).
template <typename T>
bool ts_tn(dh_ctx *ctx, size_t m, size_t n, size_t K, const T *A, size_t lda, const T *B, size_t ldb, T *C, size_t ldc,
           dh_status *status) {
    constexpr int V = TsSide<T>::V, R64 = TsSide<T>::R64;
    if (m == 0 || n == 0 || m > 128 || n > 128 || K < 4096)
        return false;
    const int cls_a = m <= 16 ? 0 : (m <= 64 ? 1 : 2), cls_b = n <= 16 ? 0 : (n <= 64 ? 1 : 2);
    // vector loads need aligned rows and must not run past the end of the last row
    auto vec_ok = [&](const T *p, size_t ld, size_t cols) {
        return dh_aligned(p, 16) && ld % V == 0 && (cols % V == 0 || ld >= (cols + V - 1) / V * V);
    };
    if ((cls_a > 0 && !vec_ok(A, lda, m)) || (cls_b > 0 && !vec_ok(B, ldb, n)))
        return false;
    const int wm = cls_a == 2 ? 2 : 1, wn = cls_b == 2 ? 2 : 1, kw = 4 / (wm * wn);
    const int nacc = (cls_a == 0 ? 1 : V * R64) * (cls_b == 0 ? 1 : V * R64);
    const bool sym = static_cast<const void *>(A) == static_cast<const void *>(B) && m == n && lda == ldb && cls_a == 1;
    const int unroll = nacc >= 16 ? (sym ? TS_SYM_U : 2) : 4; // quads per register set, as in the kernel
    const size_t gran = static_cast<size_t>(4) * kw * unroll;
    // Workgroups: two per CU keep enough loads in flight (more were slower in every shape measured), and
    // each must stream at least eight times the bytes of the slab it writes at the end.
    const size_t slabf = 8;
    // The symmetric form is bound by the matrix cores as much as by memory; a second workgroup per CU only gets in
    // the way there (20M x 64 floats: 0.90 ms with one, 1.36 ms with two).
    size_t blocks = static_cast<size_t>(ctx->num_cus) * (sym ? 1 : 2);
    size_t k_chunk = dh_ceil_div(dh_ceil_div(K, blocks), gran) * gran;
    size_t min_chunk = dh_ceil_div(slabf * m * n, m + n);
    if (min_chunk < gran * 4)
        min_chunk = gran * 4;
    min_chunk = dh_ceil_div(min_chunk, gran) * gran;
    if (k_chunk < min_chunk)
        k_chunk = min_chunk;
    blocks = dh_ceil_div(K, k_chunk);
    void *wsv = nullptr;
    *status = dh_workspace(ctx, blocks * m * n * sizeof(T), &wsv);
    if (*status != DH_OK)
        return true;
    TsTnArgs g{};
    g.A = A;
    g.B = B;
    g.slabs = wsv;
    g.lda = lda;
    g.ldb = ldb;
    g.K = K;
    g.k_chunk = k_chunk;
    g.m = static_cast<unsigned>(m);
    g.n = static_cast<unsigned>(n);
    g.stream = (wm * wn == 1 && static_cast<const void *>(A) != static_cast<const void *>(B)) ? 1 : 0;
    const unsigned nb = static_cast<unsigned>(blocks);
    const size_t elems = m * n;
    if (sym) {
        // t(X) X with up to 64 columns: upper MFMA tiles only (10 of 16 per step). With 65..128 columns the four
        // waves own one 64 x 64 quadrant each and the slowest of them still has a full one, so nothing is gained.
        ts_tn_launch_sym<T, V, R64, 1>(ctx, g, nb);
        hipLaunchKernelGGL((ts_slab_reduce_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(elems, 32))), dim3(256), 0,
                           ctx->stream, C, ldc, static_cast<const T *>(wsv), nb, g.m, g.n);
        *status = DH_OK;
        return true;
    }
#define DH_TS_B(VA_, RA_, WM_)                                                                     \
    do {                                                                                           \
        if (cls_b == 0)                                                                            \
            ts_tn_launch<T, VA_, RA_, WM_, 1, 1, 1>(ctx, g, nb);                                   \
        else if (cls_b == 1)                                                                       \
            ts_tn_launch<T, VA_, RA_, WM_, V, R64, 1>(ctx, g, nb);                                 \
        else                                                                                       \
            ts_tn_launch<T, VA_, RA_, WM_, V, R64, 2>(ctx, g, nb);                                 \
    } while (0)
    if (cls_a == 0)
        DH_TS_B(1, 1, 1);
    else if (cls_a == 1)
        DH_TS_B(V, R64, 1);
    else
        DH_TS_B(V, R64, 2);
#undef DH_TS_B
    hipLaunchKernelGGL((ts_slab_reduce_kernel<T>), dim3(static_cast<unsigned>(dh_ceil_div(elems, 32))), dim3(256), 0,
                       ctx->stream, C, ldc, static_cast<const T *>(wsv), nb, g.m, g.n);
    *status = DH_OK;
    return true;
}

// Dynamic LDS of ts_nt_kernel: B (nb blocks of 16 rows, kpad + V a row) and a staging piece per wave.
template <typename T> inline size_t ts_nt_lds_bytes(int nb, unsigned kpad, int cpg) {
    constexpr size_t V = 16 / sizeof(T), KC = 4 * V;
    return (static_cast<size_t>(nb) * 16 * (kpad + V) + 4 * 16 * (cpg * KC + V)) * sizeof(T);
}
// ... of the one-pass form: the staging piece holds both row blocks of a pair, and at the end the waves exchange their
// sums (16 nb positions x 64 lanes each) through the same area
template <typename T> inline size_t ts_nt_update_lds_bytes(int nb, unsigned kpad, int cpg) {
    constexpr size_t V = 16 / sizeof(T), KC = 4 * V;
    const size_t groups = kpad / (static_cast<size_t>(cpg) * KC);
    const size_t stage = 4 * groups * 2 * 16 * (static_cast<size_t>(cpg) * KC + V), exchange = 4 * static_cast<size_t>(nb) * 16 * 64;
    return (static_cast<size_t>(nb) * 16 * (kpad + V) + (stage > exchange ? stage : exchange)) * sizeof(T);
}
// chunks of k per step: the largest of 4, 2, 1 that divides their number
template <typename T> inline int ts_nt_chunks_per_step(unsigned kpad) {
    const unsigned chunks = kpad / (4 * (16 / sizeof(T)));
    return chunks % 4 == 0 ? 4 : (chunks % 2 == 0 ? 2 : 1);
}

template <typename T, int NB, bool ASSIGN, int CPG>
inline dh_status ts_nt_launch_cpg(dh_ctx *ctx, const TsNtArgs &g, size_t lds) {
    const void *kernel = reinterpret_cast<const void *>(&ts_nt_kernel<T, NB, ASSIGN, CPG>);
    // dynamic LDS beyond 64 KiB has to be asked for, per kernel and device (the call is cheap next to the kernel)
    if (lds > 65536)
        DH_CHECK_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    const size_t blocks = dh_ceil_div(dh_ceil_div(g.M, 32), 4 * TS_NT_PAIRS);
    if (blocks >= (size_t(1) << 31))
        return dh_fail(DH_ERR_RUNTIME, "MatMul: too many rows for one launch of the streaming kernel");
    hipLaunchKernelGGL((ts_nt_kernel<T, NB, ASSIGN, CPG>), dim3(static_cast<unsigned>(blocks)), dim3(256), lds, ctx->stream, g);
    return DH_OK;
}
// The one-pass form (UPDATE): a grid of as many workgroups as the device holds at once; *blocks_out receives their
// number (that of the partial results in g.slabs, which must hold blocks * (16 NB K + 16 NB) values: ask with
// g.slabs == nullptr first).
template <typename T, int NB, int CPG = 4> inline dh_status ts_nt_update_launch(dh_ctx *ctx, const TsNtArgs &g, size_t *blocks_out) {
    const void *kernel = reinterpret_cast<const void *>(&ts_nt_kernel<T, NB, true, CPG, true>);
    const size_t lds = ts_nt_update_lds_bytes<T>(NB, g.kpad, CPG);
    // three workgroups per CU (measured 2 .. 4 per CU: 104 .. 110 us at 2M x 64, no trend; a loop that only loads the
    // rows this way and stores the assignment takes 86 us, 74 us without the stores)
    if (lds > 65536)
        DH_CHECK_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    constexpr int per_cu = sizeof(T) == 4 ? 3 : 2; // double: two waves per SIMD by registers, two workgroups per CU by LDS
    size_t blocks = static_cast<size_t>(ctx->num_cus) * per_cu;
    const size_t needed = dh_ceil_div(dh_ceil_div(g.M, 32), 4 * 2); // at least two pairs per wavefront
    if (blocks > needed)
        blocks = needed > 0 ? needed : 1;
    *blocks_out = blocks;
    if (g.slabs == nullptr)
        return DH_OK;
    hipLaunchKernelGGL((ts_nt_kernel<T, NB, true, CPG, true>), dim3(static_cast<unsigned>(blocks)), dim3(256), lds, ctx->stream, g);
    return DH_OK;
}

// ts_nt_kernel<double, 1, false, 8>, launched from a translation unit of its own (ts_nt_wide_f64.hip): the kernel
// needs more registers than a wave has vector registers, and built with the matrix instructions in their
// accumulator-register form the compiler parks loaded rows in accumulator registers and copies them back in every step.
dh_status ts_nt_launch_wide_f64(dh_ctx *ctx, const TsNtArgs &g, size_t lds);

template <typename T, int NB, bool ASSIGN> inline dh_status ts_nt_launch(dh_ctx *ctx, const TsNtArgs &g) {
    const int cpg = ts_nt_chunks_per_step<T>(g.kpad);
    // 64 doubles a row, product stored: all eight chunks in one step, which takes the loop that finishes a pair beside
    // the matrix instructions of the next (10M x 64 by 16: 1240 -> 1090 us, at one wave per SIMD instead of two). The
    // arg-min form loses by it (1060 -> 1250 us, with or without that loop).
    if constexpr (sizeof(T) == 8 && NB == 1 && !ASSIGN) {
        if (g.kpad == 64)
            return ts_nt_launch_wide_f64(ctx, g, ts_nt_lds_bytes<T>(NB, g.kpad, 8));
    }
    const size_t lds = ts_nt_lds_bytes<T>(NB, g.kpad, cpg);
    return cpg == 4 ? ts_nt_launch_cpg<T, NB, ASSIGN, 4>(ctx, g, lds)
                    : (cpg == 2 ? ts_nt_launch_cpg<T, NB, ASSIGN, 2>(ctx, g, lds) : ts_nt_launch_cpg<T, NB, ASSIGN, 1>(ctx, g, lds));
}

template <typename T>
bool ts_nt(dh_ctx *ctx, size_t M, size_t n, size_t K, const T *A, size_t lda, const T *B, size_t ldb, T *C, size_t ldc,
           dh_status *status) {
    constexpr int V = 16 / sizeof(T), KC = 4 * V;
    if (n == 0 || n > 32 || K == 0 || K > 512 || M < 65536 || lda * sizeof(T) >= (size_t(1) << 24))
        return false;
    if (!dh_aligned(A, 16) || !dh_aligned(B, 16) || lda % V || ldb % V || K % V)
        return false;
    const int nb = n <= 16 ? 1 : 2;
    TsNtArgs g{};
    g.A = A;
    g.B = B;
    g.C = C;
    g.lda = lda;
    g.ldb = ldb;
    g.ldc = ldc;
    g.M = M;
    g.n = static_cast<unsigned>(n);
    g.K = static_cast<unsigned>(K);
    g.kpad = static_cast<unsigned>(dh_ceil_div(K, KC) * KC);
    g.vec_store = dh_aligned(C, 16) && (ldc * sizeof(T)) % 16 == 0;
    if (static_cast<size_t>(nb) * 16 * (g.kpad + V) * sizeof(T) > (size_t(48) << 10))
        return false;
    *status = nb == 1 ? ts_nt_launch<T, 1, false>(ctx, g) : ts_nt_launch<T, 2, false>(ctx, g);
    return true;
}

} // namespace dh_gemm
