// Dense linear solve A x = b for one right-hand side: LU with partial pivoting in a single
// workgroup, then forward elimination of b (done alongside) and back substitution.
//
// Stands in for CUDA::Solve (src/runtime/local/kernels/CUDA/Solve.cpp:75-151, cuSOLVER
// getrf + getrs) with the result of the CPU kernel (src/runtime/local/kernels/Solve.h:86-116,
// LAPACKE_?gesv): same pivot choice (first row of maximal magnitude), multipliers formed with
// the reciprocal of the pivot. The systems on this path are small (100 x 100 normal equations),
// so the work is latency-bound: a system that fits in LDS (up to 128 doubles / 184 floats a
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

// The whole system in LDS, the right-hand side as one more column of the matrix, factored in panels of NB columns
// (right-looking LU with partial pivoting; U and the eliminated right-hand side are all that is needed afterwards).
// The work is a chain of dependent steps, not of arithmetic, and a single compute unit issues instructions slowly
// (a wavefront on its own gets one out every four to eight cycles, whatever the instruction), so the kernel is
// built around the number of instructions on the critical path and around keeping everything else off that path.
//   P   wave 0 alone factors a panel in registers: a lane holds the panel's NB values of rows lane, lane + 64, ...
//       Rows are not exchanged there; each keeps track of the position it currently has in the matrix. Per column:
//       a wave-wide maximum over a 32-bit image of the magnitudes (the high word of a double) names the pivot's lane
//       when it is the only one with that image - otherwise the full magnitudes and then the positions decide, so the
//       choice is always that of ?gesv (first row of the largest magnitude); the pivot row's remaining values are
//       broadcast with readlane and the rows whose position lies below are eliminated. At the end the rows go back to
//       LDS at their positions (the multipliers of the rows below the panel to a packed copy), with the list of rows
//       that are not where they were.
//   C   everything a panel does to a column right of it touches that column only, so a wave takes whole columns and
//       needs no barrier in between. First half, a lane per column: the rows that moved (all read, then all written)
//       and the NB x NB unit-lower triangle for the column's part of U. Second half, a lane per row and four columns
//       at a time: the rank-NB update of the rows below, the row's multipliers in registers for the whole panel.
// Look-ahead: after panel k the eight waves first bring the NB columns of panel k + 1 up to date, a column each (both
// halves at once there: every lane solves the triangle); after a barrier wave 0 factors panel k + 1 while the other
// seven waves take panel k through all remaining columns. Two barriers per panel, and the trailing update is off the
// critical path.
// Multipliers are formed with the reciprocal of the pivot, as ?getf2 does. Back substitution runs in wave 0 alone,
// right-hand side in registers, eight unknowns per pass; the diagonal is inverted beforehand, all rows at once, so
// that no division stands in the chain (x = r * (1 / u) differs from r / u by one rounding at most).
// The kernel clears the singularity flag itself.
constexpr int LDS_SOLVE_MAX_SLOTS = 3;   // rows per lane of a wave: n <= 192
constexpr int LDS_SOLVE_NB = 8;          // panel width; also the number of waves
constexpr unsigned LDS_SOLVE_THREADS = 64 * LDS_SOLVE_NB;

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

// The magnitude of v as an unsigned integer of the same width (monotone in |v|; NaNs above everything).
__device__ __forceinline__ unsigned mag_bits(float v) { return __builtin_bit_cast(unsigned, v) & 0x7fffffffu; }
__device__ __forceinline__ unsigned long long mag_bits(double v) {
    return __builtin_bit_cast(unsigned long long, v) & 0x7fffffffffffffffull;
}
// Its leading 32 bits plus one: monotone (not strictly, for doubles) in |v| and never zero.
__device__ __forceinline__ unsigned mag_key(float v) { return mag_bits(v) + 1u; }
__device__ __forceinline__ unsigned mag_key(double v) { return static_cast<unsigned>(mag_bits(v) >> 32) + 1u; }

// Maximum of h over the 64 lanes of a fully active wave, as a wave-uniform value.
__device__ __forceinline__ unsigned wave_max_u32(unsigned h) {
    unsigned t;
    t = dh_dpp<0xB1>(h), h = t > h ? t : h;
    t = dh_dpp<0x4E>(h), h = t > h ? t : h;
    t = dh_dpp<0x141>(h), h = t > h ? t : h;
    t = dh_dpp<0x140>(h), h = t > h ? t : h;
    const unsigned r0 = read_lane(h, 0), r1 = read_lane(h, 16), r2 = read_lane(h, 32), r3 = read_lane(h, 48);
    const unsigned m0 = r0 > r1 ? r0 : r1, m1 = r2 > r3 ? r2 : r3;
    return m0 > m1 ? m0 : m1;
}

// Shape of the system in LDS: the order rounded up to whole panels (the added rows and columns are those of an identity
// matrix, so no panel is ever partial), an odd row stride (column walks spread over the banks), the right-hand side as
// column npad, one spare row (the target of the unused entries of the list of moved rows), and the packed multipliers.
template <typename T> struct LdsSolveShape {
    unsigned npad, ld;
    size_t lp_offset, bytes;
    __host__ __device__ explicit LdsSolveShape(size_t n) {
        npad = static_cast<unsigned>((n + LDS_SOLVE_NB - 1) / LDS_SOLVE_NB * LDS_SOLVE_NB);
        ld = (npad + 1) | 1u;
        lp_offset = (static_cast<size_t>(npad + 1) * ld * sizeof(T) + 15) & ~size_t(15);
        bytes = lp_offset + static_cast<size_t>(npad) * LDS_SOLVE_NB * sizeof(T);
    }
};

template <typename T, int SLOTS>
__global__ __launch_bounds__(LDS_SOLVE_THREADS) void lu_solve_lds_kernel(T *x_out, const T *A, size_t lda, const T *b, unsigned n,
                                                                         int *flag) {
    constexpr int NB = LDS_SOLVE_NB;
    constexpr unsigned WAVES = LDS_SOLVE_THREADS / 64;
    constexpr int V = 16 / sizeof(T);
    constexpr int UPDATE_COLS = 4; // columns a wave updates at a time
    extern __shared__ __attribute__((aligned(16))) unsigned char solve_lds[];
    __shared__ int s_stop;
    __shared__ unsigned s_nmoved;
    __shared__ unsigned short s_from[2 * NB], s_to[2 * NB];
    const LdsSolveShape<T> shape(n);
    const unsigned npad = shape.npad, ld = shape.ld;
    T *a = reinterpret_cast<T *>(solve_lds);
    // packed multipliers of the current panel, one 16-byte aligned row of NB values per matrix row
    T *lp = reinterpret_cast<T *>(solve_lds + shape.lp_offset);
    const unsigned tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    {
        // copy-in: a thread's loads go out in batches of eight before the first LDS store (positions past the
        // matrix read its last row and are not stored)
        constexpr unsigned TX = 128, TY = LDS_SOLVE_THREADS / 128;
        const unsigned tx = tid % TX, ty = tid / TX;
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
    }
    // right-hand side and the padding: columns n .. npad of the matrix rows, rows n .. npad whole
    {
        const unsigned wpad = npad + 1 - n;
        for (unsigned i = tid; i < n * wpad; i += LDS_SOLVE_THREADS) {
            const unsigned r = i / wpad, c = n + i % wpad;
            a[r * ld + c] = c == npad ? b[r] : T(0);
        }
        for (unsigned i = tid; i < wpad * (npad + 1); i += LDS_SOLVE_THREADS) {
            const unsigned r = n + i / (npad + 1), c = i % (npad + 1);
            a[r * ld + c] = r == c ? T(1) : T(0);
        }
    }
    if (tid == 0) {
        s_stop = 0;
        *flag = 0;
    }
    DH_PROF_DECL;
    __syncthreads();
    DH_PROF(0);

    // ---- what a wave keeps of the panel it applies to its columns (set between the two barriers of an iteration)
    T l11[NB * (NB - 1) / 2]; // the unit-lower triangle below the diagonal, row by row
    T lrow[SLOTS][NB];        // multipliers of rows lane + 64 s (zero for rows that are not below the panel)
    unsigned mv_from = 0, mv_to = 0, cnm = 0;
    unsigned ck0 = 0;

    auto load_triangle = [&]() { // of the panel [ck0, ck0 + NB)
#pragma unroll
        for (int jj = 1; jj < NB; jj++) {
#pragma unroll
            for (int m = 0; m < jj; m++)
                l11[jj * (jj - 1) / 2 + m] = a[(ck0 + jj) * ld + ck0 + m];
        }
    };
    auto load_moved = [&]() {
        mv_from = s_from[lane % (2 * NB)];
        mv_to = s_to[lane % (2 * NB)];
        cnm = s_nmoved;
    };
    // ---- C, whole, for the one column c: every lane solves the triangle (the operands are broadcast reads), lane e
    // moves entry e of the list, lanes are rows in the update
    auto column = [&](unsigned c) {
        if (cnm != 0) {
            const T t = a[mv_from * ld + c];
            if (lane < 2 * NB)
                a[mv_to * ld + c] = t;
        }
        T u[NB], v[SLOTS];
#pragma unroll
        for (int m = 0; m < NB; m++)
            u[m] = a[(ck0 + m) * ld + c];
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const unsigned i = lane + 64 * s;
            v[s] = a[(i < npad ? i : 0) * ld + c]; // rows below the panel: not among those that U is written to
        }
#pragma unroll
        for (int jj = 1; jj < NB; jj++) {
#pragma unroll
            for (int m = 0; m < jj; m++)
                u[jj] -= l11[jj * (jj - 1) / 2 + m] * u[m];
        }
        if (lane == 0) {
#pragma unroll
            for (int jj = 1; jj < NB; jj++)
                a[(ck0 + jj) * ld + c] = u[jj];
        }
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const unsigned i = lane + 64 * s;
#pragma unroll
            for (int m = 0; m < NB; m++)
                v[s] -= lrow[s][m] * u[m];
            if (i >= ck0 + NB && i < npad)
                a[i * ld + c] = v[s];
        }
    };
    // ---- C, first half, for the count columns c_first + stride * lane (a lane per column; the other lanes repeat the
    // first column and store nothing): the rows that moved, and the column's part of U
    auto triangles = [&](unsigned c_first, unsigned stride, unsigned count) {
        const bool live = lane < count;
        const unsigned c = live ? c_first + stride * lane : c_first;
        if (cnm != 0) {
            T t[2 * NB];
#pragma unroll
            for (int e = 0; e < 2 * NB; e++)
                t[e] = a[read_lane(mv_from, e) * ld + c];
            if (live) {
#pragma unroll
                for (int e = 0; e < 2 * NB; e++)
                    a[read_lane(mv_to, e) * ld + c] = t[e];
            }
        }
        T u[NB];
#pragma unroll
        for (int m = 0; m < NB; m++)
            u[m] = a[(ck0 + m) * ld + c];
#pragma unroll
        for (int jj = 1; jj < NB; jj++) {
#pragma unroll
            for (int m = 0; m < jj; m++)
                u[jj] -= l11[jj * (jj - 1) / 2 + m] * u[m];
        }
        if (live) {
#pragma unroll
            for (int jj = 1; jj < NB; jj++)
                a[(ck0 + jj) * ld + c] = u[jj];
        }
    };
    // ---- C, second half, for up to CB columns c0, c0 + stride, ... at a time (count of them; a column index past
    // the count repeats the first and stores nothing): the rank-NB update of the rows below, lanes are rows
    auto update = [&](auto width, unsigned c0, unsigned stride, unsigned count) {
        constexpr int CB = decltype(width)::value;
        unsigned cq[CB];
        bool live[CB];
#pragma unroll
        for (int q = 0; q < CB; q++) {
            live[q] = static_cast<unsigned>(q) < count;
            cq[q] = live[q] ? c0 + q * stride : c0;
        }
        T u[CB][NB];
#pragma unroll
        for (int q = 0; q < CB; q++) {
#pragma unroll
            for (int m = 0; m < NB; m++)
                u[q][m] = a[(ck0 + m) * ld + cq[q]];
        }
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const unsigned i = lane + 64 * s;
            if (64u * (s + 1) > ck0 + NB) {
                const bool below = i >= ck0 + NB && i < npad;
                T v[CB];
#pragma unroll
                for (int q = 0; q < CB; q++)
                    v[q] = a[(i < npad ? i : 0) * ld + cq[q]];
#pragma unroll
                for (int m = 0; m < NB; m++) {
#pragma unroll
                    for (int q = 0; q < CB; q++)
                        v[q] -= lrow[s][m] * u[q][m];
                }
#pragma unroll
                for (int q = 0; q < CB; q++)
                    if (below && live[q])
                        a[i * ld + cq[q]] = v[q];
            }
        }
    };

    for (unsigned k0 = 0; k0 < npad; k0 += NB) {
        const unsigned cfirst = k0 + NB; // first row below / column right of the panel; column npad is the right-hand side
        if (wave != 0) {
            // the previous panel's remaining columns, while wave 0 factors this one
            if (k0 > 0 && cfirst + (wave - 1) <= npad) {
                triangles(cfirst + (wave - 1), WAVES - 1, (npad - (cfirst + (wave - 1))) / (WAVES - 1) + 1);
                for (unsigned c = cfirst + (wave - 1); c <= npad; c += UPDATE_COLS * (WAVES - 1))
                    update(std::integral_constant<int, UPDATE_COLS>{}, c, WAVES - 1, (npad - c) / (WAVES - 1) + 1);
            }
        } else {
            // ---- P: the panel, rows k0 .. npad - 1, in registers; pos[s] is the position the row has in the matrix now
            T pv[SLOTS][NB];
            int pos[SLOTS]; // -1: not a row of this panel
#pragma unroll
            for (int s = 0; s < SLOTS; s++) {
                const unsigned r = lane + 64 * s;
                const bool valid = r >= k0 && r < npad;
                pos[s] = valid ? static_cast<int>(r) : -1;
#pragma unroll
                for (int c = 0; c < NB; c++) {
                    const T v = a[(valid ? r : k0) * ld + k0 + c];
                    pv[s][c] = valid ? v : T(0);
                }
            }
#pragma unroll
            for (int jj = 0; jj < NB; jj++) {
                const int j = static_cast<int>(k0) + jj;
                // pivot: among the rows at positions >= j, the largest |value| in column jj, the first position
                // among equals
                unsigned h[SLOTS], hm = 0;
#pragma unroll
                for (int s = 0; s < SLOTS; s++) {
                    h[s] = pos[s] >= j ? mag_key(pv[s][jj]) : 0u;
                    hm = h[s] > hm ? h[s] : hm;
                }
                hm = wave_max_u32(hm);
                unsigned long long e[SLOTS];
                unsigned cnt = 0;
#pragma unroll
                for (int s = 0; s < SLOTS; s++) {
                    e[s] = __ballot(h[s] == hm);
                    cnt += static_cast<unsigned>(__popcll(e[s]));
                }
                int os = 0, ol;
                if (cnt == 1) {
                    unsigned long long eo = e[0];
#pragma unroll
                    for (int s = 1; s < SLOTS; s++) {
                        os = e[s] != 0 ? s : os;
                        eo |= e[s];
                    }
                    ol = __builtin_ctzll(eo);
                } else {
                    // several rows share the leading bits: the whole magnitude decides, then the position
                    using Bits = decltype(mag_bits(T(0)));
                    Bits best = 0;
                    unsigned key = 0xffffffffu;
#pragma unroll
                    for (int s = 0; s < SLOTS; s++) {
                        const Bits mb = mag_bits(pv[s][jj]);
                        const unsigned k = (static_cast<unsigned>(pos[s]) << 8) | (static_cast<unsigned>(s) << 6) | lane;
                        if (h[s] == hm && (key == 0xffffffffu || mb > best || (mb == best && k < key))) {
                            best = mb;
                            key = k;
                        }
                    }
                    Bits top = best;
                    dh_butterfly(64, [&](auto peer) {
                        const Bits o = peer(top);
                        top = o > top ? o : top;
                    });
                    if (best != top)
                        key = 0xffffffffu;
                    dh_butterfly(64, [&](auto peer) {
                        const unsigned ok = peer(key);
                        key = ok < key ? ok : key;
                    });
                    const unsigned ukey = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(key)));
                    ol = static_cast<int>(ukey & 63u);
                    os = static_cast<int>((ukey >> 6) & 3u);
                }
                // the pivot row's position, and its values from column jj on
                int p = j;
                T prow[NB];
                auto take = [&](auto slot) {
                    constexpr int s = decltype(slot)::value;
                    p = read_lane(pos[s], ol);
#pragma unroll
                    for (int c = jj; c < NB; c++)
                        prow[c] = read_lane(pv[s][c], ol);
                };
                if (SLOTS == 1 || os == 0)
                    take(std::integral_constant<int, 0>{});
                else if (SLOTS == 2 || os == 1)
                    take(std::integral_constant<int, SLOTS >= 2 ? 1 : 0>{});
                else
                    take(std::integral_constant<int, SLOTS >= 3 ? 2 : 0>{});
                if (prow[jj] == T(0)) { // info > 0 of ?gesv
                    if (lane == 0) {
                        *flag = j + 1;
                        s_stop = 1;
                    }
                    break;
                }
                // the exchange of positions j and p
                if (p != j) {
#pragma unroll
                    for (int s = 0; s < SLOTS; s++)
                        pos[s] = pos[s] == j ? p : (pos[s] == p ? j : pos[s]);
                }
                const T inv = T(1) / prow[jj];
#pragma unroll
                for (int s = 0; s < SLOTS; s++) {
                    if (pos[s] > j) {
                        const T l = pv[s][jj] * inv;
                        pv[s][jj] = l;
#pragma unroll
                        for (int c = jj + 1; c < NB; c++)
                            pv[s][c] -= l * prow[c];
                    }
                }
            }
            // back to LDS by position: the panel's own rows into the matrix, the multipliers below into the packed
            // copy; and the list of the rows that are not where they were, filled up with the spare row
            unsigned nmoved = 0;
#pragma unroll
            for (int s = 0; s < SLOTS; s++) {
                const int r = static_cast<int>(lane) + 64 * s;
                if (pos[s] >= 0) {
                    if (static_cast<unsigned>(pos[s]) < cfirst) {
#pragma unroll
                        for (int c = 0; c < NB; c++)
                            a[static_cast<unsigned>(pos[s]) * ld + k0 + c] = pv[s][c];
                    } else {
#pragma unroll
                        for (int c = 0; c < NB; c++)
                            lp[static_cast<unsigned>(pos[s]) * NB + c] = pv[s][c];
                    }
                }
                const bool moved = pos[s] >= 0 && pos[s] != r;
                const unsigned long long m = __ballot(moved);
                if (moved) {
                    const unsigned at = nmoved + static_cast<unsigned>(__popcll(m & ((1ull << lane) - 1ull)));
                    s_from[at] = static_cast<unsigned short>(r);
                    s_to[at] = static_cast<unsigned short>(pos[s]);
                }
                nmoved += static_cast<unsigned>(__popcll(m));
            }
            if (lane >= nmoved && lane < 2 * NB) {
                s_from[lane] = static_cast<unsigned short>(npad);
                s_to[lane] = static_cast<unsigned short>(npad);
            }
            if (lane == 0)
                s_nmoved = nmoved;
        }
        __syncthreads();
        DH_PROF(1); // panel (and, beside it, the previous panel's remaining columns)
        if (s_stop)
            return;
        // ---- what a wave keeps of this panel (triangle, its rows' multipliers, the rows that moved), and the next
        // panel's columns, a wave each
        ck0 = k0;
        load_triangle();
        load_moved();
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const unsigned i = lane + 64 * s;
            const bool below = i >= cfirst && i < npad;
#pragma unroll
            for (int m = 0; m < NB; m += V) {
                T part[V];
                dh_load_vec<T, V>(lp + (below ? i : 0) * NB + m, part);
#pragma unroll
                for (int q = 0; q < V; q++)
                    lrow[s][m + q] = below ? part[q] : T(0);
            }
        }
        if (cfirst + wave <= npad)
            column(cfirst + wave);
        __syncthreads();
        DH_PROF(2); // the next panel's columns
    }
    if (wave != 0)
        return;
    // back substitution, column oriented, eight unknowns at a time from the last (padding included: those come out as
    // zero): x[j] = rhs[j] / U[j][j]; rhs[r] -= U[r][j] x[j]. The rows below j are updated along with those above -
    // they are solved already and their right-hand side is not read again - so a step is a multiplication, a
    // broadcast and one fused multiply-add per slot that still has unsolved rows.
    T rhs[SLOTS], res[SLOTS], dinv[SLOTS];
    unsigned rowat[SLOTS];
#pragma unroll
    for (int s = 0; s < SLOTS; s++) {
        const unsigned r = lane + 64 * s;
        rowat[s] = (r < npad ? r : 0) * ld;
        rhs[s] = a[rowat[s] + npad];
        dinv[s] = T(1) / a[rowat[s] + (r < npad ? r : 0)];
        res[s] = T(0);
    }
    auto solve_block = [&](auto owner_slot, unsigned j0) {
        constexpr int S = decltype(owner_slot)::value; // the slot of rows j0 .. j0 + 7; higher slots are solved
        T col[NB][S + 1];
#pragma unroll
        for (int t = 0; t < NB; t++) {
#pragma unroll
            for (int s = 0; s <= S; s++)
                col[t][s] = a[rowat[s] + j0 + t];
        }
        const int l0 = static_cast<int>(j0 % 64);
#pragma unroll
        for (int t = NB - 1; t >= 0; t--) {
            const T xj = read_lane(rhs[S] * dinv[S], l0 + t);
#pragma unroll
            for (int s = 0; s <= S; s++)
                rhs[s] -= col[t][s] * xj;
            res[S] = static_cast<int>(lane) == l0 + t ? xj : res[S];
        }
    };
    for (unsigned j0 = npad; j0 >= NB;) {
        j0 -= NB;
        if (SLOTS >= 3 && j0 >= 128)
            solve_block(std::integral_constant<int, SLOTS >= 3 ? 2 : 0>{}, j0);
        else if (SLOTS >= 2 && j0 >= 64)
            solve_block(std::integral_constant<int, SLOTS >= 2 ? 1 : 0>{}, j0);
        else
            solve_block(std::integral_constant<int, 0>{}, j0);
    }
#pragma unroll
    for (int s = 0; s < SLOTS; s++) {
        const unsigned r = lane + 64 * s;
        if (r < n)
            x_out[r] = res[s];
    }
    DH_PROF(3); // back substitution
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
    // where the verdict goes: the pinned host word that the wait below reads, or - with deferred verdicts - the
    // context's flag on the device, which a one-thread kernel then keeps for dh_check_deferred
    const bool deferred = ctx->deferred_depth > 0;
    int *verdict = deferred ? ctx->flag_dev : ctx->flag_host_dev;
    const size_t lds_bytes = LdsSolveShape<T>(n).bytes;
    if (n <= 64 * LDS_SOLVE_MAX_SLOTS && lds_bytes <= (size_t(150) << 10)) {
        // Systems beyond 64 KB of LDS need the limit of the kernel raised, once per kernel instantiation and device
        // (the three instantiations have the same pointer type, so the bookkeeping is keyed by SLOTS, not by type).
        auto launch = [&](auto kernel, int slots) -> dh_status {
            if (lds_bytes > (size_t(64) << 10)) {
                constexpr int MAX_DEVICES = 64;
                static std::mutex attr_lock;
                static bool attr_set[LDS_SOLVE_MAX_SLOTS + 1][MAX_DEVICES] = {};
                std::lock_guard<std::mutex> guard(attr_lock);
                const bool tracked = ctx->device >= 0 && ctx->device < MAX_DEVICES;
                if (!tracked || !attr_set[slots][ctx->device]) {
                    DH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                     150 << 10));
                    if (tracked)
                        attr_set[slots][ctx->device] = true;
                }
            }
            hipLaunchKernelGGL(kernel, dim3(1), dim3(LDS_SOLVE_THREADS), lds_bytes, ctx->stream, x, A, lda, b,
                               static_cast<unsigned>(n), verdict);
            return DH_OK;
        };
        dh_status lst;
        if (n <= 64)
            lst = launch(&lu_solve_lds_kernel<T, 1>, 1);
        else if (n <= 128)
            lst = launch(&lu_solve_lds_kernel<T, 2>, 2);
        else
            lst = launch(&lu_solve_lds_kernel<T, 3>, 3);
        if (lst != DH_OK)
            return lst;
    } else {
        hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(1), 0, ctx->stream, verdict);
        void *wsv = nullptr;
        dh_status st = dh_workspace(ctx, n * n * sizeof(T), &wsv);
        if (st != DH_OK)
            return st;
        hipLaunchKernelGGL((lu_solve_kernel<T>), dim3(1), dim3(SOLVE_THREADS), 0, ctx->stream, static_cast<T *>(wsv), x,
                           A, lda, b, static_cast<unsigned>(n), verdict);
    }
    DH_CHECK_LAUNCH();
    if (deferred)
        return dh_latch_deferred(ctx, 0, DH_DEFERRED_SOLVE_SINGULAR, 0, nullptr, 0, 0);
    // the kernels write the flag into the pinned host word itself: no copy back, only the wait
    DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (*static_cast<volatile int *>(ctx->flag_host) != 0)
        return dh_fail_solve_singular();
    return DH_OK;
}

} // namespace

extern "C" dh_status dh_solve_f32(dh_ctx *ctx, float *x, const float *A, size_t n, size_t lda, const float *b) {
    return solve<float>(ctx, x, A, n, lda, b);
}
extern "C" dh_status dh_solve_f64(dh_ctx *ctx, double *x, const double *A, size_t n, size_t lda, const double *b) {
    return solve<double>(ctx, x, A, n, lda, b);
}
