// Fused execution of a row-split ("vectorized") operator pipeline on the device.
//
// In the reference, VectorizedPipeline (src/runtime/local/kernels/VectorizedPipeline.h:35-69)
// hands row chunks to workers that run the pipeline body one kernel call per operator, each
// intermediate materialised (vectorized/TasksCUDA.cpp:21-63 for the device worker). On MI355X the
// whole body runs as ONE kernel over the device-resident matrix: every wavefront keeps the rows
// it is working on in registers, interprets the (wave-uniform) operator list on them, and only
// the declared outputs go back to HBM. A z-score + row-sum + threshold-count body thus reads X
// once and writes 4 bytes per row instead of moving six intermediates.
//
// Execution model: an accumulator machine with two implicit values per row,
//   t - the current row tile (cols values, spread over the G lanes that share the row), and
//   r - the current row scalar (result of the last row aggregation),
// and a list of at most DH_PIPE_MAX_INSTR instructions:
//   EW_BINARY  t = op(t, operand)  or  r = op(r, operand)          (swap: operand on the left)
//   EW_UNARY   t = op(t)           or  r = op(r)
//   ROW_AGG    r = agg(t)          SUM PROD MIN MAX MEAN VAR STDDEV IDXMIN IDXMAX
//   STORE_TILE / STORE_ROW / STORE_ROW_IDX   write t, r, or r as a 64-bit index
//   REDUCE_ALL combine r (or all of t) over all rows with SUM / MIN / MAX -> one device scalar
// Operands: an immediate scalar, t itself, a 1 x cols row vector (held in registers), a
// rows x 1 column vector, another rows x cols matrix, or r broadcast over the row.
// All branches on the instruction stream are uniform across the wavefront; the element loops
// inside each case are fully unrolled over the 16 (float) / 8 (double) values a lane holds.
//
// Scalar semantics per element are those of the stand-alone kernels (ew_impl.h, agg_impl.h),
// i.e. of the reference's CPU kernels.
#pragma once

#include "ew_ops.h"

namespace dh_pipe {

constexpr int THREADS = 256;

template <typename T> struct PipeIO {
    const T *x;
    size_t ld_x;
    const T *matrix[DH_PIPE_MAX_OPERANDS];
    size_t ld_matrix[DH_PIPE_MAX_OPERANDS];
    const T *rowvec[DH_PIPE_MAX_OPERANDS];
    const T *colvec[DH_PIPE_MAX_OPERANDS];
    size_t ld_colvec[DH_PIPE_MAX_OPERANDS];
    T *out_tile[DH_PIPE_MAX_OPERANDS];
    size_t ld_out_tile[DH_PIPE_MAX_OPERANDS];
    void *out_row[DH_PIPE_MAX_OPERANDS];
    size_t ld_out_row[DH_PIPE_MAX_OPERANDS];
};

struct Program {
    int n;
    dh_pipe_instr ins[DH_PIPE_MAX_INSTR];
};
// The immediates of a body, in instruction order: an argument of the specialised kernel, so that a body
// compiled once serves every value of its scalars.
struct Immediates {
    double v[DH_PIPE_MAX_INSTR];
};

template <typename T, int N> __device__ __forceinline__ void apply_binary(int op, T (&a)[N], const T (&b)[N], bool swap) {
    using namespace dh_ew;
#define DH_CASE(CODE, FUN)                                                                         \
    case CODE:                                                                                     \
        if (swap) {                                                                                \
            _Pragma("unroll") for (int i = 0; i < N; i++) a[i] = FUN<T>::apply(b[i], a[i]);        \
        } else {                                                                                   \
            _Pragma("unroll") for (int i = 0; i < N; i++) a[i] = FUN<T>::apply(a[i], b[i]);        \
        }                                                                                          \
        break;
    switch (op) {
        DH_CASE(DH_BIN_ADD, BAdd)
        DH_CASE(DH_BIN_SUB, BSub)
        DH_CASE(DH_BIN_MUL, BMul)
        DH_CASE(DH_BIN_DIV, BDiv)
        DH_CASE(DH_BIN_POW, BPow)
        DH_CASE(DH_BIN_MOD, BMod)
        DH_CASE(DH_BIN_LOG, BLog)
        DH_CASE(DH_BIN_EQ, BEq)
        DH_CASE(DH_BIN_NEQ, BNeq)
        DH_CASE(DH_BIN_LT, BLt)
        DH_CASE(DH_BIN_LE, BLe)
        DH_CASE(DH_BIN_GT, BGt)
        DH_CASE(DH_BIN_GE, BGe)
        DH_CASE(DH_BIN_MIN, BMin)
        DH_CASE(DH_BIN_MAX, BMax)
        DH_CASE(DH_BIN_AND, BAnd)
        DH_CASE(DH_BIN_OR, BOr)
    default:
        break;
    }
#undef DH_CASE
}

template <typename T, int N> __device__ __forceinline__ bool apply_unary(int op, T (&a)[N], const bool (&ok)[N]) {
    using namespace dh_ew;
    bool bad = false;
#define DH_CASE(CODE, FUN)                                                                         \
    case CODE:                                                                                     \
        _Pragma("unroll") for (int i = 0; i < N; i++) {                                            \
            if constexpr (FUN<T>::checks)                                                          \
                bad |= ok[i] && FUN<T>::bad(a[i]);                                                 \
            a[i] = FUN<T>::apply(a[i], T(0));                                                      \
        }                                                                                          \
        break;
    switch (op) {
        DH_CASE(DH_UN_MINUS, UMinus)
        DH_CASE(DH_UN_ABS, UAbs)
        DH_CASE(DH_UN_SIGN, USign)
        DH_CASE(DH_UN_SQRT, USqrt)
        DH_CASE(DH_UN_EXP, UExp)
        DH_CASE(DH_UN_LN, ULn)
        DH_CASE(DH_UN_SIN, USin)
        DH_CASE(DH_UN_COS, UCos)
        DH_CASE(DH_UN_TAN, UTan)
        DH_CASE(DH_UN_ASIN, UAsin)
        DH_CASE(DH_UN_ACOS, UAcos)
        DH_CASE(DH_UN_ATAN, UAtan)
        DH_CASE(DH_UN_SINH, USinh)
        DH_CASE(DH_UN_COSH, UCosh)
        DH_CASE(DH_UN_TANH, UTanh)
        DH_CASE(DH_UN_FLOOR, UFloor)
        DH_CASE(DH_UN_CEIL, UCeil)
        DH_CASE(DH_UN_ROUND, URound)
        DH_CASE(DH_UN_ISNAN, UIsNan)
    default:
        break;
    }
#undef DH_CASE
    return bad;
}

// t[i] / d[i] for divisors that do not change from step to step (a row-vector operand): the correctly
// rounded quotient from the same operation sequence as the general division (reciprocal, one / two
// Newton steps on it, quotient, two / one residual corrections - the sequence the compiler emits for
// a / b), minus its scaling and special-case handling. That is valid while no operand needs scaling:
// every |t[i]| and |d[i]| within [2^-40, 2^40] (float) or [2^-300, 2^300] (double). The reciprocal part
// depends on d alone and moves out of the row loop, which leaves 5 (float) / 3 (double) operations per
// item instead of 11 / 13. Returns false, having changed nothing, when a value of this wavefront is
// outside that range (zeros, infinities, subnormals); the caller then divides the ordinary way.
__device__ __forceinline__ float pipe_abs(float v) { return __builtin_fabsf(v); }
__device__ __forceinline__ double pipe_abs(double v) { return __builtin_fabs(v); }
__device__ __forceinline__ float pipe_max(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double pipe_max(double a, double b) { return __builtin_fmax(a, b); }
__device__ __forceinline__ float pipe_min(float a, float b) { return __builtin_fminf(a, b); }
__device__ __forceinline__ double pipe_min(double a, double b) { return __builtin_fmin(a, b); }
template <typename T, int N> __device__ __forceinline__ bool div_by_invariant(T (&t)[N], const T (&d)[N]) {
    const T hi = sizeof(T) == 4 ? T(0x1p40) : T(0x1p300), lo = sizeof(T) == 4 ? T(0x1p-40) : T(0x1p-300);
    T tmax = T(0), tmin = hi, dmax = T(0), dmin = hi;
#pragma unroll
    for (int i = 0; i < N; i++) {
        const T at = pipe_abs(t[i]), ad = pipe_abs(d[i]);
        tmax = pipe_max(tmax, at);
        tmin = pipe_min(tmin, at);
        dmax = pipe_max(dmax, ad);
        dmin = pipe_min(dmin, ad);
    }
    const bool ok = tmax <= hi && tmin >= lo && dmax <= hi && dmin >= lo;
    if (__builtin_amdgcn_ballot_w64(!ok) != 0)
        return false;
#pragma unroll
    for (int i = 0; i < N; i++) {
        const T n = t[i], b = d[i];
        if constexpr (sizeof(T) == 4) {
            const T r0 = __builtin_amdgcn_rcpf(b);
            const T r = __builtin_fmaf(__builtin_fmaf(-b, r0, 1.0f), r0, r0);
            const T q0 = n * r;
            const T q1 = __builtin_fmaf(__builtin_fmaf(-b, q0, n), r, q0);
            t[i] = __builtin_fmaf(__builtin_fmaf(-b, q1, n), r, q1);
        } else {
            const T r0 = __builtin_amdgcn_rcp(b);
            const T r1 = __builtin_fma(r0, __builtin_fma(-b, r0, 1.0), r0);
            const T r = __builtin_fma(r1, __builtin_fma(-b, r1, 1.0), r1);
            const T q0 = n * r;
            t[i] = __builtin_fma(__builtin_fma(-b, q0, n), r, q0);
        }
    }
    return true;
}


// The instruction source. RuntimeProgram reads the list from the kernel argument (generic
// interpreter, compiled ahead of time). A program type with is_const = true and a constexpr
// table makes the same body a straight-line kernel: the instruction loop is fully unrolled and
// every switch folds away. Such types are generated and compiled at run time (hiprtc) per
// distinct pipeline, like the reference JIT-compiles the body of each VectorizedPipelineOp.
struct RuntimeProgram {
    static constexpr bool is_const = false;
    static constexpr int N = 1;
    static __device__ __forceinline__ dh_pipe_instr get(const Program &P, int ip) { return P.ins[ip]; }
};

// One instantiation per (value type, vector width, vectors per lane, program source). U rows are
// in flight per lane group so that a lane always holds U*KV*VEC = 16 bytes * 4 of data.
// G lanes share a row; a wavefront works through runs of S consecutive steps. The run-time
// specialisation passes cols, G and S as literals, so that everything derived from them folds.
template <typename T, int VEC, int KV, class PG>
__device__ __forceinline__ void pipeline_body(const Program &P, const PipeIO<T> &io, size_t rows, size_t cols, int G, int S,
                                                           T *all_partials /* [2][gridDim.x * waves per workgroup] */, int *flag) {
    constexpr int U = 4 / KV;
    constexpr int N = U * KV * VEC;

    const int tid = threadIdx.x;
    const int lane = tid % G;
    const size_t cvecs = cols / VEC;
    // Rows are dealt to wavefronts in contiguous runs: per step a wavefront owns GPW * U
    // consecutive rows, row (u, g) = base + u * GPW + g for its lane group g, so that load u of
    // the wavefront covers GPW whole rows back to back and the per-row results of a step are one
    // contiguous run that the first GPW * U lanes can store together.
    const int wlane = tid % DH_WAVE;
    const int GPW = DH_WAVE / G;            // lane groups (rows) per wavefront and load
    const int g_in_wave = wlane / G;
    const size_t rows_per_step = static_cast<size_t>(GPW) * (4 / KV);
    // wave-uniform values are kept in scalar registers (the index of the wavefront in its workgroup is
    // uniform, which the compiler cannot see from threadIdx alone)
    const size_t wave_id = static_cast<size_t>(blockIdx.x) * (THREADS / DH_WAVE) +
                           static_cast<size_t>(__builtin_amdgcn_readfirstlane(tid / DH_WAVE));
    const size_t n_waves = static_cast<size_t>(gridDim.x) * (THREADS / DH_WAVE);
    const size_t rows_per_run = rows_per_step * static_cast<size_t>(S);
    // vmask: does this lane's j-th vector exist in the row? coff: its element offset, clamped
    // into the row so that every load is in bounds without a guard (masked values are never
    // stored, reduced or domain-checked).
    bool vmask[KV];
    size_t coff[KV];
#pragma unroll
    for (int j = 0; j < KV; j++) {
        vmask[j] = static_cast<size_t>(lane + j * G) < cvecs;
        coff[j] = (vmask[j] ? static_cast<size_t>(lane + j * G) : 0) * VEC;
    }
    // element offset of this lane's (u, j) vector of X from the first row of a step
    size_t xoff[U][KV];
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
        for (int j = 0; j < KV; j++)
            xoff[u][j] = static_cast<size_t>(u * GPW + g_in_wave) * io.ld_x + coff[j];
    // The tile of a step: U rows x KV vectors per lane, every load unconditional (rows past the end read the
    // step's first row; their values are never stored, reduced or domain-checked).
    auto load_tile = [&](size_t base, T (&t)[N]) {
        const T *xbase = io.x + base * io.ld_x; // the step's first row, which always exists
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool live_u = base + static_cast<size_t>(u * GPW + g_in_wave) < rows;
#pragma unroll
            for (int j = 0; j < KV; j++) {
                T x[VEC];
                dh_load_vec_stream<T, VEC>(xbase + (live_u ? xoff[u][j] : coff[j]), x);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    t[(u * KV + j) * VEC + e] = x[e];
            }
        }
    };
    // The wavefront's first tile is asked for before the operand vectors: what the steps derive from those
    // vectors once (reciprocals of a divisor, for one) is then computed while the tile is on its way, instead
    // of holding the first loads back by a memory round trip.
    const size_t first_base = wave_id * rows_per_run;
    T t_first[N];
    load_tile(first_base < rows ? first_base : 0, t_first); // unconditional: a wavefront without rows reads row 0 in vain
    // this lane's share of every bound row-vector operand lives in registers for the whole kernel
    T rv0[KV * VEC], rv1[KV * VEC], rv2[KV * VEC], rv3[KV * VEC];
    // (loaded without a branch: an operand that is not bound reads the first row of X instead and becomes zero;
    // bound ones are 16-byte aligned whenever VEC > 1, which the launch checks)
    auto load_rowvec = [&](const T *p, T (&rv)[KV * VEC]) {
        const T *q = p ? p : io.x;
#pragma unroll
        for (int j = 0; j < KV; j++) {
            T x[VEC];
            dh_load_vec<T, VEC>(q + coff[j], x);
#pragma unroll
            for (int e = 0; e < VEC; e++)
                rv[j * VEC + e] = p ? x[e] : T(0);
        }
    };
    load_rowvec(io.rowvec[0], rv0);
    load_rowvec(io.rowvec[1], rv1);
    load_rowvec(io.rowvec[2], rv2);
    load_rowvec(io.rowvec[3], rv3);

    // running values of the (at most two) REDUCE_ALL slots, and which combine they use
    T all_acc0 = T(0), all_acc1 = T(0);
    bool all_init0 = false, all_init1 = false;
    bool any_bad = false;
    auto fold = [](T &a, bool &init, T v, int op) {
        if (!init && op != DH_AGG_SUM)
            a = (op == DH_AGG_MIN) ? dh_inf<T>() : -dh_inf<T>();
        init = true;
        a = (op == DH_AGG_SUM) ? a + v : (op == DH_AGG_MIN) ? ((v < a) ? v : a) : ((a < v) ? v : a);
    };

    auto run_step = [&](size_t base, T (&t)[N]) {
        T o[N], r[U];
        size_t row[U], lrow[U]; // lrow: row index for loads, clamped to the last row
        bool live[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            row[u] = base + static_cast<size_t>(u * GPW + g_in_wave);
            live[u] = row[u] < rows;
            lrow[u] = live[u] ? row[u] : rows - 1;
            r[u] = T(0);
        }
        #pragma unroll(PG::is_const ? PG::N : 1)
        for (int ip = 0; ip < (PG::is_const ? PG::N : P.n); ip++) {
            const dh_pipe_instr ins = PG::get(P, ip);
            switch (ins.kind) {
            case DH_PIPE_EW_BINARY: {
                if (ins.domain == 0) {
                    switch (ins.operand) {
                    case DH_OPD_SCALAR:
#pragma unroll
                        for (int i = 0; i < N; i++)
                            o[i] = static_cast<T>(ins.scalar);
                        break;
                    case DH_OPD_SELF:
#pragma unroll
                        for (int i = 0; i < N; i++)
                            o[i] = t[i];
                        break;
                    case DH_OPD_ROWVEC:
#pragma unroll
                        for (int u = 0; u < U; u++)
#pragma unroll
                            for (int i = 0; i < KV * VEC; i++)
                                o[u * KV * VEC + i] = ins.index == 0   ? rv0[i]
                                                      : ins.index == 1 ? rv1[i]
                                                      : ins.index == 2 ? rv2[i]
                                                                       : rv3[i];
                        break;
                    case DH_OPD_COLVEC: {
                        const T *cvp = io.colvec[ins.index];
                        const size_t cld = io.ld_colvec[ins.index];
#pragma unroll
                        for (int u = 0; u < U; u++) {
                            const T s = cvp[lrow[u] * cld];
#pragma unroll
                            for (int i = 0; i < KV * VEC; i++)
                                o[u * KV * VEC + i] = s;
                        }
                        break;
                    }
                    case DH_OPD_MATRIX: {
                        const T *mp = io.matrix[ins.index];
                        const size_t mld = io.ld_matrix[ins.index];
#pragma unroll
                        for (int u = 0; u < U; u++)
#pragma unroll
                            for (int j = 0; j < KV; j++) {
                                T x[VEC];
                                dh_load_vec_stream<T, VEC>(mp + lrow[u] * mld + coff[j], x);
#pragma unroll
                                for (int e = 0; e < VEC; e++)
                                    o[(u * KV + j) * VEC + e] = x[e];
                            }
                        break;
                    }
                    default: // DH_OPD_ROWREG
#pragma unroll
                        for (int u = 0; u < U; u++)
#pragma unroll
                            for (int i = 0; i < KV * VEC; i++)
                                o[u * KV * VEC + i] = r[u];
                        break;
                    }
                    // the specialised kernel divides by a row vector with the loop-invariant part hoisted
                    if (!(PG::is_const && ins.op == DH_BIN_DIV && ins.operand == DH_OPD_ROWVEC && ins.swap == 0 &&
                          div_by_invariant<T, N>(t, o)))
                        apply_binary<T, N>(ins.op, t, o, ins.swap != 0);
                } else {
                    T ov[U];
#pragma unroll
                    for (int u = 0; u < U; u++) {
                        if (ins.operand == DH_OPD_COLVEC)
                            ov[u] = io.colvec[ins.index][lrow[u] * io.ld_colvec[ins.index]];
                        else if (ins.operand == DH_OPD_SELF)
                            ov[u] = r[u];
                        else
                            ov[u] = static_cast<T>(ins.scalar);
                    }
                    apply_binary<T, U>(ins.op, r, ov, ins.swap != 0);
                }
                break;
            }
            case DH_PIPE_EW_UNARY:
                // values of masked-out lanes / rows beyond the end must not trip a domain check
                if (ins.domain == 0) {
                    bool ok[N];
#pragma unroll
                    for (int u = 0; u < U; u++)
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                ok[(u * KV + j) * VEC + e] = live[u] && vmask[j];
                    any_bad |= apply_unary<T, N>(ins.op, t, ok);
                } else {
                    any_bad |= apply_unary<T, U>(ins.op, r, live);
                }
                break;
            case DH_PIPE_ROW_AGG: {
                const int op = ins.op;
                const int base = (tid % DH_WAVE) / G * G; // first lane of this group in the wave
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const T first = __shfl(t[u * KV * VEC], base, DH_WAVE);
                    if (op == DH_AGG_IDXMIN || op == DH_AGG_IDXMAX) {
                        const bool is_min = (op == DH_AGG_IDXMIN);
                        T best = is_min ? dh_inf<T>() : -dh_inf<T>();
                        unsigned bi = ~0u;
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++) {
                                const T x = t[(u * KV + j) * VEC + e];
                                const unsigned idx = static_cast<unsigned>((lane + j * G) * VEC + e);
                                const bool better = is_min ? (x < best) : (x > best);
                                const bool first_seen = (bi == ~0u) && !(x != x);
                                if (vmask[j] && (better || first_seen)) {
                                    best = x;
                                    bi = idx;
                                }
                            }
                        dh_butterfly(G, [&](auto peer) {
                            const T ov = peer(best);
                            const unsigned oi = peer(bi);
                            const bool better = is_min ? (ov < best) : (ov > best);
                            if (better || (ov == best && oi < bi)) {
                                best = ov;
                                bi = oi;
                            }
                        });
                        if ((first != first) || bi == ~0u)
                            bi = 0;
                        r[u] = static_cast<T>(bi);
                    } else if (op == DH_AGG_MIN || op == DH_AGG_MAX) {
                        const bool is_min = (op == DH_AGG_MIN);
                        T a = is_min ? dh_inf<T>() : -dh_inf<T>();
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++) {
                                const T x = t[(u * KV + j) * VEC + e];
                                if (vmask[j])
                                    a = is_min ? ((x < a) ? x : a) : ((a < x) ? x : a);
                            }
                        dh_butterfly(G, [&](auto peer) {
                            const T ov = peer(a);
                            a = is_min ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
                        });
                        r[u] = (first != first) ? first : a;
                    } else if (op == DH_AGG_PROD) {
                        T a = T(1);
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                if (vmask[j])
                                    a = a * t[(u * KV + j) * VEC + e];
                        dh_butterfly(G, [&](auto peer) { a = a * peer(a); });
                        r[u] = a;
                    } else { // SUM MEAN VAR STDDEV
                        T a = T(0);
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                if (vmask[j])
                                    a = a + t[(u * KV + j) * VEC + e];
                        dh_butterfly(G, [&](auto peer) { a = a + peer(a); });
                        if (op != DH_AGG_SUM)
                            a = a / static_cast<T>(cols);
                        if (op == DH_AGG_VAR || op == DH_AGG_STDDEV) {
                            const T mean = a;
                            T s = T(0);
#pragma unroll
                            for (int j = 0; j < KV; j++)
#pragma unroll
                                for (int e = 0; e < VEC; e++)
                                    if (vmask[j]) {
                                        const T d = t[(u * KV + j) * VEC + e] - mean;
                                        s = s + d * d;
                                    }
                            dh_butterfly(G, [&](auto peer) { s = s + peer(s); });
                            s = s / static_cast<T>(cols);
                            a = (op == DH_AGG_STDDEV) ? dh_ew::dh_sqrt<T>(s) : s;
                        }
                        r[u] = a;
                    }
                }
                break;
            }
            case DH_PIPE_STORE_TILE:
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int j = 0; j < KV; j++)
                        if (live[u] && vmask[j]) {
                            T x[VEC];
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                x[e] = t[(u * KV + j) * VEC + e];
                            dh_store_vec<T, VEC>(io.out_tile[ins.index] + row[u] * io.ld_out_tile[ins.index] +
                                                     static_cast<size_t>(lane + j * G) * VEC,
                                                 x);
                        }
                break;
            case DH_PIPE_STORE_ROW:
            case DH_PIPE_STORE_ROW_IDX: {
                // lane j < GPW * U takes the result of row base + j (held by every lane of group
                // j % GPW as r[j / GPW]) so that the step's results leave as one contiguous store
                if (GPW * U <= DH_WAVE) {
                    T mine = T(0);
#pragma unroll
                    for (int u = 0; u < U; u++) {
                        const T v = __shfl(r[u], (wlane % GPW) * G, DH_WAVE);
                        if (wlane / GPW == u)
                            mine = v;
                    }
                    const size_t orow = base + static_cast<size_t>(wlane);
                    if (wlane < GPW * U && orow < rows) {
                        if (ins.kind == DH_PIPE_STORE_ROW)
                            dh_store_stream(static_cast<T *>(io.out_row[ins.index]) + orow * io.ld_out_row[ins.index], mine);
                        else
                            dh_store_stream(static_cast<uint64_t *>(io.out_row[ins.index]) + orow * io.ld_out_row[ins.index],
                                            static_cast<uint64_t>(mine));
                    }
                } else {
                    // fewer than 4 lanes per row: every lane group stores its own results
#pragma unroll
                    for (int u = 0; u < U; u++)
                        if (live[u] && lane == 0) {
                            if (ins.kind == DH_PIPE_STORE_ROW)
                                static_cast<T *>(io.out_row[ins.index])[row[u] * io.ld_out_row[ins.index]] = r[u];
                            else
                                static_cast<uint64_t *>(io.out_row[ins.index])[row[u] * io.ld_out_row[ins.index]] =
                                    static_cast<uint64_t>(r[u]);
                        }
                }
                break;
            }
            default: { // DH_PIPE_REDUCE_ALL
                const int slot = ins.index & 1;
                const int op = ins.op;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    if (ins.domain == 1) {
                        if (live[u] && lane == 0) {
                            if (slot == 0)
                                fold(all_acc0, all_init0, r[u], op);
                            else
                                fold(all_acc1, all_init1, r[u], op);
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                if (live[u] && vmask[j]) {
                                    if (slot == 0)
                                        fold(all_acc0, all_init0, t[(u * KV + j) * VEC + e], op);
                                    else
                                        fold(all_acc1, all_init1, t[(u * KV + j) * VEC + e], op);
                                }
                    }
                }
                break;
            }
            }
        }
    };
    // The first step uses the tile asked for above; the later ones (step k of the wavefront: step k % S of its
    // run k / S) load theirs. Bases grow with k, so the first one past the end ends the walk.
    if (first_base < rows) {
        run_step(first_base, t_first);
#pragma unroll 1
        for (unsigned k = 1;; k++) {
            const size_t base = (wave_id + static_cast<size_t>(k / static_cast<unsigned>(S)) * n_waves) * rows_per_run +
                                static_cast<size_t>(k % static_cast<unsigned>(S)) * rows_per_step;
            if (base >= rows)
                break;
            T t[N];
            load_tile(base, t);
            run_step(base, t);
        }
    }

    // wave-level fold of the REDUCE_ALL slots
    #pragma unroll(PG::is_const ? PG::N : 1)
    for (int ip = 0; ip < (PG::is_const ? PG::N : P.n); ip++) {
        const dh_pipe_instr ins = PG::get(P, ip);
        if (ins.kind != DH_PIPE_REDUCE_ALL)
            continue;
        const int slot = ins.index & 1;
        const int op = ins.op;
        T a = slot == 0 ? all_acc0 : all_acc1;
        if (!(slot == 0 ? all_init0 : all_init1))
            a = (op == DH_AGG_SUM) ? T(0)
                                   : (op == DH_AGG_MIN) ? dh_inf<T>() : -dh_inf<T>();
        dh_butterfly(DH_WAVE, [&](auto peer) {
            const T ov = peer(a);
            a = (op == DH_AGG_SUM) ? a + ov : (op == DH_AGG_MIN) ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
        });
        // one partial per wavefront: no workgroup fold, so a wavefront retires without waiting for the others
        if ((tid % DH_WAVE) == 0)
            all_partials[static_cast<size_t>(slot) * gridDim.x * (THREADS / DH_WAVE) +
                         static_cast<size_t>(blockIdx.x) * (THREADS / DH_WAVE) + tid / DH_WAVE] = a;
    }
    if (any_bad)
        *flag = 1;
}

template <typename T, int VEC, int KV>
__global__ __launch_bounds__(THREADS) void pipeline_kernel(Program P, PipeIO<T> io, size_t rows, size_t cols, int G,
                                                           int S, T *all_partials, int *flag) {
    pipeline_body<T, VEC, KV, RuntimeProgram>(P, io, rows, cols, G, S, all_partials, flag);
}

} // namespace dh_pipe
