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
// Operands: an immediate scalar, t itself, a 1 x cols row vector (staged once in LDS), a
// rows x 1 column vector, another rows x cols matrix, or r broadcast over the row.
// All branches on the instruction stream are uniform across the wavefront; the element loops
// inside each case are fully unrolled over the 16 (float) / 8 (double) values a lane holds.
//
// Scalar semantics per element are those of the stand-alone kernels (ew_impl.h, agg_impl.h),
// i.e. of the reference's CPU kernels.
#pragma once

#include "agg_impl.h"
#include "ew_impl.h"

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

// One instantiation per (value type, vector width, vectors per lane). U rows are in flight per
// lane group so that a lane always holds U*KV*VEC = 16 bytes * 4 of data.
template <typename T, int VEC, int KV>
__global__ __launch_bounds__(THREADS) void pipeline_kernel(Program P, PipeIO<T> io, size_t rows, size_t cols, int G,
                                                           T *all_partials /* [2][gridDim.x] */, int *flag) {
    constexpr int U = 4 / KV;
    constexpr int N = U * KV * VEC;
    extern __shared__ unsigned char lds_raw[];
    T *lds_rv = reinterpret_cast<T *>(lds_raw); // [DH_PIPE_MAX_OPERANDS][cols]
    __shared__ T lds_red[2][THREADS / DH_WAVE];

    const int tid = threadIdx.x;
    const int lane = tid % G;
    const size_t cvecs = cols / VEC;
    for (int v = 0; v < DH_PIPE_MAX_OPERANDS; v++)
        if (io.rowvec[v])
            for (size_t c = tid; c < cols; c += THREADS)
                lds_rv[v * cols + c] = io.rowvec[v][c];
    __syncthreads();

    const size_t groups_per_block = THREADS / G;
    const size_t group = static_cast<size_t>(blockIdx.x) * groups_per_block + tid / G;
    const size_t group_stride = static_cast<size_t>(gridDim.x) * groups_per_block;
    bool vmask[KV];
#pragma unroll
    for (int j = 0; j < KV; j++)
        vmask[j] = static_cast<size_t>(lane + j * G) < cvecs;

    // running values of the (at most two) REDUCE_ALL slots, and which combine they use
    T all_acc0 = T(0), all_acc1 = T(0);
    bool all_init0 = false, all_init1 = false;
    bool any_bad = false;
    auto fold = [](T &a, bool &init, T v, int op) {
        if (!init && op != DH_AGG_SUM)
            a = (op == DH_AGG_MIN) ? std::numeric_limits<T>::infinity() : -std::numeric_limits<T>::infinity();
        init = true;
        a = (op == DH_AGG_SUM) ? a + v : (op == DH_AGG_MIN) ? ((v < a) ? v : a) : ((a < v) ? v : a);
    };

    for (size_t r0 = group; r0 < rows; r0 += group_stride * U) {
        T t[N], o[N], r[U];
        size_t row[U];
        bool live[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            row[u] = r0 + u * group_stride;
            live[u] = row[u] < rows;
            r[u] = T(0);
#pragma unroll
            for (int j = 0; j < KV; j++) {
                T x[VEC];
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    x[e] = T(0);
                if (live[u] && vmask[j])
                    dh_load_vec<T, VEC>(io.x + row[u] * io.ld_x + static_cast<size_t>(lane + j * G) * VEC, x);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    t[(u * KV + j) * VEC + e] = x[e];
            }
        }
        for (int ip = 0; ip < P.n; ip++) {
            const dh_pipe_instr ins = P.ins[ip];
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
                            for (int j = 0; j < KV; j++)
#pragma unroll
                                for (int e = 0; e < VEC; e++)
                                    o[(u * KV + j) * VEC + e] =
                                        vmask[j] ? lds_rv[ins.index * cols + static_cast<size_t>(lane + j * G) * VEC + e] : T(0);
                        break;
                    case DH_OPD_COLVEC:
#pragma unroll
                        for (int u = 0; u < U; u++) {
                            const T s = live[u] ? io.colvec[ins.index][row[u] * io.ld_colvec[ins.index]] : T(0);
#pragma unroll
                            for (int i = 0; i < KV * VEC; i++)
                                o[u * KV * VEC + i] = s;
                        }
                        break;
                    case DH_OPD_MATRIX:
#pragma unroll
                        for (int u = 0; u < U; u++)
#pragma unroll
                            for (int j = 0; j < KV; j++) {
                                T x[VEC];
#pragma unroll
                                for (int e = 0; e < VEC; e++)
                                    x[e] = T(0);
                                if (live[u] && vmask[j])
                                    dh_load_vec<T, VEC>(io.matrix[ins.index] + row[u] * io.ld_matrix[ins.index] +
                                                            static_cast<size_t>(lane + j * G) * VEC,
                                                        x);
#pragma unroll
                                for (int e = 0; e < VEC; e++)
                                    o[(u * KV + j) * VEC + e] = x[e];
                            }
                        break;
                    default: // DH_OPD_ROWREG
#pragma unroll
                        for (int u = 0; u < U; u++)
#pragma unroll
                            for (int i = 0; i < KV * VEC; i++)
                                o[u * KV * VEC + i] = r[u];
                        break;
                    }
                    apply_binary<T, N>(ins.op, t, o, ins.swap != 0);
                } else {
                    T ov[U];
#pragma unroll
                    for (int u = 0; u < U; u++) {
                        if (ins.operand == DH_OPD_COLVEC)
                            ov[u] = live[u] ? io.colvec[ins.index][row[u] * io.ld_colvec[ins.index]] : T(0);
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
                        T best = is_min ? std::numeric_limits<T>::infinity() : -std::numeric_limits<T>::infinity();
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
                        for (int off = G / 2; off >= 1; off >>= 1) {
                            const T ov = dh_shfl_xor(best, off);
                            const unsigned oi = dh_shfl_xor(bi, off);
                            const bool better = is_min ? (ov < best) : (ov > best);
                            if (better || (ov == best && oi < bi)) {
                                best = ov;
                                bi = oi;
                            }
                        }
                        if ((first != first) || bi == ~0u)
                            bi = 0;
                        r[u] = static_cast<T>(bi);
                    } else if (op == DH_AGG_MIN || op == DH_AGG_MAX) {
                        const bool is_min = (op == DH_AGG_MIN);
                        T a = is_min ? std::numeric_limits<T>::infinity() : -std::numeric_limits<T>::infinity();
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++) {
                                const T x = t[(u * KV + j) * VEC + e];
                                if (vmask[j])
                                    a = is_min ? ((x < a) ? x : a) : ((a < x) ? x : a);
                            }
                        for (int off = G / 2; off >= 1; off >>= 1) {
                            const T ov = dh_shfl_xor(a, off);
                            a = is_min ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
                        }
                        r[u] = (first != first) ? first : a;
                    } else if (op == DH_AGG_PROD) {
                        T a = T(1);
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                if (vmask[j])
                                    a = a * t[(u * KV + j) * VEC + e];
                        for (int off = G / 2; off >= 1; off >>= 1)
                            a = a * dh_shfl_xor(a, off);
                        r[u] = a;
                    } else { // SUM MEAN VAR STDDEV
                        T a = T(0);
#pragma unroll
                        for (int j = 0; j < KV; j++)
#pragma unroll
                            for (int e = 0; e < VEC; e++)
                                if (vmask[j])
                                    a = a + t[(u * KV + j) * VEC + e];
                        for (int off = G / 2; off >= 1; off >>= 1)
                            a = a + dh_shfl_xor(a, off);
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
                            for (int off = G / 2; off >= 1; off >>= 1)
                                s = s + dh_shfl_xor(s, off);
                            s = s / static_cast<T>(cols);
                            a = (op == DH_AGG_STDDEV) ? dh_agg::dev_sqrt<T>(s) : s;
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
#pragma unroll
                for (int u = 0; u < U; u++)
                    if (live[u] && lane == 0)
                        static_cast<T *>(io.out_row[ins.index])[row[u] * io.ld_out_row[ins.index]] = r[u];
                break;
            case DH_PIPE_STORE_ROW_IDX:
#pragma unroll
                for (int u = 0; u < U; u++)
                    if (live[u] && lane == 0)
                        static_cast<uint64_t *>(io.out_row[ins.index])[row[u] * io.ld_out_row[ins.index]] =
                            static_cast<uint64_t>(r[u]);
                break;
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
    }

    // block-level fold of the REDUCE_ALL slots
    for (int ip = 0; ip < P.n; ip++) {
        const dh_pipe_instr ins = P.ins[ip];
        if (ins.kind != DH_PIPE_REDUCE_ALL)
            continue;
        const int slot = ins.index & 1;
        const int op = ins.op;
        T a = slot == 0 ? all_acc0 : all_acc1;
        if (!(slot == 0 ? all_init0 : all_init1))
            a = (op == DH_AGG_SUM) ? T(0)
                                   : (op == DH_AGG_MIN) ? std::numeric_limits<T>::infinity() : -std::numeric_limits<T>::infinity();
        for (int off = DH_WAVE / 2; off >= 1; off >>= 1) {
            const T ov = dh_shfl_xor(a, off);
            a = (op == DH_AGG_SUM) ? a + ov : (op == DH_AGG_MIN) ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
        }
        if ((tid % DH_WAVE) == 0)
            lds_red[slot][tid / DH_WAVE] = a;
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < THREADS / DH_WAVE; w++) {
                const T ov = lds_red[slot][w];
                a = (op == DH_AGG_SUM) ? a + ov : (op == DH_AGG_MIN) ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
            }
            all_partials[static_cast<size_t>(slot) * gridDim.x + blockIdx.x] = a;
        }
        __syncthreads();
    }
    if (any_bad)
        *flag = 1;
}

template <typename T>
__global__ __launch_bounds__(THREADS) void pipeline_all_stage2(const T *partials, size_t np, int op, T *out) {
    __shared__ T lds[THREADS / DH_WAVE];
    T a = (op == DH_AGG_SUM) ? T(0)
                             : (op == DH_AGG_MIN) ? std::numeric_limits<T>::infinity() : -std::numeric_limits<T>::infinity();
    for (size_t i = threadIdx.x; i < np; i += THREADS) {
        const T v = partials[i];
        a = (op == DH_AGG_SUM) ? a + v : (op == DH_AGG_MIN) ? ((v < a) ? v : a) : ((a < v) ? v : a);
    }
    for (int off = DH_WAVE / 2; off >= 1; off >>= 1) {
        const T ov = dh_shfl_xor(a, off);
        a = (op == DH_AGG_SUM) ? a + ov : (op == DH_AGG_MIN) ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
    }
    if ((threadIdx.x % DH_WAVE) == 0)
        lds[threadIdx.x / DH_WAVE] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < THREADS / DH_WAVE; w++) {
            const T ov = lds[w];
            a = (op == DH_AGG_SUM) ? a + ov : (op == DH_AGG_MIN) ? ((ov < a) ? ov : a) : ((a < ov) ? ov : a);
        }
        out[0] = a;
    }
}

static __global__ void pipe_clear_flag(int *flag) { *flag = 0; }

template <typename T, typename IO_C>
dh_status run(dh_ctx *ctx, const dh_pipe_instr *prog, int n, const IO_C *cio, size_t rows, size_t cols) {
    DH_REQUIRE_CTX(ctx);
    if (prog == nullptr || cio == nullptr)
        return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: program or io is null");
    if (n < 0 || n > DH_PIPE_MAX_INSTR)
        return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: %d instructions, at most %d are supported", n, DH_PIPE_MAX_INSTR);
    if (rows == 0 || cols == 0)
        return DH_OK;
    Program P{};
    P.n = n;
    PipeIO<T> io{};
    io.x = cio->x;
    io.ld_x = cio->ld_x;
    if (io.x == nullptr || io.ld_x < cols)
        return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: the primary input is null or its leading dimension is too small");
    for (int i = 0; i < DH_PIPE_MAX_OPERANDS; i++) {
        io.matrix[i] = cio->matrix[i];
        io.ld_matrix[i] = cio->ld_matrix[i];
        io.rowvec[i] = cio->rowvec[i];
        io.colvec[i] = cio->colvec[i];
        io.ld_colvec[i] = cio->ld_colvec[i];
        io.out_tile[i] = cio->out_tile[i];
        io.ld_out_tile[i] = cio->ld_out_tile[i];
        io.out_row[i] = cio->out_row[i];
        io.ld_out_row[i] = cio->ld_out_row[i];
    }
    constexpr int V = 16 / sizeof(T);
    bool vec_ok = (cols % V == 0) && (io.ld_x % V == 0) && dh_aligned(io.x, 16);
    bool checks = false;
    int reduce_ops[2] = {-1, -1};
    T *reduce_out[2] = {nullptr, nullptr};
    for (int i = 0; i < n; i++) {
        const dh_pipe_instr &in = prog[i];
        P.ins[i] = in;
        const int idx = in.index;
        auto bad_index = [&]() { return idx < 0 || idx >= DH_PIPE_MAX_OPERANDS; };
        switch (in.kind) {
        case DH_PIPE_EW_BINARY:
            if (in.op < DH_BIN_ADD || in.op > DH_BIN_OR)
                return dh_fail(DH_ERR_RUNTIME, "unknown BinaryOpCode: %d", in.op);
            switch (in.operand) {
            case DH_OPD_SCALAR:
            case DH_OPD_SELF:
                break;
            case DH_OPD_ROWREG:
                if (in.domain != 0)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: ROWREG operand needs the tile domain", i);
                break;
            case DH_OPD_ROWVEC:
                if (in.domain != 0 || bad_index() || io.rowvec[idx] == nullptr)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: row-vector operand %d is not bound", i, idx);
                break;
            case DH_OPD_COLVEC:
                if (bad_index() || io.colvec[idx] == nullptr || io.ld_colvec[idx] < 1)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: column-vector operand %d is not bound", i, idx);
                break;
            case DH_OPD_MATRIX:
                if (in.domain != 0 || bad_index() || io.matrix[idx] == nullptr || io.ld_matrix[idx] < cols)
                    return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: matrix operand %d is not bound", i, idx);
                vec_ok = vec_ok && (io.ld_matrix[idx] % V == 0) && dh_aligned(io.matrix[idx], 16);
                break;
            default:
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: unknown operand kind %d", i, in.operand);
            }
            break;
        case DH_PIPE_EW_UNARY:
            if (in.op < DH_UN_MINUS || in.op > DH_UN_ISNAN)
                return dh_fail(DH_ERR_RUNTIME, "unknown UnaryOpCode: %d", in.op);
            checks |= (in.op == DH_UN_SQRT || in.op == DH_UN_LN || in.op == DH_UN_ASIN || in.op == DH_UN_ACOS);
            break;
        case DH_PIPE_ROW_AGG:
            if (in.op < DH_AGG_SUM || in.op > DH_AGG_VAR)
                return dh_fail(DH_ERR_RUNTIME, "unsupported AggOpCode");
            break;
        case DH_PIPE_STORE_TILE:
            if (bad_index() || io.out_tile[idx] == nullptr || io.ld_out_tile[idx] < cols)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: tile output %d is not bound", i, idx);
            vec_ok = vec_ok && (io.ld_out_tile[idx] % V == 0) && dh_aligned(io.out_tile[idx], 16);
            break;
        case DH_PIPE_STORE_ROW:
        case DH_PIPE_STORE_ROW_IDX:
            if (bad_index() || io.out_row[idx] == nullptr || io.ld_out_row[idx] < 1)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: row output %d is not bound", i, idx);
            break;
        case DH_PIPE_REDUCE_ALL:
            // the combines a vectorized pipeline knows: ADD MIN MAX
            // (ir/daphneir/DaphneVectorizableOpInterface.cpp:306-311)
            if (in.op != DH_AGG_SUM && in.op != DH_AGG_MIN && in.op != DH_AGG_MAX)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: REDUCE_ALL supports SUM, MIN and MAX");
            if (idx < 0 || idx > 1 || cio->out_all[idx] == nullptr)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: scalar output %d is not bound", i, idx);
            if (reduce_ops[idx] != -1)
                return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: scalar output %d is reduced twice", idx);
            reduce_ops[idx] = in.op;
            reduce_out[idx] = cio->out_all[idx];
            break;
        default:
            return dh_fail(DH_ERR_RUNTIME, "vectorizedPipeline: instruction %d: unknown kind %d", i, in.kind);
        }
    }
    const int vec = vec_ok ? V : 1;
    const size_t cvecs = cols / vec;
    int G = 1;
    while (G < DH_WAVE && static_cast<size_t>(G) < cvecs)
        G <<= 1;
    const size_t per_lane = dh_ceil_div(cvecs, G);
    if (per_lane > 4)
        return dh_fail(DH_ERR_RUNTIME,
                       "vectorizedPipeline: rows of %zu values do not fit the register tile (at most %d per row here); "
                       "run the operators one by one instead",
                       cols, 64 * vec * 4);
    const int KV = per_lane <= 1 ? 1 : (per_lane <= 2 ? 2 : 4);
    const int U = 4 / KV;
    const size_t groups_per_block = THREADS / G;
    size_t grid = dh_ceil_div(rows, groups_per_block * U);
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 16;
    if (grid > cap)
        grid = cap;
    void *wsv = nullptr;
    dh_status st = dh_workspace(ctx, 2 * grid * sizeof(T) + 256, &wsv);
    if (st != DH_OK)
        return st;
    T *partials = static_cast<T *>(wsv);
    if (checks)
        hipLaunchKernelGGL(pipe_clear_flag, dim3(1), dim3(1), 0, ctx->stream, ctx->flag_dev);
    const size_t lds = static_cast<size_t>(DH_PIPE_MAX_OPERANDS) * cols * sizeof(T);
    const dim3 g(static_cast<unsigned>(grid)), b(THREADS);
#define DH_LAUNCH(VEC_, KV_)                                                                       \
    hipLaunchKernelGGL((pipeline_kernel<T, VEC_, KV_>), g, b, lds, ctx->stream, P, io, rows, cols, G, partials,      \
                       ctx->flag_dev)
    if (vec_ok) {
        if (KV == 1)
            DH_LAUNCH(V, 1);
        else if (KV == 2)
            DH_LAUNCH(V, 2);
        else
            DH_LAUNCH(V, 4);
    } else {
        if (KV == 1)
            DH_LAUNCH(1, 1);
        else if (KV == 2)
            DH_LAUNCH(1, 2);
        else
            DH_LAUNCH(1, 4);
    }
#undef DH_LAUNCH
    DH_CHECK_LAUNCH();
    for (int s = 0; s < 2; s++)
        if (reduce_ops[s] != -1) {
            hipLaunchKernelGGL((pipeline_all_stage2<T>), dim3(1), dim3(THREADS), 0, ctx->stream, partials + s * grid, grid,
                               reduce_ops[s], reduce_out[s]);
            DH_CHECK_LAUNCH();
        }
    if (checks) {
        DH_CHECK_HIP(hipMemcpyAsync(ctx->flag_host, ctx->flag_dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        DH_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        if (*ctx->flag_host != 0)
            return dh_fail(DH_ERR_DOMAIN, "invalid argument passed to a unary function inside the pipeline");
    }
    return DH_OK;
}

} // namespace dh_pipe
