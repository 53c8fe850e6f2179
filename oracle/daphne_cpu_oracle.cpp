// TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
//
// CPU restatement of the reference's (daphne-eu/daphne) CPU kernels for DenseMatrix<float|double>
// on raw row-major pointers. It is the checker the HIP kernels are compared against. Only the
// tests, the smoke check and the cpu_baseline leg of the benchmark may load this library; the
// product never does.
//
// Every function follows the loop order and quirks of the reference file it cites (paths
// relative to the reference's src/runtime/local/kernels/). The BLAS/LAPACK-backed kernels
// (MatMul, Syrk, Solve call OpenBLAS 0.3.23 / LAPACKE, which are not part of the reference
// checkout) are restated from the published definitions of ?gemm / ?syrk / ?gesv.
//
// How each function is pinned is listed in oracle/README.md; in short: the reference's own
// unit-test vectors (tests/golden/*.json), closed forms, and independent numpy / float128
// evaluations in tests/test_oracle_*.py.
//
// Status codes returned by the functions: 0 ok, 1 std::runtime_error, 2 std::invalid_argument,
// 3 std::domain_error, 6 std::out_of_range - the exception the reference would have thrown.
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

namespace {

enum { ST_OK = 0, ST_RUNTIME = 1, ST_INVALID = 2, ST_DOMAIN = 3 };

// ---------------------------------------------------------------------------------------
// scalar ops: EwBinarySca.h:143-167, reached through a function pointer per element exactly
// like EwBinaryMat.h:70 (getEwBinaryScaFuncPtr) - this is what makes the reference slow and
// is kept so that the timed baseline is the reference's algorithm.
// ---------------------------------------------------------------------------------------
template <typename T> using BinFn = T (*)(T, T);

template <typename T> T b_add(T l, T r) { return l + r; }
template <typename T> T b_sub(T l, T r) { return l - r; }
template <typename T> T b_mul(T l, T r) { return l * r; }
template <typename T> T b_div(T l, T r) { return l / r; }
template <typename T> T b_pow(T l, T r) { return std::pow(l, r); }
template <typename T> T b_mod(T l, T r) { return std::fmod(l, r); }
template <typename T> T b_log(T l, T r) { return std::log(l) / std::log(r); }
template <typename T> T b_eq(T l, T r) { return l == r; }
template <typename T> T b_neq(T l, T r) { return l != r; }
template <typename T> T b_lt(T l, T r) { return l < r; }
template <typename T> T b_le(T l, T r) { return l <= r; }
template <typename T> T b_gt(T l, T r) { return l > r; }
template <typename T> T b_ge(T l, T r) { return l >= r; }
template <typename T> T b_min(T l, T r) { return std::min(l, r); }
template <typename T> T b_max(T l, T r) { return std::max(l, r); }
template <typename T> T b_and(T l, T r) { return l && r; }
template <typename T> T b_or(T l, T r) { return l || r; }

// BinaryOpCode.h:29-55 order. Returns nullptr for ops unsupported on floating point
// (BITWISE_AND, CONCAT: BinaryOpCode.h:178-180) and sets *unknown for codes outside the enum.
template <typename T> BinFn<T> bin_fn(int op, bool *unknown) {
    *unknown = false;
    switch (op) {
    case 0: return b_add<T>;
    case 1: return b_sub<T>;
    case 2: return b_mul<T>;
    case 3: return b_div<T>;
    case 4: return b_pow<T>;
    case 5: return b_mod<T>;
    case 6: return b_log<T>;
    case 7: return b_eq<T>;
    case 8: return b_neq<T>;
    case 9: return b_lt<T>;
    case 10: return b_le<T>;
    case 11: return b_gt<T>;
    case 12: return b_ge<T>;
    case 13: return b_min<T>;
    case 14: return b_max<T>;
    case 15: return b_and<T>;
    case 16: return b_or<T>;
    case 17:
    case 18: return nullptr;
    default: *unknown = true; return nullptr;
    }
}

// Integer DIV by zero (and INT_MIN / -1) is a hardware trap in the reference's process, and MOD by zero converts
// a NaN to an integer (undefined): both are reported as a domain error here, with 0 stored, instead of being executed.
template <typename T> struct SafeBin {
    BinFn<T> f;
    int op;
    bool bad = false;
    T operator()(T l, T r) {
        if constexpr (std::numeric_limits<T>::is_integer) {
            const bool div_traps = r == T(0) || (std::numeric_limits<T>::is_signed && r == T(-1) &&
                                                 l == std::numeric_limits<T>::min());
            if ((op == 3 && div_traps) || (op == 5 && r == T(0))) {
                bad = true;
                return T(0);
            }
        }
        return f(l, r);
    }
};

// EwBinaryMat.h:54-108
template <typename T>
int ew_binary(int op, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs, const T *rhs,
              size_t rr, size_t rc, size_t ld_rhs) {
    bool unknown;
    BinFn<T> fp = bin_fn<T>(op, &unknown);
    if (!fp)
        return ST_RUNTIME;
    SafeBin<T> f{fp, op};
    if (lr == rr && lc == rc) {
        for (size_t r = 0; r < lr; r++) {
            for (size_t c = 0; c < lc; c++)
                res[c] = f(lhs[c], rhs[c]);
            lhs += ld_lhs;
            rhs += ld_rhs;
            res += ld_res;
        }
    } else if (lc == rc && (rr == 1 || lr == 1)) {
        for (size_t r = 0; r < lr; r++) {
            for (size_t c = 0; c < lc; c++)
                res[c] = f(lhs[c], rhs[c]);
            lhs += ld_lhs;
            res += ld_res;
        }
    } else if (lr == rr && (rc == 1 || lc == 1)) {
        for (size_t r = 0; r < lr; r++) {
            for (size_t c = 0; c < lc; c++)
                res[c] = f(lhs[c], rhs[0]);
            lhs += ld_lhs;
            rhs += ld_rhs;
            res += ld_res;
        }
    } else
        return ST_RUNTIME;
    return f.bad ? ST_DOMAIN : ST_OK;
}

// EwBinaryObjSca.h:57-79
template <typename T>
int ew_binary_sca(int op, T *res, size_t ld_res, const T *lhs, size_t rows, size_t cols, size_t ld_lhs, T rhs) {
    bool unknown;
    BinFn<T> fp = bin_fn<T>(op, &unknown);
    if (!fp)
        return ST_RUNTIME;
    SafeBin<T> f{fp, op};
    for (size_t r = 0; r < rows; r++) {
        for (size_t c = 0; c < cols; c++)
            res[c] = f(lhs[c], rhs);
        lhs += ld_lhs;
        res += ld_res;
    }
    return f.bad ? ST_DOMAIN : ST_OK;
}

// EwUnarySca.h:182-206 (+ domain checks :129-157); UnaryOpCode.h:28-55 order.
template <typename T> using UnFn = T (*)(T, bool *);
template <typename T> T u_minus(T a, bool *) { return -a; }
template <typename T> T u_abs(T a, bool *) { return std::abs(a); }
template <typename T> T u_sign(T a, bool *) {
    return (a == 0) ? T(0) : ((a < 0) ? T(-1) : ((a > 0) ? T(1) : std::numeric_limits<T>::quiet_NaN()));
}
template <typename T> T u_sqrt(T a, bool *bad) {
    if (-0.0 > a)
        *bad = true;
    return std::sqrt(a);
}
template <typename T> T u_exp(T a, bool *) { return std::exp(a); }
template <typename T> T u_ln(T a, bool *bad) {
    if (-0.0 > a)
        *bad = true;
    return std::log(a);
}
template <typename T> T u_sin(T a, bool *) { return std::sin(a); }
template <typename T> T u_cos(T a, bool *) { return std::cos(a); }
template <typename T> T u_tan(T a, bool *) { return std::tan(a); }
template <typename T> T u_asin(T a, bool *bad) {
    if (-1.0 > a || a > 1.0)
        *bad = true;
    return std::asin(a);
}
template <typename T> T u_acos(T a, bool *bad) {
    if (-1.0 > a || a > 1.0)
        *bad = true;
    return std::acos(a);
}
template <typename T> T u_atan(T a, bool *) { return std::atan(a); }
template <typename T> T u_sinh(T a, bool *) { return std::sinh(a); }
template <typename T> T u_cosh(T a, bool *) { return std::cosh(a); }
template <typename T> T u_tanh(T a, bool *) { return std::tanh(a); }
template <typename T> T u_floor(T a, bool *) { return std::floor(a); }
template <typename T> T u_ceil(T a, bool *) { return std::ceil(a); }
template <typename T> T u_round(T a, bool *) { return std::round(a); }
template <typename T> T u_isnan(T a, bool *) { return std::isnan(a); }

template <typename T> UnFn<T> un_fn(int op) {
    static const UnFn<T> table[19] = {u_minus<T>, u_abs<T>,  u_sign<T>, u_sqrt<T>, u_exp<T>,  u_ln<T>,   u_sin<T>,
                                      u_cos<T>,   u_tan<T>,  u_asin<T>, u_acos<T>, u_atan<T>, u_sinh<T>, u_cosh<T>,
                                      u_tanh<T>,  u_floor<T>, u_ceil<T>, u_round<T>, u_isnan<T>};
    if (op < 0 || op >= 19)
        return nullptr;
    return table[op];
}

// EwUnaryMat.h:57-77. The reference throws at the first offending element; here the whole
// result is still produced (NaN at those positions) and ST_DOMAIN is returned.
template <typename T> int ew_unary(int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld_arg) {
    UnFn<T> f = un_fn<T>(op);
    if (!f)
        return ST_RUNTIME;
    bool bad = false;
    for (size_t r = 0; r < rows; r++) {
        for (size_t c = 0; c < cols; c++)
            res[c] = f(arg[c], &bad);
        arg += ld_arg;
        res += ld_res;
    }
    return bad ? ST_DOMAIN : ST_OK;
}

// ---------------------------------------------------------------------------------------
// aggregations
// ---------------------------------------------------------------------------------------
enum { A_SUM = 0, A_PROD = 1, A_MIN = 2, A_MAX = 3, A_IDXMIN = 4, A_IDXMAX = 5, A_MEAN = 6, A_STDDEV = 7, A_VAR = 8 };

template <typename T> bool agg_pure(int op) { return op == A_SUM || op == A_PROD || op == A_MIN || op == A_MAX; }
template <typename T> BinFn<T> agg_fn(int op) {
    switch (op) {
    case A_SUM: return b_add<T>;
    case A_PROD: return b_mul<T>;
    case A_MIN: return b_min<T>;
    case A_MAX: return b_max<T>;
    default: return b_add<T>; // MEAN / VAR / STDDEV sum first (AggRow.h:99-104)
    }
}
// AggOpCode.h:69-89
template <typename T> T agg_neutral(int op) {
    switch (op) {
    case A_SUM: return T(0);
    case A_PROD: return T(1);
    case A_MIN: return std::numeric_limits<T>::has_infinity ? std::numeric_limits<T>::infinity() : std::numeric_limits<T>::max();
    case A_MAX: return std::numeric_limits<T>::has_infinity ? -std::numeric_limits<T>::infinity() : std::numeric_limits<T>::min();
    default: return T(0);
    }
}

// AggAll.h:64-96: four interleaved accumulators, then (a0+a1)+(a2+a3), then the tail.
template <typename T> T agg_all_array(BinFn<T> f, const T *v, size_t n, T neutral) {
    T agg;
    if (n) {
        T a0 = neutral, a1 = neutral, a2 = neutral, a3 = neutral;
        for (size_t i = 0; i < n / 4 * 4; i += 4) {
            a0 = f(a0, v[i]);
            a1 = f(a1, v[i + 1]);
            a2 = f(a2, v[i + 2]);
            a3 = f(a3, v[i + 3]);
        }
        agg = f(f(a0, a1), f(a2, a3));
        for (size_t i = 0; i < n % 4; i++)
            agg = f(agg, v[n / 4 * 4 + i]);
    } else
        agg = neutral;
    return agg;
}

// AggAll.h:124-193
template <typename T> int agg_all(int op, const T *arg, size_t rows, size_t cols, size_t ld, T *out) {
    if (op == A_IDXMIN || op == A_IDXMAX || op < 0 || op > A_VAR)
        return ST_RUNTIME;
    BinFn<T> f = agg_fn<T>(op);
    T neutral = agg_pure<T>(op) ? agg_neutral<T>(op) : T(0);
    T agg;
    const T *v = arg;
    if (cols == ld || rows == 1)
        agg = agg_all_array<T>(f, v, rows * cols, neutral);
    else {
        agg = neutral;
        for (size_t r = 0; r < rows; r++) {
            agg = f(agg, agg_all_array<T>(f, v, cols, neutral));
            v += ld;
        }
    }
    if (agg_pure<T>(op)) {
        *out = agg;
        return ST_OK;
    }
    agg /= cols * rows;
    if (op == A_MEAN) {
        *out = agg;
        return ST_OK;
    }
    T stddev = 0;
    v = arg;
    for (size_t r = 0; r < rows; r++) {
        for (size_t c = 0; c < cols; c++) {
            T val = v[c] - agg;
            stddev = stddev + val * val;
        }
        v += ld;
    }
    stddev /= cols * rows;
    *out = (op == A_VAR) ? stddev : std::sqrt(stddev);
    return ST_OK;
}

// AggRow.h:96-160
template <typename T> int agg_row(int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    if (op == A_IDXMIN || op == A_IDXMAX || op < 0 || op > A_VAR)
        return ST_RUNTIME;
    BinFn<T> f = agg_fn<T>(op);
    const T *v = arg;
    T *o = res;
    for (size_t r = 0; r < rows; r++) {
        T agg = *v;
        for (size_t c = 1; c < cols; c++)
            agg = f(agg, v[c]);
        *o = agg;
        v += ld;
        o += ld_res;
    }
    if (agg_pure<T>(op))
        return ST_OK;
    o = res;
    for (size_t r = 0; r < rows; r++) {
        *o = (*o) / cols;
        o += ld_res;
    }
    if (op == A_MEAN)
        return ST_OK;
    std::vector<T> tmp(rows, T(0));
    v = arg;
    o = res;
    for (size_t r = 0; r < rows; r++) {
        for (size_t c = 0; c < cols; c++) {
            T val = v[c] - (*o);
            tmp[r] = tmp[r] + val * val;
        }
        v += ld;
        o += ld_res;
    }
    o = res;
    for (size_t r = 0; r < rows; r++) {
        tmp[r] /= cols;
        *o = (op == A_STDDEV) ? std::sqrt(tmp[r]) : tmp[r];
        o += ld_res;
    }
    return ST_OK;
}

// AggRow.h:71-94
template <typename T>
int agg_row_idx(int op, uint64_t *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    if (op != A_IDXMIN && op != A_IDXMAX)
        return ST_RUNTIME;
    const T *v = arg;
    for (size_t r = 0; r < rows; r++) {
        T best = v[0];
        size_t idx = 0;
        for (size_t c = 1; c < cols; c++)
            if (op == A_IDXMIN ? (v[c] < best) : (v[c] > best)) {
                best = v[c];
                idx = c;
            }
        *res = static_cast<uint64_t>(idx);
        v += ld;
        res += ld_res;
    }
    return ST_OK;
}

// AggCol.h:123-177
template <typename T> int agg_col(int op, T *res, const T *arg, size_t rows, size_t cols, size_t ld) {
    if (op == A_IDXMIN || op == A_IDXMAX || op < 0 || op > A_VAR)
        return ST_RUNTIME;
    BinFn<T> f = agg_fn<T>(op);
    const T *v = arg;
    for (size_t c = 0; c < cols; c++)
        res[c] = v[c];
    for (size_t r = 1; r < rows; r++) {
        v += ld;
        for (size_t c = 0; c < cols; c++)
            res[c] = f(res[c], v[c]);
    }
    if (agg_pure<T>(op))
        return ST_OK;
    for (size_t c = 0; c < cols; c++)
        res[c] /= rows;
    if (op == A_MEAN)
        return ST_OK;
    std::vector<T> tmp(cols, T(0));
    v = arg;
    for (size_t r = 0; r < rows; r++) {
        for (size_t c = 0; c < cols; c++) {
            T val = v[c] - res[c];
            tmp[c] = tmp[c] + val * val;
        }
        v += ld;
    }
    for (size_t c = 0; c < cols; c++) {
        tmp[c] /= rows;
        if (op == A_STDDEV)
            tmp[c] = std::sqrt(tmp[c]);
    }
    std::memcpy(res, tmp.data(), cols * sizeof(T));
    return ST_OK;
}

// AggCol.h:70-122
template <typename T> int agg_col_idx(int op, uint64_t *res, const T *arg, size_t rows, size_t cols, size_t ld) {
    if (op != A_IDXMIN && op != A_IDXMAX)
        return ST_RUNTIME;
    std::vector<T> tmp(arg, arg + cols);
    for (size_t c = 0; c < cols; c++)
        res[c] = 0;
    const T *v = arg + ld;
    for (size_t r = 1; r < rows; r++) {
        for (size_t c = 0; c < cols; c++)
            if (op == A_IDXMIN ? (v[c] < tmp[c]) : (v[c] > tmp[c])) {
                tmp[c] = v[c];
                res[c] = r;
            }
        v += ld;
    }
    return ST_OK;
}

// ---------------------------------------------------------------------------------------
// contractions (OpenBLAS 0.3.23 cblas_?gemm / ?gemv / ?dot / ?syrk in the reference:
// MatMul.cpp:248-290, Syrk.h:51-93). Restated from the BLAS definitions. Like a blocked BLAS
// the inner dimension is accumulated in slabs of 256 and the slab sums are added to the
// result, all in the value type T.
// ---------------------------------------------------------------------------------------
template <typename T>
void gemm_def(bool ta, bool tb, size_t m, size_t n, size_t k, const T *A, size_t lda, const T *B, size_t ldb, T *C,
              size_t ldc) {
    const size_t KB = 256;
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            T total = 0;
            for (size_t k0 = 0; k0 < k; k0 += KB) {
                T s = 0;
                const size_t k1 = std::min(k, k0 + KB);
                for (size_t kk = k0; kk < k1; kk++) {
                    const T a = ta ? A[kk * lda + i] : A[i * lda + kk];
                    const T b = tb ? B[j * ldb + kk] : B[kk * ldb + j];
                    s += a * b;
                }
                total += s;
            }
            C[i * ldc + j] = total;
        }
}

// MatMul.cpp:248-290: shape check, then dot / gemv / gemm; mathematically all three are
// res = op(lhs) op(rhs).
template <typename T>
int matmul(T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs, const T *rhs, size_t rr, size_t rc,
           size_t ld_rhs, int ta, int tb) {
    const size_t nr1 = ta ? lc : lr, nc1 = ta ? lr : lc;
    const size_t nr2 = tb ? rc : rr, nc2 = tb ? rr : rc;
    if (nc1 != nr2)
        return ST_RUNTIME;
    gemm_def<T>(ta, tb, nr1, nc2, nc1, lhs, ld_lhs, rhs, ld_rhs, res, ld_res);
    return ST_OK;
}

// Syrk.h:51-93: upper triangle by ?syrk, then mirrored to the lower one.
template <typename T> int syrk(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld, int trans_left) {
    const size_t n = trans_left ? cols : rows;
    const size_t k = trans_left ? rows : cols;
    const size_t KB = 256;
    for (size_t i = 0; i < n; i++)
        for (size_t j = i; j < n; j++) {
            T total = 0;
            for (size_t k0 = 0; k0 < k; k0 += KB) {
                T s = 0;
                const size_t k1 = std::min(k, k0 + KB);
                for (size_t kk = k0; kk < k1; kk++) {
                    const T a = trans_left ? arg[kk * ld + i] : arg[i * ld + kk];
                    const T b = trans_left ? arg[kk * ld + j] : arg[j * ld + kk];
                    s += a * b;
                }
                total += s;
            }
            res[i * ld_res + j] = total;
        }
    for (size_t r = 0; r < n; r++)
        for (size_t c = r + 1; c < n; c++)
            res[c * ld_res + r] = res[r * ld_res + c];
    return ST_OK;
}

// Solve.h:86-116 -> LAPACKE_?gesv: LU with partial pivoting (row interchanges), then forward
// and back substitution. Returns ST_RUNTIME for an exactly singular factor (info > 0).
template <typename T> int solve(T *x, const T *A, size_t n, const T *b) {
    std::vector<T> lu(A, A + n * n);
    for (size_t i = 0; i < n; i++)
        x[i] = b[i];
    for (size_t j = 0; j < n; j++) {
        size_t p = j;
        T best = std::abs(lu[j * n + j]);
        for (size_t i = j + 1; i < n; i++)
            if (std::abs(lu[i * n + j]) > best) {
                best = std::abs(lu[i * n + j]);
                p = i;
            }
        if (lu[p * n + j] == T(0))
            return ST_RUNTIME;
        if (p != j) {
            for (size_t c = 0; c < n; c++)
                std::swap(lu[p * n + c], lu[j * n + c]);
            std::swap(x[p], x[j]);
        }
        const T inv = T(1) / lu[j * n + j];
        for (size_t i = j + 1; i < n; i++) {
            const T l = lu[i * n + j] * inv;
            lu[i * n + j] = l;
            for (size_t c = j + 1; c < n; c++)
                lu[i * n + c] -= l * lu[j * n + c];
            x[i] -= l * x[j];
        }
    }
    for (size_t ii = n; ii-- > 0;) {
        T s = x[ii];
        for (size_t c = ii + 1; c < n; c++)
            s -= lu[ii * n + c] * x[c];
        x[ii] = s / lu[ii * n + ii];
    }
    return ST_OK;
}

// ---------------------------------------------------------------------------------------
// DNN ops
// ---------------------------------------------------------------------------------------
// Padding.h:6-9
uint32_t get_pq(uint32_t img, uint32_t filt, uint32_t pad, uint32_t stride) { return (img + 2 * pad - filt) / stride + 1; }

// Conv2DForward.h:77-140 (+ Padding.h:11-22). Same loop nest and accumulation order (per output:
// channels outermost, then filter rows, then filter columns, into a zero-initialised result;
// bias added last). bias == nullptr skips the bias (the reference's CUDA kernel allows that;
// its CPU kernel would dereference null).
template <typename T>
int conv2d(T *res, size_t *res_h, size_t *res_w, const T *data, const T *filter, const T *bias, size_t N, size_t C,
           size_t H, size_t W, size_t F, size_t Hf, size_t Wf, size_t sh, size_t sw, size_t ph, size_t pw) {
    if (H + 2 * ph < Hf || W + 2 * pw < Wf || sh == 0 || sw == 0)
        return ST_INVALID;
    const size_t HW = H * W, CHW = C * HW;
    const size_t P = get_pq(H, Hf, ph, sh), Q = get_pq(W, Wf, pw, sw);
    const size_t PQ = P * Q, CPQ = F * PQ;
    *res_h = P;
    *res_w = Q;
    const size_t pH = H + 2 * ph, pW = W + 2 * pw;
    std::vector<T> padded(pH * pW, T(0));
    std::fill(res, res + N * CPQ, T(0));
    for (size_t i = 0; i < N; i++)
        for (size_t f = 0; f < F; f++) {
            for (size_t c = 0; c < C; c++) {
                const size_t off_i = i * CHW + c * HW;
                for (size_t y = 0; y < H; y++)
                    for (size_t x = 0; x < W; x++)
                        padded[(ph + y) * pW + pw + x] = data[off_i + y * W + x];
                for (size_t p = 0; p < P; p++)
                    for (size_t h = 0; h < std::min(Hf, pH - p * sh); h++)
                        for (size_t q = 0; q < Q; q++)
                            for (size_t w = 0; w < std::min(Wf, pW - q * sw); w++) {
                                const size_t off_o = i * CPQ + f * PQ + p * Q + q;
                                const size_t off_p = (p * sh + h) * pW + q * sw + w;
                                const size_t off_f = f * C * Hf * Wf + c * Hf * Wf + h * Wf + w;
                                res[off_o] = res[off_o] + padded[off_p] * filter[off_f];
                            }
            }
            if (bias)
                for (size_t l = 0; l < PQ; l++)
                    res[i * CPQ + f * PQ + l] += bias[f];
        }
    return ST_OK;
}

// Pooling.cpp:28-107 with OP = MAX (Pooling.h:46-58), via MaxPoolForward.h:35-44. Quirks kept:
// P uses stride_w and Q uses stride_h (:38-39); the result starts at zero and the window is
// folded into it with std::max (so the result is max(0, window)); the P==1 && Q==1 && W==1 quick
// path starts from numeric_limits::max() instead and therefore returns that value (:57-66).
template <typename T>
int maxpool(T *res, size_t *res_h, size_t *res_w, const T *data, size_t N, size_t C, size_t H, size_t W, size_t ph_,
            size_t pw_, size_t sh, size_t sw, size_t padh, size_t padw) {
    if (H + 2 * padh < ph_ || W + 2 * padw < pw_ || sh == 0 || sw == 0)
        return ST_INVALID;
    const size_t HW = H * W, CHW = C * HW;
    const size_t P = get_pq(H, ph_, padh, sw), Q = get_pq(W, pw_, padw, sh);
    const size_t CPQ = C * P * Q;
    *res_h = P;
    *res_w = Q;
    const size_t pH = H + 2 * padh, pW = W + 2 * padw;
    std::fill(res, res + N * CPQ, T(0));
    auto fold = [](T init, const T *in, size_t start, size_t len) {
        T ret = init;
        for (size_t i = start; i < start + len; i++)
            ret = std::max(ret, in[i]);
        return ret;
    };
    if (P == 1 && Q == 1 && W == 1) {
        const size_t lenh = std::min(ph_, H);
        for (size_t i = 0; i < N; i++)
            for (size_t c = 0; c < C; c++)
                res[i * C + c] = fold(std::numeric_limits<T>::max(), data, i * CHW + c * H, lenh);
        return ST_OK;
    }
    std::vector<T> padded(pH * pW, T(0));
    for (size_t i = 0; i < N; i++)
        for (size_t c = 0; c < C; c++) {
            const size_t off = i * CHW + c * HW;
            for (size_t y = 0; y < H; y++)
                for (size_t x = 0; x < W; x++)
                    padded[(padh + y) * pW + padw + x] = data[off + y * W + x];
            T *o = res + i * CPQ + c * P * Q;
            for (size_t p = 0; p < P; p++)
                for (size_t h = p * sh; h < std::min(p * sh + ph_, pH); h++)
                    for (size_t q = 0; q < Q; q++) {
                        // A window starting beyond the padded row is undefined in the reference
                        // (unsigned wrap-around in Pooling.cpp:102); it is treated as empty here.
                        const size_t len = (q * sw < pW) ? std::min(pw_, pW - q * sw) : 0;
                        o[p * Q + q] = fold(o[p * Q + q], padded.data(), h * pW + q * sw, len);
                    }
        }
    return ST_OK;
}

// BiasAdd.h:34-52 with the channel count taken from the bias item count.
template <typename T> int bias_add(T *res, const T *data, size_t rows, size_t cols, const T *bias, size_t C) {
    if (C == 0 || cols % C != 0)
        return ST_RUNTIME;
    const size_t HW = cols / C;
    for (size_t i = 0; i < rows; i++)
        for (size_t c = 0; c < C; c++)
            for (size_t j = 0; j < HW; j++)
                res[i * cols + c * HW + j] = data[i * cols + c * HW + j] + bias[c];
    return ST_OK;
}

// BatchNorm2DTestForward.h:77-101. stat_index 1 is the reference CPU loop verbatim (statistics
// indexed by the row i); stat_index 0 applies the same expression with the statistics of the
// element's channel, which is what the reference's CUDA kernel (cuDNN spatial mode) computes.
template <typename T>
int batchnorm(T *res, const T *in, size_t rows, size_t cols, const T *gamma, const T *beta, const T *mean,
              const T *var, size_t C, T eps, int stat_index) {
    if (stat_index == 0 && (C == 0 || cols % C != 0))
        return ST_RUNTIME;
    const size_t HW = stat_index == 0 ? cols / C : 1;
    for (size_t i = 0; i < rows; i++)
        for (size_t j = 0; j < cols; j++) {
            const size_t s = stat_index == 0 ? j / HW : i;
            const size_t off = i * cols + j;
            const T x_hat = (in[off] - mean[s]) / std::sqrt(var[s] + eps);
            res[off] = gamma[s] * x_hat + beta[s];
        }
    return ST_OK;
}

// Softmax.h:22-58
template <typename T> int softmax(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    for (size_t r = 0; r < rows; r++) {
        T mx = arg[0];
        for (size_t c = 1; c < cols; c++)
            mx = std::max(mx, arg[c]);
        T sum = 0;
        for (size_t c = 0; c < cols; c++) {
            res[c] = std::exp(arg[c] - mx);
            sum += res[c];
        }
        const T inv = T(1) / sum;
        for (size_t c = 0; c < cols; c++)
            res[c] *= inv;
        arg += ld;
        res += ld_res;
    }
    return ST_OK;
}

// Pooling.cpp:28-107 with OP = AVG (Pooling.h:33-44), via AvgPoolForward.h. Each window row is summed
// left to right from zero, multiplied by plen = 1 / (pool_h * pool_w) (:50, the full window even where it
// is clipped or padded) and added to the running result. The reference's quick paths (:57-91) apply the
// same expression to the same values as the padded general path (:92-105), which is restated here; the
// P==1 && Q==1 && W==1 path (:57-66) sums the first min(pool_h, H) values of the plane.
template <typename T>
int avgpool(T *res, size_t *res_h, size_t *res_w, const T *data, size_t N, size_t C, size_t H, size_t W, size_t ph_,
            size_t pw_, size_t sh, size_t sw, size_t padh, size_t padw) {
    if (H + 2 * padh < ph_ || W + 2 * padw < pw_ || sh == 0 || sw == 0 || ph_ == 0 || pw_ == 0)
        return ST_INVALID;
    const size_t HW = H * W, CHW = C * HW;
    const size_t P = get_pq(H, ph_, padh, sw), Q = get_pq(W, pw_, padw, sh);
    const size_t CPQ = C * P * Q;
    *res_h = P;
    *res_w = Q;
    const size_t pH = H + 2 * padh, pW = W + 2 * padw;
    const T plen = static_cast<T>(1) / static_cast<T>(pw_ * ph_);
    std::fill(res, res + N * CPQ, T(0));
    auto run = [plen](T init, const T *in, size_t start, size_t len) {
        T ret = 0;
        for (size_t i = start; i < start + len; i++)
            ret += in[i];
        return ret * plen + init;
    };
    if (P == 1 && Q == 1 && W == 1) {
        const size_t lenh = std::min(ph_, H);
        for (size_t i = 0; i < N; i++)
            for (size_t c = 0; c < C; c++)
                res[i * C + c] = run(T(0), data, i * CHW + c * H, lenh);
        return ST_OK;
    }
    std::vector<T> padded(pH * pW, T(0));
    for (size_t i = 0; i < N; i++)
        for (size_t c = 0; c < C; c++) {
            const size_t off = i * CHW + c * HW;
            for (size_t y = 0; y < H; y++)
                for (size_t x = 0; x < W; x++)
                    padded[(padh + y) * pW + padw + x] = data[off + y * W + x];
            T *o = res + i * CPQ + c * P * Q;
            for (size_t p = 0; p < P; p++)
                for (size_t h = p * sh; h < std::min(p * sh + ph_, pH); h++)
                    for (size_t q = 0; q < Q; q++) {
                        const size_t len = (q * sw < pW) ? std::min(pw_, pW - q * sw) : 0;
                        o[p * Q + q] = run(o[p * Q + q], padded.data(), h * pW + q * sw, len);
                    }
        }
    return ST_OK;
}

// CUDA/Activation.cpp:21-47 (cudnnActivationForward, CUDNN_ACTIVATION_RELU, CUDNN_PROPAGATE_NAN): max(0, x),
// a NaN stays a NaN. There is no CPU kernel; the elementwise MAX with 0 (EwBinarySca.h std::max) gives the same.
template <typename T> int relu(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++) {
            const T x = arg[r * ld + c];
            res[r * ld_res + c] = (x < T(0)) ? T(0) : x;
        }
    return ST_OK;
}

// Fill.h (CPU) / CUDA/Fill.cu:27-49
template <typename T> int fill(T *res, size_t ld_res, T value, size_t rows, size_t cols) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++)
            res[r * ld_res + c] = value;
    return ST_OK;
}

// ColBind.h:58-91
template <typename T>
int col_bind(T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs, const T *rhs, size_t rr, size_t rc,
             size_t ld_rhs) {
    if (lr != rr)
        return ST_RUNTIME;
    for (size_t r = 0; r < lr; r++) {
        if (lc)
            std::memcpy(res + r * ld_res, lhs + r * ld_lhs, lc * sizeof(T));
        if (rc)
            std::memcpy(res + r * ld_res + lc, rhs + r * ld_rhs, rc * sizeof(T));
    }
    return ST_OK;
}

// ExtractCol.h:57-114: positions as int64, a negative one counts from the end, anything still outside
// [0, cols) is std::out_of_range (status 6); more than one selection column is a runtime error.
template <typename T>
int extract_col(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld, const int64_t *sel,
                size_t sel_rows, size_t sel_cols) {
    if (sel_cols != 1)
        return ST_RUNTIME;
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < sel_rows; c++) {
            int64_t idx = sel[c];
            if (idx < 0)
                idx += static_cast<int64_t>(cols);
            if (idx < 0 || cols <= static_cast<size_t>(idx))
                return 6;
            res[r * ld_res + c] = arg[r * ld + static_cast<size_t>(idx)];
        }
    return ST_OK;
}

// Transpose.h:51-76
template <typename T> int transpose(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++)
            res[c * ld_res + r] = arg[r * ld + c];
    return ST_OK;
}

} // namespace

// ---------------------------------------------------------------------------------------
// C exports: oracle_<name>_{f32,f64}
// ---------------------------------------------------------------------------------------
#define ORACLE_EXPORTS(SUF, T)                                                                                          \
    extern "C" int oracle_ew_binary_##SUF(int op, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc,            \
                                          size_t ld_lhs, const T *rhs, size_t rr, size_t rc, size_t ld_rhs) {           \
        return ew_binary<T>(op, res, ld_res, lhs, lr, lc, ld_lhs, rhs, rr, rc, ld_rhs);                                 \
    }                                                                                                                   \
    extern "C" int oracle_ew_binary_sca_##SUF(int op, T *res, size_t ld_res, const T *lhs, size_t rows, size_t cols,    \
                                              size_t ld_lhs, T rhs) {                                                   \
        return ew_binary_sca<T>(op, res, ld_res, lhs, rows, cols, ld_lhs, rhs);                                         \
    }                                                                                                                   \
    extern "C" int oracle_ew_unary_##SUF(int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,         \
                                         size_t ld_arg) {                                                               \
        return ew_unary<T>(op, res, ld_res, arg, rows, cols, ld_arg);                                                   \
    }                                                                                                                   \
    extern "C" int oracle_agg_all_##SUF(int op, const T *arg, size_t rows, size_t cols, size_t ld, T *out) {            \
        return agg_all<T>(op, arg, rows, cols, ld, out);                                                                \
    }                                                                                                                   \
    extern "C" int oracle_agg_row_##SUF(int op, T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,          \
                                        size_t ld) {                                                                    \
        return agg_row<T>(op, res, ld_res, arg, rows, cols, ld);                                                        \
    }                                                                                                                   \
    extern "C" int oracle_agg_row_idx_##SUF(int op, uint64_t *res, size_t ld_res, const T *arg, size_t rows,            \
                                            size_t cols, size_t ld) {                                                   \
        return agg_row_idx<T>(op, res, ld_res, arg, rows, cols, ld);                                                    \
    }                                                                                                                   \
    extern "C" int oracle_agg_col_##SUF(int op, T *res, const T *arg, size_t rows, size_t cols, size_t ld) {            \
        return agg_col<T>(op, res, arg, rows, cols, ld);                                                                \
    }                                                                                                                   \
    extern "C" int oracle_agg_col_idx_##SUF(int op, uint64_t *res, const T *arg, size_t rows, size_t cols,              \
                                            size_t ld) {                                                                \
        return agg_col_idx<T>(op, res, arg, rows, cols, ld);                                                            \
    }                                                                                                                   \
    extern "C" int oracle_matmul_##SUF(T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs,        \
                                       const T *rhs, size_t rr, size_t rc, size_t ld_rhs, int ta, int tb) {             \
        return matmul<T>(res, ld_res, lhs, lr, lc, ld_lhs, rhs, rr, rc, ld_rhs, ta, tb);                                \
    }                                                                                                                   \
    extern "C" int oracle_syrk_##SUF(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld,          \
                                     int trans_left) {                                                                  \
        return syrk<T>(res, ld_res, arg, rows, cols, ld, trans_left);                                                   \
    }                                                                                                                   \
    extern "C" int oracle_solve_##SUF(T *x, const T *A, size_t n, const T *b) { return solve<T>(x, A, n, b); }          \
    extern "C" int oracle_conv2d_forward_##SUF(T *res, size_t *res_h, size_t *res_w, const T *data, const T *filter,    \
                                               const T *bias, size_t N, size_t C, size_t H, size_t W, size_t F,         \
                                               size_t Hf, size_t Wf, size_t sh, size_t sw, size_t ph, size_t pw) {      \
        return conv2d<T>(res, res_h, res_w, data, filter, bias, N, C, H, W, F, Hf, Wf, sh, sw, ph, pw);                 \
    }                                                                                                                   \
    extern "C" int oracle_maxpool_forward_##SUF(T *res, size_t *res_h, size_t *res_w, const T *data, size_t N,          \
                                                size_t C, size_t H, size_t W, size_t ph, size_t pw, size_t sh,          \
                                                size_t sw, size_t padh, size_t padw) {                                  \
        return maxpool<T>(res, res_h, res_w, data, N, C, H, W, ph, pw, sh, sw, padh, padw);                             \
    }                                                                                                                   \
    extern "C" int oracle_bias_add_##SUF(T *res, const T *data, size_t rows, size_t cols, const T *bias, size_t C) {    \
        return bias_add<T>(res, data, rows, cols, bias, C);                                                             \
    }                                                                                                                   \
    extern "C" int oracle_batchnorm_inference_##SUF(T *res, const T *in, size_t rows, size_t cols, const T *gamma,      \
                                                    const T *beta, const T *mean, const T *var, size_t C, T eps,        \
                                                    int stat_index) {                                                   \
        return batchnorm<T>(res, in, rows, cols, gamma, beta, mean, var, C, eps, stat_index);                           \
    }                                                                                                                   \
    extern "C" int oracle_softmax_##SUF(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {     \
        return softmax<T>(res, ld_res, arg, rows, cols, ld);                                                            \
    }                                                                                                                   \
    extern "C" int oracle_avgpool_forward_##SUF(T *res, size_t *res_h, size_t *res_w, const T *data, size_t N,          \
                                                size_t C, size_t H, size_t W, size_t ph, size_t pw, size_t sh,          \
                                                size_t sw, size_t padh, size_t padw) {                                  \
        return avgpool<T>(res, res_h, res_w, data, N, C, H, W, ph, pw, sh, sw, padh, padw);                             \
    }                                                                                                                   \
    extern "C" int oracle_relu_forward_##SUF(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols,             \
                                             size_t ld) {                                                               \
        return relu<T>(res, ld_res, arg, rows, cols, ld);                                                               \
    }                                                                                                                   \
    extern "C" int oracle_fill_##SUF(T *res, size_t ld_res, T value, size_t rows, size_t cols) {                        \
        return fill<T>(res, ld_res, value, rows, cols);                                                                 \
    }                                                                                                                   \
    extern "C" int oracle_col_bind_##SUF(T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc, size_t ld_lhs,      \
                                         const T *rhs, size_t rr, size_t rc, size_t ld_rhs) {                           \
        return col_bind<T>(res, ld_res, lhs, lr, lc, ld_lhs, rhs, rr, rc, ld_rhs);                                      \
    }                                                                                                                   \
    extern "C" int oracle_extract_col_##SUF(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld,   \
                                            const int64_t *sel, size_t sel_rows, size_t sel_cols) {                     \
        return extract_col<T>(res, ld_res, arg, rows, cols, ld, sel, sel_rows, sel_cols);                               \
    }                                                                                                                   \
    extern "C" int oracle_transpose_##SUF(T *res, size_t ld_res, const T *arg, size_t rows, size_t cols, size_t ld) {   \
        return transpose<T>(res, ld_res, arg, rows, cols, ld);                                                          \
    }

ORACLE_EXPORTS(f32, float)
ORACLE_EXPORTS(f64, double)

// Integer value types (the reference instantiates these device kernels for them: kernels/CUDA/EwBinaryMat.cu:267-270,
// EwBinaryObjSca.cu:91-94, AggAll.cu:155, AggRow.cu:146, AggCol.cu:89, Fill.cu:47,49, ColBind.cu:75, ExtractCol.cu:58):
// the same templates as above, i.e. the reference's expressions evaluated in C++ integer arithmetic.
#define ORACLE_EW_INT_EXPORTS(SUF, T)                                                                                   \
    extern "C" int oracle_ew_binary_##SUF(int op, T *res, size_t ld_res, const T *lhs, size_t lr, size_t lc,            \
                                          size_t ld_lhs, const T *rhs, size_t rr, size_t rc, size_t ld_rhs) {           \
        return ew_binary<T>(op, res, ld_res, lhs, lr, lc, ld_lhs, rhs, rr, rc, ld_rhs);                                 \
    }                                                                                                                   \
    extern "C" int oracle_ew_binary_sca_##SUF(int op, T *res, size_t ld_res, const T *lhs, size_t rows, size_t cols,    \
                                              size_t ld_lhs, T rhs) {                                                   \
        return ew_binary_sca<T>(op, res, ld_res, lhs, rows, cols, ld_lhs, rhs);                                         \
    }
ORACLE_EW_INT_EXPORTS(si64, int64_t)
ORACLE_EW_INT_EXPORTS(ui64, uint64_t)
ORACLE_EW_INT_EXPORTS(si32, int32_t)
ORACLE_EW_INT_EXPORTS(ui32, uint32_t)

extern "C" int oracle_agg_all_si64(int op, const int64_t *arg, size_t rows, size_t cols, size_t ld, int64_t *out) {
    return agg_all<int64_t>(op, arg, rows, cols, ld, out);
}
extern "C" int oracle_agg_row_si64(int op, int64_t *res, size_t ld_res, const int64_t *arg, size_t rows, size_t cols, size_t ld) {
    return agg_row<int64_t>(op, res, ld_res, arg, rows, cols, ld);
}
extern "C" int oracle_agg_row_idx_si64(int op, uint64_t *res, size_t ld_res, const int64_t *arg, size_t rows, size_t cols,
                                       size_t ld) {
    return agg_row_idx<int64_t>(op, res, ld_res, arg, rows, cols, ld);
}
extern "C" int oracle_agg_col_si64(int op, int64_t *res, const int64_t *arg, size_t rows, size_t cols, size_t ld) {
    return agg_col<int64_t>(op, res, arg, rows, cols, ld);
}
extern "C" int oracle_agg_col_idx_si64(int op, uint64_t *res, const int64_t *arg, size_t rows, size_t cols, size_t ld) {
    return agg_col_idx<int64_t>(op, res, arg, rows, cols, ld);
}
extern "C" int oracle_fill_si64(int64_t *res, size_t ld_res, int64_t value, size_t rows, size_t cols) {
    return fill<int64_t>(res, ld_res, value, rows, cols);
}
extern "C" int oracle_fill_ui64(uint64_t *res, size_t ld_res, uint64_t value, size_t rows, size_t cols) {
    return fill<uint64_t>(res, ld_res, value, rows, cols);
}
extern "C" int oracle_col_bind_si64(int64_t *res, size_t ld_res, const int64_t *lhs, size_t lr, size_t lc, size_t ld_lhs,
                                    const int64_t *rhs, size_t rr, size_t rc, size_t ld_rhs) {
    return col_bind<int64_t>(res, ld_res, lhs, lr, lc, ld_lhs, rhs, rr, rc, ld_rhs);
}
extern "C" int oracle_extract_col_si64(int64_t *res, size_t ld_res, const int64_t *arg, size_t rows, size_t cols, size_t ld,
                                       const int64_t *sel, size_t sel_rows, size_t sel_cols) {
    return extract_col<int64_t>(res, ld_res, arg, rows, cols, ld, sel, sel_rows, sel_cols);
}
extern "C" int oracle_transpose_si64(int64_t *res, size_t ld_res, const int64_t *arg, size_t rows, size_t cols, size_t ld) {
    return transpose<int64_t>(res, ld_res, arg, rows, cols, ld);
}
