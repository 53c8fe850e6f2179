// Scalar semantics of the elementwise operators, as device functors. Also compiled at run time by
// hiprtc (fused pipeline bodies), so no host or standard-library headers here.
//
// Binary ops follow the reference's EwBinarySca (src/runtime/local/kernels/EwBinarySca.h:143-167,
// op codes BinaryOpCode.h:29-55), unary ops its EwUnarySca (EwUnarySca.h:182-206, domain checks
// :129-157, op codes UnaryOpCode.h:28-55).
#pragma once

#include "dev_common.h"

namespace dh_ew {

#define DH_MATH1(FN)                                                                               \
    template <typename T> __device__ __forceinline__ T dh_##FN(T a);                               \
    template <> __device__ __forceinline__ float dh_##FN<float>(float a) { return FN##f(a); }      \
    template <> __device__ __forceinline__ double dh_##FN<double>(double a) { return FN(a); }
DH_MATH1(sqrt)
DH_MATH1(exp)
DH_MATH1(log)
DH_MATH1(sin)
DH_MATH1(cos)
DH_MATH1(tan)
DH_MATH1(asin)
DH_MATH1(acos)
DH_MATH1(atan)
DH_MATH1(sinh)
DH_MATH1(cosh)
DH_MATH1(tanh)
DH_MATH1(floor)
DH_MATH1(ceil)
DH_MATH1(round)
DH_MATH1(fabs)
#undef DH_MATH1
template <typename T> __device__ __forceinline__ T dh_pow(T a, T b);
template <> __device__ __forceinline__ float dh_pow<float>(float a, float b) { return powf(a, b); }
template <> __device__ __forceinline__ double dh_pow<double>(double a, double b) { return pow(a, b); }
template <typename T> __device__ __forceinline__ T dh_fmod(T a, T b);
template <> __device__ __forceinline__ float dh_fmod<float>(float a, float b) { return fmodf(a, b); }
template <> __device__ __forceinline__ double dh_fmod<double>(double a, double b) { return fmod(a, b); }

// Floating-point value types evaluate the expressions of EwBinarySca.h:143-167 directly. Integer value types go
// the way C++ takes for the same expressions: pow / fmod / log promote both operands to double and the result is
// converted back (truncated); comparisons and logic give 0 / 1. An integer division or remainder by zero, and the
// signed overflow INT_MIN / -1, stop the reference's process with a hardware trap; here bad() reports them and the
// call fails with a domain error. Conversions of out-of-range or NaN doubles back to an integer are undefined in
// C++ and unspecified here.
template <typename T> struct dh_is_int {
    static constexpr bool value = false;
};
template <> struct dh_is_int<int> {
    static constexpr bool value = true;
};
template <> struct dh_is_int<unsigned> {
    static constexpr bool value = true;
};
template <> struct dh_is_int<long> {
    static constexpr bool value = true;
};
template <> struct dh_is_int<unsigned long> {
    static constexpr bool value = true;
};
template <typename T> __device__ __forceinline__ bool dh_int_div_traps(T a, T b) {
    if constexpr (!dh_is_int<T>::value) {
        return false;
    } else {
        if (b == T(0))
            return true;
        if constexpr (T(-1) < T(0)) // signed: the most negative value divided by -1 does not fit
            return b == T(-1) && a == static_cast<T>(T(1) << (sizeof(T) * 8 - 1));
        return false;
    }
}
template <typename T> __device__ __forceinline__ T dh_pow_any(T a, T b) {
    if constexpr (!dh_is_int<T>::value) {
        return dh_pow<T>(a, b);
    } else {
        // The exact power of two integers is an integer; where it fits the 53 bits of a double, a correctly rounded
        // pow() returns exactly that. Rounding to the nearest integer removes the last-bit error a device pow() may
        // have there (negative exponents give |result| <= 1, which truncates as it stands).
        const double r = pow(static_cast<double>(a), static_cast<double>(b));
        return static_cast<T>((b >= T(0)) ? rint(r) : r);
    }
}
template <typename T> __device__ __forceinline__ T dh_mod_any(T a, T b) {
    if constexpr (!dh_is_int<T>::value)
        return dh_fmod<T>(a, b);
    else
        return static_cast<T>(fmod(static_cast<double>(a), static_cast<double>(b))); // exact in double, as on the host
}
template <typename T> __device__ __forceinline__ T dh_log_any(T a, T b) {
    if constexpr (!dh_is_int<T>::value)
        return dh_log<T>(a) / dh_log<T>(b);
    else
        return static_cast<T>(log(static_cast<double>(a)) / log(static_cast<double>(b)));
}

#define DH_BIN_FUNCTOR_C(NAME, EXPR, CHK, BAD)                                                     \
    template <typename T> struct NAME {                                                            \
        static constexpr bool checks = dh_is_int<T>::value && (CHK);                               \
        static __device__ __forceinline__ T apply(T a, T b) { return EXPR; }                       \
        static __device__ __forceinline__ bool bad(T a, T b) { return (BAD); }                     \
    };
#define DH_BIN_FUNCTOR(NAME, EXPR) DH_BIN_FUNCTOR_C(NAME, EXPR, false, false)
DH_BIN_FUNCTOR(BAdd, a + b)
DH_BIN_FUNCTOR(BSub, a - b)
DH_BIN_FUNCTOR(BMul, a *b)
// IEEE division, as the CPU kernel (the CUDA kernel multiplies by 1/b); a trapping integer division yields 0 and is reported
DH_BIN_FUNCTOR_C(BDiv, (dh_int_div_traps<T>(a, b) ? T(0) : a / b), true, dh_int_div_traps<T>(a, b))
DH_BIN_FUNCTOR(BPow, dh_pow_any<T>(a, b))
// fmod(a, 0) is NaN, which no integer can hold: reported like the division
DH_BIN_FUNCTOR_C(BMod, ((dh_is_int<T>::value && b == T(0)) ? T(0) : dh_mod_any<T>(a, b)), true, (b == T(0)))
DH_BIN_FUNCTOR(BLog, dh_log_any<T>(a, b))
DH_BIN_FUNCTOR(BEq, static_cast<T>(a == b))
DH_BIN_FUNCTOR(BNeq, static_cast<T>(a != b))
DH_BIN_FUNCTOR(BLt, static_cast<T>(a < b))
DH_BIN_FUNCTOR(BLe, static_cast<T>(a <= b))
DH_BIN_FUNCTOR(BGt, static_cast<T>(a > b))
DH_BIN_FUNCTOR(BGe, static_cast<T>(a >= b))
DH_BIN_FUNCTOR(BMin, (b < a) ? b : a) // std::min(a, b): NaN in b never wins, NaN in a stays
DH_BIN_FUNCTOR(BMax, (a < b) ? b : a) // std::max(a, b)
DH_BIN_FUNCTOR(BAnd, static_cast<T>((a != T(0)) && (b != T(0))))
DH_BIN_FUNCTOR(BOr, static_cast<T>((a != T(0)) || (b != T(0))))
#undef DH_BIN_FUNCTOR
#undef DH_BIN_FUNCTOR_C

template <typename T> __device__ __forceinline__ T dh_sign(T a) {
    return (a == T(0)) ? T(0) : ((a < T(0)) ? T(-1) : ((a > T(0)) ? T(1) : dh_nan<T>()));
}

// Unary functors also expose bad(a): true where the CPU kernel throws std::domain_error, and
// `checks`: whether the op has a domain at all.
#define DH_UN_FUNCTOR(NAME, EXPR, CHECKS, BAD)                                                     \
    template <typename T> struct NAME {                                                            \
        static constexpr bool checks = CHECKS;                                                     \
        static __device__ __forceinline__ T apply(T a, T) { return EXPR; }                         \
        static __device__ __forceinline__ bool bad(T a) { return BAD; }                            \
    };
DH_UN_FUNCTOR(UMinus, -a, false, false)
DH_UN_FUNCTOR(UAbs, dh_fabs<T>(a), false, false)
DH_UN_FUNCTOR(USign, dh_sign<T>(a), false, false)
DH_UN_FUNCTOR(USqrt, dh_sqrt<T>(a), true, (T(-0.0) > a))
DH_UN_FUNCTOR(UExp, dh_exp<T>(a), false, false)
DH_UN_FUNCTOR(ULn, dh_log<T>(a), true, (T(-0.0) > a))
DH_UN_FUNCTOR(USin, dh_sin<T>(a), false, false)
DH_UN_FUNCTOR(UCos, dh_cos<T>(a), false, false)
DH_UN_FUNCTOR(UTan, dh_tan<T>(a), false, false)
DH_UN_FUNCTOR(UAsin, dh_asin<T>(a), true, (T(-1.0) > a || a > T(1.0)))
DH_UN_FUNCTOR(UAcos, dh_acos<T>(a), true, (T(-1.0) > a || a > T(1.0)))
DH_UN_FUNCTOR(UAtan, dh_atan<T>(a), false, false)
DH_UN_FUNCTOR(USinh, dh_sinh<T>(a), false, false)
DH_UN_FUNCTOR(UCosh, dh_cosh<T>(a), false, false)
DH_UN_FUNCTOR(UTanh, dh_tanh<T>(a), false, false)
DH_UN_FUNCTOR(UFloor, dh_floor<T>(a), false, false)
DH_UN_FUNCTOR(UCeil, dh_ceil<T>(a), false, false)
DH_UN_FUNCTOR(URound, dh_round<T>(a), false, false)
DH_UN_FUNCTOR(UIsNan, static_cast<T>(a != a), false, false)
#undef DH_UN_FUNCTOR

} // namespace dh_ew
