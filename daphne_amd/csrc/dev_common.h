// Device-side helpers shared by every kernel. This header is also compiled at run time by hiprtc
// (for fused pipeline bodies), so it must not include host or standard-library headers.
#pragma once

#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

constexpr int DH_WAVE = 64;

template <typename T> struct dh_vec; // 16-byte vector of T
template <> struct dh_vec<float> {
    using type = float4;
    static constexpr int N = 4;
};
template <> struct dh_vec<double> {
    using type = double2;
    static constexpr int N = 2;
};

typedef float dh_f32x4_native __attribute__((ext_vector_type(4)));
typedef double dh_f64x2_native __attribute__((ext_vector_type(2)));
template <typename T> struct dh_native_vec;
template <> struct dh_native_vec<float> {
    using type = dh_f32x4_native;
};
template <> struct dh_native_vec<double> {
    using type = dh_f64x2_native;
};

template <typename T> __device__ __forceinline__ T dh_inf();
template <> __device__ __forceinline__ float dh_inf<float>() { return __builtin_inff(); }
template <> __device__ __forceinline__ double dh_inf<double>() { return __builtin_inf(); }
template <typename T> __device__ __forceinline__ T dh_nan();
template <> __device__ __forceinline__ float dh_nan<float>() { return __builtin_nanf(""); }
template <> __device__ __forceinline__ double dh_nan<double>() { return __builtin_nan(""); }

template <typename T> __device__ __forceinline__ T dh_shfl_xor(T v, int mask) { return __shfl_xor(v, mask, DH_WAVE); }
template <typename T> __device__ __forceinline__ T dh_shfl_down(T v, int d) { return __shfl_down(v, d, DH_WAVE); }

// 16-byte (VEC = 16 / sizeof(T)) or scalar (VEC = 1) global load / store into a register array.
template <typename T, int VEC> __device__ __forceinline__ void dh_load_vec(const T *p, T (&v)[VEC]) {
    if constexpr (VEC == 1) {
        v[0] = *p;
    } else {
        using V = typename dh_native_vec<T>::type;
        const V t = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int i = 0; i < VEC; i++)
            v[i] = t[i];
    }
}
template <typename T, int VEC> __device__ __forceinline__ void dh_store_vec(T *p, const T (&v)[VEC]) {
    if constexpr (VEC == 1) {
        *p = v[0];
    } else {
        using V = typename dh_native_vec<T>::type;
        V t;
#pragma unroll
        for (int i = 0; i < VEC; i++)
            t[i] = v[i];
        *reinterpret_cast<V *>(p) = t;
    }
}
// Streaming variant: non-temporal load for data that is read exactly once (keeps the stream from
// evicting reused operands and measurably raises HBM read throughput on gfx950).
template <typename T, int VEC> __device__ __forceinline__ void dh_load_vec_stream(const T *p, T (&v)[VEC]) {
    if constexpr (VEC == 1) {
        v[0] = __builtin_nontemporal_load(p);
    } else {
        using V = typename dh_native_vec<T>::type;
        const V t = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
#pragma unroll
        for (int i = 0; i < VEC; i++)
            v[i] = t[i];
    }
}
