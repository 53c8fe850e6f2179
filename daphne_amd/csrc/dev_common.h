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

// integer value types (the reference instantiates its elementwise kernels for si64 / ui64 / si32 / ui32 and its
// aggregations for si64, kernels/CUDA/EwBinaryMat.cu:265-270, AggAll.cu:153-155)
template <> struct dh_vec<int> {
    using type = int4;
    static constexpr int N = 4;
};
template <> struct dh_vec<unsigned> {
    using type = uint4;
    static constexpr int N = 4;
};
template <> struct dh_vec<long> {
    using type = longlong2;
    static constexpr int N = 2;
};
template <> struct dh_vec<unsigned long> {
    using type = ulonglong2;
    static constexpr int N = 2;
};

typedef float dh_f32x4_native __attribute__((ext_vector_type(4)));
typedef double dh_f64x2_native __attribute__((ext_vector_type(2)));
typedef int dh_i32x4_native __attribute__((ext_vector_type(4)));
typedef unsigned dh_u32x4_native __attribute__((ext_vector_type(4)));
typedef long dh_i64x2_native __attribute__((ext_vector_type(2)));
typedef unsigned long dh_u64x2_native __attribute__((ext_vector_type(2)));
template <typename T> struct dh_native_vec;
template <> struct dh_native_vec<float> {
    using type = dh_f32x4_native;
};
template <> struct dh_native_vec<double> {
    using type = dh_f64x2_native;
};
template <> struct dh_native_vec<int> {
    using type = dh_i32x4_native;
};
template <> struct dh_native_vec<unsigned> {
    using type = dh_u32x4_native;
};
template <> struct dh_native_vec<long> {
    using type = dh_i64x2_native;
};
template <> struct dh_native_vec<unsigned long> {
    using type = dh_u64x2_native;
};

template <typename T> __device__ __forceinline__ T dh_inf();
template <> __device__ __forceinline__ float dh_inf<float>() { return __builtin_inff(); }
template <> __device__ __forceinline__ double dh_inf<double>() { return __builtin_inf(); }
template <typename T> __device__ __forceinline__ T dh_nan();
template <> __device__ __forceinline__ float dh_nan<float>() { return __builtin_nanf(""); }
template <> __device__ __forceinline__ double dh_nan<double>() { return __builtin_nan(""); }

// One data-parallel-primitive move of a 32-bit or 64-bit value (CTRL: quad_perm 0x00-0xff,
// row_half_mirror 0x141, row_mirror 0x140); source lanes that are inactive read as zero.
template <int CTRL, typename T> __device__ __forceinline__ T dh_dpp(T v) {
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32-bit or 64-bit values only");
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
    } else {
        const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b), CTRL, 0xf, 0xf, true));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b >> 32), CTRL, 0xf, 0xf, true));
        return __builtin_bit_cast(T, (static_cast<unsigned long long>(hi) << 32) | lo);
    }
}
template <typename T> __device__ __forceinline__ T dh_shfl_xor(T v, int mask) { return __shfl_xor(v, mask, DH_WAVE); }

// Butterfly all-reduce over aligned groups of G lanes (G a power of two <= 64): step(peer) is called
// once per level, and peer(v) returns the value v of this lane's partner at that level. Below 16
// lanes the partner is the lane's image under a quad swap or a mirror of the 8 / 16 lanes around it
// (one register move), above it is lane ^ 16 / lane ^ 32 (a swap of 16-lane rows between two registers). Each level pairs
// the two halves of a block that the previous levels have made uniform, so after the last one every
// lane of a group holds the combination of the whole group - provided the combine is commutative.
// Partners are always in the same group: a group must be wholly active or wholly inactive.
template <int CTRL> struct dh_peer_dpp {
    template <typename T> __device__ __forceinline__ T operator()(T v) const { return dh_dpp<CTRL>(v); }
};
template <int OFF> struct dh_peer_xor {
    template <typename T> __device__ __forceinline__ T operator()(T v) const { return __shfl_xor(v, OFF, DH_WAVE); }
};
// lane ^ 16 (ROWS = 16) or lane ^ 32 (ROWS = 32) by the row-swap instructions of gfx950: with both operands equal,
// v_permlane16_swap / v_permlane32_swap leave the partner's value in the first result for lanes of the upper rows
// and in the second for lanes of the lower rows - one ALU instruction and a select instead of a trip through LDS.
template <int ROWS> struct dh_peer_swap {
    static __device__ __forceinline__ unsigned word(unsigned w, bool upper) {
        if constexpr (ROWS == 16) {
            const auto r = __builtin_amdgcn_permlane16_swap(w, w, false, false);
            return upper ? r[0] : r[1];
        } else {
            const auto r = __builtin_amdgcn_permlane32_swap(w, w, false, false);
            return upper ? r[0] : r[1];
        }
    }
    template <typename T> __device__ __forceinline__ T operator()(T v) const {
        static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32-bit or 64-bit values only");
        const unsigned lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        const bool upper = (lane & ROWS) != 0;
        if constexpr (sizeof(T) == 4) {
            return __builtin_bit_cast(T, word(__builtin_bit_cast(unsigned, v), upper));
        } else {
            const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
            const unsigned lo = word(static_cast<unsigned>(b), upper), hi = word(static_cast<unsigned>(b >> 32), upper);
            return __builtin_bit_cast(T, (static_cast<unsigned long long>(hi) << 32) | lo);
        }
    }
};
template <class Step> __device__ __forceinline__ void dh_butterfly(int G, Step &&step) {
    if (G >= 2)
        step(dh_peer_dpp<0xB1>{}); // quad_perm [1,0,3,2]
    if (G >= 4)
        step(dh_peer_dpp<0x4E>{}); // quad_perm [2,3,0,1]
    if (G >= 8)
        step(dh_peer_dpp<0x141>{}); // row_half_mirror: lane i of 8 <-> 7 - i
    if (G >= 16)
        step(dh_peer_dpp<0x140>{}); // row_mirror: lane i of 16 <-> 15 - i
    if (G >= 32)
        step(dh_peer_swap<16>{});
    if (G >= 64)
        step(dh_peer_swap<32>{});
}
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
// Streaming counterpart of dh_store_vec for results that this kernel does not read again.
template <typename T, int VEC> __device__ __forceinline__ void dh_store_vec_stream(T *p, const T (&v)[VEC]) {
    if constexpr (VEC == 1) {
        __builtin_nontemporal_store(v[0], p);
    } else {
        using V = typename dh_native_vec<T>::type;
        V t;
#pragma unroll
        for (int i = 0; i < VEC; i++)
            t[i] = v[i];
        __builtin_nontemporal_store(t, reinterpret_cast<V *>(p));
    }
}
// Streaming store of one value that this kernel does not read again (results of a pass over a large input).
template <typename T> __device__ __forceinline__ void dh_store_stream(T *p, T v) { __builtin_nontemporal_store(v, p); }
