// Shared device/host helpers for the gfx950 Mamba-2 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <type_traits>

#include "../../include/mamba2_hip.h"

namespace m2 {

// ----------------------------------------------------------------------------- errors
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

#define M2_REQUIRE(cond, code, ...) \
    do { if (!(cond)) return ::m2::fail((code), __VA_ARGS__); } while (0)

// ----------------------------------------------------------------------------- element types
typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }   // round-to-nearest-even

template <typename T> struct VecTraits;
template <> struct VecTraits<float> { static constexpr int kVec = 4; };     // 16-byte vectors
template <> struct VecTraits<bf16_t> { static constexpr int kVec = 8; };

// 16-byte vector of T, loaded/stored as one transaction; elements converted to fp32 on the fly.
template <typename T> struct Vec16 {
    static constexpr int N = VecTraits<T>::kVec;
    T v[N];
};
template <typename T>
__device__ __forceinline__ void load16(const T* __restrict__ p, float (&out)[VecTraits<T>::kVec]) {
    constexpr int N = VecTraits<T>::kVec;
    uint4 raw = *reinterpret_cast<const uint4*>(p);
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = to_f32(e[i]);
}
template <typename T>
__device__ __forceinline__ void store16(T* __restrict__ p, const float (&in)[VecTraits<T>::kVec]) {
    constexpr int N = VecTraits<T>::kVec;
    uint4 raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < N; ++i) e[i] = from_f32<T>(in[i]);
    *reinterpret_cast<uint4*>(p) = raw;
}

// Raw vector of V elements of T (8 or 16 bytes), kept unconverted in registers until used.
template <int BYTES> struct RawBytes;
template <> struct RawBytes<16> { using type = uint4; };
template <> struct RawBytes<8> { using type = uint2; };
template <> struct RawBytes<4> { using type = uint32_t; };
template <> struct RawBytes<2> { using type = uint16_t; };
template <typename T, int V> using RawVec = typename RawBytes<V * (int)sizeof(T)>::type;
template <typename T, int V>
__device__ __forceinline__ RawVec<T, V> loadv_raw(const T* __restrict__ p) { return *reinterpret_cast<const RawVec<T, V>*>(p); }
template <typename T, int V>
__device__ __forceinline__ void cvtv(const RawVec<T, V>& raw, float (&out)[V]) {
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int i = 0; i < V; ++i) out[i] = to_f32(e[i]);
}
template <typename T, int V>
__device__ __forceinline__ void loadv(const T* __restrict__ p, float (&out)[V]) { cvtv<T, V>(loadv_raw<T, V>(p), out); }
template <typename T, int V>
__device__ __forceinline__ void storev(T* __restrict__ p, const float (&in)[V]) {
    RawVec<T, V> raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < V; ++i) e[i] = from_f32<T>(in[i]);
    *reinterpret_cast<RawVec<T, V>*>(p) = raw;
}

// raw 16-byte load (kept unconverted in 4 registers until used) and its conversion
template <typename T>
__device__ __forceinline__ uint4 load16_raw(const T* __restrict__ p) { return *reinterpret_cast<const uint4*>(p); }
template <typename T>
__device__ __forceinline__ void cvt16(const uint4& raw, float (&out)[VecTraits<T>::kVec]) {
    constexpr int N = VecTraits<T>::kVec;
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = to_f32(e[i]);
}

// sigmoid through the hardware reciprocal (1 ulp) rather than an IEEE division (ten more VALU instructions per element)
__device__ __forceinline__ float sigmoid_f(float z) { return __builtin_amdgcn_rcpf(1.0f + __expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z * sigmoid_f(z); }
// d/dz silu(z) = s * (1 + z * (1 - s)),  s = sigmoid(z)
__device__ __forceinline__ float silu_grad_f(float z) {
    float s = sigmoid_f(z);
    return s * (1.0f + z * (1.0f - s));
}

// softplus in the threshold form of the reference's torch twin (mamba2/mamba2_mixer.py:36-38): x itself from 10 on.
constexpr float kSoftplusThreshold = 10.0f;
__device__ __forceinline__ float softplus_f(float v) { return v < kSoftplusThreshold ? log1pf(__expf(v)) : v; }
// d softplus / dv expressed through the VALUE s = softplus(v): sigmoid(v) = 1 - e^{-s} (1 from the threshold on)
__device__ __forceinline__ float softplus_grad_of_value(float s) { return s < kSoftplusThreshold ? -expm1f(-s) : 1.f; }

template <int ACT> __device__ __forceinline__ float act_f(float z) {
    if (ACT == M2_ACT_SILU) return silu_f(z);
    if (ACT == M2_ACT_RELU) return z > 0.f ? z : 0.f;
    return z;
}
template <int ACT> __device__ __forceinline__ float act_grad_f(float z) {
    if (ACT == M2_ACT_SILU) return silu_grad_f(z);
    if (ACT == M2_ACT_RELU) return z > 0.f ? 1.f : 0.f;
    return 1.f;
}

// Value of lane (l ^ M) for M in {1, 2, 4, 8, 16, 32}, without the LDS crossbar (a generic shuffle is a ds_bpermute):
// DPP quad permutes / row rotation / two masked row shifts inside a row of 16 lanes, and the row / half-wave swaps of
// gfx950 (v_permlane16_swap, v_permlane32_swap) across rows.  All 64 lanes must be active.
template <int CTRL, int BANK>
__device__ __forceinline__ float dpp_move(float old, float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, x), CTRL, 0xF, BANK, false));
}
template <int M>
__device__ __forceinline__ float lane_xor(float x) {
    static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "lane_xor: single-bit masks");
    if constexpr (M == 1) return dpp_move<0xB1, 0xF>(x, x);                  // quad_perm [1,0,3,2]
    else if constexpr (M == 2) return dpp_move<0x4E, 0xF>(x, x);             // quad_perm [2,3,0,1]
    else if constexpr (M == 4) return dpp_move<0x114, 0xA>(dpp_move<0x104, 0x5>(x, x), x);     // row_shl:4 into banks 0, 2; row_shr:4 into banks 1, 3
    else if constexpr (M == 8) return dpp_move<0x128, 0xF>(x, x);            // row_ror:8
    else {
        const uint32_t u = __builtin_bit_cast(uint32_t, x);
        uint32_t r0, r1;
        if constexpr (M == 16) { const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false); r0 = r[0]; r1 = r[1]; }
        else { const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false); r0 = r[0]; r1 = r[1]; }
        // r0 = { own | partner } and r1 = { partner | own } for the lower | upper member of each pair
        return __builtin_bit_cast(float, (threadIdx.x & M) ? r0 : r1);
    }
}
// x + (value of lane l ^ M): for the two swap masks both outputs of the swap are simply added
template <int M>
__device__ __forceinline__ float lane_xor_add(float x) {
    if constexpr (M == 16 || M == 32) {
        const uint32_t u = __builtin_bit_cast(uint32_t, x);
        uint32_t r0, r1;
        if constexpr (M == 16) { const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false); r0 = r[0]; r1 = r[1]; }
        else { const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false); r0 = r[0]; r1 = r[1]; }
        return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
    } else {
        return x + lane_xor<M>(x);
    }
}

__device__ __forceinline__ float warp_sum(float v) {
    v = lane_xor_add<32>(v); v = lane_xor_add<16>(v); v = lane_xor_add<8>(v);
    v = lane_xor_add<4>(v); v = lane_xor_add<2>(v); v = lane_xor_add<1>(v);
    return v;
}

// Number of compute units of the current device (queried once per process; 256 on MI355X).
inline int64_t device_cus() {
    static int64_t cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return (int64_t)n;
    }();
    return cus;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Dispatch a runtime dtype to a template type.
#define M2_DISPATCH_DTYPE(dtype, T, ...)                                  \
    do {                                                                  \
        if ((dtype) == M2_F32) { using T = float; __VA_ARGS__; }          \
        else if ((dtype) == M2_BF16) { using T = ::m2::bf16_t; __VA_ARGS__; } \
        else return ::m2::fail(M2_ERR_DTYPE, "unsupported dtype %d", (int)(dtype)); \
    } while (0)

}  // namespace m2
