// Shared device/host helpers for the Flux block kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/flux_hip.h"

namespace flux {

// ------------------------------------------------------------------------------------------------
// Host side: error text per thread, argument checks.
// ------------------------------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ------------------------------------------------------------------------------------------------
// Device side: storage types and conversions.
// ------------------------------------------------------------------------------------------------
typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf2f(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }

// Round-to-nearest-even fp32 -> bf16 (the hardware convert on gfx950).
__device__ __forceinline__ bf16_t f2bf(float f) {
    __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(bf16_t, b);
}

// fp32 -> nearest bf16 -> fp32 in one instruction: the convert packs two values into the halves of a
// register, and a value placed in the high half over a zero low half is already the fp32 bit
// pattern of its rounded self (v_cvt_pk_bf16_f32 dst, 0, f), so no shift follows.
__device__ __forceinline__ float round_bf16(float f) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {0.0f, f};
    return __uint_as_float(__builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t)));
}

// Rounds through the storage type: identity for fp32, bf16 round trip for bf16.
template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
    static constexpr int VEC = 8;  // elements per 16-byte access
    static __device__ __forceinline__ float load(bf16_t v) { return bf2f(v); }
    static __device__ __forceinline__ bf16_t store(float f) { return f2bf(f); }
    static __device__ __forceinline__ float round(float f) { return round_bf16(f); }
};
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ float load(float v) { return v; }
    static __device__ __forceinline__ float store(float f) { return f; }
    static __device__ __forceinline__ float round(float f) { return f; }
};

// One 16-byte access worth of elements.
template <typename T> struct alignas(16) Vec16 {
    T v[Elem<T>::VEC];
};

template <typename T> __device__ __forceinline__ Vec16<T> ld16(const T* p) {
    return *reinterpret_cast<const Vec16<T>*>(p);
}
template <typename T> __device__ __forceinline__ void st16(T* p, const Vec16<T>& v) {
    *reinterpret_cast<Vec16<T>*>(p) = v;
}

// ------------------------------------------------------------------------------------------------
// Sum all-reduce over groups of G adjacent lanes (G = 1..64, power of two), wave64.
// The first four butterfly steps stay inside a 16-lane DPP row and use DPP permutations; the
// 32- and 64-lane steps go through the cross-lane permute unit.
// ------------------------------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
    return __int_as_float(r);
}

template <int G> __device__ __forceinline__ float group_sum(float v) {
    static_assert(G >= 1 && G <= 64 && (G & (G - 1)) == 0, "group size");
    if (G >= 2) v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]  : lane ^ 1
    if (G >= 4) v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]  : lane ^ 2
    if (G >= 8) v += dpp_f32<0x141>(v);  // row_half_mirror      : lane -> 7 - lane within 8
    if (G >= 16) v += dpp_f32<0x140>(v); // row_mirror           : lane -> 15 - lane within 16
    if (G >= 32) v += __shfl_xor(v, 16, 64);
    if (G >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ float gelu_tanh_f32(float x) {
    // 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3)  ==  x * sigmoid(2u)
    const float c = 0.7978845608028654f;
    float u = c * (x + 0.044715f * x * x * x);
    // 1 / (1 + exp(-2u)); exp via exp2 on the transcendental unit
    float e = __builtin_amdgcn_exp2f(-2.885390081777927f * u);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

}  // namespace flux
