// Device-side helpers shared by the gfx950 kernels: wave64 cross-lane
// primitives built on DPP, vector types for MFMA operands, static loops.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lg {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned uint2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// compile-time loop: f(std::integral_constant<int, I>) for I in [0, N)
template <int I>
struct ic {
    static constexpr int value = I;
    constexpr operator int() const { return I; }
};
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(ic<I>{});
        static_for<N, I + 1>(f);
    }
}

// DPP controls (GFX9 encoding)
constexpr int kDppRowRor = 0x120;       // + n, rotate right within a row of 16
constexpr int kDppRowNewBcast = 0x150;  // + n, lane n of each row of 16 to the whole row

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}

// value held by lane (row_base + N) broadcast to its row of 16 lanes
template <int N>
__device__ __forceinline__ float row_bcast(float v) {
    return dpp_f32<kDppRowNewBcast + N>(v);
}

// sum over each row of 16 lanes; every lane of the row gets the row total
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<kDppRowRor + 8>(v);
    v += dpp_f32<kDppRowRor + 4>(v);
    v += dpp_f32<kDppRowRor + 2>(v);
    v += dpp_f32<kDppRowRor + 1>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<kDppRowRor + 8>(v));
    v = fmaxf(v, dpp_f32<kDppRowRor + 4>(v));
    v = fmaxf(v, dpp_f32<kDppRowRor + 2>(v));
    v = fmaxf(v, dpp_f32<kDppRowRor + 1>(v));
    return v;
}

// sum over the 64 lanes of the wave; the result is wave-uniform
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    int b = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_readlane(b, 0)) +
           __int_as_float(__builtin_amdgcn_readlane(b, 16)) +
           __int_as_float(__builtin_amdgcn_readlane(b, 32)) +
           __int_as_float(__builtin_amdgcn_readlane(b, 48));
}

__device__ __forceinline__ float shfl_xor_f32(float v, int mask) {
    return __shfl_xor(v, mask, kWave);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace lg
