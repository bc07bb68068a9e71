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

// (every control used here reads a live lane for every lane, so the value a disabled or
// unfed lane would keep is never needed: with none given, the compiler has no register to
// clear before each of these and can fold them into the instruction that uses the result)
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_mov_dpp(v, CTRL, 0xf, 0xf, true);
}

// value held by lane (row_base + N) broadcast to its row of 16 lanes
template <int N>
__device__ __forceinline__ float row_bcast(float v) {
    return dpp_f32<kDppRowNewBcast + N>(v);
}

// Split-K parts are added in part order, several loads in flight per round: body(ic<N>{}, q0)
// is called for the parts q0 .. q0 + N - 1, N = MAXR for full rounds and exactly what is left
// for the last one (a round padded with repeated loads of its first part costs the
// workgroup's L1 bandwidth as if they were real).
template <int N, class F>
__device__ __forceinline__ void part_round_of(int left, int q0, F&& body) {
    if (left == N) body(ic<N>{}, q0);
    else if constexpr (N > 1) part_round_of<N - 1>(left, q0, body);
}
template <int MAXR, class F>
__device__ __forceinline__ void for_part_rounds(int num_parts, F&& body) {
    for (int q0 = 0; q0 < num_parts; q0 += MAXR) {
        const int left = num_parts - q0;
        part_round_of<MAXR>(left < MAXR ? left : MAXR, q0, body);
    }
}

// value held by lane N of each group of four lanes, broadcast to the four (quad_perm)
template <int N>
__device__ __forceinline__ float quad_bcast(float v) {
    return dpp_f32<N | (N << 2) | (N << 4) | (N << 6)>(v);
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


// Value of lane (lane ^ M) for a power of two M, without the LDS crossbar that __shfl_xor
// goes through: quad permutes (1, 2), two masked row rotations (4: the banks of four lanes
// with bit 2 clear read four lanes up, the others four lanes down), a row rotation (8), and
// the gfx950 row / half-wave swaps (16, 32), whose two results hold the upper and the lower
// partner's values.
template <int M>
__device__ __forceinline__ int lane_xor_i32(int v) {
    static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "one bit");
    if constexpr (M == 1) {
        return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false);  // quad_perm [1,0,3,2]
    } else if constexpr (M == 2) {
        return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false);  // quad_perm [2,3,0,1]
    } else if constexpr (M == 4) {
        const int up = __builtin_amdgcn_update_dpp(0, v, kDppRowRor + 12, 0xf, 0x5, false);
        return __builtin_amdgcn_update_dpp(up, v, kDppRowRor + 4, 0xf, 0xa, false);
    } else if constexpr (M == 8) {
        return __builtin_amdgcn_update_dpp(0, v, kDppRowRor + 8, 0xf, 0xf, false);
    } else if constexpr (M == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
        return (int)((threadIdx.x & 16) ? r[0] : r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
        return (int)((threadIdx.x & 32) ? r[0] : r[1]);
    }
}
template <int M>
__device__ __forceinline__ float lane_xor_f32(float v) {
    return __int_as_float(lane_xor_i32<M>(__float_as_int(v)));
}

// through the LDS crossbar: one instruction and no temporaries, for register-tight kernels
__device__ __forceinline__ float shfl_xor_lds_f32(float v, int mask) {
    return __shfl_xor(v, mask, kWave);
}

// the same for a mask that is a constant once the caller's loop is unrolled
__device__ __forceinline__ float shfl_xor_f32(float v, int mask) {
    switch (mask) {
        case 1: return lane_xor_f32<1>(v);
        case 2: return lane_xor_f32<2>(v);
        case 4: return lane_xor_f32<4>(v);
        case 8: return lane_xor_f32<8>(v);
        case 16: return lane_xor_f32<16>(v);
        case 32: return lane_xor_f32<32>(v);
        default: return __shfl_xor(v, mask, kWave);
    }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace lg
