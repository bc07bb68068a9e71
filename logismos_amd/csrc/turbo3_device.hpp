// TurboQuant 3-bit head-row encoder shared by the kernels that write turbo3 KV pools
// (`encode_turbo3_0_head`, crates/quant/src/lib.rs:316-353): one wave encodes one 128-value
// head row, lane l holding elements l and l + 64.  The arithmetic follows the reference
// operation by operation -- the sum of squares is accumulated in element order, the
// butterflies run h = 1, 2, .., 64, division and square root are the correctly rounded
// ones -- so the encoded bytes are identical to the CPU function's.
#pragma once

#include "device_utils.hpp"

#include <hip/hip_fp16.h>

namespace lg {

constexpr int kTurbo3HeadBytes = 56;
constexpr int kTurbo3BlockBytes = 14;

static __device__ __constant__ const float kTurbo3Codebook[8] = {
    -0.1883972972f, -0.1181399059f, -0.0665857641f, -0.0216044751f,
    0.0216041461f,  0.0665854520f,  0.1181396281f,  0.1883970748f,
};

// fwht_128 over elements (a = element lane, b = element lane + 64) of a wave
template <int H>
__device__ __forceinline__ void wave_fwht_stage(float& a, float& b, int lane) {
    const float pa = lane_xor_f32<H>(a);
    const float pb = lane_xor_f32<H>(b);
    const bool hi = (lane & H) != 0;
    a = hi ? __fsub_rn(pa, a) : __fadd_rn(a, pa);
    b = hi ? __fsub_rn(pb, b) : __fadd_rn(b, pb);
}

__device__ __forceinline__ void wave_fwht_128(float& a, float& b, int lane) {
    wave_fwht_stage<1>(a, b, lane);
    wave_fwht_stage<2>(a, b, lane);
    wave_fwht_stage<4>(a, b, lane);
    wave_fwht_stage<8>(a, b, lane);
    wave_fwht_stage<16>(a, b, lane);
    wave_fwht_stage<32>(a, b, lane);
    const float x = a, y = b;
    a = __fadd_rn(x, y);
    b = __fsub_rn(x, y);
    const float scale = 0.08838834764831844f;  // the reference's f32 literal of 1/sqrt(128)
    a = __fmul_rn(a, scale);
    b = __fmul_rn(b, scale);
}

__device__ __forceinline__ unsigned turbo3_nearest(float v) {
    unsigned best = 0;
    float bd = fabsf(__fsub_rn(v, kTurbo3Codebook[0]));
#pragma unroll
    for (int i = 1; i < 8; ++i) {
        const float d = fabsf(__fsub_rn(v, kTurbo3Codebook[i]));
        if (d < bd) {  // the first minimum wins
            bd = d;
            best = i;
        }
    }
    return best;
}

// Encodes the row held as (a, b) by the 64 lanes of a wave into the 56 bytes at dst; `norm`
// is the row's L2 norm as turbo3_row_norm / turbo3_row_norm_serial compute it.
__device__ __forceinline__ void turbo3_encode_row_normed(float a, float b, float norm, int lane,
                                                         uint8_t* dst) {
    const bool live = norm > 1e-12f;
    a = live ? __fdiv_rn(a, norm) : 0.0f;
    b = live ? __fdiv_rn(b, norm) : 0.0f;
    wave_fwht_128(a, b, lane);

    // 3-bit indices of this lane's two elements, OR-reduced into their blocks' 96 bits
    const int p = lane & 31;
    const int bit = 3 * p;
    const int word = bit >> 5, sh = bit & 31;
    unsigned wa[3] = {0, 0, 0}, wb[3] = {0, 0, 0};
    {
        const unsigned long long va = (unsigned long long)turbo3_nearest(a) << sh;
        const unsigned long long vb = (unsigned long long)turbo3_nearest(b) << sh;
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            if (w == word) {
                wa[w] |= (unsigned)va;
                wb[w] |= (unsigned)vb;
            }
            if (w == word + 1) {
                wa[w] |= (unsigned)(va >> 32);
                wb[w] |= (unsigned)(vb >> 32);
            }
        }
    }
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        wa[w] |= (unsigned)lane_xor_i32<1>((int)wa[w]);
        wb[w] |= (unsigned)lane_xor_i32<1>((int)wb[w]);
        wa[w] |= (unsigned)lane_xor_i32<2>((int)wa[w]);
        wb[w] |= (unsigned)lane_xor_i32<2>((int)wb[w]);
        wa[w] |= (unsigned)lane_xor_i32<4>((int)wa[w]);
        wb[w] |= (unsigned)lane_xor_i32<4>((int)wb[w]);
        wa[w] |= (unsigned)lane_xor_i32<8>((int)wa[w]);
        wb[w] |= (unsigned)lane_xor_i32<8>((int)wb[w]);
        wa[w] |= (unsigned)lane_xor_i32<16>((int)wa[w]);
        wb[w] |= (unsigned)lane_xor_i32<16>((int)wb[w]);
    }
    // halfword p (< 7) of the two 14-byte blocks this half-wave owns: the norm, then the
    // six halfwords of the payload
    if (p < 7) {
        const unsigned short nh = __builtin_bit_cast(unsigned short, __float2half_rn(norm));
        const int k = p - 1;
        const unsigned short ha =
            p == 0 ? nh : (unsigned short)(wa[k < 0 ? 0 : (k >> 1)] >> (16 * (k & 1)));
        const unsigned short hb =
            p == 0 ? nh : (unsigned short)(wb[k < 0 ? 0 : (k >> 1)] >> (16 * (k & 1)));
        const int blk_a = lane >> 5, blk_b = 2 + (lane >> 5);
        reinterpret_cast<unsigned short*>(dst + kTurbo3BlockBytes * blk_a)[p] = ha;
        reinterpret_cast<unsigned short*>(dst + kTurbo3BlockBytes * blk_b)[p] = hb;
    }
}

// L2 norm of the row held as (a, b) by a wave: squares summed in element order, as the
// reference's loop does (128 dependent additions)
__device__ __forceinline__ float turbo3_row_norm(float a, float b) {
    const int asq = __float_as_int(__fmul_rn(a, a));
    const int bsq = __float_as_int(__fmul_rn(b, b));
    float sum_sq = 0.0f;
#pragma unroll
    for (int i = 0; i < 64; ++i)
        sum_sq = __fadd_rn(sum_sq, __int_as_float(__builtin_amdgcn_readlane(asq, i)));
#pragma unroll
    for (int i = 0; i < 64; ++i)
        sum_sq = __fadd_rn(sum_sq, __int_as_float(__builtin_amdgcn_readlane(bsq, i)));
    return __fsqrt_rn(sum_sq);
}

// The same norm computed by ONE lane from the row's 128 fp16 values in memory: 64 lanes do
// 64 rows at once, which is what makes the dependent chain affordable when many rows are
// encoded.  `row` is 16-byte aligned.
__device__ __forceinline__ float turbo3_row_norm_serial(const _Float16* row) {
    float sum_sq = 0.0f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const half8_t v = *reinterpret_cast<const half8_t*>(row + 8 * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = (float)v[e];
            sum_sq = __fadd_rn(sum_sq, __fmul_rn(x, x));
        }
    }
    return __fsqrt_rn(sum_sq);
}

__device__ __forceinline__ void turbo3_encode_row(float a, float b, int lane, uint8_t* dst) {
    turbo3_encode_row_normed(a, b, turbo3_row_norm(a, b), lane, dst);
}

}  // namespace lg
