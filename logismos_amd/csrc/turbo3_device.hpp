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
__device__ __forceinline__ void wave_fwht_128(float& a, float& b, int lane) {
#pragma unroll
    for (int h = 1; h < 64; h <<= 1) {
        const float pa = shfl_xor_f32(a, h);
        const float pb = shfl_xor_f32(b, h);
        const bool hi = (lane & h) != 0;
        a = hi ? __fsub_rn(pa, a) : __fadd_rn(a, pa);
        b = hi ? __fsub_rn(pb, b) : __fadd_rn(b, pb);
    }
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

// Encodes the row held as (a, b) by the 64 lanes of a wave into the 56 bytes at dst.
__device__ __forceinline__ void turbo3_encode_row(float a, float b, int lane, uint8_t* dst) {
    // L2 norm: squares summed in element order, as the reference's loop does
    const int asq = __float_as_int(__fmul_rn(a, a));
    const int bsq = __float_as_int(__fmul_rn(b, b));
    float sum_sq = 0.0f;
#pragma unroll
    for (int i = 0; i < 64; ++i)
        sum_sq = __fadd_rn(sum_sq, __int_as_float(__builtin_amdgcn_readlane(asq, i)));
#pragma unroll
    for (int i = 0; i < 64; ++i)
        sum_sq = __fadd_rn(sum_sq, __int_as_float(__builtin_amdgcn_readlane(bsq, i)));
    const float norm = __fsqrt_rn(sum_sq);
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
    for (int m = 1; m < 32; m <<= 1)
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            wa[w] |= (unsigned)__shfl_xor((int)wa[w], m, 64);
            wb[w] |= (unsigned)__shfl_xor((int)wb[w], m, 64);
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

}  // namespace lg
