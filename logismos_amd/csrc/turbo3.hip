// TurboQuant 3-bit KV codec on the GPU: encoding new K/V rows into turbo3 paged pools and
// decoding rows back (`encode_turbo3_0_head` / `decode_turbo3_0_head`,
// crates/quant/src/lib.rs:316-353,376-413).
//
// A head row (128 values) becomes four 14-byte blocks {fp16 norm, 32 x 3-bit indices}: the
// values are divided by their L2 norm, Walsh-Hadamard transformed (`fwht_128`, :88-113) and
// each coefficient replaced by the index of the nearest of eight centroids
// (`TURBO3_CODEBOOK`, :66-80).  One wave handles one head row; lane l holds elements l and
// l + 64.  The arithmetic follows the reference operation by operation -- the sum of
// squares is accumulated in element order, the butterflies run h = 1, 2, .., 64, division
// and square root are the correctly rounded ones -- so the encoded bytes and the decoded
// f32 values are bit-identical to the CPU functions.
//
// Pool layout: `[num_blocks][block_size][num_kv_heads][56]` bytes, same slots and block
// tables as the fp16 pools.
#include "device_utils.hpp"
#include "launch_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

constexpr int kTurbo3HeadBytes = 56;
constexpr int kTurbo3BlockBytes = 14;

__device__ __constant__ float kTurbo3Codebook[8] = {
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

// one wave per (token, kv head, K|V); block = 4 waves
__global__ __launch_bounds__(256) void kv_write_turbo3_kernel(
    const _Float16* __restrict__ k_new, const _Float16* __restrict__ v_new,
    uint8_t* __restrict__ k_pool, uint8_t* __restrict__ v_pool,
    const int64_t* __restrict__ slot_mapping, int total_tokens, int hkv) {
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (int64_t)total_tokens * hkv * 2) return;
    const int which = (int)(item & 1);
    const int64_t th = item >> 1;
    const int t = (int)(th / hkv);
    const int h = (int)(th - (int64_t)t * hkv);
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    const _Float16* src = (which ? v_new : k_new) + ((int64_t)t * hkv + h) * 128;
    float a = (float)src[lane];
    float b = (float)src[lane + 64];

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
        uint8_t* dst = (which ? v_pool : k_pool) + (slot * hkv + h) * kTurbo3HeadBytes;
        const int blk_a = lane >> 5, blk_b = 2 + (lane >> 5);
        reinterpret_cast<unsigned short*>(dst + kTurbo3BlockBytes * blk_a)[p] = ha;
        reinterpret_cast<unsigned short*>(dst + kTurbo3BlockBytes * blk_b)[p] = hb;
    }
}

__device__ __forceinline__ unsigned turbo3_index_at(const uint8_t* head, int e) {
    const int blk = e >> 5, bit = 3 * (e & 31);
    const uint8_t* pay = head + kTurbo3BlockBytes * blk + 2;
    unsigned v = pay[bit >> 3];
    if ((bit & 7) > 5) v |= (unsigned)pay[(bit >> 3) + 1] << 8;
    return (v >> (bit & 7)) & 7u;
}

// Rows [start_pos, start_pos + n_tokens) of one sequence, decoded to f32; one wave per
// (token, kv head, K|V)
__global__ __launch_bounds__(256) void kv_gather_turbo3_kernel(
    const uint8_t* __restrict__ k_pool, const uint8_t* __restrict__ v_pool,
    const int32_t* __restrict__ bt_row, float* __restrict__ k_out, float* __restrict__ v_out,
    int start_pos, int n_tokens, int hkv, int block_size) {
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (int64_t)n_tokens * hkv * 2) return;
    const int which = (int)(item & 1);
    const int64_t th = item >> 1;
    const int t = (int)(th / hkv);
    const int h = (int)(th - (int64_t)t * hkv);
    const int pos = start_pos + t;
    const int bi = pos / block_size;
    const int64_t slot = (int64_t)bt_row[bi] * block_size + (pos - bi * block_size);
    const uint8_t* head = (which ? v_pool : k_pool) + (slot * hkv + h) * kTurbo3HeadBytes;
    float a = kTurbo3Codebook[turbo3_index_at(head, lane)];
    float b = kTurbo3Codebook[turbo3_index_at(head, lane + 64)];
    wave_fwht_128(a, b, lane);
    const unsigned short nh = *reinterpret_cast<const unsigned short*>(head);  // first block's
    const float norm = __half2float(__builtin_bit_cast(__half, nh));
    float* dst = (which ? v_out : k_out) + ((int64_t)t * hkv + h) * 128;
    dst[lane] = __fmul_rn(a, norm);
    dst[lane + 64] = __fmul_rn(b, norm);
}

}  // namespace lg

extern "C" logismos_status_t logismos_launch_kv_write_turbo3(
    const void* k_new_f16, const void* v_new_f16, void* k_pool_t3, void* v_pool_t3,
    const int64_t* slot_mapping, int total_tokens, int num_kv_heads, logismos_stream_t stream) {
    if (total_tokens < 0 || num_kv_heads <= 0) return hipErrorInvalidValue;
    if ((int64_t)total_tokens * num_kv_heads > (int64_t)INT32_MAX / 128) return hipErrorInvalidValue;
    if (total_tokens == 0) return hipSuccess;
    if (!k_new_f16 || !v_new_f16 || !k_pool_t3 || !v_pool_t3 || !slot_mapping)
        return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(k_pool_t3) | reinterpret_cast<uintptr_t>(v_pool_t3)) & 1u)
        return hipErrorInvalidValue;
    const int64_t items = (int64_t)total_tokens * num_kv_heads * 2;
    lg::kv_write_turbo3_kernel<<<dim3((unsigned)((items + 3) / 4)), dim3(256), 0,
                                 static_cast<hipStream_t>(stream)>>>(
        static_cast<const _Float16*>(k_new_f16), static_cast<const _Float16*>(v_new_f16),
        static_cast<uint8_t*>(k_pool_t3), static_cast<uint8_t*>(v_pool_t3), slot_mapping,
        total_tokens, num_kv_heads);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_kv_gather_turbo3_f32(
    const void* k_pool_t3, const void* v_pool_t3, const int32_t* block_table_row, void* k_out_f32,
    void* v_out_f32, int start_pos, int n_tokens, int num_kv_heads, int block_size,
    logismos_stream_t stream) {
    if (start_pos < 0 || n_tokens < 0 || num_kv_heads <= 0 || block_size <= 0)
        return hipErrorInvalidValue;
    if ((int64_t)start_pos + n_tokens > (int64_t)INT32_MAX ||
        (int64_t)n_tokens * num_kv_heads > (int64_t)INT32_MAX / 128)
        return hipErrorInvalidValue;
    if (n_tokens == 0) return hipSuccess;
    if (!k_pool_t3 || !v_pool_t3 || !block_table_row || !k_out_f32 || !v_out_f32)
        return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(k_pool_t3) | reinterpret_cast<uintptr_t>(v_pool_t3)) & 1u)
        return hipErrorInvalidValue;
    const int64_t items = (int64_t)n_tokens * num_kv_heads * 2;
    lg::kv_gather_turbo3_kernel<<<dim3((unsigned)((items + 3) / 4)), dim3(256), 0,
                                  static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint8_t*>(k_pool_t3), static_cast<const uint8_t*>(v_pool_t3),
        block_table_row, static_cast<float*>(k_out_f32), static_cast<float*>(v_out_f32), start_pos,
        n_tokens, num_kv_heads, block_size);
    return hipGetLastError();
}
