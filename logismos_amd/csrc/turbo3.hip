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
#include "turbo3_device.hpp"

#include <hip/hip_fp16.h>

namespace lg {

// One wave per kT3RowsPerWave rows, a row being one (token, kv head, K|V): first a lane per
// row computes that row's norm on its own (the reference adds the 128 squares one after the
// other; done across a wave that chain costs 256 dependent instructions per row), then the
// wave encodes the rows one at a time, lane l holding elements l and l + 64, the next row's
// elements already requested.  block = 4 waves
constexpr int kT3RowsPerWave = 16;

__global__ __launch_bounds__(256) void kv_write_turbo3_kernel(
    const _Float16* __restrict__ k_new, const _Float16* __restrict__ v_new,
    uint8_t* __restrict__ k_pool, uint8_t* __restrict__ v_pool,
    const int64_t* __restrict__ slot_mapping, int total_tokens, int hkv) {
    constexpr int RW = kT3RowsPerWave;
    const int lane = threadIdx.x & 63;
    const int64_t items = (int64_t)total_tokens * hkv * 2;
    const int64_t first = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RW;
    if (first >= items) return;
    auto source = [&](int64_t item) {
        const int64_t th = item >> 1;
        return ((item & 1) ? v_new : k_new) + th * 128;
    };
    const int rows = (int)(items - first < RW ? items - first : RW);
    float my_norm = 0.0f;
    if (lane < rows) my_norm = turbo3_row_norm_serial(source(first + lane));
    const _Float16* src = source(first);
    float a = (float)src[lane], b = (float)src[lane + 64];
    for (int r = 0; r < rows; ++r) {
        const int64_t item = first + r;
        const float norm = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_norm), r));
        const float ca = a, cb = b;
        if (r + 1 < rows) {
            const _Float16* nxt = source(item + 1);
            a = (float)nxt[lane];
            b = (float)nxt[lane + 64];
        }
        const int64_t th = item >> 1;
        const int t = (int)(th / hkv);
        const int h = (int)(th - (int64_t)t * hkv);
        const int64_t slot = slot_mapping[t];
        if (slot < 0) continue;  // uniform
        uint8_t* dst = ((item & 1) ? v_pool : k_pool) + (slot * hkv + h) * kTurbo3HeadBytes;
        turbo3_encode_row_normed(ca, cb, norm, lane, dst);
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
    if ((reinterpret_cast<uintptr_t>(k_new_f16) | reinterpret_cast<uintptr_t>(v_new_f16)) & 15u)
        return hipErrorInvalidValue;
    const int64_t items = (int64_t)total_tokens * num_kv_heads * 2;
    const int64_t per_block = 4 * lg::kT3RowsPerWave;
    lg::kv_write_turbo3_kernel<<<dim3((unsigned)((items + per_block - 1) / per_block)), dim3(256), 0,
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
