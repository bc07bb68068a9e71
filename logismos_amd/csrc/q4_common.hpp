// Helpers shared by the Q4G128 kernels: bf16 bit tricks, the pair order of x,
// the nibble mask of the magic-number unpack.
#pragma once

#include "device_utils.hpp"

namespace lg {

__device__ __forceinline__ float bf16_lo_to_f32(unsigned v) { return __uint_as_float(v << 16); }
__device__ __forceinline__ float bf16_hi_to_f32(unsigned v) {
    return __uint_as_float(v & 0xffff0000u);
}
__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float dot2_bf16(unsigned a, unsigned b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), c, false);
}

// 8 consecutive bf16 (x0..x7 in four dwords) -> pairs (x0,x4) (x1,x5) (x2,x6) (x3,x7)
__device__ __forceinline__ uint4_t pair_order(uint4_t d) {
    uint4_t o;
    o[0] = (d[0] & 0xffffu) | (d[2] << 16);
    o[1] = (d[0] >> 16) | (d[2] & 0xffff0000u);
    o[2] = (d[1] & 0xffffu) | (d[3] << 16);
    o[3] = (d[1] >> 16) | (d[3] & 0xffff0000u);
    return o;
}
__device__ __forceinline__ float sum8_bf16(uint4_t d) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s += bf16_lo_to_f32(d[i]) + bf16_hi_to_f32(d[i]);
    return s;
}

constexpr unsigned kNibMask = 0x000F000Fu;


// "Prepared" form of a batch of activations for the Q4G128 MFMA kernels: what the
// kernels otherwise build in LDS per workgroup, built once by the producer.
//   xp  uint4 [K/8][BP]   chunk c of batch row r: its 8 bf16 in pair order
//   xg  float [K/128][BP] sum of the (bf16-rounded) x over each group
// BP = 16 for up to 16 batch rows, else 32; rows >= b are never read for a stored
// result (row i of the MFMA A operand only reaches row i of the product).
__host__ __device__ inline int xprep_bp(int b) { return b <= 16 ? 16 : 32; }
__host__ __device__ inline size_t xprep_xg_offset(int b, int k) {
    return (size_t)(k / 8) * xprep_bp(b) * 16;
}
__host__ __device__ inline size_t xprep_bytes(int b, int k) {
    return xprep_xg_offset(b, k) + (size_t)(k / 128) * xprep_bp(b) * 4;
}

// Workspace of the Q4G128 GEMM for many rows (qgemm_q4_tallp.hip), first part: what its first
// pass -- or the operator that produces x -- writes.
//   xp  bf16  [m_pad][K]  x in pair order per 16-byte chunk, rows >= m zero, m_pad = m rounded
//                         up to the kernel's 128-row tiles
//   xs  float             the sum of the bf16 values of every row and group of 128 columns,
//                         as [row tile][block of w pairs of groups][group's place in its
//                         pair][row of the tile][pair]; w = pairs of groups the kernel loads
//                         at once (tall_pairs_per_load)
constexpr int kTallTileRows = 128;
__host__ __device__ inline int tall_padded_rows(int m) {
    return (m + kTallTileRows - 1) / kTallTileRows * kTallTileRows;
}
__host__ __device__ inline size_t tall_sums_offset(int m, int k) {
    return ((size_t)tall_padded_rows(m) * k * 2 + 255) & ~(size_t)255;
}
__host__ __device__ inline int64_t tall_sum_index(int64_t row, int g, int k, int w) {
    const int bl = 2 * w;
    const int64_t block = (row / kTallTileRows) * ((k >> 7) / bl) + g / bl;
    const int in_block = g % bl;
    return ((block * 2 + (in_block & 1)) * kTallTileRows + row % kTallTileRows) * w + (in_block >> 1);
}
// as many pairs of groups per load as K (whole blocks) and the alignment of the scales and
// zeros (a load of 4, 8 or 16 bytes per row) allow
inline int tall_pairs_per_load(int k, const void* scale, const void* zero) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(scale) | reinterpret_cast<uintptr_t>(zero);
    if (k % 1024 == 0 && (a & 15u) == 0) return 4;
    if (k % 512 == 0 && (a & 7u) == 0) return 2;
    return 1;
}

inline int device_cu_count() {
    static const int count = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0)
            return 256;
        return cus;
    }();
    return count;
}

}  // namespace lg
