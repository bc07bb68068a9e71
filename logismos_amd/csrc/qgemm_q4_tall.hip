// Q4G128 GEMM for a tall x (many activation rows: the prefill chunks of a mixed batch):
//   y[m][n] = bf16( sum_k x[m][k] * (q[n][k] - zero[n][k/128]) * scale[n][k/128] + bias[n] )
// `cpu_f32::linear_t` (crates/kernels/src/cpu_f32/mod.rs:271-345) at m = `seq` rows
// (crates/transformers/src/mlp.rs:104-111) over the dequantised matrix.
//
// The decode kernels keep at most 32 rows of x per workgroup and are bound by the weight
// stream; with hundreds of rows every weight byte is reused enough for the matrix cores to
// be the bound.  A workgroup of four waves owns a 128 x 128 tile of y (128 rows of x, 128
// weight rows) and walks K one group of 128 columns at a time:
//
// * x: the 128 x 128 bf16 slab of the group goes global -> registers -> LDS (double
//   buffered, one barrier per group), each 16-byte chunk in "pair order" (x0,x4,x1,x5,..) so
//   that it matches what the nibble unpack below produces; the threads that move a row's 16
//   chunks also reduce them to the row's sum over the group (one DPP row reduction), kept in
//   LDS beside the slab for the zero-point term.
// * weights: never touch LDS.  A lane of the v_mfma_f32_32x32x16_bf16 B operand is one weight
//   row and eight consecutive k = one dword of nibbles; lane (row, half h) reads the 32 bytes
//   [64 g + 32 h, +32) of its row for the whole group (two 16-byte loads, next group's in
//   flight), dword j feeding MFMA j.  A nibble becomes the bf16 value 128 + q with one
//   and-or per pair (exponent bits 0x4300), exact, so the products are exact and
//   accumulation is fp32; per group and output element
//       y += scale * (acc - (128 + zero) * sum_x),
//   where acc starts from zero at every group (the MFMA's C operand).
// * a wave owns a 64 x 64 quarter: 2 x 2 MFMA tiles, 32 MFMAs per group against 16 LDS
//   operand reads and 16 dwords of weights.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

constexpr int kTallTile = 128;               // rows of x and weight rows per workgroup
constexpr int kTallStride = 128 + 8;         // halfs per x row in LDS (272 bytes)
constexpr int kTallSlab = kTallTile * kTallStride;  // halfs per buffer

// NW: waves side by side on the weight rows, 2 (tile 128 x 128) or 4 (128 x 256).  F32OUT: y is
// fp32 (what the step executor keeps between operators) instead of bf16.
template <int NW, bool F32OUT>
__global__ __launch_bounds__(128 * NW, NW == 2 ? 2 : 1) void qgemm_q4g128_tall_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero,
    const float* __restrict__ bias, void* __restrict__ y_out, int m, int n, int k) {
    extern __shared__ uint4_t tall_lds[];
    uint16_t* const xs_lds = reinterpret_cast<uint16_t*>(tall_lds);              // 2 slabs of x
    float* const sum_lds = reinterpret_cast<float*>(xs_lds + 2 * kTallSlab);     // 2 x 128 sums

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int row0 = blockIdx.y * kTallTile;
    constexpr int THREADS = 128 * NW;
    constexpr int UPT = 2048 / THREADS;  // 16-byte chunks of a group's slab per thread
    constexpr int UH = UPT / 2;          // ... per half
    const int col0 = blockIdx.x * (64 * NW);
    const int wr = (wave / NW) * 64;  // this wave's 64 x 64 part of the tile
    const int wc = (wave % NW) * 64;
    const int r = lane & 31;
    const int h = lane >> 5;
    const int groups = k >> 7;

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    // ---- staging role for x: thread -> chunk tid % 16 of rows tid / 16 + (THREADS / 16) u
    const int s_chunk = tid & 15, s_row = tid >> 4;
    // a group's slab is moved in two halves (half as many registers in flight): a thread's
    // rows are s_row + (THREADS / 16) * u, u = UH * part .. + UH - 1
    uint4_t ra[UH];
    auto gload_x = [&](int g, int part) {
#pragma unroll
        for (int u = 0; u < UH; ++u) {
            const int gr = row0 + s_row + (THREADS / 16) * (UH * part + u);
            // rows past m re-read the last row (their results are never stored)
            const uint16_t* src = x + (int64_t)min(gr, m - 1) * k + g * 128 + s_chunk * 8;
            ra[u] = *reinterpret_cast<const uint4_t*>(src);
        }
    };
    auto lstore_x = [&](int buf, int part) {
#pragma unroll
        for (int u = 0; u < UH; ++u) {
            const int row = s_row + (THREADS / 16) * (UH * part + u);
            // the row's sum over this group: four two-element dot products with (1, 1), then
            // the 16 lanes that hold the row
            float psum = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) psum = dot2_bf16(ra[u][e], 0x3f803f80u, psum);
            const float gs = row16_sum(psum);
            // pair order (x0,x4)(x1,x5)(x2,x6)(x3,x7): one byte permute per dword
            uint4_t po;
            po[0] = __builtin_amdgcn_perm(ra[u][2], ra[u][0], 0x05040100u);
            po[1] = __builtin_amdgcn_perm(ra[u][2], ra[u][0], 0x07060302u);
            po[2] = __builtin_amdgcn_perm(ra[u][3], ra[u][1], 0x05040100u);
            po[3] = __builtin_amdgcn_perm(ra[u][3], ra[u][1], 0x07060302u);
            *reinterpret_cast<uint4_t*>(xs_lds + buf * kTallSlab + row * kTallStride + s_chunk * 8) =
                po;
            if (s_chunk == 0) sum_lds[buf * kTallTile + row] = gs;
        }
    };

    // ---- weights: lane (r, h) of n-tile j reads 32 bytes of row col0 + wc + 32 j + r
    // (32-bit element offsets: N * K and batch * K are below 2^31)
    unsigned woff[2], soff[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int gn = min(col0 + wc + 32 * j + r, n - 1);  // a row past n re-reads the last row
        woff[j] = (unsigned)gn * (unsigned)(k >> 1) + 32u * h;
        soff[j] = (unsigned)gn * (unsigned)groups;
    }
    // the 32 bytes of a group are consumed 16 at a time (MFMAs 0-3, then 4-7); each half is
    // requested again, for the next group, as soon as its last MFMA has been issued
    uint4_t wcur[2][2];
    // scales and zeros of two consecutive groups per request (one dword: a 2-byte request per
    // lane costs the texture addresser as much as a 16-byte one)
    unsigned scur[2], zcur[2], snext[2], znext[2];
    auto gload_w_half = [&](int g, int half) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            wcur[j][half] = reinterpret_cast<const uint4_t*>(qw + (woff[j] + (unsigned)g * 64u))[half];
    };
    auto gload_sz = [&](int g, unsigned (&s)[2], unsigned (&z)[2]) {  // g even: groups g, g + 1
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (g + 1 < groups) {
                __builtin_memcpy(&s[j], scale + soff[j] + (unsigned)g, 4);
                __builtin_memcpy(&z[j], zero + soff[j] + (unsigned)g, 4);
            } else {  // an odd number of groups: the last one alone
                s[j] = __builtin_bit_cast(unsigned short, scale[soff[j] + (unsigned)g]);
                z[j] = __builtin_bit_cast(unsigned short, zero[soff[j] + (unsigned)g]);
            }
        }
    };

    float16_t yacc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) yacc[i][j][e] = 0.0f;

    gload_x(0, 0);
    gload_w_half(0, 0);
    gload_w_half(0, 1);
    gload_sz(0, scur, zcur);
    lstore_x(0, 0);
    gload_x(0, 1);
    lstore_x(0, 1);
    __syncthreads();
    for (int g = 0; g < groups; ++g) {
        const int buf = g & 1;
        const bool more = g + 1 < groups;
        if (more) {
            gload_x(g + 1, 0);
            if (((g + 1) & 1) == 0) gload_sz(g + 1, snext, znext);
        }
        const uint16_t* xt = xs_lds + buf * kTallSlab;
        float16_t acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) {
            bf16x8_t av[2], bv[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                av[i] = *reinterpret_cast<const bf16x8_t*>(xt + (wr + 32 * i + r) * kTallStride +
                                                           64 * h + 8 * s8);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const unsigned wd = wcur[j][s8 >> 2][s8 & 3];
                uint4_t e4;
#pragma unroll
                for (int sft = 0; sft < 4; ++sft) e4[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                bv[j] = __builtin_bit_cast(bf16x8_t, e4);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i], bv[j], acc[i][j], 0,
                                                                        0, 0);
            if (more && s8 == 3) {
                gload_w_half(g + 1, 0);
                lstore_x(buf ^ 1, 0);  // that buffer's last readers passed the barrier of g - 1
                gload_x(g + 1, 1);
            }
            if (more && s8 == 7) gload_w_half(g + 1, 1);
        }
        // y += scale * (acc - (128 + zero) * sum_x): a lane's 16 results of a tile belong to one
        // weight row (one scale, one zero) and to the rows 8 (e / 4) + 4 h + e % 4 of x
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            float sx[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4_t v = *reinterpret_cast<const float4_t*>(
                    sum_lds + buf * kTallTile + wr + 32 * i + 8 * q + 4 * h);
#pragma unroll
                for (int e = 0; e < 4; ++e) sx[4 * q + e] = v[e];
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const unsigned short sb = (unsigned short)((g & 1) ? (scur[j] >> 16) : scur[j]);
                const unsigned short zb = (unsigned short)((g & 1) ? (zcur[j] >> 16) : zcur[j]);
                const float sf = __half2float(__builtin_bit_cast(__half, sb));
                const float off = 128.0f + __half2float(__builtin_bit_cast(__half, zb));
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    yacc[i][j][e] = fmaf(sf, fmaf(-off, sx[e], acc[i][j][e]), yacc[i][j][e]);
            }
        }
        if (more) {
            lstore_x(buf ^ 1, 1);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (((g + 1) & 1) == 0) {
                    scur[j] = snext[j];
                    zcur[j] = znext[j];
                }
        }
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int gn = col0 + wc + 32 * j + r;
        if (gn >= n) continue;
        const float bv = bias ? bias[gn] : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int gr = row0 + wr + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
                if (gr < m) {
                    if constexpr (F32OUT)
                        static_cast<float*>(y_out)[(int64_t)gr * n + gn] = yacc[i][j][e] + bv;
                    else
                        static_cast<uint16_t*>(y_out)[(int64_t)gr * n + gn] =
                            f32_to_bf16_rne(yacc[i][j][e] + bv);
                }
            }
    }
}

// Rows of x from which the tiled kernel is used: below, the decode kernels taken 32 rows at a
// time stream the weights at most three times and keep more workgroups busy.
bool qgemm_q4_tall_applies(int b, int n, int k) {
    return b > 96 && n >= 128 && k % 128 == 0;
}

template <int NW, bool F32OUT>
static hipError_t launch_tall(const void* x_bf16, const void* qw, const void* scale,
                              const void* zero, const float* bias, void* y, int b, int n, int k,
                              hipStream_t stream) {
    const dim3 grid((n + 64 * NW - 1) / (64 * NW), (b + kTallTile - 1) / kTallTile);
    if (grid.y > 65535u) return hipErrorInvalidValue;
    constexpr size_t lds = (size_t)2 * kTallSlab * 2 + (size_t)2 * kTallTile * 4;  // 70656 bytes
    static const hipError_t opt = hipFuncSetAttribute(
        reinterpret_cast<const void*>(qgemm_q4g128_tall_kernel<NW, F32OUT>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (opt != hipSuccess) return opt;
    qgemm_q4g128_tall_kernel<NW, F32OUT><<<grid, dim3(128 * NW), lds, stream>>>(
        static_cast<const uint16_t*>(x_bf16), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero), bias, y, b, n, k);
    return hipGetLastError();
}

// 128 x 128 tiles, two workgroups per CU.  (128 x 256 tiles with eight waves, where a staged
// slab of x serves twice the weight rows, measured 0-10 % slower on 8240-row problems: the
// kernel waits for its loads, not for the staging arithmetic.)
hipError_t qgemm_q4_tall_launch(const void* x_bf16, const void* qw, const void* scale,
                                const void* zero, const float* bias, void* y_bf16, int b, int n,
                                int k, hipStream_t stream) {
    return launch_tall<2, false>(x_bf16, qw, scale, zero, bias, y_bf16, b, n, k, stream);
}

hipError_t qgemm_q4_tall_f32_launch(const void* x_bf16, const void* qw, const void* scale,
                                    const void* zero, const float* bias, void* y_f32, int b,
                                    int n, int k, hipStream_t stream) {
    return launch_tall<2, true>(x_bf16, qw, scale, zero, bias, y_f32, b, n, k, stream);
}

}  // namespace lg
