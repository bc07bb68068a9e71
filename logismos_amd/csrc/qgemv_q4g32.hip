// Q4G32 dequant-fused row-GEMV for gfx950 and the repack of ggml Q4_0 / Q4_1 block
// streams into the planar form it reads:
//   y[n] = sum_k x[k] * (q[n][k] * scale[n][k/32] + min[n][k/32])
//
// Same shape as the Q8G32 kernel: one wave64 owns R consecutive rows; a lane's 16-byte
// load is exactly one group of 32 nibbles (low nibble first, k order), so a lane applies
// one scale and one min per load: acc += scale * sum(q * x) + min * sum(x), the group's
// sum(x) being computed once per step and shared by the R rows.  Nibbles are split into
// bytes with two masks and converted with v_cvt_f32_ubyteN.  All R rows' loads are
// issued before the first use.
//
// Algorithmic bytes per call: n*k/2 (nibbles) + n*(k/32)*4 (scale, min) + 4k + 4n.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

template <int R>
__global__ __launch_bounds__(256) void qgemv_q4g32_kernel(const float* __restrict__ x,
                                                          const uint8_t* __restrict__ qw,
                                                          const __half* __restrict__ scale,
                                                          const __half* __restrict__ minv,
                                                          float* __restrict__ y,
        const float* __restrict__ bias, int n, int k) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t row0 = wave * R;
    if (row0 >= n) return;
    const int groups = k >> 5;
    const int64_t row_bytes = k >> 1;

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;

    for (int g = lane; g < groups; g += kWave) {
        uint4_t w[R];
        __half sc[R], mn[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // rows past the end re-read the last row (their result is dropped)
            const int64_t row = (row0 + r < n) ? (row0 + r) : (int64_t)(n - 1);
            w[r] = *reinterpret_cast<const uint4_t*>(qw + row * row_bytes + (int64_t)g * 16);
            sc[r] = scale[row * groups + g];
            mn[r] = minv[row * groups + g];
        }
        float xv[32];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float4_t t = *reinterpret_cast<const float4_t*>(x + g * 32 + 4 * i);
            xv[4 * i + 0] = t[0];
            xv[4 * i + 1] = t[1];
            xv[4 * i + 2] = t[2];
            xv[4 * i + 3] = t[3];
        }
        __builtin_amdgcn_sched_barrier(0);  // every load of the step is issued before any math
        float xsum = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) xsum += xv[i];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // word i: nibbles of elements 8i .. 8i+7; even elements in the low nibbles
                const unsigned v = w[r][i];
                const unsigned ev = v & 0x0F0F0F0Fu;         // elements 8i, 8i+2, 8i+4, 8i+6
                const unsigned od = (v >> 4) & 0x0F0F0F0Fu;  // elements 8i+1, 8i+3, ...
                s = fmaf(xv[8 * i + 0], (float)(ev & 0xffu), s);
                s = fmaf(xv[8 * i + 1], (float)(od & 0xffu), s);
                s = fmaf(xv[8 * i + 2], (float)((ev >> 8) & 0xffu), s);
                s = fmaf(xv[8 * i + 3], (float)((od >> 8) & 0xffu), s);
                s = fmaf(xv[8 * i + 4], (float)((ev >> 16) & 0xffu), s);
                s = fmaf(xv[8 * i + 5], (float)((od >> 16) & 0xffu), s);
                s = fmaf(xv[8 * i + 6], (float)(ev >> 24), s);
                s = fmaf(xv[8 * i + 7], (float)(od >> 24), s);
            }
            acc[r] = fmaf(s, __half2float(sc[r]), acc[r]);
            acc[r] = fmaf(xsum, __half2float(mn[r]), acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < n) y[row0 + r] = bias ? total + bias[row0 + r] : total;
    }
}

// The same product for rows of 32 .. 512 groups (K = 1024 .. 16384), with every load of a
// wave issued at once.  A wave's R consecutive rows are one contiguous run of R*K/2 bytes (and
// of R*K/32 scales / mins): lane l takes the groups l, l + 64, ... of that run, NP of them,
// whichever row they fall into, so that the wave pays the memory latency once.  x is staged
// in LDS in eight planes (quarter j of group c at xl[j * K/32 + c]) with the group sums of x
// beside them; a group's result goes to the accumulator of its row by comparison.  Eight
// waves per workgroup share one copy of x.
constexpr int kFlatWaves = 8;
template <int R, int NP>
__global__ __launch_bounds__(64 * kFlatWaves) void qgemv_q4g32_flat_kernel(const float* __restrict__ x,
                                                               const uint8_t* __restrict__ qw,
                                                               const __half* __restrict__ scale,
                                                               const __half* __restrict__ minv,
                                                               float* __restrict__ y,
        const float* __restrict__ bias, int n, int k) {
    extern __shared__ float4_t xl[];
    const int groups = k >> 5;
    float* xs = reinterpret_cast<float*>(xl + (size_t)8 * groups);
    const int lane = threadIdx.x & 63;
    const int64_t row0 = ((int64_t)blockIdx.x * kFlatWaves + (threadIdx.x >> 6)) * R;
    const int rows = row0 < n ? (int)min((int64_t)R, (int64_t)n - row0) : 0;
    const int valid = rows * groups;
    // a wave past the end, and groups past a wave's rows, re-read a group that exists
    const uint8_t* wbase = rows > 0 ? qw + row0 * (int64_t)(k >> 1) : qw;
    const int64_t g0 = rows > 0 ? row0 * groups : 0;

    uint4_t w[NP];
    __half sc[NP], mn[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = lane + 64 * i;
        const int pc = p < valid ? p : 0;
        w[i] = *reinterpret_cast<const uint4_t*>(wbase + (int64_t)pc * 16);
        sc[i] = scale[g0 + pc];
        mn[i] = minv[g0 + pc];
    }
    for (int c = threadIdx.x; c < groups; c += 64 * kFlatWaves) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float4_t v = reinterpret_cast<const float4_t*>(x)[c * 8 + j];
            xl[j * groups + c] = v;
            s += (v[0] + v[1]) + (v[2] + v[3]);
        }
        xs[c] = s;
    }
    __syncthreads();

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = lane + 64 * i;
        int r = 0;
#pragma unroll
        for (int j = 1; j < R; ++j) r += (p >= j * groups) ? 1 : 0;
        const bool live = p < valid;
        const int c = live ? p - r * groups : 0;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // word j: nibbles of elements 8j .. 8j+7; even elements in the low nibbles
            const unsigned v = w[i][j];
            const unsigned ev = v & 0x0F0F0F0Fu;
            const unsigned od = (v >> 4) & 0x0F0F0F0Fu;
            const float4_t xa = xl[(2 * j) * groups + c];
            const float4_t xb = xl[(2 * j + 1) * groups + c];
            s = fmaf(xa[0], (float)(ev & 0xffu), s);
            s = fmaf(xa[1], (float)(od & 0xffu), s);
            s = fmaf(xa[2], (float)((ev >> 8) & 0xffu), s);
            s = fmaf(xa[3], (float)((od >> 8) & 0xffu), s);
            s = fmaf(xb[0], (float)((ev >> 16) & 0xffu), s);
            s = fmaf(xb[1], (float)((od >> 16) & 0xffu), s);
            s = fmaf(xb[2], (float)(ev >> 24), s);
            s = fmaf(xb[3], (float)(od >> 24), s);
        }
        float v = fmaf(s, __half2float(sc[i]), xs[c] * __half2float(mn[i]));
        v = live ? v : 0.0f;
#pragma unroll
        for (int rr = 0; rr < R; ++rr) acc[rr] += (r == rr) ? v : 0.0f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && r < rows) y[row0 + r] = bias ? total + bias[row0 + r] : total;
    }
}

template <int R, int NP = 1>
static hipError_t launch_q4g32_flat(int np, const float* x, const uint8_t* qw, const __half* scale,
                                    const __half* minv, float* y, const float* bias, int n, int k,
                                    hipStream_t stream) {
    if constexpr (NP > (R == 1 ? 8 : 4)) {
        return hipErrorInvalidValue;
    } else {
        if (np != NP) return launch_q4g32_flat<R, NP + 1>(np, x, qw, scale, minv, y, bias, n, k, stream);
        const size_t lds = (size_t)(k / 32) * (8 * 16 + 4);  // at most 66 KiB (K = 16384)
        auto kern = qgemv_q4g32_flat_kernel<R, NP>;
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        const int64_t waves = ((int64_t)n + R - 1) / R;
        kern<<<dim3((unsigned)((waves + kFlatWaves - 1) / kFlatWaves)), dim3(64 * kFlatWaves), lds,
               stream>>>(x, qw, scale, minv, y, bias, n, k);
        return hipGetLastError();
    }
}

// Rows per wave of the flat kernel, 0 when it does not apply.  At most 256 groups (four per
// lane) per wave unless a single row is longer; fewer rows per wave while that leaves fewer
// than four waves per CU.
static int q4g32_flat_rows(int n, int k, int cus) {
    const int groups = k / 32;
    if (groups < 32 || groups > 512) return 0;
    int r = 8;
    while (r > 1 && r * groups > 256) r >>= 1;
    while (r > 1 && (n + r - 1) / r < 4 * cus) r >>= 1;
    return r;
}

// ggml Q4_0 (18-byte blocks: f16 d, 16 bytes) or Q4_1 (20-byte blocks: f16 d, f16 m, 16
// bytes) stream -> planar Q4G32.  ggml keeps value j in the low and value j + 16 in the
// high nibble of byte j; the planar form is in k order.  One thread per block.
template <bool HAS_MIN>
__global__ __launch_bounds__(256) void repack_q4_blocks_kernel(const uint8_t* __restrict__ blocks,
                                                               uint8_t* __restrict__ qw,
                                                               uint16_t* __restrict__ scale,
                                                               uint16_t* __restrict__ minv,
                                                               int64_t num_blocks) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= num_blocks) return;
    constexpr int BS = HAS_MIN ? 20 : 18;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(blocks + b * BS);  // 2-byte aligned
    const uint16_t dh = src[0];
    scale[b] = dh;
    if (HAS_MIN) {
        minv[b] = src[1];
    } else {
        const __half d = __builtin_bit_cast(__half, dh);
        const __half m = __float2half_rn(-8.0f * __half2float(d));
        minv[b] = __builtin_bit_cast(uint16_t, m);
    }
    const uint16_t* qs = src + (HAS_MIN ? 2 : 1);
    uint8_t lo[8], hi[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const unsigned two = qs[t];  // ggml bytes 2t, 2t+1
        const unsigned b0 = two & 0xffu, b1 = two >> 8;
        lo[t] = (uint8_t)((b0 & 0x0Fu) | ((b1 & 0x0Fu) << 4));
        hi[t] = (uint8_t)((b0 >> 4) | ((b1 >> 4) << 4));
    }
    uint2_t o0, o1;
    o0[0] = lo[0] | (lo[1] << 8) | (lo[2] << 16) | ((unsigned)lo[3] << 24);
    o0[1] = lo[4] | (lo[5] << 8) | (lo[6] << 16) | ((unsigned)lo[7] << 24);
    o1[0] = hi[0] | (hi[1] << 8) | (hi[2] << 16) | ((unsigned)hi[3] << 24);
    o1[1] = hi[4] | (hi[5] << 8) | (hi[6] << 16) | ((unsigned)hi[7] << 24);
    uint2_t* dst = reinterpret_cast<uint2_t*>(qw + b * 16);
    dst[0] = o0;
    dst[1] = o1;
}

}  // namespace lg

extern "C" logismos_status_t logismos_check_qgemv_q4g32_shape(int n, int k, char* msg,
                                                              size_t msg_cap) {
    if (n <= 0) return lg::reject(msg, msg_cap, "qgemv_q4g32: N must be positive, got %d", n);
    if (k <= 0) return lg::reject(msg, msg_cap, "qgemv_q4g32: K must be positive, got %d", k);
    if (k % 32 != 0)
        return lg::reject(msg, msg_cap, "qgemv_q4g32: K = %d is not a multiple of the group size 32", k);
    if ((int64_t)n * (int64_t)k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "qgemv_q4g32: N*K = %lld exceeds i32::MAX",
                          (long long)((int64_t)n * k));
    return 0;
}

extern "C" logismos_status_t logismos_launch_qgemv_q4g32_f32_bias(
    const void* x_f32, const void* qw_u8, const void* scale_f16, const void* min_f16,
    const void* bias_f32, void* y_f32, int n, int k, logismos_stream_t stream) {
    if (logismos_check_qgemv_q4g32_shape(n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!x_f32 || !qw_u8 || !scale_f16 || !min_f16 || !y_f32) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) & 15u) || (reinterpret_cast<uintptr_t>(x_f32) & 15u))
        return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* xp = static_cast<const float*>(x_f32);
    auto* qp = static_cast<const uint8_t*>(qw_u8);
    auto* sp = static_cast<const __half*>(scale_f16);
    auto* mp = static_cast<const __half*>(min_f16);
    auto* yp = static_cast<float*>(y_f32);
    auto* bp = static_cast<const float*>(bias_f32);  // may be null: no bias
    if (const int fr = lg::q4g32_flat_rows(n, k, lg::device_cu_count()); fr > 0) {
        const int np = (fr * (k / 32) + 63) / 64;
        switch (fr) {
            case 8: return lg::launch_q4g32_flat<8>(np, xp, qp, sp, mp, yp, bp, n, k, st);
            case 4: return lg::launch_q4g32_flat<4>(np, xp, qp, sp, mp, yp, bp, n, k, st);
            case 2: return lg::launch_q4g32_flat<2>(np, xp, qp, sp, mp, yp, bp, n, k, st);
            default: return lg::launch_q4g32_flat<1>(np, xp, qp, sp, mp, yp, bp, n, k, st);
        }
    }
    constexpr int R = 4;
    const int waves = (n + R - 1) / R;
    const int wpb = 4;
    dim3 grid((waves + wpb - 1) / wpb), block(wpb * 64);
    lg::qgemv_q4g32_kernel<R><<<grid, block, 0, st>>>(xp, qp, sp, mp, yp, bp, n, k);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_qgemv_q4g32_f32(const void* x_f32, const void* qw_u8,
                                                             const void* scale_f16,
                                                             const void* min_f16, void* y_f32,
                                                             int n, int k,
                                                             logismos_stream_t stream) {
    return logismos_launch_qgemv_q4g32_f32_bias(x_f32, qw_u8, scale_f16, min_f16, nullptr, y_f32, n,
                                                k, stream);
}

static logismos_status_t repack_q4(bool has_min, const void* blocks, void* qw_u8, void* scale_f16,
                                   void* min_f16, int n, int k, logismos_stream_t stream) {
    if (logismos_check_qgemv_q4g32_shape(n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!blocks || !qw_u8 || !scale_f16 || !min_f16) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(blocks) & 1u) || (reinterpret_cast<uintptr_t>(qw_u8) & 7u))
        return hipErrorInvalidValue;
    const int64_t num_blocks = (int64_t)n * (k / 32);
    dim3 grid((unsigned)((num_blocks + 255) / 256)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* b = static_cast<const uint8_t*>(blocks);
    auto* q = static_cast<uint8_t*>(qw_u8);
    auto* s = static_cast<uint16_t*>(scale_f16);
    auto* m = static_cast<uint16_t*>(min_f16);
    if (has_min)
        lg::repack_q4_blocks_kernel<true><<<grid, block, 0, st>>>(b, q, s, m, num_blocks);
    else
        lg::repack_q4_blocks_kernel<false><<<grid, block, 0, st>>>(b, q, s, m, num_blocks);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_repack_q4_0(const void* blocks_q4_0, void* qw_u8,
                                                         void* scale_f16, void* min_f16, int n,
                                                         int k, logismos_stream_t stream) {
    return repack_q4(false, blocks_q4_0, qw_u8, scale_f16, min_f16, n, k, stream);
}

extern "C" logismos_status_t logismos_launch_repack_q4_1(const void* blocks_q4_1, void* qw_u8,
                                                         void* scale_f16, void* min_f16, int n,
                                                         int k, logismos_stream_t stream) {
    return repack_q4(true, blocks_q4_1, qw_u8, scale_f16, min_f16, n, k, stream);
}
