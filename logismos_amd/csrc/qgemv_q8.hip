// Q8G32 dequant-fused row-GEMV for gfx950: y[n] = sum_k x[k] * d[n][k/32] * qs[n][k].
//
// Bandwidth-bound streaming kernel.  One wave64 owns R consecutive rows of
// the weight; each lane reads 16-byte pieces of the int8 plane
// (global_load_dwordx4, a row is contiguous so a wave instruction covers 1 KiB
// of one row), converts the bytes in registers (sign-extending SDWA converts),
// multiplies by the 16 matching x values and applies the group's fp16 scale
// once per 16 elements.  All R rows' loads are issued before the first use so
// that R*16 B per lane are in flight.  Per-row totals are reduced with DPP row
// rotations and four v_readlane.
//
// Algorithmic bytes per call: n*k (int8) + n*(k/32)*2 (scales) + 4k + 4n.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

template <int R>
__global__ __launch_bounds__(256) void qgemv_q8g32_kernel(const float* __restrict__ x,
                                                          const int8_t* __restrict__ qs,
                                                          const __half* __restrict__ d,
                                                          float* __restrict__ y,
        const float* __restrict__ bias, int n, int k) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t row0 = wave * R;
    if (row0 >= n) return;
    const int groups = k >> 5;

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;

    for (int k0 = lane * 16; k0 < k; k0 += kWave * 16) {
        int4_t w[R];
        __half sc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // rows past the end re-read the last row (their result is dropped)
            const int64_t row = (row0 + r < n) ? (row0 + r) : (int64_t)(n - 1);
            w[r] = *reinterpret_cast<const int4_t*>(qs + row * k + k0);
            sc[r] = d[row * groups + (k0 >> 5)];
        }
        float xv[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4_t t = *reinterpret_cast<const float4_t*>(x + k0 + 4 * i);
            xv[4 * i + 0] = t[0];
            xv[4 * i + 1] = t[1];
            xv[4 * i + 2] = t[2];
            xv[4 * i + 3] = t[3];
        }
        __builtin_amdgcn_sched_barrier(0);  // every load of the step is issued before any math
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int v = w[r][i];
                s = fmaf(xv[4 * i + 0], (float)(int8_t)(v), s);
                s = fmaf(xv[4 * i + 1], (float)(int8_t)(v >> 8), s);
                s = fmaf(xv[4 * i + 2], (float)(int8_t)(v >> 16), s);
                s = fmaf(xv[4 * i + 3], (float)(int8_t)(v >> 24), s);
            }
            acc[r] = fmaf(s, __half2float(sc[r]), acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < n) y[row0 + r] = bias ? total + bias[row0 + r] : total;
    }
}

// The same product for rows of 512 .. 8192 bytes, with every load of a wave issued at once.
// A wave's R consecutive rows are one contiguous run of R*K bytes (and of R*K/32 scales):
// lane l takes the 16-byte pieces l, l + 64, ... of that run, NP of them, whatever row they
// fall into, so that no lane idles when K is not a multiple of 1024 and the wave pays the
// memory latency once instead of once per 1024 columns.  x is staged in LDS in four planes
// (quarter j of piece c at xl[j * K/16 + c]) so that neighbouring lanes read neighbouring
// 16-byte words.  A piece's partial sum goes to the accumulator of its row by comparison.
// Eight waves per workgroup share one copy of x (8960 x 1536: 5.5 us against 5.75 with four).
constexpr int kFlatWaves = 8;
template <int R, int NP>
__global__ __launch_bounds__(64 * kFlatWaves) void qgemv_q8g32_flat_kernel(const float* __restrict__ x,
                                                               const int8_t* __restrict__ qs,
                                                               const __half* __restrict__ d,
                                                               float* __restrict__ y,
        const float* __restrict__ bias, int n, int k) {
    extern __shared__ float4_t xl[];
    const int lane = threadIdx.x & 63;
    const int ppr = k >> 4;  // pieces per row
    const int64_t wave = (int64_t)blockIdx.x * kFlatWaves + (threadIdx.x >> 6);
    const int64_t row0 = wave * R;
    const int rows = row0 < n ? (int)min((int64_t)R, (int64_t)n - row0) : 0;
    const int valid = rows * ppr;
    // a wave past the end, and pieces past a wave's rows, re-read a piece that exists
    const int8_t* wbase = rows > 0 ? qs + row0 * k : qs;
    const __half* dbase = rows > 0 ? d + row0 * (k >> 5) : d;

    int4_t w[NP];
    __half sc[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = lane + 64 * i;
        const int pc = p < valid ? p : 0;
        w[i] = *reinterpret_cast<const int4_t*>(wbase + (int64_t)pc * 16);
        sc[i] = dbase[pc >> 1];
    }
    for (int f = threadIdx.x; f < (k >> 2); f += 64 * kFlatWaves)
        xl[(f & 3) * ppr + (f >> 2)] = reinterpret_cast<const float4_t*>(x)[f];
    __syncthreads();

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = lane + 64 * i;
        int r = 0;
#pragma unroll
        for (int j = 1; j < R; ++j) r += (p >= j * ppr) ? 1 : 0;
        const bool live = p < valid;
        const int c = live ? p - r * ppr : 0;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4_t xv = xl[j * ppr + c];
            const int v = w[i][j];
            s = fmaf(xv[0], (float)(int8_t)(v), s);
            s = fmaf(xv[1], (float)(int8_t)(v >> 8), s);
            s = fmaf(xv[2], (float)(int8_t)(v >> 16), s);
            s = fmaf(xv[3], (float)(int8_t)(v >> 24), s);
        }
        const float v = live ? s * __half2float(sc[i]) : 0.0f;
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
static hipError_t launch_flat(int np, const float* x, const int8_t* qs, const __half* d, float* y,
                              const float* bias, int n, int k, hipStream_t stream) {
    if constexpr (NP > 8) {
        return hipErrorInvalidValue;
    } else {
        if (np != NP) return launch_flat<R, NP + 1>(np, x, qs, d, y, bias, n, k, stream);
        const int64_t waves = ((int64_t)n + R - 1) / R;
        qgemv_q8g32_flat_kernel<R, NP>
            <<<dim3((unsigned)((waves + kFlatWaves - 1) / kFlatWaves)), dim3(64 * kFlatWaves),
               (size_t)k * 4, stream>>>(x, qs, d, y, bias, n, k);
        return hipGetLastError();
    }
}

// Rows per wave of the flat kernel for this shape, 0 when it does not apply (rows shorter than
// 512 or longer than 8192 bytes).  At most 256 pieces (four per lane) per wave unless a
// single row is longer: on 8960 x 1536 and 4096 x 4096 matrices two to four pieces per lane
// measured 8 % faster than six or eight; fewer rows per wave while that leaves fewer than
// four waves per CU.
static int flat_rows(int n, int k) {
    const int ppr = k / 16;
    if (k % 16 != 0 || ppr < 32 || ppr > 512) return 0;
    int r = 8;
    while (r > 1 && r * ppr > 256) r >>= 1;
    while (r > 1 && (n + r - 1) / r < 4 * device_cu_count()) r >>= 1;
    return r;
}

// ggml Q8_0 block stream -> planar.  One thread per 34-byte block.
__global__ __launch_bounds__(256) void repack_q8_0_kernel(const uint8_t* __restrict__ blocks,
                                                          int8_t* __restrict__ qs,
                                                          uint16_t* __restrict__ d,
                                                          int64_t num_blocks) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= num_blocks) return;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(blocks + b * 34);  // 2-byte aligned
    d[b] = src[0];
    uint16_t* dst = reinterpret_cast<uint16_t*>(qs + b * 32);
#pragma unroll
    for (int i = 0; i < 16; ++i) dst[i] = src[1 + i];
}

}  // namespace lg

extern "C" logismos_status_t logismos_check_qgemv_q8g32_shape(int n, int k, char* msg,
                                                              size_t msg_cap) {
    if (n <= 0) return lg::reject(msg, msg_cap, "qgemv_q8g32: N must be positive, got %d", n);
    if (k <= 0) return lg::reject(msg, msg_cap, "qgemv_q8g32: K must be positive, got %d", k);
    if (k % 32 != 0)
        return lg::reject(msg, msg_cap, "qgemv_q8g32: K = %d is not a multiple of the group size 32", k);
    if ((int64_t)n * (int64_t)k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "qgemv_q8g32: N*K = %lld exceeds i32::MAX",
                          (long long)((int64_t)n * k));
    return 0;
}

extern "C" logismos_status_t logismos_launch_qgemv_q8g32_f32_bias(
    const void* x_f32, const void* qs_i8, const void* d_f16, const void* bias_f32, void* y_f32,
    int n, int k, logismos_stream_t stream) {
    if (logismos_check_qgemv_q8g32_shape(n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!x_f32 || !qs_i8 || !d_f16 || !y_f32) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qs_i8) & 15u) || (reinterpret_cast<uintptr_t>(x_f32) & 15u))
        return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* xp = static_cast<const float*>(x_f32);
    auto* qp = static_cast<const int8_t*>(qs_i8);
    auto* dp = static_cast<const __half*>(d_f16);
    auto* yp = static_cast<float*>(y_f32);
    auto* bp = static_cast<const float*>(bias_f32);  // may be null: no bias
    if (const int fr = lg::flat_rows(n, k); fr > 0) {
        const int np = (fr * (k / 16) + 63) / 64;
        switch (fr) {
            case 8: return lg::launch_flat<8>(np, xp, qp, dp, yp, bp, n, k, st);
            case 4: return lg::launch_flat<4>(np, xp, qp, dp, yp, bp, n, k, st);
            case 2: return lg::launch_flat<2>(np, xp, qp, dp, yp, bp, n, k, st);
            default: return lg::launch_flat<1>(np, xp, qp, dp, yp, bp, n, k, st);
        }
    }
    constexpr int R = 4;
    const int waves = (n + R - 1) / R;
    const int wpb = 4;
    dim3 grid((waves + wpb - 1) / wpb), block(wpb * 64);
    lg::qgemv_q8g32_kernel<R><<<grid, block, 0, st>>>(xp, qp, dp, yp, bp, n, k);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_qgemv_q8g32_f32(const void* x_f32, const void* qs_i8,
                                                             const void* d_f16, void* y_f32, int n,
                                                             int k, logismos_stream_t stream) {
    return logismos_launch_qgemv_q8g32_f32_bias(x_f32, qs_i8, d_f16, nullptr, y_f32, n, k, stream);
}

extern "C" logismos_status_t logismos_launch_repack_q8_0(const void* blocks_q8_0, void* qs_i8,
                                                         void* d_f16, int n, int k,
                                                         logismos_stream_t stream) {
    if (logismos_check_qgemv_q8g32_shape(n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!blocks_q8_0 || !qs_i8 || !d_f16) return hipErrorInvalidValue;
    const int64_t num_blocks = (int64_t)n * (k / 32);
    dim3 grid((unsigned)((num_blocks + 255) / 256)), block(256);
    lg::repack_q8_0_kernel<<<grid, block, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint8_t*>(blocks_q8_0), static_cast<int8_t*>(qs_i8),
        static_cast<uint16_t*>(d_f16), num_blocks);
    return hipGetLastError();
}
