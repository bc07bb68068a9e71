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

#include <hip/hip_fp16.h>

namespace lg {

template <int R>
__global__ __launch_bounds__(256) void qgemv_q8g32_kernel(const float* __restrict__ x,
                                                          const int8_t* __restrict__ qs,
                                                          const __half* __restrict__ d,
                                                          float* __restrict__ y, int n, int k) {
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
        if (lane == 0 && row0 + r < n) y[row0 + r] = total;
    }
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

extern "C" logismos_status_t logismos_launch_qgemv_q8g32_f32(const void* x_f32, const void* qs_i8,
                                                             const void* d_f16, void* y_f32, int n,
                                                             int k, logismos_stream_t stream) {
    if (logismos_check_qgemv_q8g32_shape(n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!x_f32 || !qs_i8 || !d_f16 || !y_f32) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qs_i8) & 15u) || (reinterpret_cast<uintptr_t>(x_f32) & 15u))
        return hipErrorInvalidValue;
    constexpr int R = 4;
    const int waves = (n + R - 1) / R;
    const int wpb = 4;
    dim3 grid((waves + wpb - 1) / wpb), block(wpb * 64);
    lg::qgemv_q8g32_kernel<R><<<grid, block, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const float*>(x_f32), static_cast<const int8_t*>(qs_i8),
        static_cast<const __half*>(d_f16), static_cast<float*>(y_f32), n, k);
    return hipGetLastError();
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
