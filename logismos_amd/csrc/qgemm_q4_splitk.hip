// Q4G128 GEMM for a decode batch (up to 32 rows of x) with fp32 partial
// outputs, the form the decode step uses:
//   part[j][b][n] = sum over the j-th K part of x[b][k] * w[n][k]          (fp32)
// and the consumer (residual add + RMSNorm, RoPE, SiLU*up) adds the J parts.
//
// Why another kernel: at batch 32 every workgroup of a row-parallel GEMM needs
// x for all of its K range, and x for all of K (256 KiB at K = 4096, 768 KiB
// at K = 12288) dwarfs the 32..96 KiB of weights a workgroup streams when the
// matrix is spread over 256 CUs.  Here a workgroup is "tall": R = 64..256
// weight rows times a short K part of GP groups (GP*128 columns), so the x it
// needs is R/128 times smaller than its weights, sits in LDS after one
// coalesced copy, and the K parts of different workgroups are summed by the
// consumer instead of through shared accumulators.
//
// Per workgroup (1024 threads): x part -> LDS in pair order (+ per-group sums of
// x), scale/zero of its rows and groups -> LDS; wave w owns row tile w, w+16, ..
// and for each issues its GP 16-byte loads per lane (one per group) up front.
// Dequantisation is the same magic-number trick as in qgemm_q4.hip; the weight
// tile is the MFMA B operand, x from LDS the A operand.  Loads retire in order,
// so x, scale and zero are requested BEFORE the weights: waiting for them does
// not wait for the weight stream.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>
#include <math.h>

namespace lg {

constexpr int kSplitkThreads = 1024;

template <int BT, int GP>
__global__ __launch_bounds__(kSplitkThreads) void qgemm_q4g128_splitk_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero, float* __restrict__ part,
    int b, int n, int k, int tiles_per_wg) {
    extern __shared__ uint4_t lds[];
    constexpr int BP = BT * 16;
    constexpr int QS = GP * 16 + 1;  // row stride of xl in 16-byte words, == 1 (mod 16)
    const int groups = k >> 7;
    const int j = blockIdx.y;
    const int g0 = j * GP;
    const int gcount = min(GP, groups - g0);
    const int rows_wg = tiles_per_wg * 16;
    const int64_t row0 = (int64_t)blockIdx.x * rows_wg;
    const int rows_here = (int)min((int64_t)rows_wg, (int64_t)n - row0);

    uint4_t* xl = lds;                                          // [BP][QS]
    float* xg = reinterpret_cast<float*>(lds + BP * QS);        // [GP][BP]
    __half* szl = reinterpret_cast<__half*>(xg + GP * BP);      // scale [rows_wg][GP], zero [..]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int kc = lane >> 4;

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    // ---- requests, in the order they must retire: x, scale/zero, weights
    constexpr int U = (BP * GP * 16 + kSplitkThreads - 1) / kSplitkThreads;
    const int chunks = gcount * 16;
    const int x_total = chunks * b;
    uint4_t xd[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        const int idc = idx < x_total ? idx : x_total - 1;
        const int bi = idc / chunks, q = idc - bi * chunks;
        xd[u] = *reinterpret_cast<const uint4_t*>(x + (int64_t)bi * k + (int64_t)g0 * 128 +
                                                  (int64_t)q * 8);
    }
    constexpr int SZU = (256 * GP + kSplitkThreads - 1) / kSplitkThreads;  // rows_wg <= 256
    const int sz_total = rows_here * gcount;
    __half sd[SZU], zd[SZU];
#pragma unroll
    for (int u = 0; u < SZU; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        const int idc = idx < sz_total ? idx : sz_total - 1;
        const int r = idc / gcount, g = idc - r * gcount;
        sd[u] = scale[(row0 + r) * groups + g0 + g];
        zd[u] = zero[(row0 + r) * groups + g0 + g];
    }
    __builtin_amdgcn_sched_barrier(0);

    auto load_tile = [&](int t, uint4_t (&w)[GP]) {
        const int r = t * 16 + col;
        const uint8_t* wrow =
            qw + (row0 + (r < rows_here ? r : rows_here - 1)) * (int64_t)(k >> 1) + kc * 16;
#pragma unroll
        for (int i = 0; i < GP; ++i) {
            const int g = (i < gcount) ? (g0 + i) : (g0 + gcount - 1);
            w[i] = *reinterpret_cast<const uint4_t*>(wrow + (int64_t)g * 64);
        }
    };
    uint4_t w[GP];
    int t = wave;
    if (t < tiles_per_wg) load_tile(t, w);
    __builtin_amdgcn_sched_barrier(0);

    // ---- x, scale, zero into LDS
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        const int idc = idx < x_total ? idx : x_total - 1;
        const int bi = idc / chunks, q = idc - bi * chunks;
        const float gs = row16_sum(sum8_bf16(xd[u]));  // 16 chunks of a group = 16 lanes
        if (idx < x_total) {
            xl[bi * QS + q] = pair_order(xd[u]);
            if ((lane & 15) == 0) xg[(q >> 4) * BP + bi] = gs;
        }
    }
#pragma unroll
    for (int u = 0; u < SZU; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        if (idx < sz_total) {
            const int r = idx / gcount, g = idx - r * gcount;
            szl[r * GP + g] = sd[u];
            szl[rows_wg * GP + r * GP + g] = zd[u];
        }
    }
    __syncthreads();
    const __half* zl = szl + rows_wg * GP;

    for (; t < tiles_per_wg; t += kSplitkThreads / 64) {
        if (t != wave) load_tile(t, w);
        const int r = t * 16 + col;
        const int rl = r < rows_here ? r : rows_here - 1;
        float4_t ysum[BT];
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) ysum[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < GP; ++i) {
            const bool valid = i < gcount;  // uniform
            const float sf = __half2float(szl[rl * GP + (valid ? i : 0)]);
            const float off = 128.0f + __half2float(zl[rl * GP + (valid ? i : 0)]);
            float4_t acc[BT];
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const unsigned wd = w[i][s4];
                uint4_t h;
#pragma unroll
                for (int sft = 0; sft < 4; ++sft) h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
                const int q = i * 16 + 4 * kc + s4;
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
                    acc[bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, xl[(bt * 16 + col) * QS + q]), bop, acc[bt], 0,
                        0, 0);
            }
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) {
                const float4_t xsum =
                    *reinterpret_cast<const float4_t*>(xg + i * BP + bt * 16 + 4 * kc);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = fmaf(sf, fmaf(-off, xsum[e], acc[bt][e]), ysum[bt][e]);
                    ysum[bt][e] = valid ? v : ysum[bt][e];
                }
            }
        }
        if (r < rows_here) {
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int bi = bt * 16 + 4 * kc + e;
                    if (bi < b) part[((int64_t)j * b + bi) * n + row0 + r] = ysum[bt][e];
                }
        }
    }
}

struct SplitkPlan {
    int tiles_per_wg;  // 16-row tiles per workgroup (rows = 16 * tiles_per_wg <= 256)
    int gp;            // groups per K part
    int parts;         // J = ceil(groups / gp)
};

// Deterministic in (b, n, k) and the CU count.  Cost relative to the weight
// bytes: 1 (weights) + x re-reads (128/R per 32 batch rows, served by L2)
// + partial write + read (4/gp per 32 batch rows), times the idle fraction when
// fewer workgroups than CUs exist.
static SplitkPlan splitk_plan(int b, int n, int k) {
    const int groups = k / 128;
    const int tiles = (n + 15) / 16;
    const int cus = device_cu_count();
    const double bs = (double)b / 32.0;
    SplitkPlan best{1, 1, groups};
    double best_cost = 1e30;
    const int tpws[] = {4, 8, 16};
    const int gps[] = {1, 2, 4, 8};
    for (int tpw : tpws)
        for (int gp : gps) {
            if (gp > groups && gp != 1) continue;
            const int parts = (groups + gp - 1) / gp;
            const long wgs = (long)((tiles + tpw - 1) / tpw) * parts;
            const double r = 16.0 * tpw;
            double cost = 1.0 + 0.35 * bs * 128.0 / r + bs * 4.0 / gp;
            const double waves_of_wgs = (double)wgs / cus;
            // a partially filled last round of workgroups idles part of the chip
            const double rounds = waves_of_wgs <= 1.0 ? 1.0 : ceil(waves_of_wgs);
            cost *= rounds / waves_of_wgs;
            if (cost < best_cost) {
                best_cost = cost;
                best = SplitkPlan{tpw, gp, parts};
            }
        }
    return best;
}

template <int BT, int GP>
static hipError_t launch_splitk(const void* x, const void* qw, const void* scale, const void* zero,
                                void* part, int b, int n, int k, const SplitkPlan& plan,
                                hipStream_t stream) {
    constexpr int BP = BT * 16;
    const int tiles = (n + 15) / 16;
    const size_t lds = (size_t)BP * (GP * 16 + 1) * 16 + (size_t)GP * BP * 4 +
                       (size_t)2 * plan.tiles_per_wg * 16 * GP * 2;
    auto kern = qgemm_q4g128_splitk_kernel<BT, GP>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    dim3 grid((tiles + plan.tiles_per_wg - 1) / plan.tiles_per_wg, plan.parts);
    kern<<<grid, dim3(kSplitkThreads), lds, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<float*>(part), b, n, k, plan.tiles_per_wg);
    return hipGetLastError();
}

template <int BT>
static hipError_t launch_splitk_bt(const void* x, const void* qw, const void* scale,
                                   const void* zero, void* part, int b, int n, int k,
                                   const SplitkPlan& plan, hipStream_t stream) {
    switch (plan.gp) {
        case 1: return launch_splitk<BT, 1>(x, qw, scale, zero, part, b, n, k, plan, stream);
        case 2: return launch_splitk<BT, 2>(x, qw, scale, zero, part, b, n, k, plan, stream);
        case 4: return launch_splitk<BT, 4>(x, qw, scale, zero, part, b, n, k, plan, stream);
        default: return launch_splitk<BT, 8>(x, qw, scale, zero, part, b, n, k, plan, stream);
    }
}

}  // namespace lg

extern "C" int logismos_qgemm_q4g128_splitk_parts(int b, int n, int k) {
    if (logismos_check_qgemm_q4g128_shape(b, n, k, nullptr, 0) != 0) return 0;
    return lg::splitk_plan(b, n, k).parts;
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_f32_splitk(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* parts_f32, int b, int n, int k, logismos_stream_t stream) {
    if (logismos_check_qgemm_q4g128_shape(b, n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!x_bf16 || !qw_u8 || !scale_f16 || !zero_f16 || !parts_f32) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) & 15u) || (reinterpret_cast<uintptr_t>(x_bf16) & 15u))
        return hipErrorInvalidValue;
    const lg::SplitkPlan plan = lg::splitk_plan(b, n, k);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (b <= 16)
        return lg::launch_splitk_bt<1>(x_bf16, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, plan,
                                       st);
    return lg::launch_splitk_bt<2>(x_bf16, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, plan, st);
}
