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
// Per workgroup (4 waves): x part -> LDS in pair order (+ per-group sums of x),
// scale/zero of its rows and groups -> LDS; every wave owns TW row tiles and
// issues their TW*GP 16-byte loads per lane (one per tile and group) up front.
// Dequantisation is the same magic-number trick as in qgemm_q4.hip; the weight
// tile is the MFMA B operand, x from LDS the A operand.  Loads retire in order,
// so x, scale and zero are requested BEFORE the weights: waiting for them does
// not wait for the weight stream.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>
#include <math.h>
#include <stdlib.h>

namespace lg {

constexpr int kSplitkWaves = 4;
constexpr int kSplitkThreads = 64 * kSplitkWaves;

// BT batch tiles of 16 rows of x, GP groups per K part, TW row tiles per wave
// (a workgroup owns 4*TW*16 weight rows).  Small workgroups on purpose: several
// are resident per CU at different stages (staging x / waiting for weights /
// MFMA), which overlaps what a single big workgroup would serialise.
template <int BT, int GP, int TW, bool PREP>
__global__ __launch_bounds__(kSplitkThreads) void qgemm_q4g128_splitk_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero, float* __restrict__ part,
    int b, int n, int k) {
    extern __shared__ uint4_t lds[];
    constexpr int BP = BT * 16;
    // xl: PREP ? [GP*16 chunks][BP] (the prepared layout itself) : [BP][QS], QS == 1 (mod 16)
    constexpr int QS = GP * 16 + 1;
    constexpr int ROWS = kSplitkWaves * TW * 16;
    const int groups = k >> 7;
    const int j = blockIdx.y;
    const int g0 = j * GP;
    const int gcount = min(GP, groups - g0);
    const int64_t row0 = (int64_t)blockIdx.x * ROWS;
    const int rows_here = (int)min((int64_t)ROWS, (int64_t)n - row0);

    uint4_t* xl = lds;                                      // [BP][QS]
    float* xg = reinterpret_cast<float*>(lds + BP * QS);    // [GP][BP]
    __half* szl = reinterpret_cast<__half*>(xg + GP * BP);  // scale [ROWS][GP], zero [ROWS][GP]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int kc = lane >> 4;

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    // ---- requests, in the order they must retire: x, scale/zero, weights
    constexpr int U = (BP * GP * 16 + kSplitkThreads - 1) / kSplitkThreads;
    const int chunks = gcount * 16;
    const int x_total = PREP ? chunks * BP : chunks * b;
    uint4_t xd[U];
    float xgd = 0.0f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        const int idc = idx < x_total ? idx : x_total - 1;
        if constexpr (PREP) {
            // the K part of the prepared x is one contiguous block of 16-byte words
            const uint4_t* xb = reinterpret_cast<const uint4_t*>(x) + (int64_t)g0 * 16 * BP;
            xd[u] = xb[(unsigned)idc];
        } else {
            const int bi = idc / chunks, q = idc - bi * chunks;
            xd[u] = *reinterpret_cast<const uint4_t*>(x + (int64_t)bi * k + (int64_t)g0 * 128 +
                                                      (int64_t)q * 8);
        }
    }
    if constexpr (PREP) {
        static_assert(GP * BP <= kSplitkThreads, "one group sum per thread");
        const float* xg_src = reinterpret_cast<const float*>(
            reinterpret_cast<const char*>(x) + xprep_xg_offset(b, k));
        const int t = (int)threadIdx.x < gcount * BP ? (int)threadIdx.x : 0;
        xgd = xg_src[(int64_t)g0 * BP + t];
    }
    // scale / zero of (row r, group g): thread idx -> r = idx / GP, g = idx % GP; rows and
    // groups past the end repeat the last valid one (their products are dropped below)
    constexpr int SZU = (ROWS * GP + kSplitkThreads - 1) / kSplitkThreads;
    const __half* sbase = scale + row0 * groups + g0;  // workgroup-uniform
    const __half* zbase = zero + row0 * groups + g0;
    __half sd[SZU], zd[SZU];
#pragma unroll
    for (int u = 0; u < SZU; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        const int r = min(idx / GP, rows_here - 1), g = min(idx % GP, gcount - 1);
        const unsigned off = (unsigned)r * (unsigned)groups + (unsigned)g;
        sd[u] = sbase[off];
        zd[u] = zbase[off];
    }
    __builtin_amdgcn_sched_barrier(0);

    // this wave's TW tiles: rows (wave*TW + t)*16 .. +16
    uint4_t w[TW][GP];
    const uint8_t* wbase = qw + row0 * (int64_t)(k >> 1) + (int64_t)g0 * 64;  // uniform
#pragma unroll
    for (int t = 0; t < TW; ++t) {
        const int r = (wave * TW + t) * 16 + col;
        const unsigned woff =
            (unsigned)(r < rows_here ? r : rows_here - 1) * (unsigned)(k >> 1) + (unsigned)kc * 16u;
#pragma unroll
        for (int i = 0; i < GP; ++i)
            w[t][i] = *reinterpret_cast<const uint4_t*>(wbase + woff +
                                                        64u * (unsigned)(i < gcount ? i : gcount - 1));
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- x, scale, zero into LDS
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        if constexpr (PREP) {
            if (idx < x_total) xl[idx] = xd[u];
        } else {
            const int idc = idx < x_total ? idx : x_total - 1;
            const int bi = idc / chunks, q = idc - bi * chunks;
            const float gs = row16_sum(sum8_bf16(xd[u]));  // 16 chunks of a group = 16 lanes
            if (idx < x_total) {
                xl[bi * QS + q] = pair_order(xd[u]);
                if ((lane & 15) == 0) xg[(q >> 4) * BP + bi] = gs;
            }
        }
    }
    if constexpr (PREP) {
        if ((int)threadIdx.x < gcount * BP) xg[threadIdx.x] = xgd;
    }
#pragma unroll
    for (int u = 0; u < SZU; ++u) {
        const int idx = u * kSplitkThreads + (int)threadIdx.x;
        if (idx < ROWS * GP) {
            szl[idx] = sd[u];
            szl[ROWS * GP + idx] = zd[u];
        }
    }
    __syncthreads();
    const __half* zl = szl + ROWS * GP;

#pragma unroll
    for (int t = 0; t < TW; ++t) {
        const int r = (wave * TW + t) * 16 + col;
        const int rl = r < rows_here ? r : rows_here - 1;
        float4_t ysum[BT];
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) ysum[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < GP; ++i) {
            // a group past the end of K (last part only): scale 0, operands of group 0
            const bool valid = i < gcount;  // uniform
            const int ix = valid ? i : 0;
            const float sf = valid ? __half2float(szl[rl * GP + i]) : 0.0f;
            const float off = 128.0f + __half2float(zl[rl * GP + ix]);
            float4_t acc[BT];
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const unsigned wd = w[t][i][s4];
                uint4_t h;
#pragma unroll
                for (int sft = 0; sft < 4; ++sft) h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
                const int q = ix * 16 + 4 * kc + s4;
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
                    acc[bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, PREP ? xl[q * BP + bt * 16 + col]
                                                          : xl[(bt * 16 + col) * QS + q]),
                        bop, acc[bt], 0, 0, 0);
            }
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) {
                const float4_t xsum =
                    *reinterpret_cast<const float4_t*>(xg + ix * BP + bt * 16 + 4 * kc);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    ysum[bt][e] = fmaf(sf, fmaf(-off, xsum[e], acc[bt][e]), ysum[bt][e]);
            }
            // pin the running sums here: otherwise the compiler sinks every group's update to
            // the store and keeps all their accumulators alive
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) asm volatile("" : "+v"(ysum[bt]));
            // one group at a time: without this the scheduler hoists the LDS reads of
            // every group (GP*4*BT operands of four registers) and spills
            __builtin_amdgcn_sched_barrier(0);
        }
        if (r < rows_here) {
            float* pbase = part + (int64_t)j * b * n + row0;  // uniform
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int bi = bt * 16 + 4 * kc + e;
                    if (bi < b) pbase[(unsigned)bi * (unsigned)n + (unsigned)r] = ysum[bt][e];
                }
        }
    }
}

struct SplitkPlan {
    int tw;     // row tiles per wave (rows per workgroup = 64 * tw)
    int gp;     // groups per K part
    int parts;  // J = ceil(groups / gp)
};

// Deterministic in (b, n, k) and the CU count.  Cost relative to the weight
// bytes: 1 (weights) + x re-reads (128/R per 32 batch rows, served by L2)
// + the fp32 parts (4/gp per 32 batch rows, written here and read back by the
// consumer, whose few workgroups read them slowly: weighted 1.5), times a mild
// penalty when the workgroups do not fill the CUs evenly (measured kernels lose far
// less than the idle fraction suggests, because fewer resident workgroups run faster).
static SplitkPlan splitk_plan(int b, int n, int k) {
    const int groups = k / 128;
    const int tiles = (n + 15) / 16;
    const int cus = device_cu_count();
    const double bs = (double)b / 32.0;
    // shapes the streaming kernel takes (prepared x) use its K parts in both entry points
    if (stream_steps(b, n, k) > 0) return SplitkPlan{1, 8, groups / 8};
    SplitkPlan best{1, 1, groups};
    double best_cost = 1e30;
    const int tws[] = {1, 2, 4};
    const int gps[] = {1, 2, 4, 8};
    for (int tw : tws)
        for (int gp : gps) {
            if (gp > groups && gp != 1) continue;
            if (b > 16 && tw * gp > 8) continue;  // register budget with two batch tiles
            if (gp == 8 && tw > 2) continue;      // instantiated: (8,1), (8,2)
            const int parts = (groups + gp - 1) / gp;
            const int tpw = kSplitkWaves * tw;
            const long wgs = (long)((tiles + tpw - 1) / tpw) * parts;
            const double r = 16.0 * tpw;
            double cost = 1.0 + 0.35 * bs * 128.0 / r + 1.5 * bs * 4.0 / gp;
            // resident workgroups per CU: four, two when the x part takes 64 KiB of LDS
            const double fill = (double)wgs / ((gp == 8 ? 2.0 : 4.0) * cus);
            if (fill <= 1.0)
                cost *= 1.0 + 0.3 * (1.0 - fill);
            else
                cost *= 1.0 + 0.5 * (ceil(fill) / fill - 1.0);
            if (cost < best_cost) {
                best_cost = cost;
                best = SplitkPlan{tw, gp, parts};
            }
        }
    return best;
}

template <int BT, int GP, int TW, bool PREP>
static hipError_t launch_splitk(const void* x, const void* qw, const void* scale, const void* zero,
                                void* part, int b, int n, int k, const SplitkPlan& plan,
                                hipStream_t stream) {
    constexpr int BP = BT * 16;
    constexpr int ROWS = kSplitkWaves * TW * 16;
    const int tiles = (n + 15) / 16;
    const size_t lds =
        (size_t)BP * (GP * 16 + 1) * 16 + (size_t)GP * BP * 4 + (size_t)2 * ROWS * GP * 2;
    auto kern = qgemm_q4g128_splitk_kernel<BT, GP, TW, PREP>;
    if (lds > 64 * 1024) {
        // above the default dynamic-LDS limit: opt in once per instantiation
        static const hipError_t opt = hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
            160 * 1024 - 1024);
        if (opt != hipSuccess) return opt;
    }
    dim3 grid((tiles + kSplitkWaves * TW - 1) / (kSplitkWaves * TW), plan.parts);
    kern<<<grid, dim3(kSplitkThreads), lds, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<float*>(part), b, n, k);
    return hipGetLastError();
}

template <int BT, bool PREP>
static hipError_t launch_splitk_bt(const void* x, const void* qw, const void* scale,
                                   const void* zero, void* part, int b, int n, int k,
                                   const SplitkPlan& plan, hipStream_t stream) {
#define LG_SPLITK_CASE(GP, TW)                                                                  \
    if (plan.gp == GP && plan.tw == TW)                                                         \
        return launch_splitk<BT, GP, TW, PREP>(x, qw, scale, zero, part, b, n, k, plan, stream);
    LG_SPLITK_CASE(1, 1) LG_SPLITK_CASE(1, 2) LG_SPLITK_CASE(1, 4)
    LG_SPLITK_CASE(2, 1) LG_SPLITK_CASE(2, 2) LG_SPLITK_CASE(2, 4)
    LG_SPLITK_CASE(4, 1) LG_SPLITK_CASE(4, 2)
    LG_SPLITK_CASE(8, 1) LG_SPLITK_CASE(8, 2)
    if constexpr (BT == 1) {
        LG_SPLITK_CASE(4, 4)
    }
#undef LG_SPLITK_CASE
    return hipErrorInvalidValue;
}

}  // namespace lg

// The split-K forms hold the whole batch in one launch (and the prepared layout has 32 rows).
extern "C" int logismos_qgemm_q4g128_splitk_parts(int b, int n, int k) {
    if (b > 32 || logismos_check_qgemm_q4g128_shape(b, n, k, nullptr, 0) != 0) return 0;
    return lg::splitk_plan(b, n, k).parts;
}

extern "C" int logismos_qgemm_q4g128_splitk_xprep_parts(int b, int n, int k) {
    if (b > 32 || logismos_check_qgemm_q4g128_shape(b, n, k, nullptr, 0) != 0) return 0;
    if (const lg::RegxPlan rp = lg::regx_plan(b, n, k); rp.parts > 0) return rp.parts;
    return lg::splitk_plan(b, n, k).parts;
}

static logismos_status_t splitk_dispatch(const void* x, bool prepared, const void* qw_u8,
                                         const void* scale_f16, const void* zero_f16,
                                         void* parts_f32, int b, int n, int k,
                                         logismos_stream_t stream) {
    if (b > 32 || logismos_check_qgemm_q4g128_shape(b, n, k, nullptr, 0) != 0)
        return hipErrorInvalidValue;
    if (!x || !qw_u8 || !scale_f16 || !zero_f16 || !parts_f32) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) & 15u) || (reinterpret_cast<uintptr_t>(x) & 15u))
        return hipErrorInvalidValue;
    const lg::SplitkPlan plan = lg::splitk_plan(b, n, k);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (prepared) {
        if (const lg::RegxPlan rp = lg::regx_plan(b, n, k); rp.parts > 0)
            return lg::qgemm_q4_regx_launch(rp, x, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, st);
        if (const int steps = lg::stream_steps(b, n, k))
            return lg::qgemm_q4_stream_launch(x, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k,
                                              steps, st);
        if (b <= 16)
            return lg::launch_splitk_bt<1, true>(x, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k,
                                                 plan, st);
        return lg::launch_splitk_bt<2, true>(x, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, plan,
                                             st);
    }
    if (b <= 16)
        return lg::launch_splitk_bt<1, false>(x, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k,
                                              plan, st);
    return lg::launch_splitk_bt<2, false>(x, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, plan,
                                          st);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_f32_splitk(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* parts_f32, int b, int n, int k, logismos_stream_t stream) {
    return splitk_dispatch(x_bf16, false, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, stream);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_f32_splitk_xprep(
    const void* x_prepared, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* parts_f32, int b, int n, int k, logismos_stream_t stream) {
    return splitk_dispatch(x_prepared, true, qw_u8, scale_f16, zero_f16, parts_f32, b, n, k, stream);
}

extern "C" size_t logismos_q4_xprep_bytes(int b, int k) {
    if (b <= 0 || b > 32 || k <= 0 || k % 128 != 0) return 0;
    return lg::xprep_bytes(b, k);
}

namespace lg {
// bf16 x [b][k] -> prepared form; one thread per 8-element chunk
__global__ __launch_bounds__(256) void q4_prepare_x_kernel(const uint16_t* __restrict__ x,
                                                           void* __restrict__ xprep, int b, int k) {
    const int bp = xprep_bp(b);
    const int chunks = k >> 3;
    const int idx = blockIdx.x * 256 + threadIdx.x;  // chunk-major inside a batch row
    const int bi = idx / chunks, c = idx - bi * chunks;
    const bool live = bi < b;
    uint4_t d = uint4_t{0u, 0u, 0u, 0u};
    if (live) d = *reinterpret_cast<const uint4_t*>(x + (int64_t)bi * k + (int64_t)c * 8);
    const float gs = row16_sum(sum8_bf16(d));
    if (live) {
        reinterpret_cast<uint4_t*>(xprep)[(int64_t)c * bp + bi] = pair_order(d);
        if ((threadIdx.x & 15) == 0)
            reinterpret_cast<float*>(reinterpret_cast<char*>(xprep) +
                                     xprep_xg_offset(b, k))[(int64_t)(c >> 4) * bp + bi] = gs;
    }
}
}  // namespace lg

extern "C" logismos_status_t logismos_launch_q4_prepare_x_bf16(const void* x_bf16, void* x_prepared,
                                                               int b, int k,
                                                               logismos_stream_t stream) {
    if (b <= 0 || b > 32 || k <= 0 || k % 128 != 0 || (int64_t)b * k > (int64_t)INT32_MAX)
        return hipErrorInvalidValue;
    if (!x_bf16 || !x_prepared || (reinterpret_cast<uintptr_t>(x_bf16) & 15u) ||
        (reinterpret_cast<uintptr_t>(x_prepared) & 15u))
        return hipErrorInvalidValue;
    const int items = b * (k / 8);
    lg::q4_prepare_x_kernel<<<dim3((items + 255) / 256), dim3(256), 0,
                              static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint16_t*>(x_bf16), x_prepared, b, k);
    return hipGetLastError();
}
