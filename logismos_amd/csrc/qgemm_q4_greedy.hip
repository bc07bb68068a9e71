// Output projection and token selection of a decode step in one pass:
//   logits[b][n] = sum_k x[b][k] * w[n][k]   (Q4G128 weights, PREPARED activations)
//   token[b]     = first index of the maximum of logits[b][:]
//                  (`decode::greedy`, crates/decode/src/lib.rs:73-83: strict >, first wins)
//
// A vocabulary projection has so many rows (151936 x 4096 for the Qwen3 geometry) that the
// fp32 K parts of the split-K kernels would cost half as much traffic again as the weights
// themselves.  Here a workgroup owns a contiguous range of 16-row tiles and ALL of K: it
// walks the K parts (8 groups = 1024 columns each) one after the other, with that part of x
// in LDS, and keeps the running sums of its tiles in LDS between parts (2 KiB per tile at
// batch 32).  In the last part a finished tile's logits are compared against the lane's
// running best and, if the caller wants them, stored.  The inner loop is the streaming loop
// of qgemm_q4_stream.hip: a wave's next tile is in flight while the current one is
// dequantised and multiplied.  A second, tiny kernel picks the winner among the workgroups.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>
#include <math.h>

namespace lg {

constexpr int kGreedyGP = 8;
constexpr int kGreedyWaves = 8;
constexpr int kNoIndex = 0x7fffffff;

struct GreedyTile {
    uint4_t w[kGreedyGP];
    uint4_t s, z;
};

// (value, index) of the better of two candidates: the larger value, the lower index on a tie
__device__ __forceinline__ void take_better(float& v, int& i, float ov, int oi) {
    const bool take = ov > v || (ov == v && oi < i);
    v = take ? ov : v;
    i = take ? oi : i;
}

template <int BT>
__global__ __launch_bounds__(64 * kGreedyWaves) void qgemm_q4g128_greedy_kernel(
    const uint4_t* __restrict__ xprep, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero,
    float* __restrict__ logits, float* __restrict__ best_val, int* __restrict__ best_idx, int b,
    int n, int k, int tiles_per_worker) {
    extern __shared__ uint4_t lds[];
    constexpr int BP = BT * 16;
    constexpr int GP = kGreedyGP;
    constexpr int NT = 64 * kGreedyWaves;
    const int groups = k >> 7;
    const int parts = groups / GP;
    const int tiles = (n + 15) >> 4;
    const int t_begin = blockIdx.x * tiles_per_worker;  // < tiles by the launch's grid
    const int t_end = min(tiles, t_begin + tiles_per_worker);

    uint4_t* xl = lds;                                          // [GP*16 chunks][BP]
    float* xg = reinterpret_cast<float*>(lds + GP * 16 * BP);  // [GP][BP]
    float* acc = xg + GP * BP;  // [tiles_per_worker][BT*4][64 lanes] sums over the parts so far

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int kc = lane >> 4;

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    float bv[BT][4];
    int bi[BT][4];
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            bv[bt][e] = -INFINITY;
            bi[bt][e] = kNoIndex;
        }

    constexpr int U = GP * 16 * BP / NT;
    static_assert(GP * 16 * BP % NT == 0 && GP * BP <= NT, "x part divides over the threads");
    const float* xg_src = reinterpret_cast<const float*>(reinterpret_cast<const char*>(xprep) +
                                                         xprep_xg_offset(b, k));
    const unsigned khalf = (unsigned)(k >> 1);
    const int t_first = t_begin + wave;
    const int t_last = t_end - 1;

    for (int j = 0; j < parts; ++j) {
        const int g0 = j * GP;
        const bool last_part = j == parts - 1;
        // ---- requests in the order they must retire: x part, then the wave's first tile
        const uint4_t* xb = xprep + (int64_t)g0 * 16 * BP;
        uint4_t xd[U];
#pragma unroll
        for (int u = 0; u < U; ++u) xd[u] = xb[u * NT + (int)threadIdx.x];
        const float xgd =
            xg_src[(int64_t)g0 * BP + ((int)threadIdx.x < GP * BP ? (int)threadIdx.x : 0)];
        __builtin_amdgcn_sched_barrier(0);

        const uint8_t* wbase = qw + (int64_t)g0 * 64;  // uniform; lane offsets fit 32 bits
        const __half* sbase = scale + g0;
        const __half* zbase = zero + g0;
        auto load_tile = [&](int t, GreedyTile& tl) {
            const int row = min(t * 16 + col, n - 1);
            const unsigned woff = (unsigned)row * khalf + (unsigned)kc * 16u;
#pragma unroll
            for (int i = 0; i < GP; ++i)
                tl.w[i] = *reinterpret_cast<const uint4_t*>(wbase + woff + 64u * i);
            const unsigned soff = (unsigned)row * (unsigned)groups;
            tl.s = *reinterpret_cast<const uint4_t*>(sbase + soff);
            tl.z = *reinterpret_cast<const uint4_t*>(zbase + soff);
        };
        GreedyTile ta, tb;
        load_tile(min(t_first, t_last), ta);
        __builtin_amdgcn_sched_barrier(0);

        // ---- x part into LDS once every wave is done with the previous one
        if (j > 0) __syncthreads();
#pragma unroll
        for (int u = 0; u < U; ++u) xl[u * NT + (int)threadIdx.x] = xd[u];
        if ((int)threadIdx.x < GP * BP) xg[threadIdx.x] = xgd;
        __syncthreads();

        auto compute_tile = [&](int t, const GreedyTile& tl) {
            float4_t ysum[BT];
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) ysum[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int i = 0; i < GP; ++i) {
                const unsigned sw = tl.s[i >> 1], zw = tl.z[i >> 1];
                const unsigned short sh =
                    (unsigned short)((i & 1) ? (sw >> 16) : (sw & 0xffffu));
                const unsigned short zh =
                    (unsigned short)((i & 1) ? (zw >> 16) : (zw & 0xffffu));
                const float sf = __half2float(__builtin_bit_cast(__half, sh));
                const float off = 128.0f + __half2float(__builtin_bit_cast(__half, zh));
                float4_t a[BT];
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) a[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) {
                    const unsigned wd = tl.w[i][s4];
                    uint4_t h;
#pragma unroll
                    for (int sft = 0; sft < 4; ++sft)
                        h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                    const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
                    const int q = i * 16 + 4 * kc + s4;
#pragma unroll
                    for (int bt = 0; bt < BT; ++bt)
                        a[bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, xl[q * BP + bt * 16 + col]), bop, a[bt],
                            0, 0, 0);
                }
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) {
                    const float4_t xsum =
                        *reinterpret_cast<const float4_t*>(xg + i * BP + bt * 16 + 4 * kc);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        ysum[bt][e] = fmaf(sf, fmaf(-off, xsum[e], a[bt][e]), ysum[bt][e]);
                }
                // pin the running sums here: otherwise the compiler sinks every group's update
                // to the end and keeps all their accumulators alive
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) asm volatile("" : "+v"(ysum[bt]));
                __builtin_amdgcn_sched_barrier(0);
            }
            // this wave's own slots: no other wave touches the sums of this tile
            float* slot = acc + (size_t)(t - t_begin) * (BT * 4 * 64) + lane;
            const int row = t * 16 + col;
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = ysum[bt][e];
                    if (j > 0) v += slot[(bt * 4 + e) * 64];
                    if (!last_part) {
                        slot[(bt * 4 + e) * 64] = v;
                    } else if (row < n) {
                        const int r = bt * 16 + 4 * kc + e;
                        if (logits && r < b) logits[(unsigned)r * (unsigned)n + (unsigned)row] = v;
                        if (v > bv[bt][e]) {  // rows ascend with t: the first maximum stays
                            bv[bt][e] = v;
                            bi[bt][e] = row;
                        }
                    }
                }
        };

        for (int t = t_first; t < t_end; t += 2 * kGreedyWaves) {
            load_tile(min(t + kGreedyWaves, t_last), tb);
            __builtin_amdgcn_sched_barrier(0);
            compute_tile(t, ta);
            __builtin_amdgcn_sched_barrier(0);
            load_tile(min(t + 2 * kGreedyWaves, t_last), ta);
            __builtin_amdgcn_sched_barrier(0);
            if (t + kGreedyWaves < t_end) compute_tile(t + kGreedyWaves, tb);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- best of the workgroup per batch row: over the 16 weight rows a wave tile spans,
    // then over the waves
    __syncthreads();  // the x part in LDS is no longer needed; reuse its space
    float* wv = reinterpret_cast<float*>(lds);         // [waves][BP]
    int* wi = reinterpret_cast<int*>(wv + kGreedyWaves * BP);
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v = bv[bt][e];
            int i = bi[bt][e];
#pragma unroll
            for (int m = 1; m < 16; m <<= 1) {
                const float ov = __shfl_xor(v, m, kWave);
                const int oi = __shfl_xor(i, m, kWave);
                take_better(v, i, ov, oi);
            }
            if (col == 0) {
                wv[wave * BP + bt * 16 + 4 * kc + e] = v;
                wi[wave * BP + bt * 16 + 4 * kc + e] = i;
            }
        }
    __syncthreads();
    if ((int)threadIdx.x < BP) {
        float v = wv[threadIdx.x];
        int i = wi[threadIdx.x];
        for (int w = 1; w < kGreedyWaves; ++w)
            take_better(v, i, wv[w * BP + threadIdx.x], wi[w * BP + threadIdx.x]);
        best_val[(int64_t)blockIdx.x * BP + threadIdx.x] = v;
        best_idx[(int64_t)blockIdx.x * BP + threadIdx.x] = i;
    }
}

// token[r] = index of the best candidate over the workers; a row whose logits never exceeded
// -inf (all -inf or NaN) gives 0, like the CPU loop that never updates.  One workgroup: thread
// (g = t / bp, r = t % bp) folds workers g, g + groups, ...; the groups are folded through LDS.
constexpr int kPickThreads = 1024;

__global__ __launch_bounds__(kPickThreads) void greedy_pick_kernel(
    const float* __restrict__ best_val, const int* __restrict__ best_idx,
    uint32_t* __restrict__ out, int b, int bp, int workers) {
    __shared__ float sv[kPickThreads];
    __shared__ int si[kPickThreads];
    const int r = threadIdx.x % bp;
    const int g = threadIdx.x / bp;
    const int groups = kPickThreads / bp;
    float v = -INFINITY;
    int i = kNoIndex;
    for (int w = g; w < workers; w += groups)
        take_better(v, i, best_val[(int64_t)w * bp + r], best_idx[(int64_t)w * bp + r]);
    sv[threadIdx.x] = v;
    si[threadIdx.x] = i;
    __syncthreads();
    if (g == 0 && r < b) {
        for (int k = 1; k < groups; ++k) take_better(v, i, sv[k * bp + r], si[k * bp + r]);
        out[r] = i == kNoIndex ? 0u : (uint32_t)i;
    }
}

struct GreedyPlan {
    int tiles_per_worker, workers;
    size_t lds;
};

static GreedyPlan greedy_plan(int b, int n) {
    const int bp = xprep_bp(b);
    const int bt = bp / 16;
    const int tiles = (n + 15) / 16;
    const int cus = device_cu_count();
    const size_t fixed = (size_t)kGreedyGP * 16 * bp * 16 + (size_t)kGreedyGP * bp * 4;
    const size_t per_tile = (size_t)bt * 4 * 64 * 4;
    const int cap = (int)((150 * 1024 - fixed) / per_tile);
    int tpw = (tiles + cus - 1) / cus;
    if (tpw > cap) tpw = cap;
    if (tpw < 1) tpw = 1;
    GreedyPlan p;
    p.tiles_per_worker = tpw;
    p.workers = (tiles + tpw - 1) / tpw;
    p.lds = fixed + per_tile * tpw;
    return p;
}

template <int BT>
static hipError_t launch_greedy(const void* xprep, const void* qw, const void* scale,
                                const void* zero, void* out_tokens, void* logits, void* workspace,
                                int b, int n, int k, hipStream_t stream) {
    const GreedyPlan p = greedy_plan(b, n);
    auto kern = qgemm_q4g128_greedy_kernel<BT>;
    static const hipError_t opt = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
        160 * 1024 - 1024);
    if (opt != hipSuccess) return opt;
    constexpr int BP = BT * 16;
    float* best_val = static_cast<float*>(workspace);
    int* best_idx = reinterpret_cast<int*>(best_val + (size_t)p.workers * BP);
    kern<<<dim3(p.workers), dim3(64 * kGreedyWaves), p.lds, stream>>>(
        static_cast<const uint4_t*>(xprep), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<float*>(logits), best_val, best_idx, b, n, k, p.tiles_per_worker);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    greedy_pick_kernel<<<dim3(1), dim3(kPickThreads), 0, stream>>>(
        best_val, best_idx, static_cast<uint32_t*>(out_tokens), b, BP, p.workers);
    return hipGetLastError();
}

}  // namespace lg

extern "C" logismos_status_t logismos_check_qgemm_q4g128_greedy_shape(int b, int n, int k,
                                                                      char* msg, size_t msg_cap) {
    const char* kn = "qgemm_q4g128_greedy";
    if (b <= 0 || b > 32)
        return lg::reject(msg, msg_cap, "%s: batch must be in 1..32, got %d", kn, b);
    if (n <= 0) return lg::reject(msg, msg_cap, "%s: N must be positive, got %d", kn, n);
    if (k <= 0 || k % 1024 != 0)
        return lg::reject(msg, msg_cap,
                          "%s: K = %d is not a positive multiple of 1024 (8 groups of 128)", kn, k);
    if ((int64_t)n * k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "%s: N*K = %lld exceeds i32::MAX", kn,
                          (long long)((int64_t)n * k));
    if ((int64_t)b * n > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "%s: batch*N exceeds i32::MAX", kn);
    return 0;
}

extern "C" size_t logismos_qgemm_q4g128_greedy_workspace_bytes(int b, int n, int k) {
    if (logismos_check_qgemm_q4g128_greedy_shape(b, n, k, nullptr, 0) != 0) return 0;
    const lg::GreedyPlan p = lg::greedy_plan(b, n);
    return (size_t)p.workers * lg::xprep_bp(b) * 8;
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_greedy_xprep(
    const void* x_prepared, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* out_tokens_u32, void* logits_f32, void* workspace, int b, int n, int k,
    logismos_stream_t stream) {
    if (logismos_check_qgemm_q4g128_greedy_shape(b, n, k, nullptr, 0) != 0)
        return hipErrorInvalidValue;
    if (!x_prepared || !qw_u8 || !scale_f16 || !zero_f16 || !out_tokens_u32 || !workspace)
        return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) & 15u) || (reinterpret_cast<uintptr_t>(x_prepared) & 15u) ||
        (reinterpret_cast<uintptr_t>(scale_f16) & 15u) || (reinterpret_cast<uintptr_t>(zero_f16) & 15u) ||
        (reinterpret_cast<uintptr_t>(workspace) & 3u))
        return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (b <= 16)
        return lg::launch_greedy<1>(x_prepared, qw_u8, scale_f16, zero_f16, out_tokens_u32,
                                    logits_f32, workspace, b, n, k, st);
    return lg::launch_greedy<2>(x_prepared, qw_u8, scale_f16, zero_f16, out_tokens_u32, logits_f32,
                                workspace, b, n, k, st);
}
