// Q4G128 GEMM for a decode batch over PREPARED activations, streaming form:
//   part[j][b][n] = sum over K part j (8 groups = 1024 columns) of x[b][k] * w[n][k]   (fp32)
//
// The split-K kernel of qgemm_q4_splitk.hip gives every workgroup one 64-row slab of one K
// part and stages that part of x (64 KiB at batch 32) again for each slab; with two such
// workgroups per CU the large matrices need 1.5 .. 3 rounds of them, each paying the x
// copy, a barrier and a cold weight load.  Here a workgroup stays on one K part: it copies
// the x part to LDS once and then walks down its share of the row tiles, eight tiles (one
// per wave) per step, with the next step's weights, scales and zeros already in flight
// while the current tile is dequantised and multiplied.  No barrier after the prologue.
//
// Per wave and tile (16 weight rows x 1024 columns): lane (kc = lane/16, col = lane%16)
// loads the 16 bytes of row `col`, piece kc, of each of the 8 groups (the MFMA B operand
// after the magic-number unpack of qgemm_q4.hip), plus the row's 8 scales and 8 zeros as
// one 16-byte load each.  x from LDS is the A operand.  Used when K/128 is a multiple of
// 8 (so that every part is full and the scale/zero loads are aligned) and the matrix is
// large enough to give every CU more than one step.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

constexpr int kStreamGP = 8;
constexpr int kStreamWaves = 8;

struct StreamTile {
    uint4_t w[kStreamGP];
    uint4_t s, z;  // 8 fp16 scales, 8 fp16 zeros of this lane's row
};

template <int BT>
__global__ __launch_bounds__(64 * kStreamWaves) void qgemm_q4g128_stream_kernel(
    const uint4_t* __restrict__ xprep, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero, float* __restrict__ part,
    int b, int n, int k, int tiles_per_worker) {
    extern __shared__ uint4_t lds[];
    constexpr int BP = BT * 16;
    constexpr int GP = kStreamGP;
    constexpr int NT = 64 * kStreamWaves;
    const int groups = k >> 7;
    const int j = blockIdx.y;
    const int g0 = j * GP;
    const int tiles = (n + 15) >> 4;
    const int t_begin = blockIdx.x * tiles_per_worker;
    if (t_begin >= tiles) return;
    const int t_end = min(tiles, t_begin + tiles_per_worker);

    uint4_t* xl = lds;                                          // [GP*16 chunks][BP]
    float* xg = reinterpret_cast<float*>(lds + GP * 16 * BP);  // [GP][BP]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int kc = lane >> 4;

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    // ---- requests in the order they must retire: x part, then the first tile
    constexpr int U = GP * 16 * BP / NT;
    static_assert(GP * 16 * BP % NT == 0 && GP * BP <= NT, "x part divides over the threads");
    const uint4_t* xb = xprep + (int64_t)g0 * 16 * BP;
    uint4_t xd[U];
#pragma unroll
    for (int u = 0; u < U; ++u) xd[u] = xb[u * NT + (int)threadIdx.x];
    const float* xg_src = reinterpret_cast<const float*>(
        reinterpret_cast<const char*>(xprep) + xprep_xg_offset(b, k));
    const float xgd = xg_src[(int64_t)g0 * BP + ((int)threadIdx.x < GP * BP ? (int)threadIdx.x : 0)];
    __builtin_amdgcn_sched_barrier(0);

    const uint8_t* wbase = qw + (int64_t)g0 * 64;  // uniform; lane offsets fit 32 bits (N*K < 2^31)
    const __half* sbase = scale + g0;
    const __half* zbase = zero + g0;
    const unsigned khalf = (unsigned)(k >> 1);
    auto load_tile = [&](int t, StreamTile& tl) {
        const int row = min(t * 16 + col, n - 1);
        const unsigned woff = (unsigned)row * khalf + (unsigned)kc * 16u;
#pragma unroll
        for (int i = 0; i < GP; ++i)
            tl.w[i] = *reinterpret_cast<const uint4_t*>(wbase + woff + 64u * i);
        const unsigned soff = (unsigned)row * (unsigned)groups;
        tl.s = *reinterpret_cast<const uint4_t*>(sbase + soff);
        tl.z = *reinterpret_cast<const uint4_t*>(zbase + soff);
    };
    const int t_first = t_begin + wave;
    const int t_last = t_end - 1;
    StreamTile ta, tb;
    load_tile(min(t_first, t_last), ta);
    __builtin_amdgcn_sched_barrier(0);

    // ---- x part into LDS (a straight copy of the prepared layout)
#pragma unroll
    for (int u = 0; u < U; ++u) xl[u * NT + (int)threadIdx.x] = xd[u];
    if ((int)threadIdx.x < GP * BP) xg[threadIdx.x] = xgd;
    __syncthreads();

    float* pbase = part + (int64_t)j * b * n;  // uniform
    auto compute_tile = [&](int t, const StreamTile& tl) {
        float4_t ysum[BT];
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) ysum[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < GP; ++i) {
            const unsigned sw = tl.s[i >> 1], zw = tl.z[i >> 1];
            const unsigned short sh = (unsigned short)((i & 1) ? (sw >> 16) : (sw & 0xffffu));
            const unsigned short zh = (unsigned short)((i & 1) ? (zw >> 16) : (zw & 0xffffu));
            const float sf = __half2float(__builtin_bit_cast(__half, sh));
            const float off = 128.0f + __half2float(__builtin_bit_cast(__half, zh));
            float4_t acc[BT];
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const unsigned wd = tl.w[i][s4];
                uint4_t h;
#pragma unroll
                for (int sft = 0; sft < 4; ++sft) h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
                const int q = i * 16 + 4 * kc + s4;
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
                    acc[bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, xl[q * BP + bt * 16 + col]), bop, acc[bt], 0, 0,
                        0);
            }
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) {
                const float4_t xsum =
                    *reinterpret_cast<const float4_t*>(xg + i * BP + bt * 16 + 4 * kc);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    ysum[bt][e] = fmaf(sf, fmaf(-off, xsum[e], acc[bt][e]), ysum[bt][e]);
            }
            // pin the running sums here: otherwise the compiler sinks every group's update to
            // the store and keeps all their accumulators alive
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) asm volatile("" : "+v"(ysum[bt]));
            // one group at a time: keeps the LDS operand reads from being hoisted (and spilled)
            __builtin_amdgcn_sched_barrier(0);
        }
        const int row = t * 16 + col;
        if (row < n) {
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int bi = bt * 16 + 4 * kc + e;
                    if (bi < b) pbase[(unsigned)bi * (unsigned)n + (unsigned)row] = ysum[bt][e];
                }
        }
    };

    // two tiles per iteration in one straight-line body: the loads of the next tile are in
    // flight while the current one is multiplied (a tile index past the end re-reads the
    // last tile of the range; its result is not computed)
    for (int t = t_first; t < t_end; t += 2 * kStreamWaves) {
        load_tile(min(t + kStreamWaves, t_last), tb);
        __builtin_amdgcn_sched_barrier(0);
        compute_tile(t, ta);
        __builtin_amdgcn_sched_barrier(0);
        load_tile(min(t + 2 * kStreamWaves, t_last), ta);
        __builtin_amdgcn_sched_barrier(0);
        if (t + kStreamWaves < t_end) compute_tile(t + kStreamWaves, tb);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Steps (tiles per wave) a worker takes, 0 when the streaming kernel does not apply.  One
// workgroup per CU: spreading the same tiles over two (which fit) measured slower, the
// second copy of the x part costing more than the extra waves gain.
int stream_steps(int b, int n, int k) {
    const int groups = k / 128;
    if (b < 3 || groups % kStreamGP != 0) return 0;
    const int tiles = (n + 15) / 16;
    const int parts = groups / kStreamGP;
    const int cus = device_cu_count();
    // wave tiles per CU if spread evenly; with fewer than ten the split-K kernel's finer
    // workgroups do as well
    if ((long)tiles * parts / cus < 10) return 0;
    int steps = 1;
    while ((long)((tiles + steps * kStreamWaves - 1) / (steps * kStreamWaves)) * parts > cus) ++steps;
    return steps;
}

template <int BT>
static hipError_t launch_stream(const void* xprep, const void* qw, const void* scale,
                                const void* zero, void* part, int b, int n, int k, int steps,
                                hipStream_t stream) {
    constexpr int BP = BT * 16;
    const int tiles = (n + 15) / 16;
    const int tpw = steps * kStreamWaves;
    const size_t lds = (size_t)kStreamGP * 16 * BP * 16 + (size_t)kStreamGP * BP * 4;
    auto kern = qgemm_q4g128_stream_kernel<BT>;
    if (lds > 64 * 1024) {
        static const hipError_t opt = hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
            160 * 1024 - 1024);
        if (opt != hipSuccess) return opt;
    }
    dim3 grid((tiles + tpw - 1) / tpw, (k / 128) / kStreamGP);
    kern<<<grid, dim3(64 * kStreamWaves), lds, stream>>>(
        static_cast<const uint4_t*>(xprep), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<float*>(part), b, n, k, tpw);
    return hipGetLastError();
}

hipError_t qgemm_q4_stream_launch(const void* xprep, const void* qw, const void* scale,
                                  const void* zero, void* part, int b, int n, int k, int steps,
                                  hipStream_t stream) {
    if (b <= 16) return launch_stream<1>(xprep, qw, scale, zero, part, b, n, k, steps, stream);
    return launch_stream<2>(xprep, qw, scale, zero, part, b, n, k, steps, stream);
}

}  // namespace lg
