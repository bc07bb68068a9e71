// Q4G128 dequant-fused row-GEMV / GEMM for gfx950:
//   y[b][n] = bf16( sum_k x[b][k] * (q[n][k] - zero[n][k/128]) * scale[n][k/128] )
//
// Nibbles are never converted one by one.  OR-ing a nibble into the mantissa
// of the bf16 constant 128.0 (0x4300) yields the bf16 number 128 + q exactly,
// two per 32-bit register:  ((w >> 4s) & 0x000F000F) | 0x43004300  holds
// elements s and s+4 of the 8 nibbles of w.  Both kernels contract these
// "128 + q" values against x and remove the offset per group:
//   sum_k x_k (q_k - z) s  =  s * ( sum_k x_k (128 + q_k)  -  (128 + z) * sum_k x_k ).
// x is staged once per workgroup in LDS, already permuted to the (s, s+4)
// pair order, next to the per-chunk / per-group sums of x.
//
// Batch 1 and 2 (bandwidth-bound GEMV): VALU path.  One wave owns R rows; a lane
// reads 16 bytes (32 nibbles) of each row per step, unpacks them once and
// feeds v_dot2_f32_bf16 for every batch row.
//
// Batch >= 3, and batch 2 on large matrices: MFMA paths (the register-x kernel of
// qgemm_q4_regx.hip for K = 2048 / 4096, else qgemm_q4g128_mfma_kernel below).
//
// Algorithmic bytes per call: n*k/2 (nibbles) + n*(k/128)*4 (scale, zero)
// + b*k*2 (x) + b*n*2 (y).
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

// ---------------------------------------------------------------------------
// VALU path, batch B <= 4.  grid = ceil(n / (4*R)), block = 256 (4 waves).
// LDS: xp [B][4][nchunks] uint4 (x in pair order, piece-major so that a wave
// reads consecutive 16-byte words) and xs [B][nchunks] float (sum of x over
// the 32 elements of a chunk).
// ---------------------------------------------------------------------------
template <int B, int R>
__global__ __launch_bounds__(256) void qgemv_q4g128_kernel(const uint16_t* __restrict__ x,
                                                           const uint8_t* __restrict__ qw,
                                                           const __half* __restrict__ scale,
                                                           const __half* __restrict__ zero,
                                                           uint16_t* __restrict__ y,
                                                           const float* __restrict__ bias, int n, int k) {
    extern __shared__ uint4_t lds[];
    const int nchunks = k >> 5;  // 32 elements = 16 bytes of nibbles
    const int groups = k >> 7;
    uint4_t* xp = lds;
    float* xs = reinterpret_cast<float*>(lds + (size_t)B * 4 * nchunks);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * R;
    const int64_t row_bytes = k >> 1;

    // first step's weights go in flight before x is staged
    uint4_t w_next[R];
    {
        const int c = lane < nchunks ? lane : nchunks - 1;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t row = (row0 + r < n) ? (row0 + r) : (int64_t)(n - 1);
            w_next[r] = *reinterpret_cast<const uint4_t*>(qw + row * row_bytes + (int64_t)c * 16);
        }
    }

    for (int idx = threadIdx.x; idx < B * nchunks; idx += 256) {
        const int b = idx / nchunks, c = idx - b * nchunks;
        const uint4_t* src = reinterpret_cast<const uint4_t*>(x + (int64_t)b * k + (int64_t)c * 32);
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint4_t d = src[j];
            s += sum8_bf16(d);
            xp[((size_t)b * 4 + j) * nchunks + c] = pair_order(d);
        }
        xs[b * nchunks + c] = s;
    }
    __syncthreads();
    if (row0 >= n) return;

    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < B; ++b) acc[r][b] = 0.0f;

    // The magic constant lives in a VGPR the optimiser cannot see through, so
    // that (w & mask) | magic is one v_and_or_b32 (a VOP3 takes no literal and
    // at most one scalar operand on this target).
    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    for (int c0 = 0; c0 < nchunks; c0 += kWave) {
        const int c = c0 + lane;
        const bool live = c < nchunks;
        const int cc = live ? c : nchunks - 1;
        uint4_t w[R];
        __half sc[R], zr[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t row = (row0 + r < n) ? (row0 + r) : (int64_t)(n - 1);
            w[r] = w_next[r];
            sc[r] = scale[row * groups + (cc >> 2)];
            zr[r] = zero[row * groups + (cc >> 2)];
        }
        {   // next step's weights (clamped: the last step re-reads its own chunk)
            const int cn = (c0 + kWave + lane) < nchunks ? (c0 + kWave + lane) : cc;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int64_t row = (row0 + r < n) ? (row0 + r) : (int64_t)(n - 1);
                w_next[r] =
                    *reinterpret_cast<const uint4_t*>(qw + row * row_bytes + (int64_t)cn * 16);
            }
        }
        __builtin_amdgcn_sched_barrier(0);

        float raw[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) raw[r][b] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint4_t xv[B];
#pragma unroll
            for (int b = 0; b < B; ++b) xv[b] = xp[((size_t)b * 4 + j) * nchunks + cc];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const unsigned wd = w[r][j];
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const unsigned h = ((wd >> (4 * s)) & kNibMask) | magic;
#pragma unroll
                    for (int b = 0; b < B; ++b) raw[r][b] = dot2_bf16(h, xv[b][s], raw[r][b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const float xsum = live ? xs[b * nchunks + cc] : 0.0f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float sf = live ? __half2float(sc[r]) : 0.0f;
                const float off = 128.0f + __half2float(zr[r]);
                acc[r][b] = fmaf(sf, fmaf(-off, xsum, raw[r][b]), acc[r][b]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const float total = wave_sum(acc[r][b]);
            if (lane == 0 && row0 + r < n)
                y[(int64_t)b * n + row0 + r] =
                    f32_to_bf16_rne(bias ? total + bias[row0 + r] : total);
        }
}

template <int B, int R>
static hipError_t launch_gemv(const void* x, const void* qw, const void* scale, const void* zero,
                              void* y, const float* bias, int n, int k, hipStream_t stream) {
    const int nchunks = k / 32;
    const size_t lds = (size_t)B * nchunks * (4 * 16 + 4);
    auto kern = qgemv_q4g128_kernel<B, R>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    const int rows_per_block = 4 * R;
    dim3 grid((n + rows_per_block - 1) / rows_per_block), block(256);
    kern<<<grid, block, lds, stream>>>(static_cast<const uint16_t*>(x),
                                       static_cast<const uint8_t*>(qw),
                                       static_cast<const __half*>(scale),
                                       static_cast<const __half*>(zero),
                                       static_cast<uint16_t*>(y), bias, n, k);
    return hipGetLastError();
}

template <int B>
static hipError_t launch_gemv_b(const void* x, const void* qw, const void* scale, const void* zero,
                                void* y, const float* bias, int n, int k, hipStream_t stream) {
    // rows per wave: enough waves to cover the chip several times over
    if (n >= 8192) return launch_gemv<B, 4>(x, qw, scale, zero, y, bias, n, k, stream);
    if (n >= 4096) return launch_gemv<B, 2>(x, qw, scale, zero, y, bias, n, k, stream);
    return launch_gemv<B, 1>(x, qw, scale, zero, y, bias, n, k, stream);
}


// ---------------------------------------------------------------------------
// MFMA path, batch 5..32.  y^T is computed: the weight tile is the B operand
// of v_mfma_f32_16x16x32_bf16 (column = weight row n, 8 contraction elements
// per lane = one dword of nibbles turned into four bf16 pairs), x is the A
// operand (row = batch index), so that the four results a lane holds all
// belong to ONE weight row and need only that row's scale / zero.
//
// A workgroup owns T tiles of 16 weight rows and ALL of K, split across its W
// waves: in phase p, wave w owns the GW consecutive groups starting at
// (p*W + w)*GW.  Its slice of x (all batch rows, GW*128 columns) is loaded
// straight from global memory (L2-resident) into MFMA A-operand registers once
// per phase and reused for every tile; one 16-byte load per lane covers a whole
// group (128 nibbles) of a weight row: lane (n = lane%16, kc = lane/16) reads
// bytes [64 g + 16 kc, +16) of row n, its dword t feeds MFMA t, which therefore
// contracts over k = 128 g + 32 kc + 8 t + (0..7), kc = 0..3.  Every load of a
// phase is issued before any of it is consumed.  Waves never wait for each
// other while streaming: every wave keeps its partial results in its own LDS
// slot (LDS float atomics on shared accumulators measured 2-4x slower for the
// whole kernel), and the slots are summed once after the only barrier.  scale / zero of the
// workgroup's rows are staged in LDS with one coalesced copy (per-lane 2-byte
// loads from 16 different rows per instruction are what this avoids).
// ---------------------------------------------------------------------------
template <int BT, int GW, int T>
__global__ __launch_bounds__(1024) void qgemm_q4g128_mfma_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero, uint16_t* __restrict__ y,
    const float* __restrict__ bias, int b, int n, int k) {
    extern __shared__ uint4_t lds[];
    constexpr int BP = BT * 16;
    const int groups = k >> 7;
    float* yl = reinterpret_cast<float*>(lds);  // [waves][T][BP][16] partial results
    __half* sz = reinterpret_cast<__half*>(yl + (size_t)(blockDim.x >> 6) * T * BP * 16);
    // sz: scale [T*16][groups], then zero [T*16][groups]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int col = lane & 15;
    const int kc = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.x * T * 16;
    const int rows_here = (int)min((int64_t)(T * 16), (int64_t)n - row0);

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    struct Phase {
        uint4_t xa[GW][4][BT];
        uint4_t w[T][GW];
    };
    const uint8_t* wrow[T];
#pragma unroll
    for (int ti = 0; ti < T; ++ti) {
        const int r = ti * 16 + col;
        wrow[ti] = qw + (row0 + (r < rows_here ? r : rows_here - 1)) * (int64_t)(k >> 1) + kc * 16;
    }
    const uint16_t* xrow[BT];
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) {
        const int bi = bt * 16 + col;
        xrow[bt] = x + (int64_t)(bi < b ? bi : b - 1) * k + kc * 32;
    }
    auto issue = [&](int phase, Phase& ph) {
        const int g0 = (phase * nwaves + wave) * GW;
#pragma unroll
        for (int i = 0; i < GW; ++i) {
            const int g = (g0 + i) < groups ? (g0 + i) : (groups - 1);
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    ph.xa[i][t][bt] =
                        *reinterpret_cast<const uint4_t*>(xrow[bt] + (int64_t)g * 128 + t * 8);
        }
#pragma unroll
        for (int ti = 0; ti < T; ++ti)
#pragma unroll
            for (int i = 0; i < GW; ++i) {
                const int g = (g0 + i) < groups ? (g0 + i) : (groups - 1);
                ph.w[ti][i] = *reinterpret_cast<const uint4_t*>(wrow[ti] + (int64_t)g * 64);
            }
    };

    const int num_phases = (groups + nwaves * GW - 1) / (nwaves * GW);
    Phase ph;
    issue(0, ph);
    __builtin_amdgcn_sched_barrier(0);

    float* yw = yl + (size_t)wave * T * BP * 16;
    // while the first loads fly: stage scale / zero
    {
        const int count = rows_here * groups;
        const __half* s0 = scale + row0 * groups;
        const __half* z0 = zero + row0 * groups;
        for (int i = threadIdx.x; i < count; i += blockDim.x) {
            sz[i] = s0[i];
            sz[T * 16 * groups + i] = z0[i];
        }
    }
    __syncthreads();
    const __half* zl = sz + T * 16 * groups;

    for (int phase = 0; phase < num_phases; ++phase) {
        if (phase > 0) {
            issue(phase, ph);
            __builtin_amdgcn_sched_barrier(0);
        }
        const int g0 = (phase * nwaves + wave) * GW;
        // x slice: pair order in place, per-group sums of x in result layout
        float xsum[GW][BT][4];
#pragma unroll
        for (int i = 0; i < GW; ++i)
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) {
                float part = 0.0f;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    part += sum8_bf16(ph.xa[i][t][bt]);
                    ph.xa[i][t][bt] = pair_order(ph.xa[i][t][bt]);
                }
                part += shfl_xor_f32(part, 16);
                part += shfl_xor_f32(part, 32);  // sum over the group for batch row `col`
#pragma unroll
                for (int e = 0; e < 4; ++e) xsum[i][bt][e] = __shfl(part, 4 * kc + e, kWave);
            }
#pragma unroll
        for (int ti = 0; ti < T; ++ti) {
            float4_t ysum[BT];
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) ysum[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
            const int r = ti * 16 + col;
            const int rl = r < rows_here ? r : rows_here - 1;
#pragma unroll
            for (int i = 0; i < GW; ++i) {
                const bool valid = (g0 + i) < groups;  // wave-uniform
                const int g = valid ? (g0 + i) : (groups - 1);
                const float sf = __half2float(sz[rl * groups + g]);
                const float off = 128.0f + __half2float(zl[rl * groups + g]);
                float4_t acc[BT];
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const unsigned wd = ph.w[ti][i][t];
                    uint4_t h;
#pragma unroll
                    for (int sft = 0; sft < 4; ++sft)
                        h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                    const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
#pragma unroll
                    for (int bt = 0; bt < BT; ++bt)
                        acc[bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, ph.xa[i][t][bt]), bop, acc[bt], 0, 0, 0);
                }
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float v = fmaf(sf, fmaf(-off, xsum[i][bt][e], acc[bt][e]), ysum[bt][e]);
                        ysum[bt][e] = valid ? v : ysum[bt][e];
                    }
            }
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int e = 0; e < 4; ++e)
{
                    // this wave's own slot: no other wave touches it before the barrier
                    float* slot = &yw[(ti * BP + bt * 16 + 4 * kc + e) * 16 + col];
                    *slot = (phase == 0) ? ysum[bt][e] : (*slot + ysum[bt][e]);
                }
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < T * BP * 16; i += blockDim.x) {
        const int c = i & 15;
        const int bi = (i >> 4) % BP;
        const int ti = i / (BP * 16);
        const int r = ti * 16 + c;
        float sum = 0.0f;
        for (int w = 0; w < nwaves; ++w) sum += yl[(size_t)w * T * BP * 16 + i];
        if (r < rows_here && bi < b)
            y[(int64_t)bi * n + row0 + r] = f32_to_bf16_rne(bias ? sum + bias[row0 + r] : sum);
    }
}

constexpr size_t kMaxLds = 160 * 1024;

// LDS bytes of the MFMA path (per-wave partial slots + staged scales and zeros) for the
// template form launch_mfma picks; the shape check and the launcher share it.
static size_t mfma_lds_bytes(int b, int n, int k) {
    const int groups = k / 128;
    const int bt = b <= 16 ? 1 : 2;
    const int gw = b <= 16 ? 2 : 1;
    int waves = (groups + gw - 1) / gw;
    if (waves > 16) waves = 16;
    const int tiles = (n + 15) / 16;
    const int cus = device_cu_count();
    int t = (tiles + cus - 1) / cus;
    if (t > 3) t = 3;
    return (size_t)waves * t * bt * 16 * 16 * 4 + (size_t)2 * t * 16 * groups * 2;
}

template <int BT, int GW, int T>
static hipError_t launch_mfma_t(const void* x, const void* qw, const void* scale, const void* zero,
                                void* y, const float* bias, int b, int n, int k,
                                hipStream_t stream) {
    const int groups = k / 128;
    const int tiles = (n + 15) / 16;
    int waves = (groups + GW - 1) / GW;
    if (waves > 16) waves = 16;
    const size_t lds =
        (size_t)waves * T * BT * 16 * 16 * 4 + (size_t)2 * T * 16 * groups * 2;
    auto kern = qgemm_q4g128_mfma_kernel<BT, GW, T>;
    if (lds > kMaxLds) return hipErrorInvalidValue;  // the shape check refuses these shapes
    // opt in to the full LDS once per instantiation (the attribute is per function and device;
    // one device per process here)
    static const hipError_t attr =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds);
    if (attr != hipSuccess) return attr;
    kern<<<dim3((tiles + T - 1) / T), dim3(64 * waves), lds, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<uint16_t*>(y), bias, b, n, k);
    return hipGetLastError();
}

template <int BT, int GW>
static hipError_t launch_mfma(const void* x, const void* qw, const void* scale, const void* zero,
                              void* y, const float* bias, int b, int n, int k,
                              hipStream_t stream) {
    const int tiles = (n + 15) / 16;
    const int cus = device_cu_count();
    const int t = (tiles + cus - 1) / cus;  // row tiles per workgroup (LDS slots cap it at 3)
    if (t >= 3) return launch_mfma_t<BT, GW, 3>(x, qw, scale, zero, y, bias, b, n, k, stream);
    if (t == 2) return launch_mfma_t<BT, GW, 2>(x, qw, scale, zero, y, bias, b, n, k, stream);
    return launch_mfma_t<BT, GW, 1>(x, qw, scale, zero, y, bias, b, n, k, stream);
}

}  // namespace lg

extern "C" logismos_status_t logismos_check_qgemm_q4g128_shape(int b, int n, int k, char* msg,
                                                               size_t msg_cap) {
    const char* kn = "qgemm_q4g128_bf16";
    if (b <= 0) return lg::reject(msg, msg_cap, "%s: batch must be positive, got %d", kn, b);
    if (n <= 0) return lg::reject(msg, msg_cap, "%s: N must be positive, got %d", kn, n);
    if (k <= 0) return lg::reject(msg, msg_cap, "%s: K must be positive, got %d", kn, k);
    if (k % 128 != 0)
        return lg::reject(msg, msg_cap, "%s: K = %d is not a multiple of the group size 128", kn, k);
    if ((int64_t)n * k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "%s: N*K = %lld exceeds i32::MAX", kn,
                          (long long)((int64_t)n * k));
    if ((int64_t)b * n > (int64_t)INT32_MAX || (int64_t)b * k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "%s: batch*N or batch*K exceeds i32::MAX", kn);
    // rows beyond 32 are taken 32 at a time: the per-launch bounds hold for a full pass and for
    // the ragged last pass (which may fall to another kernel family), so that no launch of a
    // call is refused after an earlier one has written its rows
    const int passes[2] = {b < 32 ? b : 32, b > 32 ? b % 32 : 0};
    for (const int rows : passes) {
        if (rows == 0) continue;
        if (rows <= 4 && (size_t)rows * (k / 32) * 68 > lg::kMaxLds)
            return lg::reject(msg, msg_cap,
                              "%s: %d rows x K = %d do not fit the LDS staging of x", kn, rows, k);
        // the matrix-core path (3 rows or more; ..._bf16_mfma refuses such a shape at any batch)
        // stages a workgroup's scales and zeros for all of K next to its partial sums
        if (rows >= 3 && lg::mfma_lds_bytes(rows, n, k) > lg::kMaxLds)
            return lg::reject(msg, msg_cap,
                              "%s: K = %d needs %zu bytes of LDS on the matrix-core path (limit %zu)",
                              kn, k, lg::mfma_lds_bytes(rows, n, k), lg::kMaxLds);
    }
    return 0;
}

// One launch for up to 32 activation rows.
static logismos_status_t qgemm_q4_dispatch32(const void* x_bf16, const void* qw_u8,
                                             const void* scale_f16, const void* zero_f16,
                                             const float* bias, void* y_bf16, int b, int n, int k,
                                             bool force_mfma, hipStream_t st) {
    if (!force_mfma) {
        switch (b) {
            case 1:
                return lg::launch_gemv_b<1>(x_bf16, qw_u8, scale_f16, zero_f16, y_bf16, bias, n, k, st);
            case 2:
                if (lg::regx_plain_plan(b, n, k).parts == 1) break;  // large matrices, see there
                return lg::launch_gemv_b<2>(x_bf16, qw_u8, scale_f16, zero_f16, y_bf16, bias, n, k, st);
            default: break;  // batch 3 and 4: the MFMA kernels are faster (measured crossover)
        }
        // K = 2048 / 4096: x in registers, weights through the LDS ring, one workgroup per K
        if (const lg::RegxPlan rp = lg::regx_plain_plan(b, n, k); rp.parts == 1)
            return lg::qgemm_q4_regx_plain_launch(rp, x_bf16, qw_u8, scale_f16, zero_f16, y_bf16, bias,
                                                  b, n, k, st);
    }
    if (b <= 16)
        return lg::launch_mfma<1, 2>(x_bf16, qw_u8, scale_f16, zero_f16, y_bf16, bias, b, n, k, st);
    return lg::launch_mfma<2, 1>(x_bf16, qw_u8, scale_f16, zero_f16, y_bf16, bias, b, n, k, st);
}

// `linear_t` takes any m (crates/kernels/src/cpu_f32/mod.rs:271-345).  The decode kernels hold
// at most 32 activation rows per workgroup, so a somewhat taller x is taken 32 rows at a time
// (every launch streams the weights once); from about a hundred rows on (the prefill chunks
// of a mixed batch) the tiled kernel of qgemm_q4_tall.hip takes over.
static logismos_status_t qgemm_q4_dispatch(const void* x_bf16, const void* qw_u8,
                                           const void* scale_f16, const void* zero_f16,
                                           const void* bias_f32, void* y_bf16, int b, int n, int k,
                                           bool force_mfma, logismos_stream_t stream) {
    if (logismos_check_qgemm_q4g128_shape(b, n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!x_bf16 || !qw_u8 || !scale_f16 || !zero_f16 || !y_bf16) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) & 15u) || (reinterpret_cast<uintptr_t>(x_bf16) & 15u))
        return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const float* bias = static_cast<const float*>(bias_f32);
    // many rows: the tiled kernel, one pass over the weights per 128 rows of x and the matrix
    // cores as its bound
    if (!force_mfma && lg::qgemm_q4_tall_applies(b, n, k))
        return lg::qgemm_q4_tall_launch(x_bf16, qw_u8, scale_f16, zero_f16, bias, y_bf16, b, n, k,
                                        st);
    for (int m0 = 0; m0 < b; m0 += 32) {
        const int rows = b - m0 < 32 ? b - m0 : 32;
        const logismos_status_t e = qgemm_q4_dispatch32(
            static_cast<const uint16_t*>(x_bf16) + (int64_t)m0 * k, qw_u8, scale_f16, zero_f16, bias,
            static_cast<uint16_t*>(y_bf16) + (int64_t)m0 * n, rows, n, k, force_mfma, st);
        if (e != 0) return e;
    }
    return 0;
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_bf16(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* y_bf16, int b, int n, int k, logismos_stream_t stream) {
    return qgemm_q4_dispatch(x_bf16, qw_u8, scale_f16, zero_f16, nullptr, y_bf16, b, n, k, false,
                             stream);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_bf16_bias(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    const void* bias_f32, void* y_bf16, int b, int n, int k, logismos_stream_t stream) {
    return qgemm_q4_dispatch(x_bf16, qw_u8, scale_f16, zero_f16, bias_f32, y_bf16, b, n, k, false,
                             stream);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_bf16_mfma(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* y_bf16, int b, int n, int k, logismos_stream_t stream) {
    return qgemm_q4_dispatch(x_bf16, qw_u8, scale_f16, zero_f16, nullptr, y_bf16, b, n, k, true,
                             stream);
}
