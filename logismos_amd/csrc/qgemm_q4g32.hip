// Q4G32 dequant-fused GEMM for a decode batch (1 .. 32 rows) on gfx950:
//   y[b][n] = bf16( sum_k x[b][k] * (q[n][k] * scale[n][k/32] + min[n][k/32]) )
// over the planar form of ggml Q4_0 / Q4_1 weights that the repack kernels of
// qgemv_q4g32.hip write.  x and y are bf16 like those of the Q4G128 GEMM.
//
// One v_mfma_f32_16x16x32_bf16 contracts exactly one group of 32 columns, so a group's
// scale and min apply to a whole MFMA result:
//   y += d * (sum_k x_k (128 + q_k) - 128 * sum_k x_k) + m * sum_k x_k
// with the "128 + q" bf16 values of the magic-number unpack (q4_common.hpp) as the B operand
// (column = weight row), x as the A operand (row = batch index) and the group sums of x from
// one more MFMA against a B operand of ones, which leaves them in the result layout.
//
// A lane (col = lane % 16, kc = lane / 16) loads the 16 bytes of group 4c + kc of weight row
// `col` (c: a chunk of 128 columns), i.e. whole groups per lane, 64 contiguous bytes per row.
// The MFMA wants dword kc of group t in lane kc instead: a 4 x 4 transpose between the four
// lanes that share `col` and the four dwords, done with two row swaps and two half-wave
// swaps (v_permlane16_swap, v_permlane32_swap).
//
// A workgroup of 8 waves owns T tiles of 16 weight rows and all of K; wave w takes the
// chunks w, w + 8, ... with the next chunk's loads in flight while the current one is
// multiplied.  Partial sums meet once, through LDS, after the only barrier.
//
// Algorithmic bytes per call: n*k/2 (nibbles) + n*(k/32)*4 (scale, min) + 2*b*k + 2*b*n.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

constexpr int kG32Waves = 8;

// lanes (col, kc) hold w[t] = dword t of group kc  ->  w[t] = dword kc of group t
__device__ __forceinline__ uint4_t transpose_groups(uint4_t w) {
    // rows of 16 lanes: (register bit 0) <-> (kc bit 0)
    const auto a = __builtin_amdgcn_permlane16_swap(w[0], w[1], false, false);
    const auto b = __builtin_amdgcn_permlane16_swap(w[2], w[3], false, false);
    // halves of 32 lanes: (register bit 1) <-> (kc bit 1)
    const auto c = __builtin_amdgcn_permlane32_swap(a[0], b[0], false, false);
    const auto d = __builtin_amdgcn_permlane32_swap(a[1], b[1], false, false);
    return uint4_t{c[0], d[0], c[1], d[1]};
}

// What a wave has in flight for one chunk of 128 columns, in the layout it is LOADED in:
// four consecutive lanes read 64 consecutive bytes (of x: sixteen lanes read a row's 256), so
// a request touches each cache line once.  Loading straight into the MFMA operand layout
// (lane = row % 16 + 16 * piece) put the four lanes of every quad on four different rows, a
// tag look-up per lane: the texture addresser was busy 75 % of the launch and set its pace.
template <int BT, int T>
struct G32Chunk {
    uint4_t x[4][BT];  // batch row bt * 16 + 4 i + lane / 16, columns 8 (lane % 16) .. + 7
    uint4_t w[T];      // group lane % 4 of weight row ti * 16 + lane / 4
    unsigned short sc[T], mn[T];  // that group's scale and min
};

// per-wave LDS staging: the loaded layout goes in, the operand layout comes out (the LDS
// queue of a wave is in order, so no wait sits between the write and the read)
constexpr int kG32XRow = 272;                     // bytes per staged x row (256 + 16: no conflicts)
constexpr int kG32WRow = 80;                      // bytes per staged weight row (64 + 16)
constexpr int kG32StageX = 16 * kG32XRow;         // one 16-row x block
constexpr int kG32StageW = 16 * kG32WRow;
constexpr int kG32StageS = 16 * 8;                // four fp16 per row
constexpr int kG32Stage = kG32StageX + kG32StageW + 2 * kG32StageS;

template <int BT, int T>
__global__ __launch_bounds__(64 * kG32Waves) void qgemm_q4g32_mfma_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ minv, uint16_t* __restrict__ y,
    const float* __restrict__ bias, int b, int n, int k) {
    // the staging areas of the eight waves; afterwards [waves][T][BP][16] partial results
    extern __shared__ __attribute__((aligned(16))) unsigned char g32_lds[];
    float* yl = reinterpret_cast<float*>(g32_lds);
    constexpr int BP = BT * 16;
    const int nchunks = k >> 7;
    const int groups = k >> 5;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int kc = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.x * T * 16;
    const int rows_here = (int)min((int64_t)(T * 16), (int64_t)n - row0);

    unsigned magic, ones;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));
    asm volatile("v_mov_b32 %0, 0x3f803f80" : "=v"(ones));
    const bf16x8_t one_op = __builtin_bit_cast(bf16x8_t, uint4_t{ones, ones, ones, ones});

    // rows and batch rows past the end re-read the last one; their results are not stored
    const uint8_t* wrow[T];
    const __half* srow[T];
    const __half* mrow[T];
#pragma unroll
    for (int ti = 0; ti < T; ++ti) {
        const int r = ti * 16 + (lane >> 2);
        const int64_t row = row0 + (r < rows_here ? r : rows_here - 1);
        wrow[ti] = qw + row * (int64_t)(k >> 1) + (lane & 3) * 16;
        srow[ti] = scale + row * groups + (lane & 3);
        mrow[ti] = minv + row * groups + (lane & 3);
    }
    const uint16_t* xrow[4][BT];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) {
            const int bi = bt * 16 + 4 * i + kc;
            xrow[i][bt] = x + (int64_t)(bi < b ? bi : b - 1) * k + col * 8;
        }
    auto load_chunk = [&](int c, G32Chunk<BT, T>& ch) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
                ch.x[i][bt] = *reinterpret_cast<const uint4_t*>(xrow[i][bt] + c * 128);
#pragma unroll
        for (int ti = 0; ti < T; ++ti) {
            ch.w[ti] = *reinterpret_cast<const uint4_t*>(wrow[ti] + c * 64);
            ch.sc[ti] = *reinterpret_cast<const unsigned short*>(srow[ti] + c * 4);
            ch.mn[ti] = *reinterpret_cast<const unsigned short*>(mrow[ti] + c * 4);
        }
    };

    float4_t ysum[T][BT];
#pragma unroll
    for (int ti = 0; ti < T; ++ti)
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) ysum[ti][bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    unsigned char* stage = g32_lds + (size_t)wave * kG32Stage;
    unsigned char* st_x = stage;
    unsigned char* st_w = stage + kG32StageX;
    unsigned char* st_s = st_w + kG32StageW;
    unsigned char* st_m = st_s + kG32StageS;
    // a wave's LDS accesses execute in program order; this only keeps the compiler from
    // moving one across (another lane's data is not a dependence it sees)
    auto in_order = [&]() {
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };

    auto compute_chunk = [&](const G32Chunk<BT, T>& ch) {
        // x in operand layout: xa[t][bt] = group t, columns 8 kc .. 8 kc + 7, batch row
        // bt * 16 + col
        uint4_t xa[4][BT];
        // sums of x over each group, in result layout: xs[t][bt][e] belongs to batch row
        // bt * 16 + 4 kc + e (the same for every column)
        float4_t xs[4][BT];
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) {
            in_order();
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<uint4_t*>(st_x + (4 * i + kc) * kG32XRow + col * 16) = ch.x[i][bt];
            in_order();
#pragma unroll
            for (int t = 0; t < 4; ++t)
                xa[t][bt] = *reinterpret_cast<const uint4_t*>(st_x + col * kG32XRow + t * 64 + kc * 16);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) {
                xs[t][bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8_t, xa[t][bt]), one_op,
                    float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                xa[t][bt] = pair_order(xa[t][bt]);
            }
#pragma unroll
        for (int ti = 0; ti < T; ++ti) {
            in_order();
            *reinterpret_cast<uint4_t*>(st_w + (lane >> 2) * kG32WRow + (lane & 3) * 16) = ch.w[ti];
            *reinterpret_cast<unsigned short*>(st_s + (lane >> 2) * 8 + (lane & 3) * 2) = ch.sc[ti];
            *reinterpret_cast<unsigned short*>(st_m + (lane >> 2) * 8 + (lane & 3) * 2) = ch.mn[ti];
            in_order();
            const uint4_t wl = *reinterpret_cast<const uint4_t*>(st_w + col * kG32WRow + kc * 16);
            const uint2_t sc4 = *reinterpret_cast<const uint2_t*>(st_s + col * 8);
            const uint2_t mn4 = *reinterpret_cast<const uint2_t*>(st_m + col * 8);
            const uint4_t wt = transpose_groups(wl);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const unsigned sw = sc4[t >> 1], mw = mn4[t >> 1];
                const unsigned short sh = (unsigned short)((t & 1) ? (sw >> 16) : (sw & 0xffffu));
                const unsigned short mh = (unsigned short)((t & 1) ? (mw >> 16) : (mw & 0xffffu));
                const float d = __half2float(__builtin_bit_cast(__half, sh));
                const float m = __half2float(__builtin_bit_cast(__half, mh));
                const unsigned wd = wt[t];
                uint4_t h;
#pragma unroll
                for (int sft = 0; sft < 4; ++sft) h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) {
                    const float4_t acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, xa[t][bt]), bop,
                        float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float xsum = xs[t][bt][e];
                        float v = fmaf(d, fmaf(-128.0f, xsum, acc[e]), ysum[ti][bt][e]);
                        ysum[ti][bt][e] = fmaf(m, xsum, v);
                    }
                }
            }
        }
    };

    // two chunks per iteration in one straight-line body; a chunk index past the end
    // re-reads the wave's last chunk and is not computed
    if (wave < nchunks) {
        const int c_last = wave + ((nchunks - 1 - wave) / kG32Waves) * kG32Waves;
        G32Chunk<BT, T> ca, cb;
        load_chunk(wave, ca);
        for (int c = wave; c < nchunks; c += 2 * kG32Waves) {
            load_chunk(min(c + kG32Waves, c_last), cb);
            __builtin_amdgcn_sched_barrier(0);
            compute_chunk(ca);
            __builtin_amdgcn_sched_barrier(0);
            load_chunk(min(c + 2 * kG32Waves, c_last), ca);
            __builtin_amdgcn_sched_barrier(0);
            if (c + kG32Waves < nchunks) compute_chunk(cb);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();  // the partial results reuse the staging areas

    float* yw = yl + (size_t)wave * T * BP * 16;
#pragma unroll
    for (int ti = 0; ti < T; ++ti)
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                yw[(ti * BP + bt * 16 + 4 * kc + e) * 16 + col] = ysum[ti][bt][e];
    __syncthreads();
    for (int i = threadIdx.x; i < T * BP * 16; i += 64 * kG32Waves) {
        const int c = i & 15;
        const int bi = (i >> 4) % BP;
        const int ti = i / (BP * 16);
        const int r = ti * 16 + c;
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < kG32Waves; ++w) sum += yl[(size_t)w * T * BP * 16 + i];
        if (r < rows_here && bi < b)
            y[(int64_t)bi * n + row0 + r] = f32_to_bf16_rne(bias ? sum + bias[row0 + r] : sum);
    }
}

template <int BT, int T>
static hipError_t launch_g32(const void* x, const void* qw, const void* scale, const void* minv,
                             void* y, const float* bias, int b, int n, int k, hipStream_t stream) {
    const int tiles = (n + 15) / 16;
    const size_t parts = (size_t)kG32Waves * T * BT * 16 * 16 * 4;  // at most 48 KiB
    const size_t staging = (size_t)kG32Waves * kG32Stage;           // 46 KiB
    const size_t lds = parts > staging ? parts : staging;
    qgemm_q4g32_mfma_kernel<BT, T><<<dim3((tiles + T - 1) / T), dim3(64 * kG32Waves), lds, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(minv),
        static_cast<uint16_t*>(y), bias, b, n, k);
    return hipGetLastError();
}

template <int BT>
static hipError_t launch_g32_b(const void* x, const void* qw, const void* scale, const void* minv,
                               void* y, const float* bias, int b, int n, int k,
                               hipStream_t stream) {
    // row tiles per workgroup: one workgroup per CU where the matrix allows it
    const int tiles = (n + 15) / 16;
    const int t = (tiles + device_cu_count() - 1) / device_cu_count();
    if (t >= 3) return launch_g32<BT, 3>(x, qw, scale, minv, y, bias, b, n, k, stream);
    if (t == 2) return launch_g32<BT, 2>(x, qw, scale, minv, y, bias, b, n, k, stream);
    return launch_g32<BT, 1>(x, qw, scale, minv, y, bias, b, n, k, stream);
}

}  // namespace lg

extern "C" logismos_status_t logismos_check_qgemm_q4g32_shape(int b, int n, int k, char* msg,
                                                              size_t msg_cap) {
    const char* kn = "qgemm_q4g32_bf16";
    if (b <= 0) return lg::reject(msg, msg_cap, "%s: batch must be positive, got %d", kn, b);
    if (n <= 0) return lg::reject(msg, msg_cap, "%s: N must be positive, got %d", kn, n);
    if (k <= 0) return lg::reject(msg, msg_cap, "%s: K must be positive, got %d", kn, k);
    if (k % 128 != 0)
        return lg::reject(msg, msg_cap, "%s: K = %d is not a multiple of 128 (four groups of 32)",
                          kn, k);
    if ((int64_t)n * k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "%s: N*K = %lld exceeds i32::MAX", kn,
                          (long long)((int64_t)n * k));
    if ((int64_t)b * n > (int64_t)INT32_MAX || (int64_t)b * k > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "%s: batch*N or batch*K exceeds i32::MAX", kn);
    return 0;
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g32_bf16_bias(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* min_f16,
    const void* bias_f32, void* y_bf16, int b, int n, int k, logismos_stream_t stream) {
    if (logismos_check_qgemm_q4g32_shape(b, n, k, nullptr, 0) != 0) return hipErrorInvalidValue;
    if (!x_bf16 || !qw_u8 || !scale_f16 || !min_f16 || !y_bf16) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) & 15u) || (reinterpret_cast<uintptr_t>(x_bf16) & 15u) ||
        (reinterpret_cast<uintptr_t>(scale_f16) & 7u) || (reinterpret_cast<uintptr_t>(min_f16) & 7u))
        return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const float* bias = static_cast<const float*>(bias_f32);  // may be null: no bias
    // a taller x is taken 32 rows at a time (`linear_t` takes any m)
    for (int m0 = 0; m0 < b; m0 += 32) {
        const int rows = b - m0 < 32 ? b - m0 : 32;
        const uint16_t* xs = static_cast<const uint16_t*>(x_bf16) + (int64_t)m0 * k;
        uint16_t* ys = static_cast<uint16_t*>(y_bf16) + (int64_t)m0 * n;
        const hipError_t e =
            rows <= 16 ? lg::launch_g32_b<1>(xs, qw_u8, scale_f16, min_f16, ys, bias, rows, n, k, st)
                       : lg::launch_g32_b<2>(xs, qw_u8, scale_f16, min_f16, ys, bias, rows, n, k, st);
        if (e != hipSuccess) return e;
    }
    return 0;
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g32_bf16(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* min_f16,
    void* y_bf16, int b, int n, int k, logismos_stream_t stream) {
    return logismos_launch_qgemm_q4g32_bf16_bias(x_bf16, qw_u8, scale_f16, min_f16, nullptr, y_bf16,
                                                 b, n, k, stream);
}
