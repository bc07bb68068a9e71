// Probes of the part.  Memory system: a plain 16-byte-per-lane copy kernel and a read-only
// sum kernel (plain or non-temporal loads).  They give the box's achievable HBM ceiling next to the
// datasheet figure, and the calibration factor for the FETCH_SIZE /
// WRITE_SIZE hardware counters (a copy of known size).  Matrix cores: nothing but MFMAs,
// on operands that stay the same or that change with every instruction -- what the pipes
// sustain next to the datasheet rate.
#include "device_utils.hpp"
#include "launch_common.hpp"

namespace lg {

constexpr int kProbeMfmaWorkgroups = 256;  // one workgroup of eight waves per CU

__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4_t* __restrict__ src,
                                                         uint4_t* __restrict__ dst, int64_t n16) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        dst[i] = src[i];
}

// Read-only sum, 4 x 16 bytes per lane in flight.  NT: the loads are non-temporal, as the decode
// attention reads K and V (every byte used once per step).  STRIDED: the workgroups take
// chunks of blockDim.x * 4 pieces in turn (grid-stride) instead of one contiguous slab each.
template <bool NT, bool STRIDED>
__global__ __launch_bounds__(512) void probe_read_kernel(const uint4_t* __restrict__ src,
                                                         unsigned* __restrict__ sink, int64_t n16) {
    const int64_t T = blockDim.x;
    const int64_t chunks = (n16 + 4 * T - 1) / (4 * T);
    int64_t c0, c1, cs;
    if (STRIDED) {
        c0 = blockIdx.x, c1 = chunks, cs = gridDim.x;
    } else {
        const int64_t per = (chunks + gridDim.x - 1) / gridDim.x;
        c0 = (int64_t)blockIdx.x * per, c1 = c0 + per < chunks ? c0 + per : chunks, cs = 1;
    }
    auto ld = [&](int64_t j) {
        j = j < n16 ? j : n16 - 1;  // the ragged tail re-reads the last piece
        return NT ? __builtin_nontemporal_load(src + j) : src[j];
    };
    unsigned acc = 0;
    for (int64_t c = c0; c < c1; c += cs) {
        const int64_t i = c * 4 * T + threadIdx.x;
        const uint4_t a = ld(i), b = ld(i + T), e = ld(i + 2 * T), d = ld(i + 3 * T);
        acc ^= a[0] ^ a[1] ^ a[2] ^ a[3] ^ b[0] ^ b[1] ^ b[2] ^ b[3];
        acc ^= e[0] ^ e[1] ^ e[2] ^ e[3] ^ d[0] ^ d[1] ^ d[2] ^ d[3];
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;  // practically never; keeps the loads alive
}

// Back-to-back v_mfma_f32_32x32x16 on four accumulators, two waves per SIMD on every CU.
// CHANGING: both operands are rewritten between the MFMAs (fresh mantissas and signs,
// exponents of 0.5 .. 1) by vector instructions that issue under the running MFMA; otherwise
// the operands are 1.0 throughout.  Same instruction stream apart from that.  On the part
// this was written on, the first form runs at 32 clocks per MFMA and ~2.2 GHz, the second 1.6
// times slower by the wall clock: its power management holds the matrix pipes back when
// their inputs toggle, which is what they do on real data.
template <bool BF16, bool CHANGING>
__global__ __launch_bounds__(512) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
    float16_t acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.0f;
    // bit patterns: fp16 1.0 = 0x3c00, bf16 1.0 = 0x3f80; changing values keep the exponent
    // field at 0.5 .. 1 and take sign and mantissa from a multiplicative generator
    constexpr unsigned kOne = BF16 ? 0x3f803f80u : 0x3c003c00u;
    constexpr unsigned kKeep = BF16 ? 0x807f807fu : 0x83ff83ffu;
    constexpr unsigned kExp = BF16 ? 0x3f003f00u : 0x38003800u;
    unsigned h = threadIdx.x * 2654435761u + blockIdx.x * 40503u;
    uint4_t a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        h = h * 1664525u + 1013904223u;
        a[i] = CHANGING ? ((h & kKeep) | kExp) : kOne;
        h = h * 1664525u + 1013904223u;
        b[i] = CHANGING ? ((h & kKeep) | kExp) : kOne;
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if constexpr (BF16)
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                                 __builtin_bit_cast(bf16x8_t, b),
                                                                 acc[t], 0, 0, 0);
            else
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a),
                                                                __builtin_bit_cast(half8_t, b),
                                                                acc[t], 0, 0, 0);
            if constexpr (CHANGING) {
                a[t] = ((a[t] * 5u + 0x01230123u) & kKeep) | kExp;
                b[t] = ((b[t] * 9u + 0x04560456u) & kKeep) | kExp;
            } else {
                // the same number of vector instructions, on values that do not change
                asm volatile("v_mov_b32 %0, %0\n\tv_mov_b32 %1, %1\n\tv_nop\n\tv_nop\n\tv_nop\n\tv_nop"
                             : "+v"(a[t]), "+v"(b[t]));
            }
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[t][e];
    if (s == 12345.678f) sink[0] = s;  // practically never; keeps the products alive
}

}  // namespace lg

extern "C" logismos_status_t logismos_launch_probe_mfma(void* sink_f32, int iters, int flags,
                                                        logismos_stream_t stream) {
    if (!sink_f32 || iters <= 0 || (flags & ~3)) return hipErrorInvalidValue;
    float* sink = static_cast<float*>(sink_f32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(lg::kProbeMfmaWorkgroups), block(512);
    switch (flags) {
        case 0: lg::probe_mfma_kernel<false, false><<<grid, block, 0, st>>>(sink, iters); break;
        case 1: lg::probe_mfma_kernel<false, true><<<grid, block, 0, st>>>(sink, iters); break;
        case 2: lg::probe_mfma_kernel<true, false><<<grid, block, 0, st>>>(sink, iters); break;
        default: lg::probe_mfma_kernel<true, true><<<grid, block, 0, st>>>(sink, iters); break;
    }
    return hipGetLastError();
}

extern "C" double logismos_probe_mfma_flops(int iters) {
    // per launch: workgroups x 8 waves x iters x 4 MFMAs x 32 x 32 x 16 x 2
    return (double)lg::kProbeMfmaWorkgroups * 8.0 * (double)iters * 4.0 * 32768.0;
}

extern "C" logismos_status_t logismos_launch_probe_copy(const void* src, void* dst, size_t bytes,
                                                        logismos_stream_t stream) {
    if (!src || !dst || bytes == 0 || (bytes & 15u)) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u)
        return hipErrorInvalidValue;
    const int64_t n16 = (int64_t)(bytes >> 4);
    int64_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    lg::probe_copy_kernel<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const lg::uint4_t*>(src), static_cast<lg::uint4_t*>(dst), n16);
    return hipGetLastError();
}

static logismos_status_t probe_read(const void* src, void* sink_u32, size_t bytes, int flags,
                                    logismos_stream_t stream) {
    if (!src || !sink_u32 || bytes == 0 || (bytes & 15u) || (flags & ~3)) return hipErrorInvalidValue;
    if (reinterpret_cast<uintptr_t>(src) & 15u) return hipErrorInvalidValue;
    const int64_t n16 = (int64_t)(bytes >> 4);
    const lg::uint4_t* s = static_cast<const lg::uint4_t*>(src);
    unsigned* sink = static_cast<unsigned*>(sink_u32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (flags & LOGISMOS_PROBE_STRIDED) {
        // one resident workgroup of 512 threads per CU's worth of the chip
        const dim3 grid(256), block(512);
        if (flags & LOGISMOS_PROBE_NON_TEMPORAL)
            lg::probe_read_kernel<true, true><<<grid, block, 0, st>>>(s, sink, n16);
        else
            lg::probe_read_kernel<false, true><<<grid, block, 0, st>>>(s, sink, n16);
    } else {
        int64_t blocks = (n16 + 1023) / 1024;
        if (blocks > 256 * 8) blocks = 256 * 8;
        const dim3 grid((unsigned)blocks), block(256);
        if (flags & LOGISMOS_PROBE_NON_TEMPORAL)
            lg::probe_read_kernel<true, false><<<grid, block, 0, st>>>(s, sink, n16);
        else
            lg::probe_read_kernel<false, false><<<grid, block, 0, st>>>(s, sink, n16);
    }
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_probe_read(const void* src, void* sink_u32,
                                                        size_t bytes, logismos_stream_t stream) {
    return probe_read(src, sink_u32, bytes, 0, stream);
}

extern "C" logismos_status_t logismos_launch_probe_read_ex(const void* src, void* sink_u32,
                                                           size_t bytes, int flags,
                                                           logismos_stream_t stream) {
    return probe_read(src, sink_u32, bytes, flags, stream);
}
