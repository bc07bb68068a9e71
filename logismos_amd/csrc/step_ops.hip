// The small operators of a decode step, gfx950 versions of the contracts the
// reference's CPU op set defines (crates/kernels/src/cpu_f32/mod.rs):
// residual add + RMSNorm, RoPE (halves convention) fused with the KV write,
// SiLU * up, fp16 -> bf16 cast, greedy argmax.  All are tiny at decode batch
// sizes: they exist to keep the step on the GPU between the big kernels.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"
#include "turbo3_device.hpp"

#include <hip/hip_fp16.h>
#include <math.h>

namespace lg {

__device__ __forceinline__ float bf16_to_f32(unsigned short v) {
    return __uint_as_float((unsigned)v << 16);
}
__device__ __forceinline__ unsigned short f32_to_bf16(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}

// h[r][:] += y[r][:] (when y != nullptr); out[r][:] = bf16(h * inv_rms * w).
// One workgroup of 1024 threads per row, four consecutive elements per thread
// per pass kept in registers (a 4096-wide row is a single pass: one read of h,
// one write of h, one write of out).
constexpr int kNormThreads = 1024;
constexpr int kNormMaxPasses = 4;  // rows up to 16384 wide stay in registers

__global__ __launch_bounds__(kNormThreads) void add_rms_norm_kernel(
    float* __restrict__ h, const uint16_t* __restrict__ y, const float* __restrict__ yp,
    int num_parts, int64_t part_stride, const float* __restrict__ w, uint16_t* __restrict__ out,
    int n, float eps) {
    const int64_t row = blockIdx.x;
    float* hr = h + row * n;
    const bool vec = (n & 3) == 0 && n <= 4 * kNormThreads * kNormMaxPasses;
    __shared__ float part[kNormThreads / 64];
    float4_t v[kNormMaxPasses];
    float sum_sq = 0.0f;
    if (vec) {
#pragma unroll
        for (int p = 0; p < kNormMaxPasses; ++p) {
            const int j = (p * kNormThreads + (int)threadIdx.x) * 4;
            if (j < n) {
                v[p] = *reinterpret_cast<const float4_t*>(hr + j);
                if (y) {
                    const uint2_t yy = *reinterpret_cast<const uint2_t*>(y + row * n + j);
                    v[p][0] += __uint_as_float(yy[0] << 16);
                    v[p][1] += __uint_as_float(yy[0] & 0xffff0000u);
                    v[p][2] += __uint_as_float(yy[1] << 16);
                    v[p][3] += __uint_as_float(yy[1] & 0xffff0000u);
                    *reinterpret_cast<float4_t*>(hr + j) = v[p];
                } else if (yp) {
                    // fp32 partial sums of a split-K projection, added in part order
                    for_part_rounds<4>(num_parts, [&](auto nc, int q0) {
                        constexpr int N = decltype(nc)::value;
                        float4_t t4[N];
#pragma unroll
                        for (int u = 0; u < N; ++u)
                            t4[u] = *reinterpret_cast<const float4_t*>(
                                yp + (int64_t)(q0 + u) * part_stride + row * n + j);
#pragma unroll
                        for (int u = 0; u < N; ++u)
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[p][e] += t4[u][e];
                    });
                    *reinterpret_cast<float4_t*>(hr + j) = v[p];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) sum_sq = fmaf(v[p][e], v[p][e], sum_sq);
            }
        }
    } else {
        for (int j = threadIdx.x; j < n; j += kNormThreads) {
            float t = hr[j];
            if (y) {
                t += bf16_to_f32(y[row * n + j]);
                hr[j] = t;
            } else if (yp) {
                for (int q = 0; q < num_parts; ++q) t += yp[(int64_t)q * part_stride + row * n + j];
                hr[j] = t;
            }
            sum_sq = fmaf(t, t, sum_sq);
        }
    }
    sum_sq = wave_sum(sum_sq);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sum_sq;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormThreads / 64; ++i) total += part[i];
    const float inv = 1.0f / sqrtf(total / (float)n + eps);
    if (vec) {
#pragma unroll
        for (int p = 0; p < kNormMaxPasses; ++p) {
            const int j = (p * kNormThreads + (int)threadIdx.x) * 4;
            if (j < n) {
                const float4_t ww = *reinterpret_cast<const float4_t*>(w + j);
                uint2_t o;
                o[0] = (unsigned)f32_to_bf16(v[p][0] * inv * ww[0]) |
                       ((unsigned)f32_to_bf16(v[p][1] * inv * ww[1]) << 16);
                o[1] = (unsigned)f32_to_bf16(v[p][2] * inv * ww[2]) |
                       ((unsigned)f32_to_bf16(v[p][3] * inv * ww[3]) << 16);
                *reinterpret_cast<uint2_t*>(out + row * n + j) = o;
            }
        }
    } else {
        for (int j = threadIdx.x; j < n; j += kNormThreads)
            out[row * n + j] = f32_to_bf16(hr[j] * inv * w[j]);
    }
}

// The step's form of the same operator: y arrives as fp32 split-K parts and the
// normed row leaves in the prepared layout of the next Q4G128 GEMM (pair order
// + per-group sums).  512 threads per row, eight consecutive elements (one
// 16-byte chunk of the output) per thread and pass; n % 128 == 0.
constexpr int kPrepThreads = 512;
constexpr int kPrepMaxPasses = 4;  // rows up to 16384 wide

// TALL: the normed rows leave as the operand of the tiled GEMM for many rows instead
// (q4_common.hpp: row-major in pair order, `pairs` pairs of groups per block of sums; the grid
// covers the rows padded to the GEMM's 128-row tiles, and a padding row is written as zeros).
template <bool TALL>
__global__ __launch_bounds__(kPrepThreads) void add_rms_norm_xprep_kernel(
    float* __restrict__ h, const float* __restrict__ yp, int num_parts, int64_t part_stride,
    const float* __restrict__ w, void* __restrict__ xprep, int rows, int n, float eps,
    int pairs) {
    const int64_t row = blockIdx.x;
    if constexpr (TALL) {
        if (row >= rows) {
            uint4_t* xt = reinterpret_cast<uint4_t*>(xprep) + row * (n >> 3);
            float* xs = reinterpret_cast<float*>(reinterpret_cast<char*>(xprep) +
                                                 tall_sums_offset(rows, n));
            for (int c = threadIdx.x; c < (n >> 3); c += kPrepThreads) {
                xt[c] = uint4_t{0u, 0u, 0u, 0u};
                if ((c & 15) == 0) xs[tall_sum_index(row, c >> 4, n, pairs)] = 0.0f;
            }
            return;
        }
    }
    float* hr = h + row * n;
    float v[kPrepMaxPasses][8];
    float4_t wv[kPrepMaxPasses][2];  // the gains, requested with the first loads, not after the reduction
    float sum_sq = 0.0f;
#pragma unroll
    for (int p = 0; p < kPrepMaxPasses; ++p) {
        const int j = (p * kPrepThreads + (int)threadIdx.x) * 8;
        if (j < n) {
            wv[p][0] = *reinterpret_cast<const float4_t*>(w + j);
            wv[p][1] = *reinterpret_cast<const float4_t*>(w + j + 4);
            const float4_t a = *reinterpret_cast<const float4_t*>(hr + j);
            const float4_t b = *reinterpret_cast<const float4_t*>(hr + j + 4);
            float4_t s0 = a, s1 = b;
            // h + part 0 + part 1 + ... in this order; the loads of up to six parts in flight
            // per round (a round is one trip to memory: 4 parts take one, 12 take two)
            for_part_rounds<6>(num_parts, [&](auto nc, int q0) {
                constexpr int N = decltype(nc)::value;
                float4_t t0[N], t1[N];
#pragma unroll
                for (int u = 0; u < N; ++u) {
                    const float* src = yp + (int64_t)(q0 + u) * part_stride + row * n + j;
                    t0[u] = *reinterpret_cast<const float4_t*>(src);
                    t1[u] = *reinterpret_cast<const float4_t*>(src + 4);
                }
#pragma unroll
                for (int u = 0; u < N; ++u)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s0[e] += t0[u][e];
                        s1[e] += t1[u][e];
                    }
            });
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[p][e] = s0[e];
                v[p][4 + e] = s1[e];
            }
            if (num_parts > 0) {
                *reinterpret_cast<float4_t*>(hr + j) = float4_t{v[p][0], v[p][1], v[p][2], v[p][3]};
                *reinterpret_cast<float4_t*>(hr + j + 4) =
                    float4_t{v[p][4], v[p][5], v[p][6], v[p][7]};
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) sum_sq = fmaf(v[p][e], v[p][e], sum_sq);
        }
    }
    __shared__ float part[kPrepThreads / 64];
    sum_sq = wave_sum(sum_sq);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sum_sq;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < kPrepThreads / 64; ++i) total += part[i];
    const float inv = 1.0f / sqrtf(total / (float)n + eps);
    const int bp = xprep_bp(rows);
    uint4_t* xp = reinterpret_cast<uint4_t*>(xprep);
    float* xg = reinterpret_cast<float*>(reinterpret_cast<char*>(xprep) + xprep_xg_offset(rows, n));
#pragma unroll
    for (int p = 0; p < kPrepMaxPasses; ++p) {
        const int c = p * kPrepThreads + (int)threadIdx.x;  // chunk index
        const int j = c * 8;
        const bool live = j < n;  // uniform over each group of 16 threads (n % 128 == 0)
        uint4_t o = {0u, 0u, 0u, 0u};
        if (live) {
            const float4_t w0 = wv[p][0], w1 = wv[p][1];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = v[p][2 * e] * inv * (2 * e < 4 ? w0[2 * e] : w1[2 * e - 4]);
                const float hi = v[p][2 * e + 1] * inv * (2 * e + 1 < 4 ? w0[2 * e + 1] : w1[2 * e - 3]);
                o[e] = (unsigned)f32_to_bf16(lo) | ((unsigned)f32_to_bf16(hi) << 16);
            }
        }
        const float gs = row16_sum(sum8_bf16(o));
        if (live) {
            if constexpr (TALL) {
                xp[row * (n >> 3) + c] = pair_order(o);
                if ((threadIdx.x & 15) == 0)
                    reinterpret_cast<float*>(reinterpret_cast<char*>(xprep) +
                                             tall_sums_offset(rows, n))
                        [tall_sum_index(row, c >> 4, n, pairs)] = gs;
            } else {
                xp[(int64_t)c * bp + row] = pair_order(o);
                if ((threadIdx.x & 15) == 0) xg[(int64_t)(c >> 4) * bp + row] = gs;
            }
        }
    }
}

// act = silu(gate) * up from the fp32 parts of the gate_up GEMM, written in the
// prepared layout of the down projection.  One thread per 8 outputs.
__global__ __launch_bounds__(256) void silu_mul_xprep_kernel(const float* __restrict__ parts,
                                                             int num_parts, int64_t part_stride,
                                                             void* __restrict__ xprep, int rows,
                                                             int inter) {
    const int chunks = inter >> 3;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int t = idx / chunks, c = idx - t * chunks;
    const bool live = t < rows;  // uniform over groups of 16 threads (inter % 128 == 0)
    uint4_t o = {0u, 0u, 0u, 0u};
    if (live) {
        float g[8], u[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) g[e] = u[e] = 0.0f;
        const int64_t base = (int64_t)t * 2 * inter + (int64_t)c * 8;
        // parts are added in order; the loads of up to four parts are in flight per round
        for_part_rounds<4>(num_parts, [&](auto nc, int q0) {
            constexpr int N = decltype(nc)::value;
            float4_t g0[N], g1[N], u0[N], u1[N];
#pragma unroll
            for (int r = 0; r < N; ++r) {
                const float* src = parts + (int64_t)(q0 + r) * part_stride + base;
                g0[r] = *reinterpret_cast<const float4_t*>(src);
                g1[r] = *reinterpret_cast<const float4_t*>(src + 4);
                u0[r] = *reinterpret_cast<const float4_t*>(src + inter);
                u1[r] = *reinterpret_cast<const float4_t*>(src + inter + 4);
            }
#pragma unroll
            for (int r = 0; r < N; ++r)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    g[e] += g0[r][e];
                    g[4 + e] += g1[r][e];
                    u[e] += u0[r][e];
                    u[4 + e] += u1[r][e];
                }
        });
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = g[2 * e] / (1.0f + expf(-g[2 * e])) * u[2 * e];
            const float b = g[2 * e + 1] / (1.0f + expf(-g[2 * e + 1])) * u[2 * e + 1];
            o[e] = (unsigned)f32_to_bf16(a) | ((unsigned)f32_to_bf16(b) << 16);
        }
    }
    const float gs = row16_sum(sum8_bf16(o));
    if (live) {
        const int bp = xprep_bp(rows);
        reinterpret_cast<uint4_t*>(xprep)[(int64_t)c * bp + t] = pair_order(o);
        if ((threadIdx.x & 15) == 0)
            reinterpret_cast<float*>(reinterpret_cast<char*>(xprep) +
                                     xprep_xg_offset(rows, inter))[(int64_t)(c >> 4) * bp + t] = gs;
    }
}

// grid (hq + 2*hkv, total_tokens), 64 threads: thread i rotates elements i and
// i + d/2 (d = 128).  q heads go to q_out (fp16); k heads, rotated, and v heads,
// as they are, go to the pools at the token's slot: as fp16 rows, or (T3) rounded to fp16
// like those and then encoded as turbo3 head rows -- the lane layout of the rotation is
// the encoder's.
// One rotation pair.  Spelled out with fmaf so that every kernel that rotates rounds alike
// (left to the compiler, `x0 * c - x1 * s` contracts one way in a scalar loop and another in an
// unrolled one).
__device__ __forceinline__ void rope_rotate(float x0, float x1, float c, float s, float& y0,
                                            float& y1) {
    y0 = fmaf(x0, c, -(x1 * s));
    y1 = fmaf(x0, s, x1 * c);
    // (the fp32 values are the results: without this the compiler may fold the conversion to
    // fp16 that follows into the multiply-add, v_fma_mixlo_f16, which rounds once where the
    // reference rounds to fp32 and then to fp16)
    asm volatile("" : "+v"(y0), "+v"(y1));
}

template <bool T3, bool D128>
__global__ __launch_bounds__(64) void rope_kv_write_kernel(
    const uint16_t* __restrict__ qkv, const float* __restrict__ qkv_parts, int num_parts,
    int64_t part_stride, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int64_t* __restrict__ slot_mapping, __half* __restrict__ q_out,
    __half* __restrict__ k_pool, __half* __restrict__ v_pool, int hq, int hkv, int max_pos,
    const float* __restrict__ bias, int head_dim) {
    // 128-wide heads: one pair (i, i + 64) per lane; other widths walk their pairs 64 at a time
    static_assert(D128 || !T3, "turbo3 head rows are 128 wide");
    const int D = D128 ? 128 : head_dim, HALF = D / 2;
    const int head = blockIdx.x;
    const int64_t t = blockIdx.y;
    const int64_t off = (t * (hq + 2 * hkv) + head) * D;
    for (int i = threadIdx.x; i < HALF; i += 64) {
        float x0 = 0.0f, x1 = 0.0f;
        if (qkv) {
            x0 = bf16_to_f32(qkv[off + i]);
            x1 = bf16_to_f32(qkv[off + i + HALF]);
        } else {
            // parts are added in order; the loads of up to four parts are in flight per round
            for_part_rounds<4>(num_parts, [&](auto nc, int q0) {
                constexpr int N = decltype(nc)::value;
                float a[N], b[N];
#pragma unroll
                for (int r = 0; r < N; ++r) {
                    a[r] = qkv_parts[(int64_t)(q0 + r) * part_stride + off + i];
                    b[r] = qkv_parts[(int64_t)(q0 + r) * part_stride + off + i + HALF];
                }
#pragma unroll
                for (int r = 0; r < N; ++r) {
                    x0 += a[r];
                    x1 += b[r];
                }
            });
        }
        if (bias) {
            // the projection's bias (`linear_t`, one fp32 add on the finished sum), column
            // head*D + i
            x0 += bias[head * D + i];
            x1 += bias[head * D + i + HALF];
        }
        if (head < hq + hkv) {
            int pos = positions[t];
            pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
            const float c = cos_t[(int64_t)pos * HALF + i];
            const float s = sin_t[(int64_t)pos * HALF + i];
            float y0, y1;
            rope_rotate(x0, x1, c, s, y0, y1);
            if (head < hq) {
                __half* dst = q_out + (t * hq + head) * D;
                dst[i] = __float2half_rn(y0);
                dst[i + HALF] = __float2half_rn(y1);
            } else {
                const int64_t slot = slot_mapping[t];
                if (slot < 0) return;
                if constexpr (T3) {
                    turbo3_encode_row(__half2float(__float2half_rn(y0)),
                                      __half2float(__float2half_rn(y1)), i,
                                      reinterpret_cast<uint8_t*>(k_pool) +
                                          (slot * hkv + (head - hq)) * kTurbo3HeadBytes);
                } else {
                    __half* dst = k_pool + (slot * hkv + (head - hq)) * D;
                    dst[i] = __float2half_rn(y0);
                    dst[i + HALF] = __float2half_rn(y1);
                }
            }
        } else {
            const int64_t slot = slot_mapping[t];
            if (slot < 0) return;
            if constexpr (T3) {
                turbo3_encode_row(__half2float(__float2half_rn(x0)),
                                  __half2float(__float2half_rn(x1)), i,
                                  reinterpret_cast<uint8_t*>(v_pool) +
                                      (slot * hkv + (head - hq - hkv)) * kTurbo3HeadBytes);
            } else {
                __half* dst = v_pool + (slot * hkv + (head - hq - hkv)) * D;
                dst[i] = __float2half_rn(x0);
                dst[i + HALF] = __float2half_rn(x1);
            }
        }
    }
}

// The same operator for many rows (a prefill chunk's worth and more), 128-wide heads, fp16
// pools, fp32 parts in: one thread per four consecutive rotation pairs (i .. i + 3 with
// i + 64 .. i + 67), 16-byte loads and 8-byte stores, 16 heads of a token per workgroup.  The
// kernel above is one 64-thread workgroup per (token, head) with 4-byte accesses: at 8240
// tokens x 48 heads that is 400 k workgroups for 300 MB.  Same sums in the same order, same
// rotation, same rounding.
constexpr int kRopeRowsKernelFrom = 64;  // tokens from which the many-row kernel is used
__global__ __launch_bounds__(256) void rope_kv_write_rows_kernel(
    const float* __restrict__ qkv_parts, int num_parts, int64_t part_stride,
    const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int64_t* __restrict__ slot_mapping,
    __half* __restrict__ q_out, __half* __restrict__ k_pool, __half* __restrict__ v_pool, int hq,
    int hkv, int max_pos, const float* __restrict__ bias, int64_t total_quads) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= total_quads) return;
    const int heads = hq + 2 * hkv;
    const int i = 4 * (int)(gid & 15);
    const int64_t th = gid >> 4;
    const int64_t t = th / heads;
    const int head = (int)(th - t * heads);
    const int64_t off = th * 128;
    float4_t x0 = {0.0f, 0.0f, 0.0f, 0.0f}, x1 = x0;
    for (int q = 0; q < num_parts; ++q) {
        const float* src = qkv_parts + (int64_t)q * part_stride + off + i;
        const float4_t a = *reinterpret_cast<const float4_t*>(src);
        const float4_t b = *reinterpret_cast<const float4_t*>(src + 64);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x0[e] += a[e];
            x1[e] += b[e];
        }
    }
    if (bias) {
        const float4_t b0 = *reinterpret_cast<const float4_t*>(bias + head * 128 + i);
        const float4_t b1 = *reinterpret_cast<const float4_t*>(bias + head * 128 + i + 64);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x0[e] += b0[e];
            x1[e] += b1[e];
        }
    }
    auto store4 = [](__half* dst, const float4_t& v) {
        uint2_t o;
#pragma unroll
        for (int e = 0; e < 2; ++e)
            o[e] = (unsigned)__half_as_ushort(__float2half_rn(v[2 * e])) |
                   ((unsigned)__half_as_ushort(__float2half_rn(v[2 * e + 1])) << 16);
        *reinterpret_cast<uint2_t*>(dst) = o;
    };
    if (head < hq + hkv) {
        int pos = positions[t];
        pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
        const float4_t c = *reinterpret_cast<const float4_t*>(cos_t + (int64_t)pos * 64 + i);
        const float4_t sn = *reinterpret_cast<const float4_t*>(sin_t + (int64_t)pos * 64 + i);
        float4_t y0, y1;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float a, b;
            rope_rotate(x0[e], x1[e], c[e], sn[e], a, b);
            y0[e] = a;
            y1[e] = b;
        }
        __half* dst;
        if (head < hq) {
            dst = q_out + (t * hq + head) * 128;
        } else {
            const int64_t slot = slot_mapping[t];
            if (slot < 0) return;
            dst = k_pool + (slot * hkv + (head - hq)) * 128;
        }
        store4(dst + i, y0);
        store4(dst + i + 64, y1);
    } else {
        const int64_t slot = slot_mapping[t];
        if (slot < 0) return;
        __half* dst = v_pool + (slot * hkv + (head - hq - hkv)) * 128;
        store4(dst + i, x0);
        store4(dst + i + 64, x1);
    }
}

// out[t][j] = bf16( silu(gate[t][j]) * up[t][j] ), gate_up = [t][gate(0..inter) | up(0..inter)]
// V: elements per thread (8 where inter is a multiple of 8: 32-byte loads of the fp32 parts,
// one 16-byte store; over thousands of rows the operator reads a gigabyte).
template <int V>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ gate_up,
                                                       const float* __restrict__ parts,
                                                       int num_parts, int64_t part_stride,
                                                       uint16_t* __restrict__ out, int inter,
                                                       int64_t total) {
    const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (idx >= total) return;
    const int64_t t = idx / inter;
    const int64_t j = idx - t * inter;
    float g[V], u[V];
#pragma unroll
    for (int e = 0; e < V; ++e) g[e] = u[e] = 0.0f;
    if (gate_up) {
        const uint16_t* gp = gate_up + t * 2 * inter + j;
        if constexpr (V == 8) {
            const uint4_t gv = *reinterpret_cast<const uint4_t*>(gp);
            const uint4_t uv = *reinterpret_cast<const uint4_t*>(gp + inter);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                g[e] = bf16_to_f32((uint16_t)(gv[e >> 1] >> (16 * (e & 1))));
                u[e] = bf16_to_f32((uint16_t)(uv[e >> 1] >> (16 * (e & 1))));
            }
        } else {
            g[0] = bf16_to_f32(gp[0]);
            u[0] = bf16_to_f32(gp[inter]);
        }
    } else {
        for (int q = 0; q < num_parts; ++q) {
            const float* gp = parts + (int64_t)q * part_stride + t * 2 * inter + j;
            if constexpr (V == 8) {
#pragma unroll
                for (int v4 = 0; v4 < 2; ++v4) {
                    const float4_t gv = *reinterpret_cast<const float4_t*>(gp + 4 * v4);
                    const float4_t uv = *reinterpret_cast<const float4_t*>(gp + inter + 4 * v4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        g[4 * v4 + e] += gv[e];
                        u[4 * v4 + e] += uv[e];
                    }
                }
            } else {
                g[0] += gp[0];
                u[0] += gp[inter];
            }
        }
    }
    uint16_t o[V];
#pragma unroll
    for (int e = 0; e < V; ++e) {
        const float sg = g[e] / (1.0f + expf(-g[e]));
        o[e] = f32_to_bf16(sg * u[e]);
    }
    if constexpr (V == 8) {
        uint4_t ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (unsigned)o[2 * e] | ((unsigned)o[2 * e + 1] << 16);
        *reinterpret_cast<uint4_t*>(out + idx) = ov;
    } else {
        out[idx] = o[0];
    }
}

// The same operator writing the down projection's operand where the tiled GEMM for many rows
// wants it (q4_common.hpp: x in pair order, rows padded with zeros to the 128-row tiles, the
// group sums in the layout of the GEMM's loads) instead of plain bf16 rows: the GEMM's first
// pass over x (a read and a write of the whole operand) is not needed then.  One thread per
// 16-byte chunk of the padded operand; the 16 lanes of a row of lanes hold one group.
__global__ __launch_bounds__(256) void silu_mul_tall_kernel(const float* __restrict__ parts,
                                                            int num_parts, int64_t part_stride,
                                                            uint16_t* __restrict__ xp,
                                                            float* __restrict__ xs, int rows,
                                                            int rows_pad, int inter, int w) {
    const int64_t chunks_per_row = inter >> 3;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)rows_pad * chunks_per_row) return;  // (whole rows of 16 lanes: inter % 128 == 0)
    const int64_t t = id / chunks_per_row;
    const int64_t c = id - t * chunks_per_row;
    uint4_t o = {0u, 0u, 0u, 0u};
    if (t < rows) {
        float g[8], u[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) g[e] = u[e] = 0.0f;
        for (int q = 0; q < num_parts; ++q) {
            const float* gp = parts + (int64_t)q * part_stride + t * 2 * inter + c * 8;
#pragma unroll
            for (int v4 = 0; v4 < 2; ++v4) {
                const float4_t gv = *reinterpret_cast<const float4_t*>(gp + 4 * v4);
                const float4_t uv = *reinterpret_cast<const float4_t*>(gp + inter + 4 * v4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    g[4 * v4 + e] += gv[e];
                    u[4 * v4 + e] += uv[e];
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float s0 = g[2 * e] / (1.0f + expf(-g[2 * e]));
            const float s1 = g[2 * e + 1] / (1.0f + expf(-g[2 * e + 1]));
            o[e] = (unsigned)f32_to_bf16(s0 * u[2 * e]) | ((unsigned)f32_to_bf16(s1 * u[2 * e + 1]) << 16);
        }
    }
    const float gs = row16_sum(sum8_bf16(o));
    *reinterpret_cast<uint4_t*>(xp + t * inter + c * 8) = pair_order(o);
    if ((threadIdx.x & 15) == 0) xs[tall_sum_index(t, (int)(c >> 4), inter, w)] = gs;
}

// (one launcher for both element widths: 8 per thread where rows of `inter` elements and the
// buffers allow 16- and 32-byte accesses)
static hipError_t silu_mul_launch(const uint16_t* gate_up, const float* parts, int num_parts,
                                  int64_t part_stride, uint16_t* out, int inter, int64_t total,
                                  hipStream_t st) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(parts) |
                        reinterpret_cast<uintptr_t>(out) | (uintptr_t)(part_stride * 4);
    if (inter % 8 == 0 && (a & 15u) == 0) {
        const int64_t threads = total / 8;
        silu_mul_kernel<8><<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st>>>(
            gate_up, parts, num_parts, part_stride, out, inter, total);
    } else {
        silu_mul_kernel<1><<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st>>>(
            gate_up, parts, num_parts, part_stride, out, inter, total);
    }
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void cast_f16_bf16_kernel(const __half* __restrict__ in,
                                                            uint16_t* __restrict__ out,
                                                            int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx < total) out[idx] = f32_to_bf16(__half2float(in[idx]));
}

// dst[s][:] = src[cu_seqlens[s + 1] - 1][:]: the last packed row of every sequence (bf16 rows
// of `hidden` elements, hidden % 8 == 0).  One workgroup per sequence.  A sequence without new
// tokens takes the row before its position (row 0 for the first): what it gets is not used.
__global__ __launch_bounds__(256) void gather_last_rows_bf16_kernel(
    const uint4_t* __restrict__ src, const int32_t* __restrict__ cu_seqlens,
    uint4_t* __restrict__ dst, int chunks) {
    const int s = blockIdx.x;
    const int last = cu_seqlens[s + 1] - 1;
    const int64_t row = last > 0 ? last : 0;
    for (int i = threadIdx.x; i < chunks; i += 256)
        dst[(int64_t)s * chunks + i] = src[row * chunks + i];
}

// One workgroup per row: first index of the maximum (strict >, ties keep the lower index).
__global__ __launch_bounds__(256) void greedy_kernel(const float* __restrict__ logits,
                                                     uint32_t* __restrict__ out, int n) {
    const int64_t row = blockIdx.x;
    const float* lr = logits + row * n;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int j = threadIdx.x; j < n; j += 256) {
        const float v = lr[j];
        if (v > best) {
            best = v;
            best_i = j;
        }
    }
    __shared__ float sb[256];
    __shared__ int si[256];
    sb[threadIdx.x] = best;
    si[threadIdx.x] = best_i;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) {
            const float ov = sb[threadIdx.x + off];
            const int oi = si[threadIdx.x + off];
            if (ov > sb[threadIdx.x] || (ov == sb[threadIdx.x] && oi < si[threadIdx.x])) {
                sb[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    // all -inf (or NaN-only) rows: index 0, like the CPU loop that never updates
    if (threadIdx.x == 0) out[row] = si[0] == 0x7fffffff ? 0u : (uint32_t)si[0];
}

// out[r][:] = table[ids[r]][:] widened to fp32; an id outside the vocabulary gives a zero row
// (`embed_lookup`, crates/kernels/src/cpu_f32/mod.rs:106-127).
template <bool BF16>
__global__ __launch_bounds__(256) void embed_lookup_kernel(const void* __restrict__ table,
                                                           const uint32_t* __restrict__ ids,
                                                           float* __restrict__ out, int hidden,
                                                           int64_t vocab) {
    const int64_t row = blockIdx.x;
    const uint32_t id = ids[row];
    const bool valid = (int64_t)id < vocab;
    float* o = out + row * hidden;
    for (int j = threadIdx.x; j < hidden; j += 256) {
        float v = 0.0f;
        if (valid) {
            if constexpr (BF16)
                v = bf16_to_f32(static_cast<const uint16_t*>(table)[(int64_t)id * hidden + j]);
            else
                v = static_cast<const float*>(table)[(int64_t)id * hidden + j];
        }
        o[j] = v;
    }
}

}  // namespace lg

extern "C" logismos_status_t logismos_launch_add_rms_norm_bf16(void* h_f32, const void* y_bf16,
                                                               const void* w_f32, void* out_bf16,
                                                               int rows, int n, float eps,
                                                               logismos_stream_t stream) {
    if (rows <= 0 || n <= 0 || (int64_t)rows * n > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!h_f32 || !w_f32 || !out_bf16) return hipErrorInvalidValue;
    lg::add_rms_norm_kernel<<<dim3(rows), dim3(lg::kNormThreads), 0,
                              static_cast<hipStream_t>(stream)>>>(
        static_cast<float*>(h_f32), static_cast<const uint16_t*>(y_bf16), nullptr, 0, 0,
        static_cast<const float*>(w_f32), static_cast<uint16_t*>(out_bf16), n, eps);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_add_rms_norm_f32p(void* h_f32, const void* parts_f32,
                                                               int num_parts, const void* w_f32,
                                                               void* out_bf16, int rows, int n,
                                                               float eps,
                                                               logismos_stream_t stream) {
    if (rows <= 0 || n <= 0 || (int64_t)rows * n > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!h_f32 || !w_f32 || !out_bf16 || num_parts < 0 || (num_parts > 0 && !parts_f32))
        return hipErrorInvalidValue;
    lg::add_rms_norm_kernel<<<dim3(rows), dim3(lg::kNormThreads), 0,
                              static_cast<hipStream_t>(stream)>>>(
        static_cast<float*>(h_f32), nullptr,
        num_parts > 0 ? static_cast<const float*>(parts_f32) : nullptr, num_parts,
        (int64_t)rows * n, static_cast<const float*>(w_f32), static_cast<uint16_t*>(out_bf16), n,
        eps);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_rope_kv_write_fp16(
    const void* qkv_bf16, const int32_t* positions, const void* cos_f32, const void* sin_f32,
    const int64_t* slot_mapping, void* q_out_f16, void* k_pool_f16, void* v_pool_f16,
    int total_tokens, int num_q_heads, int num_kv_heads, int head_dim, int max_pos,
    logismos_stream_t stream) {
    if (total_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_pos <= 0)
        return hipErrorInvalidValue;
    // an even number of elements per head (a rotation pair is (i, i + head_dim / 2))
    if (head_dim <= 0 || head_dim % 2 != 0 || head_dim > 1024 || total_tokens > 65535)
        return hipErrorInvalidValue;
    if ((int64_t)total_tokens * (num_q_heads + 2 * num_kv_heads) * head_dim > (int64_t)INT32_MAX)
        return hipErrorInvalidValue;
    if (total_tokens == 0) return hipSuccess;
    if (!qkv_bf16 || !positions || !cos_f32 || !sin_f32 || !slot_mapping || !q_out_f16 ||
        !k_pool_f16 || !v_pool_f16)
        return hipErrorInvalidValue;
    dim3 grid(num_q_heads + 2 * num_kv_heads, total_tokens);
    const auto kernel = head_dim == 128 ? lg::rope_kv_write_kernel<false, true>
                                        : lg::rope_kv_write_kernel<false, false>;
    kernel<<<grid, dim3(64), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint16_t*>(qkv_bf16), nullptr, 0, 0, positions,
        static_cast<const float*>(cos_f32),
        static_cast<const float*>(sin_f32), slot_mapping, static_cast<__half*>(q_out_f16),
        static_cast<__half*>(k_pool_f16), static_cast<__half*>(v_pool_f16), num_q_heads,
        num_kv_heads, max_pos, nullptr, head_dim);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_rope_kv_write_f32p_bias(
    const void* qkv_parts_f32, int num_parts, const void* bias_f32, const int32_t* positions,
    const void* cos_f32, const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16,
    void* k_pool_f16, void* v_pool_f16, int total_tokens, int num_q_heads, int num_kv_heads,
    int head_dim, int max_pos, logismos_stream_t stream) {
    if (total_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_pos <= 0 || num_parts <= 0)
        return hipErrorInvalidValue;
    // an even number of elements per head (a rotation pair is (i, i + head_dim / 2))
    if (head_dim <= 0 || head_dim % 2 != 0 || head_dim > 1024 || total_tokens > 65535)
        return hipErrorInvalidValue;
    const int64_t width = (int64_t)(num_q_heads + 2 * num_kv_heads) * head_dim;
    if ((int64_t)total_tokens * width > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (total_tokens == 0) return hipSuccess;
    if (!qkv_parts_f32 || !positions || !cos_f32 || !sin_f32 || !slot_mapping || !q_out_f16 ||
        !k_pool_f16 || !v_pool_f16)
        return hipErrorInvalidValue;
    // many rows of 128-wide heads: the kernel with 16-byte accesses (everything it reads and
    // writes 16-byte aligned)
    const uintptr_t align = reinterpret_cast<uintptr_t>(qkv_parts_f32) |
                            reinterpret_cast<uintptr_t>(bias_f32) |
                            reinterpret_cast<uintptr_t>(cos_f32) |
                            reinterpret_cast<uintptr_t>(sin_f32) |
                            reinterpret_cast<uintptr_t>(q_out_f16) |
                            reinterpret_cast<uintptr_t>(k_pool_f16) |
                            reinterpret_cast<uintptr_t>(v_pool_f16);
    if (head_dim == 128 && total_tokens >= lg::kRopeRowsKernelFrom && (align & 15u) == 0 &&
        ((int64_t)total_tokens * width) % 4 == 0) {
        const int64_t quads = (int64_t)total_tokens * (num_q_heads + 2 * num_kv_heads) * 16;
        lg::rope_kv_write_rows_kernel<<<dim3((unsigned)((quads + 255) / 256)), dim3(256), 0,
                                        static_cast<hipStream_t>(stream)>>>(
            static_cast<const float*>(qkv_parts_f32), num_parts, (int64_t)total_tokens * width,
            positions, static_cast<const float*>(cos_f32), static_cast<const float*>(sin_f32),
            slot_mapping, static_cast<__half*>(q_out_f16), static_cast<__half*>(k_pool_f16),
            static_cast<__half*>(v_pool_f16), num_q_heads, num_kv_heads, max_pos,
            static_cast<const float*>(bias_f32), quads);
        return hipGetLastError();
    }
    dim3 grid(num_q_heads + 2 * num_kv_heads, total_tokens);
    const auto kernel = head_dim == 128 ? lg::rope_kv_write_kernel<false, true>
                                        : lg::rope_kv_write_kernel<false, false>;
    kernel<<<grid, dim3(64), 0, static_cast<hipStream_t>(stream)>>>(
        nullptr, static_cast<const float*>(qkv_parts_f32), num_parts, (int64_t)total_tokens * width,
        positions, static_cast<const float*>(cos_f32), static_cast<const float*>(sin_f32),
        slot_mapping, static_cast<__half*>(q_out_f16), static_cast<__half*>(k_pool_f16),
        static_cast<__half*>(v_pool_f16), num_q_heads, num_kv_heads, max_pos,
        static_cast<const float*>(bias_f32), head_dim);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_rope_kv_write_f32p(
    const void* qkv_parts_f32, int num_parts, const int32_t* positions, const void* cos_f32,
    const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16, void* k_pool_f16,
    void* v_pool_f16, int total_tokens, int num_q_heads, int num_kv_heads, int head_dim,
    int max_pos, logismos_stream_t stream) {
    return logismos_launch_rope_kv_write_f32p_bias(qkv_parts_f32, num_parts, nullptr, positions,
                                                   cos_f32, sin_f32, slot_mapping, q_out_f16,
                                                   k_pool_f16, v_pool_f16, total_tokens,
                                                   num_q_heads, num_kv_heads, head_dim, max_pos,
                                                   stream);
}

extern "C" logismos_status_t logismos_launch_rope_kv_write_f32p_turbo3_bias(
    const void* qkv_parts_f32, int num_parts, const void* bias_f32, const int32_t* positions,
    const void* cos_f32, const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16,
    void* k_pool_t3, void* v_pool_t3, int total_tokens, int num_q_heads, int num_kv_heads,
    int head_dim, int max_pos, logismos_stream_t stream) {
    if (total_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_pos <= 0 || num_parts <= 0)
        return hipErrorInvalidValue;
    if (head_dim != 128 || total_tokens > 65535) return hipErrorInvalidValue;
    const int64_t width = (int64_t)(num_q_heads + 2 * num_kv_heads) * head_dim;
    if ((int64_t)total_tokens * width > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (total_tokens == 0) return hipSuccess;
    if (!qkv_parts_f32 || !positions || !cos_f32 || !sin_f32 || !slot_mapping || !q_out_f16 ||
        !k_pool_t3 || !v_pool_t3)
        return hipErrorInvalidValue;
    dim3 grid(num_q_heads + 2 * num_kv_heads, total_tokens);
    lg::rope_kv_write_kernel<true, true><<<grid, dim3(64), 0, static_cast<hipStream_t>(stream)>>>(
        nullptr, static_cast<const float*>(qkv_parts_f32), num_parts, (int64_t)total_tokens * width,
        positions, static_cast<const float*>(cos_f32), static_cast<const float*>(sin_f32),
        slot_mapping, static_cast<__half*>(q_out_f16), static_cast<__half*>(k_pool_t3),
        static_cast<__half*>(v_pool_t3), num_q_heads, num_kv_heads, max_pos,
        static_cast<const float*>(bias_f32), 128);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_rope_kv_write_f32p_turbo3(
    const void* qkv_parts_f32, int num_parts, const int32_t* positions, const void* cos_f32,
    const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16, void* k_pool_t3,
    void* v_pool_t3, int total_tokens, int num_q_heads, int num_kv_heads, int head_dim,
    int max_pos, logismos_stream_t stream) {
    return logismos_launch_rope_kv_write_f32p_turbo3_bias(
        qkv_parts_f32, num_parts, nullptr, positions, cos_f32, sin_f32, slot_mapping, q_out_f16,
        k_pool_t3, v_pool_t3, total_tokens, num_q_heads, num_kv_heads, head_dim, max_pos, stream);
}

extern "C" logismos_status_t logismos_launch_silu_mul_f32p(const void* parts_f32, int num_parts,
                                                           void* out_bf16, int rows, int inter,
                                                           logismos_stream_t stream) {
    if (rows <= 0 || inter <= 0 || num_parts <= 0 ||
        (int64_t)rows * inter * 2 > (int64_t)INT32_MAX)
        return hipErrorInvalidValue;
    if (!parts_f32 || !out_bf16) return hipErrorInvalidValue;
    const int64_t total = (int64_t)rows * inter;
    return lg::silu_mul_launch(nullptr, static_cast<const float*>(parts_f32), num_parts,
                               (int64_t)rows * 2 * inter, static_cast<uint16_t*>(out_bf16), inter,
                               total, static_cast<hipStream_t>(stream));
}

extern "C" logismos_status_t logismos_launch_silu_mul_f32p_tall(const void* parts_f32,
                                                                int num_parts, void* workspace,
                                                                int rows, int inter,
                                                                int pairs_per_load,
                                                                logismos_stream_t stream) {
    if (rows <= 0 || inter <= 0 || inter % 256 != 0 || num_parts <= 0 ||
        (pairs_per_load != 1 && pairs_per_load != 2 && pairs_per_load != 4) ||
        inter % (256 * pairs_per_load) != 0)
        return hipErrorInvalidValue;
    const int rows_pad = lg::tall_padded_rows(rows);
    if ((int64_t)rows_pad * inter * 2 > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!parts_f32 || !workspace) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(parts_f32) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
        return hipErrorInvalidValue;
    const int64_t chunks = (int64_t)rows_pad * (inter / 8);
    lg::silu_mul_tall_kernel<<<dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                               static_cast<hipStream_t>(stream)>>>(
        static_cast<const float*>(parts_f32), num_parts, (int64_t)rows * 2 * inter,
        static_cast<uint16_t*>(workspace),
        reinterpret_cast<float*>(static_cast<char*>(workspace) + lg::tall_sums_offset(rows, inter)),
        rows, rows_pad, inter, pairs_per_load);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_silu_mul_bf16(const void* gate_up_bf16,
                                                           void* out_bf16, int rows, int inter,
                                                           logismos_stream_t stream) {
    if (rows <= 0 || inter <= 0 || (int64_t)rows * inter * 2 > (int64_t)INT32_MAX)
        return hipErrorInvalidValue;
    if (!gate_up_bf16 || !out_bf16) return hipErrorInvalidValue;
    const int64_t total = (int64_t)rows * inter;
    return lg::silu_mul_launch(static_cast<const uint16_t*>(gate_up_bf16), nullptr, 0, 0,
                               static_cast<uint16_t*>(out_bf16), inter, total,
                               static_cast<hipStream_t>(stream));
}

extern "C" logismos_status_t logismos_launch_cast_f16_bf16(const void* in_f16, void* out_bf16,
                                                           size_t count,
                                                           logismos_stream_t stream) {
    if (count == 0) return hipSuccess;
    if (!in_f16 || !out_bf16 || count > (size_t)INT32_MAX) return hipErrorInvalidValue;
    lg::cast_f16_bf16_kernel<<<dim3((unsigned)((count + 255) / 256)), dim3(256), 0,
                               static_cast<hipStream_t>(stream)>>>(
        static_cast<const __half*>(in_f16), static_cast<uint16_t*>(out_bf16), (int64_t)count);
    return hipGetLastError();
}

namespace lg {
hipError_t gather_last_rows_bf16_launch(const void* src_bf16, const int32_t* cu_seqlens,
                                        void* dst_bf16, int num_seqs, int hidden,
                                        hipStream_t stream) {
    if (num_seqs <= 0 || hidden <= 0 || (hidden & 7) || !src_bf16 || !cu_seqlens || !dst_bf16)
        return hipErrorInvalidValue;
    gather_last_rows_bf16_kernel<<<dim3(num_seqs), dim3(256), 0, stream>>>(
        static_cast<const uint4_t*>(src_bf16), cu_seqlens, static_cast<uint4_t*>(dst_bf16),
        hidden / 8);
    return hipGetLastError();
}
}  // namespace lg

extern "C" logismos_status_t logismos_launch_greedy_f32(const void* logits_f32, void* out_u32,
                                                        int rows, int n,
                                                        logismos_stream_t stream) {
    if (rows <= 0 || n <= 0 || (int64_t)rows * n > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!logits_f32 || !out_u32) return hipErrorInvalidValue;
    lg::greedy_kernel<<<dim3(rows), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const float*>(logits_f32), static_cast<uint32_t*>(out_u32), n);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_add_rms_norm_f32p_xprep(
    void* h_f32, const void* parts_f32, int num_parts, const void* w_f32, void* x_prepared, int rows,
    int n, float eps, logismos_stream_t stream) {
    if (rows <= 0 || rows > 32 || n <= 0 || n % 128 != 0 ||
        n > 8 * lg::kPrepThreads * lg::kPrepMaxPasses)
        return hipErrorInvalidValue;
    if (!h_f32 || !w_f32 || !x_prepared || num_parts < 0 || (num_parts > 0 && !parts_f32))
        return hipErrorInvalidValue;
    lg::add_rms_norm_xprep_kernel<false><<<dim3(rows), dim3(lg::kPrepThreads), 0,
                                           static_cast<hipStream_t>(stream)>>>(
        static_cast<float*>(h_f32), static_cast<const float*>(parts_f32), num_parts,
        (int64_t)rows * n, static_cast<const float*>(w_f32), x_prepared, rows, n, eps, 0);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_add_rms_norm_f32p_tall(
    void* h_f32, const void* parts_f32, int num_parts, const void* w_f32, void* workspace,
    int rows, int n, float eps, int pairs_per_load, logismos_stream_t stream) {
    if (rows <= 0 || n <= 0 || num_parts < 0 ||
        (pairs_per_load != 1 && pairs_per_load != 2 && pairs_per_load != 4) ||
        n % (256 * pairs_per_load) != 0 || n > 8 * lg::kPrepThreads * lg::kPrepMaxPasses)
        return hipErrorInvalidValue;
    const int rows_pad = lg::tall_padded_rows(rows);
    if ((int64_t)rows_pad * n * 2 > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!h_f32 || !w_f32 || !workspace || (num_parts > 0 && !parts_f32))
        return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(h_f32) | reinterpret_cast<uintptr_t>(parts_f32) |
         reinterpret_cast<uintptr_t>(w_f32) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
        return hipErrorInvalidValue;
    lg::add_rms_norm_xprep_kernel<true><<<dim3(rows_pad), dim3(lg::kPrepThreads), 0,
                                          static_cast<hipStream_t>(stream)>>>(
        static_cast<float*>(h_f32), static_cast<const float*>(parts_f32), num_parts,
        (int64_t)rows * n, static_cast<const float*>(w_f32), workspace, rows, n, eps,
        pairs_per_load);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_silu_mul_f32p_xprep(const void* parts_f32,
                                                                 int num_parts, void* x_prepared,
                                                                 int rows, int inter,
                                                                 logismos_stream_t stream) {
    if (rows <= 0 || rows > 32 || inter <= 0 || inter % 128 != 0 || num_parts <= 0 ||
        (int64_t)rows * inter * 2 > (int64_t)INT32_MAX)
        return hipErrorInvalidValue;
    if (!parts_f32 || !x_prepared) return hipErrorInvalidValue;
    const int items = rows * (inter / 8);
    lg::silu_mul_xprep_kernel<<<dim3((items + 255) / 256), dim3(256), 0,
                                static_cast<hipStream_t>(stream)>>>(
        static_cast<const float*>(parts_f32), num_parts, (int64_t)rows * 2 * inter, x_prepared, rows,
        inter);
    return hipGetLastError();
}

static logismos_status_t embed_lookup_launch(const void* table, const void* ids_u32, void* out_f32,
                                             int rows, int hidden, int64_t vocab, bool bf16,
                                             logismos_stream_t stream) {
    if (rows <= 0 || hidden <= 0 || vocab <= 0 || (int64_t)rows * hidden > (int64_t)INT32_MAX)
        return hipErrorInvalidValue;
    if (!table || !ids_u32 || !out_f32) return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (bf16)
        lg::embed_lookup_kernel<true><<<dim3(rows), dim3(256), 0, st>>>(
            table, static_cast<const uint32_t*>(ids_u32), static_cast<float*>(out_f32), hidden,
            vocab);
    else
        lg::embed_lookup_kernel<false><<<dim3(rows), dim3(256), 0, st>>>(
            table, static_cast<const uint32_t*>(ids_u32), static_cast<float*>(out_f32), hidden,
            vocab);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_embed_lookup_f32(const void* table_f32,
                                                              const void* ids_u32, void* out_f32,
                                                              int rows, int hidden,
                                                              long long vocab,
                                                              logismos_stream_t stream) {
    return embed_lookup_launch(table_f32, ids_u32, out_f32, rows, hidden, vocab, false, stream);
}

extern "C" logismos_status_t logismos_launch_embed_lookup_bf16(const void* table_bf16,
                                                               const void* ids_u32, void* out_f32,
                                                               int rows, int hidden,
                                                               long long vocab,
                                                               logismos_stream_t stream) {
    return embed_lookup_launch(table_bf16, ids_u32, out_f32, rows, hidden, vocab, true, stream);
}
