// The five launchers the reference's kernels crate already declares and its `praxis` layer
// already calls, for gfx950 (the reference builds them for gfx1100, wave32):
//
//   logismos_launch_rms_norm_fp16       crates/kernels/src/rms_norm/hip/rms_norm.hip:58-84
//   logismos_launch_softmax_fp16        crates/kernels/src/softmax/hip/softmax.hip:66-87
//   logismos_launch_rope_fp16           crates/kernels/src/rope/hip/rope.hip:45-68
//   logismos_launch_matmul_naive_fp16   crates/kernels/src/matmul/hip/matmul_launchers.cpp:14-32
//   logismos_launch_matmul_wmma_fp16    crates/kernels/src/matmul/hip/matmul_launchers.cpp:34-52
//
// Same symbols, argument lists and meaning (fp16 in and out, fp32 arithmetic inside, one
// rounding at the output; the CPU references crates/kernels/src/{rms_norm,softmax,rope,
// matmul}/cpu.rs define the results), so the crate's `extern "C"` blocks link against this
// archive unchanged.  "wmma" names the reference's RDNA3 instruction; here that entry point
// runs on the CDNA4 matrix cores (v_mfma_f32_32x32x16_f16) and, unlike the reference's,
// takes any M, N, K.
#include "device_utils.hpp"
#include "launch_common.hpp"

#include <hip/hip_fp16.h>
#include <math.h>

namespace lg {

constexpr int kRowThreads = 256;

// sum / max over the 256 threads of a workgroup; every thread gets the result
__device__ __forceinline__ float block_sum_256(float v, float* red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const float r = red[0] + red[1] + red[2] + red[3];
    __syncthreads();
    return r;
}
__device__ __forceinline__ float block_max_256(float v, float* red) {
    v = row16_max(v);
    v = fmaxf(fmaxf(__shfl(v, 0, kWave), __shfl(v, 16, kWave)),
              fmaxf(__shfl(v, 32, kWave), __shfl(v, 48, kWave)));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const float r = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return r;
}

// y[r][j] = fp16( x[r][j] * (1 / sqrt(mean_j x[r][j]^2 + eps)) * w[j] ), one workgroup per row
// (`rms_norm_fp16_ref`, crates/kernels/src/rms_norm/cpu.rs:13-45)
__global__ __launch_bounds__(kRowThreads) void rms_norm_fp16_kernel(
    const __half* __restrict__ x, const __half* __restrict__ w, __half* __restrict__ y, int n,
    float eps) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const __half* xr = x + row * n;
    __half* yr = y + row * n;
    float part = 0.0f;
    for (int j = threadIdx.x; j < n; j += kRowThreads) {
        const float v = __half2float(xr[j]);
        part = fmaf(v, v, part);
    }
    const float sum_sq = block_sum_256(part, red);
    const float inv_rms = 1.0f / sqrtf(sum_sq / (float)n + eps);
    for (int j = threadIdx.x; j < n; j += kRowThreads)
        yr[j] = __float2half_rn(__half2float(xr[j]) * inv_rms * __half2float(w[j]));
}

// Row softmax, fp32 inside: max-subtracted exponentials times the reciprocal of their sum; a
// row whose maximum is -inf (every entry -inf) becomes uniform 1/n
// (`softmax_fp16_ref`, crates/kernels/src/softmax/cpu.rs:14-74)
__global__ __launch_bounds__(kRowThreads) void softmax_fp16_kernel(const __half* __restrict__ x,
                                                                   __half* __restrict__ y, int n) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const __half* xr = x + row * n;
    __half* yr = y + row * n;
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < n; j += kRowThreads) mx = fmaxf(mx, __half2float(xr[j]));
    mx = block_max_256(mx, red);
    if (mx == -INFINITY) {
        const __half u = __float2half_rn(1.0f / (float)n);
        for (int j = threadIdx.x; j < n; j += kRowThreads) yr[j] = u;
        return;
    }
    float part = 0.0f;
    for (int j = threadIdx.x; j < n; j += kRowThreads) part += expf(__half2float(xr[j]) - mx);
    const float inv = 1.0f / block_sum_256(part, red);
    for (int j = threadIdx.x; j < n; j += kRowThreads)
        yr[j] = __float2half_rn(expf(__half2float(xr[j]) - mx) * inv);
}

// In place on fp16 (batch, seq, heads, head_dim): pair (2i, 2i+1) of every head row at
// position s is rotated by (cos, sin) = table[s][2i], table[s][2i+1]
// (`rope_apply_fp16_ref`, crates/kernels/src/rope/cpu.rs:56-127).  One thread per pair: a
// pair is one aligned 32-bit word of the tensor and one 64-bit entry of the table.
__global__ __launch_bounds__(256) void rope_fp16_kernel(unsigned* __restrict__ qk_pairs,
                                                        const float2* __restrict__ cos_sin,
                                                        int64_t total_pairs, int seq, int heads,
                                                        int pairs) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total_pairs) return;
    const int i = (int)(idx % pairs);
    const int64_t row = idx / pairs;           // (b * seq + s) * heads + h
    const int s = (int)((row / heads) % seq);
    const float2 cs = cos_sin[(int64_t)s * pairs + i];
    const unsigned word = qk_pairs[idx];
    const float x0 = __half2float(__ushort_as_half((unsigned short)(word & 0xffffu)));
    const float x1 = __half2float(__ushort_as_half((unsigned short)(word >> 16)));
    const float y0 = x0 * cs.x - x1 * cs.y;
    const float y1 = x0 * cs.y + x1 * cs.x;
    qk_pairs[idx] = (unsigned)__half_as_ushort(__float2half_rn(y0)) |
                    ((unsigned)__half_as_ushort(__float2half_rn(y1)) << 16);
}

// D = A[M,K] . B[K,N], one thread per output element, fp32 accumulation in ascending k with
// separate multiply and add -- the order and the roundings of `matmul_fp16_ref`
// (crates/kernels/src/matmul/cpu.rs:12-30), so the result is bit-identical to it.
__global__ __launch_bounds__(256) void matmul_naive_fp16_kernel(const __half* __restrict__ a,
                                                                const __half* __restrict__ b,
                                                                __half* __restrict__ d, int m,
                                                                int n, int k) {
    const int col = blockIdx.x * 64 + (threadIdx.x & 63);
    const int row = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (row >= m || col >= n) return;
    const __half* ar = a + (int64_t)row * k;
    float acc = 0.0f;
    for (int p = 0; p < k; ++p)
        acc = __fadd_rn(acc, __fmul_rn(__half2float(ar[p]), __half2float(b[(int64_t)p * n + col])));
    d[(int64_t)row * n + col] = __float2half_rn(acc);
}

// The matrix-core version: a workgroup of four waves owns a 128 x 128 tile of D, each wave a
// 64 x 64 quarter (2 x 2 accumulators of v_mfma_f32_32x32x16_f16).  Per 32-wide slab of K the
// workgroup stages A[128 x 32] and B[32 x 128] in LDS -- B transposed to [n][k] on the way,
// because the MFMA B operand wants eight consecutive k of one column and B is row-major: two
// k rows per thread, merged into (k, k+1) words, with the four 16-byte chunks of an LDS row
// XOR-swizzled by (row / 16) % 4 so that these transposed 4-byte stores are two-way instead
// of eight-way bank conflicts.  The LDS tiles are double buffered: slab s + 1 is fetched
// from memory while slab s is multiplied, one barrier per slab.  Rows, columns and k beyond
// the matrix are zero-filled.
constexpr int kMmTile = 128, kMmK = 32;
constexpr int kMmStride = kMmK + 8;  // halfs per LDS row: 80 bytes, 16-byte reads stay aligned
constexpr int kMmBuf = kMmTile * kMmStride;

__global__ __launch_bounds__(256) void matmul_mfma_fp16_kernel(const _Float16* __restrict__ a,
                                                               const _Float16* __restrict__ b,
                                                               _Float16* __restrict__ d, int m,
                                                               int n, int k) {
    __shared__ __attribute__((aligned(16))) _Float16 as[2 * kMmBuf];
    __shared__ __attribute__((aligned(16))) _Float16 bs[2 * kMmBuf];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int row0 = blockIdx.y * kMmTile;
    const int col0 = blockIdx.x * kMmTile;
    const int wr = (wave >> 1) * 64;  // this wave's quarter
    const int wc = (wave & 1) * 64;
    const int r = lane & 31;
    const int h = lane >> 5;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // staging roles.  A: thread -> rows tid / 4 and tid / 4 + 64, eight consecutive k at
    // 8 * (tid % 4).  B: thread -> k rows 2 * (tid / 16) and + 1, eight consecutive columns at
    // 8 * (tid % 16).
    const int a_row = tid >> 2, a_k = (tid & 3) * 8;
    const int b_kp = tid >> 4, b_col = (tid & 15) * 8;
    const bool a_vec = (k & 7) == 0, b_vec = (n & 7) == 0;
    half8_t ra[2], rb[2];
    auto gload = [&](int k0) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            const int gr = row0 + a_row + 64 * u, gk = k0 + a_k;
            if (gr < m && gk < k) {
                const _Float16* src = a + (int64_t)gr * k + gk;
                if (a_vec && gk + 8 <= k) {
                    v = *reinterpret_cast<const half8_t*>(src);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        if (gk + i < k) v[i] = src[i];
                }
            }
            ra[u] = v;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            const int gk = k0 + 2 * b_kp + u, gc = col0 + b_col;
            if (gk < k && gc < n) {
                const _Float16* src = b + (int64_t)gk * n + gc;
                if (b_vec && gc + 8 <= n) {
                    v = *reinterpret_cast<const half8_t*>(src);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        if (gc + i < n) v[i] = src[i];
                }
            }
            rb[u] = v;
        }
    };
    // LDS column (halfs) of k pair b_kp in a B row whose swizzle key is `key`
    auto lstore = [&](int buf) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
            *reinterpret_cast<half8_t*>(as + buf * kMmBuf + (a_row + 64 * u) * kMmStride + a_k) =
                ra[u];
        const uint4_t lo = __builtin_bit_cast(uint4_t, rb[0]);
        const uint4_t hi = __builtin_bit_cast(uint4_t, rb[1]);
        const int key = (b_col >> 4) & 3;  // (row / 16) % 4 of rows b_col .. b_col + 7
        _Float16* dst =
            bs + buf * kMmBuf + 8 * ((b_kp >> 2) ^ key) + 2 * (b_kp & 3);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const unsigned sel = (e & 1) ? 0x07060302u : 0x05040100u;
            const unsigned pr = __builtin_amdgcn_perm(hi[e >> 1], lo[e >> 1], sel);
            *reinterpret_cast<unsigned*>(dst + (b_col + e) * kMmStride) = pr;
        }
    };

    const int slabs = (k + kMmK - 1) / kMmK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int sl = 0; sl < slabs; ++sl) {
        const int buf = sl & 1;
        if (sl + 1 < slabs) gload((sl + 1) * kMmK);
        const _Float16* at = as + buf * kMmBuf;
        const _Float16* bt = bs + buf * kMmBuf;
#pragma unroll
        for (int kk = 0; kk < kMmK; kk += 16) {
            half8_t av[2], bv[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                av[i] = *reinterpret_cast<const half8_t*>(at + (wr + 32 * i + r) * kMmStride + kk +
                                                          8 * h);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int row = wc + 32 * j + r;
                bv[j] = *reinterpret_cast<const half8_t*>(
                    bt + row * kMmStride + 8 * (((kk >> 3) + h) ^ ((row >> 4) & 3)));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[j], acc[i][j], 0,
                                                                       0, 0);
        }
        if (sl + 1 < slabs) lstore(buf ^ 1);  // last read of that buffer: before the last barrier
        __syncthreads();
    }
    // lane (h, r) holds column r, rows 8 * (e / 4) + 4h + e % 4 of each 32 x 32 block
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int gc = col0 + wc + 32 * j + r;
            if (gc >= n) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int gr = row0 + wr + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
                if (gr < m) d[(int64_t)gr * n + gc] = (_Float16)acc[i][j][e];
            }
        }
}

// `check_matmul_shape` (crates/kernels/src/matmul/mod.rs:89-117)
static bool matmul_shape_ok(int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0) return false;
    const int64_t lim = INT32_MAX;
    return (int64_t)m * k <= lim && (int64_t)k * n <= lim && (int64_t)m * n <= lim;
}

}  // namespace lg

namespace lg {

// scores[r][c] = -inf where mask[r / repeat][c] == 0 (one mask row serves `repeat` consecutive
// score rows: the heads of one batch row), 16 bytes of mask per thread where n allows
template <typename T>
__global__ __launch_bounds__(256) void mask_additive_kernel(T* __restrict__ scores,
                                                            const uint8_t* __restrict__ mask,
                                                            int64_t rows, int64_t n,
                                                            int64_t repeat, T neg_inf) {
    const int64_t total = rows * n;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / n;
        const int64_t c = i - r * n;
        if (mask[(r / repeat) * n + c] == 0) scores[i] = neg_inf;
    }
}

static logismos_status_t mask_additive_check(const void* scores, const void* mask,
                                             size_t mask_len, size_t rows, size_t n,
                                             int64_t* repeat) {
    *repeat = 0;
    // `mask_additive_in_place` (crates/kernels/src/cpu_f32/mod.rs:451-486): nothing to do
    // without columns, rows or a mask, or with a mask shorter than one row
    if (n == 0 || rows == 0 || mask_len == 0 || mask_len / n == 0) return hipSuccess;
    if (!scores || !mask) return hipErrorInvalidValue;
    const size_t mask_rows = mask_len / n;
    // (the reference's debug assertion: the mask is whole rows)
    if (mask_rows * n != mask_len) return hipErrorInvalidValue;
    // the reference panics here: a row count that the mask rows do not divide would leave
    // the trailing rows unmasked
    if (rows % mask_rows != 0) return hipErrorInvalidValue;
    if (rows > (size_t)INT32_MAX || n > (size_t)INT32_MAX ||
        (uint64_t)rows * (uint64_t)n > ((uint64_t)1 << 40))
        return hipErrorInvalidValue;
    *repeat = (int64_t)(rows / mask_rows);
    return hipSuccess;
}

template <typename T>
static logismos_status_t mask_additive_launch(void* scores, const void* mask, size_t mask_len,
                                              size_t rows, size_t n, T neg_inf,
                                              logismos_stream_t stream) {
    int64_t repeat;
    const logismos_status_t st = mask_additive_check(scores, mask, mask_len, rows, n, &repeat);
    if (st != hipSuccess || repeat == 0) return st;
    const int64_t total = (int64_t)rows * (int64_t)n;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    mask_additive_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0,
                              static_cast<hipStream_t>(stream)>>>(
        static_cast<T*>(scores), static_cast<const uint8_t*>(mask), (int64_t)rows, (int64_t)n,
        repeat, neg_inf);
    return hipGetLastError();
}

}  // namespace lg

extern "C" logismos_status_t logismos_launch_mask_additive_f32(void* scores_f32,
                                                               const void* mask_u8,
                                                               size_t mask_len, size_t rows,
                                                               size_t n,
                                                               logismos_stream_t stream) {
    return lg::mask_additive_launch<float>(scores_f32, mask_u8, mask_len, rows, n, -INFINITY,
                                           stream);
}

extern "C" logismos_status_t logismos_launch_mask_additive_fp16(void* scores_fp16,
                                                                const void* mask_u8,
                                                                size_t mask_len, size_t rows,
                                                                size_t n,
                                                                logismos_stream_t stream) {
    return lg::mask_additive_launch<unsigned short>(scores_fp16, mask_u8, mask_len, rows, n,
                                                    (unsigned short)0xFC00u, stream);
}

extern "C" logismos_status_t logismos_launch_rms_norm_fp16(const void* x_fp16, const void* w_fp16,
                                                           void* y_fp16, int m, int n, float eps,
                                                           logismos_stream_t stream) {
    if (m <= 0 || n <= 0 || (int64_t)m * n > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!x_fp16 || !w_fp16 || !y_fp16) return hipErrorInvalidValue;
    lg::rms_norm_fp16_kernel<<<dim3(m), dim3(lg::kRowThreads), 0,
                               static_cast<hipStream_t>(stream)>>>(
        static_cast<const __half*>(x_fp16), static_cast<const __half*>(w_fp16),
        static_cast<__half*>(y_fp16), n, eps);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_softmax_fp16(const void* x_fp16, void* y_fp16, int m,
                                                          int n, logismos_stream_t stream) {
    if (m <= 0 || n <= 0 || (int64_t)m * n > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (!x_fp16 || !y_fp16) return hipErrorInvalidValue;
    lg::softmax_fp16_kernel<<<dim3(m), dim3(lg::kRowThreads), 0,
                              static_cast<hipStream_t>(stream)>>>(
        static_cast<const __half*>(x_fp16), static_cast<__half*>(y_fp16), n);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_rope_fp16(void* qk_fp16, const void* cos_sin_f32,
                                                       int batch, int seq, int heads, int head_dim,
                                                       logismos_stream_t stream) {
    // `check_rope_shape` (crates/kernels/src/rope/mod.rs:79-130): positive dimensions, an even
    // head_dim, element counts within i32
    if (batch <= 0 || seq <= 0 || heads <= 0 || head_dim <= 0 || (head_dim & 1))
        return hipErrorInvalidValue;
    // the product is bounded factor by factor: four i32 factors can overflow i64 as well
    int64_t total = 1;
    for (int f : {batch, seq, heads, head_dim}) {
        if (total > (int64_t)INT32_MAX / f) return hipErrorInvalidValue;
        total *= f;
    }
    if (!qk_fp16 || !cos_sin_f32) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qk_fp16) & 3u) || (reinterpret_cast<uintptr_t>(cos_sin_f32) & 7u))
        return hipErrorInvalidValue;
    const int64_t total_pairs = total / 2;
    lg::rope_fp16_kernel<<<dim3((unsigned)((total_pairs + 255) / 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream)>>>(
        static_cast<unsigned*>(qk_fp16), static_cast<const float2*>(cos_sin_f32), total_pairs, seq,
        heads, head_dim / 2);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_matmul_naive_fp16(const void* a_fp16,
                                                               const void* b_fp16, void* d_fp16,
                                                               int m, int n, int k,
                                                               logismos_stream_t stream) {
    if (!lg::matmul_shape_ok(m, n, k) || !a_fp16 || !b_fp16 || !d_fp16) return hipErrorInvalidValue;
    lg::matmul_naive_fp16_kernel<<<dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0,
                                   static_cast<hipStream_t>(stream)>>>(
        static_cast<const __half*>(a_fp16), static_cast<const __half*>(b_fp16),
        static_cast<__half*>(d_fp16), m, n, k);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_matmul_wmma_fp16(const void* a_fp16,
                                                              const void* b_fp16, void* d_fp16,
                                                              int m, int n, int k,
                                                              logismos_stream_t stream) {
    if (!lg::matmul_shape_ok(m, n, k) || !a_fp16 || !b_fp16 || !d_fp16) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(a_fp16) | reinterpret_cast<uintptr_t>(b_fp16)) & 15u)
        return hipErrorInvalidValue;
    lg::matmul_mfma_fp16_kernel<<<dim3((n + lg::kMmTile - 1) / lg::kMmTile,
                                       (m + lg::kMmTile - 1) / lg::kMmTile),
                                  dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const _Float16*>(a_fp16), static_cast<const _Float16*>(b_fp16),
        static_cast<_Float16*>(d_fp16), m, n, k);
    return hipGetLastError();
}
