/*
 * logismos_oracle.c -- CPU oracle (test infrastructure, never shipped).
 * See logismos_oracle.h for the role of this file.  Paths in comments are
 * relative to the reference tree.
 */
#include "logismos_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ conversions */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* IEEE binary32 -> binary16, round to nearest even (what `half::f16::from_f32`
 * and `__float2half_rn` do). */
uint16_t oracle_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs = x & 0x7fffffffu;
    uint32_t exp = abs >> 23;
    uint32_t man = abs & 0x7fffffu;
    if (exp == 0xff) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x0200u | (man >> 13));
    }
    if (exp > 142) return (uint16_t)(sign | 0x7c00u); /* >= 2^16 */
    if (exp >= 113) {                                 /* normal half */
        uint32_t r = ((exp - 112) << 10) | (man >> 13);
        uint32_t rem = man & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
        return (uint16_t)(sign | r); /* a carry into the exponent is the right answer */
    }
    if (exp >= 102) { /* subnormal half: unit 2^-24 */
        uint32_t full = man | 0x800000u;
        uint32_t shift = 126 - exp; /* 14..24 */
        uint32_t r = full >> shift;
        uint32_t rem = full & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return (uint16_t)(sign | r);
    }
    return (uint16_t)sign;
}

float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: man * 2^-24, exact in f32 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112) << 23) | (man << 13));
}

uint16_t oracle_f32_to_bf16(float f) {
    uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

void oracle_f32_to_f16_n(const float* x, uint16_t* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = oracle_f32_to_f16(x[i]);
}
void oracle_f16_to_f32_n(const uint16_t* x, float* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = oracle_f16_to_f32(x[i]);
}
void oracle_f32_to_bf16_n(const float* x, uint16_t* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = oracle_f32_to_bf16(x[i]);
}
void oracle_bf16_to_f32_n(const uint16_t* x, float* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = oracle_bf16_to_f32(x[i]);
}

/* ------------------------------------------------------------------ cpu_f32 */

/* crates/kernels/src/cpu_f32/mod.rs:106-127 -- out-of-range id leaves a zero row. */
void oracle_embed_lookup(const float* weight, size_t hidden, size_t vocab, const uint32_t* ids,
                         size_t n_ids, float* out) {
    memset(out, 0, n_ids * hidden * sizeof(float));
    for (size_t i = 0; i < n_ids; ++i) {
        size_t id = ids[i];
        if (id >= vocab) continue;
        memcpy(out + i * hidden, weight + id * hidden, hidden * sizeof(float));
    }
}

/* crates/kernels/src/cpu_f32/mod.rs:137-159 -- y = x * (1/sqrt(mean(x^2)+eps)) * w,
 * sequential fp32 sum of squares, product evaluated left to right. */
void oracle_rms_norm(const float* x, const float* weight, float* y, size_t rows, size_t n,
                     float eps) {
    for (size_t r = 0; r < rows; ++r) {
        const float* row = x + r * n;
        float sum_sq = 0.0f;
        for (size_t j = 0; j < n; ++j) sum_sq += row[j] * row[j];
        float inv = 1.0f / sqrtf((sum_sq / (float)n) + eps);
        for (size_t j = 0; j < n; ++j) y[r * n + j] = row[j] * inv * weight[j];
    }
}

/* crates/kernels/src/cpu_f32/mod.rs:183-249 -- C[m,n] = A[m,k] . B[k,n] (+bias).
 * The reference hands the contraction to matrixmultiply::sgemm; ascending-k
 * fp32 accumulation is used here (see header note). */
void oracle_linear(const float* a, const float* b, const float* bias, float* c, size_t m, size_t n,
                   size_t k) {
    for (size_t i = 0; i < m; ++i) {
        for (size_t j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (size_t p = 0; p < k; ++p) acc += a[i * k + p] * b[p * n + j];
            c[i * n + j] = acc;
        }
    }
    if (bias) {
        for (size_t i = 0; i < m; ++i)
            for (size_t j = 0; j < n; ++j) c[i * n + j] += bias[j];
    }
}

/* crates/kernels/src/cpu_f32/mod.rs:271-345 -- C[m,n] = A[m,k] . B[n,k]^T (+bias);
 * the weight is `[out,in]` row-major.  Bias is added after the product. */
void oracle_linear_t(const float* a, const float* b, const float* bias, float* c, size_t m,
                     size_t n, size_t k) {
    long total = (long)(m * n);
#pragma omp parallel for schedule(static) if (total * (long)k > (1L << 18))
    for (long ij = 0; ij < total; ++ij) {
        size_t i = (size_t)ij / n, j = (size_t)ij % n;
        const float* ar = a + i * k;
        const float* br = b + j * k;
        float acc = 0.0f;
        for (size_t p = 0; p < k; ++p) acc += ar[p] * br[p];
        c[ij] = acc;
    }
    if (bias) {
        for (size_t i = 0; i < m; ++i)
            for (size_t j = 0; j < n; ++j) c[i * n + j] += bias[j];
    }
}

/* crates/kernels/src/cpu_f32/mod.rs:349-351 -- v / (1 + exp(-v)). */
void oracle_silu(const float* x, float* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = x[i] / (1.0f + expf(-x[i]));
}

/* crates/kernels/src/cpu_f32/mod.rs:365-374 */
void oracle_hadamard(const float* a, const float* b, float* c, size_t n) {
    for (size_t i = 0; i < n; ++i) c[i] = a[i] * b[i];
}

/* crates/kernels/src/cpu_f32/mod.rs:380-433 -- max-subtracted exp, multiply by
 * the reciprocal of the sum; a row that is all -inf becomes uniform 1/n. */
void oracle_softmax_last_dim(const float* x, float* y, size_t rows, size_t n) {
    for (size_t r = 0; r < rows; ++r) {
        const float* row = x + r * n;
        float* out = y + r * n;
        float m = -INFINITY;
        for (size_t j = 0; j < n; ++j)
            if (row[j] > m) m = row[j];
        if (isinf(m) && m < 0) {
            float uniform = n == 0 ? 0.0f : 1.0f / (float)n;
            for (size_t j = 0; j < n; ++j) out[j] = uniform;
            continue;
        }
        float denom = 0.0f;
        for (size_t j = 0; j < n; ++j) {
            float e = expf(row[j] - m);
            out[j] = e;
            denom += e;
        }
        float inv = 1.0f / denom;
        for (size_t j = 0; j < n; ++j) out[j] *= inv;
    }
}

/* crates/kernels/src/cpu_f32/mod.rs:451-486 -- mask rows broadcast over
 * `rows / mask_rows` consecutive score rows; mask byte 0 => -inf.  Returns 0,
 * or -1 where the reference panics (rows not a multiple of mask_rows). */
int oracle_mask_additive_in_place(float* scores, const uint8_t* mask, size_t mask_len, size_t rows,
                                  size_t n) {
    if (n == 0 || rows == 0 || mask_len == 0) return 0;
    size_t mask_rows = mask_len / n;
    if (mask_rows == 0) return 0;
    if (rows % mask_rows != 0) return -1;
    size_t repeat = rows / mask_rows;
    for (size_t mr = 0; mr < mask_rows; ++mr)
        for (size_t rep = 0; rep < repeat; ++rep) {
            size_t r = mr * repeat + rep;
            for (size_t j = 0; j < n; ++j)
                if (mask[mr * n + j] == 0) scores[r * n + j] = -INFINITY;
        }
    return 0;
}

/* crates/kernels/src/cpu_f32/mod.rs:502-547 -- halves convention, per-row cos/sin
 * of length head_dim/2 (the caller gathers them by position). */
void oracle_rope_halves_in_place(float* x, const float* cos, const float* sin, size_t rows,
                                 size_t head_dim) {
    size_t half = head_dim / 2;
    for (size_t r = 0; r < rows; ++r) {
        float* row = x + r * head_dim;
        const float* cr = cos + r * half;
        const float* sr = sin + r * half;
        for (size_t i = 0; i < half; ++i) {
            float x0 = row[i], x1 = row[i + half];
            row[i] = x0 * cr[i] - x1 * sr[i];
            row[i + half] = x0 * sr[i] + x1 * cr[i];
        }
    }
}

/* crates/kernels/src/cpu_f32/mod.rs:599-619 -- angles in f64, then cast. */
void oracle_build_rope_table_f32(size_t seq, size_t head_dim, double theta, float* cos_out,
                                 float* sin_out) {
    size_t half = head_dim / 2;
    for (size_t pos = 0; pos < seq; ++pos)
        for (size_t i = 0; i < half; ++i) {
            double e = (2.0 * (double)i) / (double)head_dim;
            double inv_freq = pow(theta, -e);
            double angle = (double)pos * inv_freq;
            cos_out[pos * half + i] = (float)cos(angle);
            sin_out[pos * half + i] = (float)sin(angle);
        }
}

/* ------------------------------------------------------------------ fp16-I/O refs */

/* crates/kernels/src/matmul/cpu.rs:12-30 -- fp16 in, fp32 accumulate in
 * ascending k, one rounding to fp16; B is `[K,N]`. */
void oracle_matmul_fp16_ref(const uint16_t* a, const uint16_t* b, uint16_t* d, size_t m, size_t n,
                            size_t k) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (size_t p = 0; p < k; ++p)
                acc += oracle_f16_to_f32(a[i * k + p]) * oracle_f16_to_f32(b[p * n + j]);
            d[i * n + j] = oracle_f32_to_f16(acc);
        }
}

/* crates/kernels/src/softmax/cpu.rs:14-74 -- fp32 inside, rounded at the output only. */
void oracle_softmax_fp16_ref(const uint16_t* x, uint16_t* y, size_t m, size_t n) {
    float* xf = (float*)malloc((n ? n : 1) * sizeof(float));
    float* yf = (float*)malloc((n ? n : 1) * sizeof(float));
    for (size_t r = 0; r < m; ++r) {
        oracle_f16_to_f32_n(x + r * n, xf, n);
        oracle_softmax_last_dim(xf, yf, 1, n);
        oracle_f32_to_f16_n(yf, y + r * n, n);
    }
    free(xf);
    free(yf);
}

/* crates/kernels/src/rms_norm/cpu.rs:13-45 */
void oracle_rms_norm_fp16_ref(const uint16_t* x, const uint16_t* w, uint16_t* y, size_t m, size_t n,
                              float eps) {
    for (size_t r = 0; r < m; ++r) {
        float sum_sq = 0.0f;
        for (size_t j = 0; j < n; ++j) {
            float f = oracle_f16_to_f32(x[r * n + j]);
            sum_sq += f * f;
        }
        float inv_rms = 1.0f / sqrtf(sum_sq / (float)n + eps);
        for (size_t j = 0; j < n; ++j)
            y[r * n + j] = oracle_f32_to_f16(oracle_f16_to_f32(x[r * n + j]) * inv_rms *
                                             oracle_f16_to_f32(w[j]));
    }
}

/* crates/kernels/src/rope/cpu.rs:19-40 -- `[seq][head_dim]` f32, cos at 2i and sin at 2i+1
 * of row pos; frequency, angle, cos and sin all in f32 as there. */
void oracle_build_cos_sin_table(size_t seq, size_t head_dim, float theta_base, float* table) {
    size_t pairs = head_dim / 2;
    for (size_t pos = 0; pos < seq; ++pos)
        for (size_t i = 0; i < pairs; ++i) {
            float e = -(2.0f * (float)i) / (float)head_dim;
            float freq = powf(theta_base, e);
            float angle = (float)pos * freq;
            table[pos * head_dim + 2 * i] = cosf(angle);
            table[pos * head_dim + 2 * i + 1] = sinf(angle);
        }
}

/* crates/kernels/src/rope/cpu.rs:56-127 -- in place on fp16 (B, S, H, D), interleaved pairs. */
void oracle_rope_apply_fp16_ref(uint16_t* qk, const float* cos_sin, size_t batch, size_t seq,
                                size_t heads, size_t head_dim) {
    size_t pairs = head_dim / 2;
    for (size_t b = 0; b < batch; ++b)
        for (size_t s = 0; s < seq; ++s) {
            const float* row = cos_sin + s * head_dim;
            for (size_t h = 0; h < heads; ++h) {
                size_t base = ((b * seq + s) * heads + h) * head_dim;
                for (size_t i = 0; i < pairs; ++i) {
                    float c = row[2 * i], sn = row[2 * i + 1];
                    float x0 = oracle_f16_to_f32(qk[base + 2 * i]);
                    float x1 = oracle_f16_to_f32(qk[base + 2 * i + 1]);
                    float y0 = x0 * c - x1 * sn;
                    float y1 = x0 * sn + x1 * c;
                    qk[base + 2 * i] = oracle_f32_to_f16(y0);
                    qk[base + 2 * i + 1] = oracle_f32_to_f16(y1);
                }
            }
        }
}

/* ------------------------------------------------------------------ attention pieces */

/* crates/transformers/src/attention.rs:318-337 -- [seq,heads,d] -> [heads,seq,d] */
void oracle_transpose_seq_heads(const float* x, float* out, size_t seq, size_t heads, size_t d) {
    for (size_t s = 0; s < seq; ++s)
        for (size_t h = 0; h < heads; ++h)
            memcpy(out + (h * seq + s) * d, x + (s * heads + h) * d, d * sizeof(float));
}

/* crates/transformers/src/attention.rs:339-358 -- [heads,seq,d] -> [seq,heads,d] */
void oracle_merge_heads(const float* attn, float* out, size_t heads, size_t seq, size_t d) {
    for (size_t h = 0; h < heads; ++h)
        for (size_t s = 0; s < seq; ++s)
            memcpy(out + (s * heads + h) * d, attn + (h * seq + s) * d, d * sizeof(float));
}

/* crates/transformers/src/attention.rs:366-382 -- kv head h feeds q heads h*groups+g. */
void oracle_repeat_kv(const float* kv, float* out, size_t n_kv, size_t groups, size_t seq,
                      size_t d) {
    for (size_t h = 0; h < n_kv; ++h)
        for (size_t g = 0; g < groups; ++g)
            memcpy(out + (h * groups + g) * seq * d, kv + h * seq * d, seq * d * sizeof(float));
}

/* crates/transformers/src/attention.rs:225-296 -- scores = (q.k^T) * (1/sqrt(d)),
 * scale applied after the dot; key-column mask; fp32 softmax; out = P.V. */
void oracle_sdpa_f32(const float* q_hsd, const float* k_hsd, const float* v_hsd,
                     const uint8_t* mask, float* out_hsd, size_t n_h, size_t n_kv, size_t seq,
                     size_t d) {
    size_t groups = n_h / n_kv;
    float* k_exp = (float*)malloc(n_h * seq * d * sizeof(float));
    float* v_exp = (float*)malloc(n_h * seq * d * sizeof(float));
    oracle_repeat_kv(k_hsd, k_exp, n_kv, groups, seq, d);
    oracle_repeat_kv(v_hsd, v_exp, n_kv, groups, seq, d);
    float scale = 1.0f / sqrtf((float)d);
    float* scores = (float*)malloc(seq * seq * sizeof(float));
    float* probs = (float*)malloc(seq * seq * sizeof(float));
    uint8_t* col_mask = (uint8_t*)malloc(seq * seq);
    for (size_t i = 0; i < seq; ++i)
        for (size_t j = 0; j < seq; ++j) col_mask[i * seq + j] = mask[j];
    for (size_t h = 0; h < n_h; ++h) {
        oracle_linear_t(q_hsd + h * seq * d, k_exp + h * seq * d, NULL, scores, seq, seq, d);
        for (size_t i = 0; i < seq * seq; ++i) scores[i] = scores[i] * scale;
        oracle_mask_additive_in_place(scores, col_mask, seq * seq, seq, seq);
        oracle_softmax_last_dim(scores, probs, seq, seq);
        oracle_linear(probs, v_exp + h * seq * d, NULL, out_hsd + h * seq * d, seq, d, seq);
    }
    free(k_exp);
    free(v_exp);
    free(scores);
    free(probs);
    free(col_mask);
}

/* crates/decode/src/lib.rs:73-83 -- strict `>`: the first maximum wins. */
uint32_t oracle_greedy(const float* logits, size_t n) {
    size_t best_i = 0;
    float best = -INFINITY;
    for (size_t i = 0; i < n; ++i)
        if (logits[i] > best) {
            best = logits[i];
            best_i = i;
        }
    return best_i > 0xffffffffu ? 0xffffffffu : (uint32_t)best_i;
}

/* ------------------------------------------------------------------ nibble order */

/* crates/quant/src/lib.rs:272-285 -- index i sits at bit 4*i of a little-endian
 * integer: byte j = idx[2j] | idx[2j+1] << 4.  Returns -1 for an index > 15
 * (the reference returns Error::IndexOutOfRange). n must be even. */
int oracle_pack_nibbles(const uint8_t* idx, size_t n, uint8_t* packed) {
    for (size_t i = 0; i < n; ++i)
        if (idx[i] > 15) return -1;
    for (size_t j = 0; j < n / 2; ++j) packed[j] = (uint8_t)(idx[2 * j] | (idx[2 * j + 1] << 4));
    return 0;
}

/* crates/quant/src/lib.rs:287-301 */
void oracle_unpack_nibbles(const uint8_t* packed, size_t n, uint8_t* idx) {
    for (size_t i = 0; i < n; ++i) idx[i] = (packed[i / 2] >> (4 * (i & 1))) & 0xf;
}

/* ------------------------------------------------------------------ Q8G32 */

/* ggml Q8_0 reference quantizer (the format crates/loader/src/gguf.rs:57-78
 * tags as id 8; the struct and quantizer are ggml's published ones, not in the
 * reference): per 32 values, d = amax/127, q = roundf(w * (1/d)) with the
 * UNROUNDED d, d then stored as fp16.  roundf = half away from zero. */
void oracle_quantize_q8g32(const float* w, int8_t* qs, uint16_t* d, size_t n, size_t k) {
    size_t groups = k / 32;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const float* src = w + (size_t)r * k + g * 32;
            float amax = 0.0f;
            for (int i = 0; i < 32; ++i) {
                float a = fabsf(src[i]);
                if (a > amax) amax = a;
            }
            float dd = amax / 127.0f;
            float id = dd != 0.0f ? 1.0f / dd : 0.0f;
            d[(size_t)r * groups + g] = oracle_f32_to_f16(dd);
            for (int i = 0; i < 32; ++i) {
                float q = roundf(src[i] * id);
                if (q > 127.0f) q = 127.0f;
                if (q < -127.0f) q = -127.0f;
                qs[(size_t)r * k + g * 32 + i] = (int8_t)q;
            }
        }
}

void oracle_dequantize_q8g32(const int8_t* qs, const uint16_t* d, float* w, size_t n, size_t k) {
    size_t groups = k / 32;
    for (size_t r = 0; r < n; ++r)
        for (size_t c = 0; c < k; ++c)
            w[r * k + c] = oracle_f16_to_f32(d[r * groups + c / 32]) * (float)qs[r * k + c];
}

/* planar <-> ggml block stream `{f16 d (LE); int8 qs[32]}`, 34 bytes, align 1. */
void oracle_q8g32_to_q8_0_blocks(const int8_t* qs, const uint16_t* d, uint8_t* blocks, size_t n,
                                 size_t k) {
    size_t groups = k / 32;
    for (size_t r = 0; r < n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            uint8_t* blk = blocks + (r * groups + g) * 34;
            uint16_t dv = d[r * groups + g];
            blk[0] = (uint8_t)(dv & 0xff);
            blk[1] = (uint8_t)(dv >> 8);
            memcpy(blk + 2, qs + r * k + g * 32, 32);
        }
}

void oracle_q8_0_blocks_to_q8g32(const uint8_t* blocks, int8_t* qs, uint16_t* d, size_t n,
                                 size_t k) {
    size_t groups = k / 32;
    for (size_t r = 0; r < n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t* blk = blocks + (r * groups + g) * 34;
            d[r * groups + g] = (uint16_t)(blk[0] | (blk[1] << 8));
            memcpy(qs + r * k + g * 32, blk + 2, 32);
        }
}

/* linear_t at m = 1 (crates/kernels/src/cpu_f32/mod.rs:271-345) over the
 * dequantised matrix: y[n] = sum_k x[k] * (d * q), ascending k, fp32. */
void oracle_qgemv_q8g32_f32(const float* x, const int8_t* qs, const uint16_t* d, float* y,
                            size_t n, size_t k) {
    size_t groups = k / 32;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n; ++r) {
        const int8_t* q = qs + (size_t)r * k;
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            float dd = oracle_f16_to_f32(d[(size_t)r * groups + g]);
            for (int i = 0; i < 32; ++i) acc += x[g * 32 + i] * (dd * (float)q[g * 32 + i]);
        }
        y[r] = acc;
    }
}

/* ------------------------------------------------- ggml Q4_0 / Q4_1 and Q4G32 */

/* ggml's 4-bit block formats, the ids the reference parses and rejects (`GgmlType::Q4_0 = 2`,
 * `Q4_1 = 3`, crates/loader/src/gguf.rs:57-78,127-145).  The reference holds neither the
 * structs nor arithmetic for them and names no ggml version; what follows restates ggml's
 * published definitions (ggml-common.h `block_q4_0` = {f16 d; u8 qs[16]}, 18 bytes, and
 * `block_q4_1` = {f16 d; f16 m; u8 qs[16]}, 20 bytes, for 32 values; ggml-quants.c
 * `quantize_row_q4_0_ref`, `quantize_row_q4_1_ref`, `dequantize_row_q4_0`,
 * `dequantize_row_q4_1`): byte j of qs holds value j in its low nibble and value j + 16 in its
 * high nibble; Q4_0: w = (q - 8) * d; Q4_1: w = q * d + m. */
void oracle_quantize_q4_0_blocks(const float* w, uint8_t* blocks, size_t n, size_t k) {
    size_t groups = k / 32;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const float* src = w + (size_t)r * k + g * 32;
            float amax = 0.0f, max = 0.0f; /* the value of largest magnitude, with its sign */
            for (int i = 0; i < 32; ++i)
                if (amax < fabsf(src[i])) {
                    amax = fabsf(src[i]);
                    max = src[i];
                }
            const float d = max / -8.0f;
            const float id = d != 0.0f ? 1.0f / d : 0.0f;
            uint8_t* blk = blocks + ((size_t)r * groups + g) * 18;
            uint16_t dh = oracle_f32_to_f16(d);
            blk[0] = (uint8_t)(dh & 0xff);
            blk[1] = (uint8_t)(dh >> 8);
            for (int j = 0; j < 16; ++j) {
                const float x0 = src[j] * id, x1 = src[16 + j] * id;
                int q0 = (int)(int8_t)(x0 + 8.5f), q1 = (int)(int8_t)(x1 + 8.5f);
                if (q0 > 15) q0 = 15;
                if (q1 > 15) q1 = 15;
                blk[2 + j] = (uint8_t)(q0 | (q1 << 4));
            }
        }
}

void oracle_quantize_q4_1_blocks(const float* w, uint8_t* blocks, size_t n, size_t k) {
    size_t groups = k / 32;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const float* src = w + (size_t)r * k + g * 32;
            float mn = src[0], mx = src[0];
            for (int i = 1; i < 32; ++i) {
                if (src[i] < mn) mn = src[i];
                if (src[i] > mx) mx = src[i];
            }
            const float d = (mx - mn) / 15.0f;
            const float id = d != 0.0f ? 1.0f / d : 0.0f;
            uint8_t* blk = blocks + ((size_t)r * groups + g) * 20;
            uint16_t dh = oracle_f32_to_f16(d), mh = oracle_f32_to_f16(mn);
            blk[0] = (uint8_t)(dh & 0xff);
            blk[1] = (uint8_t)(dh >> 8);
            blk[2] = (uint8_t)(mh & 0xff);
            blk[3] = (uint8_t)(mh >> 8);
            for (int j = 0; j < 16; ++j) {
                const float x0 = (src[j] - mn) * id, x1 = (src[16 + j] - mn) * id;
                int q0 = (int)(int8_t)(x0 + 0.5f), q1 = (int)(int8_t)(x1 + 0.5f);
                if (q0 > 15) q0 = 15;
                if (q1 > 15) q1 = 15;
                blk[4 + j] = (uint8_t)(q0 | (q1 << 4));
            }
        }
}

void oracle_dequantize_q4_0_blocks(const uint8_t* blocks, float* w, size_t n, size_t k) {
    size_t groups = k / 32;
    for (size_t r = 0; r < n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t* blk = blocks + (r * groups + g) * 18;
            const float d = oracle_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            float* dst = w + r * k + g * 32;
            for (int j = 0; j < 16; ++j) {
                dst[j] = (float)((int)(blk[2 + j] & 0x0F) - 8) * d;
                dst[j + 16] = (float)((int)(blk[2 + j] >> 4) - 8) * d;
            }
        }
}

void oracle_dequantize_q4_1_blocks(const uint8_t* blocks, float* w, size_t n, size_t k) {
    size_t groups = k / 32;
    for (size_t r = 0; r < n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t* blk = blocks + (r * groups + g) * 20;
            const float d = oracle_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            const float m = oracle_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
            float* dst = w + r * k + g * 32;
            for (int j = 0; j < 16; ++j) {
                dst[j] = (float)(blk[4 + j] & 0x0F) * d + m;
                dst[j + 16] = (float)(blk[4 + j] >> 4) * d + m;
            }
        }
}

/* Planar Q4G32 [DEFINED BY BUILD], what the GPU GEMV reads: nibbles uint8 [N][K/2] in k
 * order, low nibble first (the reference's only nibble order, `pack_turbo4_indices`,
 * crates/quant/src/lib.rs:272-285), fp16 scale [N][K/32], fp16 min [N][K/32];
 * w = q * scale + min.  Q4_1 maps onto it unchanged (scale = d, min = m); Q4_0 with
 * scale = d and min = -8 * d, which is exact in fp16 short of overflow, and then
 * q * d + (-8 d) differs from (q - 8) * d by at most one fp32 rounding. */
void oracle_q4_blocks_to_q4g32(const uint8_t* blocks, int has_min, uint8_t* qw, uint16_t* scale,
                               uint16_t* minv, size_t n, size_t k) {
    size_t groups = k / 32;
    const size_t bsz = has_min ? 20 : 18;
    for (size_t r = 0; r < n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t* blk = blocks + (r * groups + g) * bsz;
            const uint16_t dh = (uint16_t)(blk[0] | (blk[1] << 8));
            scale[r * groups + g] = dh;
            minv[r * groups + g] = has_min ? (uint16_t)(blk[2] | (blk[3] << 8))
                                           : oracle_f32_to_f16(-8.0f * oracle_f16_to_f32(dh));
            const uint8_t* qs = blk + (has_min ? 4 : 2);
            uint8_t* dst = qw + r * (k / 2) + g * 16;
            for (int t = 0; t < 8; ++t) {
                dst[t] = (uint8_t)((qs[2 * t] & 0x0F) | ((qs[2 * t + 1] & 0x0F) << 4));
                dst[8 + t] = (uint8_t)((qs[2 * t] >> 4) | ((qs[2 * t + 1] >> 4) << 4));
            }
        }
}

void oracle_dequantize_q4g32(const uint8_t* qw, const uint16_t* scale, const uint16_t* minv,
                             float* w, size_t n, size_t k) {
    size_t groups = k / 32;
    for (size_t r = 0; r < n; ++r)
        for (size_t c = 0; c < k; ++c) {
            const uint8_t byte = qw[r * (k / 2) + c / 2];
            const float q = (float)((c & 1) ? (byte >> 4) : (byte & 0x0F));
            w[r * k + c] = q * oracle_f16_to_f32(scale[r * groups + c / 32]) +
                           oracle_f16_to_f32(minv[r * groups + c / 32]);
        }
}

/* linear_t at m = 1 (crates/kernels/src/cpu_f32/mod.rs:271-345) over the dequantised
 * matrix, ascending k, fp32. */
void oracle_qgemv_q4g32_f32(const float* x, const uint8_t* qw, const uint16_t* scale,
                            const uint16_t* minv, float* y, size_t n, size_t k) {
    size_t groups = k / 32;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n; ++r) {
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            const float s = oracle_f16_to_f32(scale[(size_t)r * groups + g]);
            const float m = oracle_f16_to_f32(minv[(size_t)r * groups + g]);
            for (int i = 0; i < 32; ++i) {
                const size_t c = g * 32 + i;
                const uint8_t byte = qw[(size_t)r * (k / 2) + c / 2];
                const float q = (float)((c & 1) ? (byte >> 4) : (byte & 0x0F));
                acc += x[c] * (q * s + m);
            }
        }
        y[r] = acc;
    }
}

/* ------------------------------------------------------------------ Q4G128 */

/* 4-bit asymmetric, group 128: scale = (max-min)/15, zero = -min/scale, both
 * rounded to fp16 FIRST; q = clamp(roundf(w/scale + zero), 0, 15) with the
 * rounded values, so that dequantisation uses exactly what was stored.  A
 * constant group stores scale = 1, zero = -w (q = 0). */
void oracle_quantize_q4g128(const float* w, uint8_t* qw, uint16_t* scale, uint16_t* zero, size_t n,
                            size_t k) {
    size_t groups = k / 128;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n; ++r)
        for (size_t g = 0; g < groups; ++g) {
            const float* src = w + (size_t)r * k + g * 128;
            float mn = src[0], mx = src[0];
            for (int i = 1; i < 128; ++i) {
                if (src[i] < mn) mn = src[i];
                if (src[i] > mx) mx = src[i];
            }
            float s = (mx - mn) / 15.0f;
            float z;
            if (s == 0.0f || oracle_f16_to_f32(oracle_f32_to_f16(s)) == 0.0f) {
                s = 1.0f;
                z = -mn;
            } else {
                s = oracle_f16_to_f32(oracle_f32_to_f16(s));
                z = -mn / s;
            }
            uint16_t s16 = oracle_f32_to_f16(s), z16 = oracle_f32_to_f16(z);
            scale[(size_t)r * groups + g] = s16;
            zero[(size_t)r * groups + g] = z16;
            float sf = oracle_f16_to_f32(s16), zf = oracle_f16_to_f32(z16);
            uint8_t idx[128];
            for (int i = 0; i < 128; ++i) {
                float q = roundf(src[i] / sf + zf);
                if (q < 0.0f) q = 0.0f;
                if (q > 15.0f) q = 15.0f;
                idx[i] = (uint8_t)q;
            }
            oracle_pack_nibbles(idx, 128, qw + ((size_t)r * k + g * 128) / 2);
        }
}

void oracle_dequantize_q4g128(const uint8_t* qw, const uint16_t* scale, const uint16_t* zero,
                              float* w, size_t n, size_t k) {
    size_t groups = k / 128;
    for (size_t r = 0; r < n; ++r)
        for (size_t c = 0; c < k; ++c) {
            uint8_t q = (qw[(r * k + c) / 2] >> (4 * (c & 1))) & 0xf;
            float s = oracle_f16_to_f32(scale[r * groups + c / 128]);
            float z = oracle_f16_to_f32(zero[r * groups + c / 128]);
            w[r * k + c] = ((float)q - z) * s;
        }
}

/* linear_t (crates/kernels/src/cpu_f32/mod.rs:271-345) over the dequantised
 * matrix with bf16 activations: y[b][n] = bf16( sum_k x[b][k] * ((q-z)*s) ),
 * ascending k, fp32 accumulation, one rounding at the end. */
static void qgemm_q4g128_core(const uint16_t* x_bf16, const uint8_t* qw, const uint16_t* scale,
                              const uint16_t* zero, uint16_t* y_bf16, float* y_f32, size_t b,
                              size_t n, size_t k) {
    size_t groups = k / 128;
    float* xf = (float*)malloc(b * k * sizeof(float));
    oracle_bf16_to_f32_n(x_bf16, xf, b * k);
#pragma omp parallel
    {
        float* wrow = (float*)malloc(k * sizeof(float));
#pragma omp for schedule(static)
        for (long r = 0; r < (long)n; ++r) {
            for (size_t g = 0; g < groups; ++g) {
                float s = oracle_f16_to_f32(scale[(size_t)r * groups + g]);
                float z = oracle_f16_to_f32(zero[(size_t)r * groups + g]);
                for (int i = 0; i < 128; ++i) {
                    size_t c = g * 128 + (size_t)i;
                    uint8_t q = (qw[((size_t)r * k + c) / 2] >> (4 * (c & 1))) & 0xf;
                    wrow[c] = ((float)q - z) * s;
                }
            }
            for (size_t bi = 0; bi < b; ++bi) {
                const float* xr = xf + bi * k;
                float acc = 0.0f;
                for (size_t c = 0; c < k; ++c) acc += xr[c] * wrow[c];
                if (y_f32)
                    y_f32[bi * n + (size_t)r] = acc;
                else
                    y_bf16[bi * n + (size_t)r] = oracle_f32_to_bf16(acc);
            }
        }
        free(wrow);
    }
    free(xf);
}

void oracle_qgemm_q4g128_bf16(const uint16_t* x_bf16, const uint8_t* qw, const uint16_t* scale,
                              const uint16_t* zero, uint16_t* y_bf16, size_t b, size_t n,
                              size_t k) {
    qgemm_q4g128_core(x_bf16, qw, scale, zero, y_bf16, NULL, b, n, k);
}

/* The same product before its final rounding (the decode step keeps GEMM
 * results in fp32 until the next operator). */
void oracle_qgemm_q4g128_f32(const uint16_t* x_bf16, const uint8_t* qw, const uint16_t* scale,
                             const uint16_t* zero, float* y_f32, size_t b, size_t n, size_t k) {
    qgemm_q4g128_core(x_bf16, qw, scale, zero, NULL, y_f32, b, n, k);
}

/* ------------------------------------------------------------------ ragged packing / paged KV */

/* cu_seqlens: exclusive prefix sum with leading 0 (the convention of
 * research/14-gdn-aiter-preflight.md:338); context_lens = prior + new;
 * slot of new token i of sequence s, at position pos = prior + i:
 *   block_tables[s][pos / block_size] * block_size + pos % block_size.
 * A position whose block index is >= max_blocks gets slot -1.  Returns the
 * number of such tokens, or -1 for a negative count. */
#define ORACLE_BLOCK_ID_LIMIT 0x3FFFFFF /* entries from here up, and negative ones, name no block */

int oracle_pack_ragged(const int32_t* new_tokens, const int32_t* prior_ctx,
                       const int32_t* block_tables, int32_t* cu_seqlens, int64_t* slot_mapping,
                       int32_t* context_lens, size_t num_seqs, size_t block_size,
                       size_t max_blocks) {
    int bad = 0;
    cu_seqlens[0] = 0;
    for (size_t s = 0; s < num_seqs; ++s) {
        if (new_tokens[s] < 0 || prior_ctx[s] < 0) return -1;
        cu_seqlens[s + 1] = cu_seqlens[s] + new_tokens[s];
        /* the reference cache refuses to grow past its capacity (Error::LenOverflow,
         * crates/cache/src/flat.rs:180-255); a packer cannot refuse, so the context stops at
         * what the table row can hold and the tokens past it get no slot */
        int64_t cap = (int64_t)block_size * (int64_t)max_blocks;
        int64_t ctx = (int64_t)prior_ctx[s] + (int64_t)new_tokens[s];
        context_lens[s] = (int32_t)(ctx < cap ? ctx : cap);
        for (int32_t i = 0; i < new_tokens[s]; ++i) {
            size_t pos = (size_t)prior_ctx[s] + (size_t)i;
            size_t blk = pos / block_size;
            int64_t slot;
            int32_t id = blk < max_blocks ? block_tables[s * max_blocks + blk] : -1;
            if (blk >= max_blocks || id < 0 || id >= ORACLE_BLOCK_ID_LIMIT) {
                slot = -1; /* past the table, or an entry that names no block */
                bad++;
            } else {
                slot = (int64_t)id * (int64_t)block_size + (int64_t)(pos % block_size);
            }
            slot_mapping[(size_t)cu_seqlens[s] + (size_t)i] = slot;
        }
    }
    return bad;
}

/* Row t of k_new/v_new (`[T][row_elems]`, a FlatKvCache::put row,
 * crates/cache/src/flat.rs:180-252) lands in pool row slot_mapping[t]; negative
 * slots are skipped. */
void oracle_kv_write_fp16(const uint16_t* k_new, const uint16_t* v_new, uint16_t* k_pool,
                          uint16_t* v_pool, const int64_t* slot_mapping, size_t total_tokens,
                          size_t row_elems) {
    for (size_t t = 0; t < total_tokens; ++t) {
        int64_t slot = slot_mapping[t];
        if (slot < 0) continue;
        memcpy(k_pool + (size_t)slot * row_elems, k_new + t * row_elems, row_elems * 2);
        memcpy(v_pool + (size_t)slot * row_elems, v_new + t * row_elems, row_elems * 2);
    }
}

/* The paged counterpart of FlatKvCache::get (crates/cache/src/flat.rs:254-304):
 * rows [0,ctx) of one sequence, in token order, `[ctx][row_elems]`. */
void oracle_paged_gather_fp16(const uint16_t* pool, const int32_t* block_table_row, size_t ctx,
                              size_t block_size, size_t row_elems, uint16_t* out) {
    for (size_t p = 0; p < ctx; ++p) {
        size_t slot = (size_t)block_table_row[p / block_size] * block_size + p % block_size;
        memcpy(out + p * row_elems, pool + slot * row_elems, row_elems * 2);
    }
}

/* ------------------------------------------------------------------ TurboQuant 3-bit KV */

/* `TURBO3_CODEBOOK` (crates/quant/src/lib.rs:66-80): Lloyd-Max centroids, verbatim. */
static const float kTurbo3Codebook[8] = {
    -0.1883972972f, -0.1181399059f, -0.0665857641f, -0.0216044751f,
    0.0216041461f,  0.0665854520f,  0.1181396281f,  0.1883970748f,
};

void oracle_turbo3_codebook(float* out8) { memcpy(out8, kTurbo3Codebook, sizeof kTurbo3Codebook); }

/* `fwht_128` (crates/quant/src/lib.rs:88-113): butterflies h = 1, 2, .., 64 over chunks
 * of 2h (lo += hi, hi = lo - hi), then every value times the f32 literal 1/sqrt(128). */
void oracle_fwht_128(float* data) {
    for (size_t h = 1; h < 128; h *= 2)
        for (size_t c = 0; c < 128; c += 2 * h)
            for (size_t i = 0; i < h; ++i) {
                float x = data[c + i], y = data[c + h + i];
                data[c + i] = x + y;
                data[c + h + i] = x - y;
            }
    const float scale = 0.08838834764831844f;
    for (size_t i = 0; i < 128; ++i) data[i] *= scale;
}

/* `nearest_centroid` (crates/quant/src/lib.rs:119-126): argmin |v - c| by total order,
 * the first minimum wins (Iterator::min_by keeps the first of equal elements). */
static uint8_t turbo3_nearest(float v) {
    int best = 0;
    float bd = fabsf(v - kTurbo3Codebook[0]);
    for (int i = 1; i < 8; ++i) {
        float d = fabsf(v - kTurbo3Codebook[i]);
        /* total_cmp: a NaN distance (v NaN) compares greater than every number */
        if (d < bd) {
            bd = d;
            best = i;
        }
    }
    return (uint8_t)best;
}

/* `pack_turbo3_indices` / `unpack_turbo3_indices` (crates/quant/src/lib.rs:224-268):
 * index i occupies bits [3i, 3i+3) of a little-endian 96-bit integer.  Returns the
 * position of the first index > 7, or -1. */
int oracle_pack_turbo3_indices(const uint8_t* idx32, uint8_t* packed12) {
    memset(packed12, 0, 12);
    for (int i = 0; i < 32; ++i) {
        if (idx32[i] > 7) return i;
        int bit = 3 * i;
        packed12[bit >> 3] |= (uint8_t)(idx32[i] << (bit & 7));
        if ((bit & 7) > 5) packed12[(bit >> 3) + 1] |= (uint8_t)(idx32[i] >> (8 - (bit & 7)));
    }
    return -1;
}

void oracle_unpack_turbo3_indices(const uint8_t* packed12, uint8_t* idx32) {
    for (int i = 0; i < 32; ++i) {
        int bit = 3 * i;
        unsigned v = packed12[bit >> 3] >> (bit & 7);
        if ((bit & 7) > 5) v |= (unsigned)packed12[(bit >> 3) + 1] << (8 - (bit & 7));
        idx32[i] = (uint8_t)(v & 7u);
    }
}

/* `encode_turbo3_0_head` (crates/quant/src/lib.rs:316-353): L2 norm (sequential fp32 sum
 * of squares, sqrt), v / norm (zeros when norm <= 1e-12), FWHT, nearest centroid, pack; the
 * fp16 norm is stored in each of the four 14-byte blocks {norm_f16_le[2], packed[12]}. */
void oracle_encode_turbo3_0_head(const float* values128, uint8_t* out56) {
    float sum_sq = 0.0f;
    for (int i = 0; i < 128; ++i) sum_sq += values128[i] * values128[i];
    const float norm = sqrtf(sum_sq);
    const uint16_t nh = oracle_f32_to_f16(norm);
    float t[128];
    for (int i = 0; i < 128; ++i) t[i] = norm > 1e-12f ? values128[i] / norm : 0.0f;
    oracle_fwht_128(t);
    for (int b = 0; b < 4; ++b) {
        uint8_t idx[32];
        for (int i = 0; i < 32; ++i) idx[i] = turbo3_nearest(t[b * 32 + i]);
        uint8_t* blk = out56 + 14 * b;
        blk[0] = (uint8_t)(nh & 0xff);
        blk[1] = (uint8_t)(nh >> 8);
        oracle_pack_turbo3_indices(idx, blk + 2);
    }
}

/* `decode_turbo3_0_head` (crates/quant/src/lib.rs:376-413): centroids, FWHT, times the
 * norm of the FIRST block. */
void oracle_decode_turbo3_0_head(const uint8_t* in56, float* values128) {
    for (int b = 0; b < 4; ++b) {
        uint8_t idx[32];
        oracle_unpack_turbo3_indices(in56 + 14 * b + 2, idx);
        for (int i = 0; i < 32; ++i) values128[b * 32 + i] = kTurbo3Codebook[idx[i]];
    }
    oracle_fwht_128(values128);
    const float norm = oracle_f16_to_f32((uint16_t)(in56[0] | (in56[1] << 8)));
    for (int i = 0; i < 128; ++i) values128[i] *= norm;
}

/* Paged turbo3 pools [DEFINED BY BUILD]: the fp16 pools with every 128-value head row
 * replaced by its 56 encoded bytes: `[num_blocks][block_size][num_kv_heads][56]`, same
 * block tables and slots.  Writing = `KvCache::put` of encoded rows: k_new / v_new fp16
 * `[T][num_kv_heads][128]`, widened to f32 and encoded head by head. */
void oracle_kv_write_turbo3(const uint16_t* k_new, const uint16_t* v_new, uint8_t* k_pool,
                            uint8_t* v_pool, const int64_t* slot_mapping, size_t total_tokens,
                            size_t num_kv_heads) {
#pragma omp parallel for schedule(static)
    for (long t = 0; t < (long)total_tokens; ++t) {
        int64_t slot = slot_mapping[t];
        if (slot < 0) continue;
        for (size_t h = 0; h < num_kv_heads; ++h) {
            float f[128];
            oracle_f16_to_f32_n(k_new + ((size_t)t * num_kv_heads + h) * 128, f, 128);
            oracle_encode_turbo3_0_head(f, k_pool + ((size_t)slot * num_kv_heads + h) * 56);
            oracle_f16_to_f32_n(v_new + ((size_t)t * num_kv_heads + h) * 128, f, 128);
            oracle_encode_turbo3_0_head(f, v_pool + ((size_t)slot * num_kv_heads + h) * 56);
        }
    }
}

/* First ctx rows of a sequence, decoded to f32 `[ctx][num_kv_heads*128]`. */
void oracle_paged_gather_turbo3(const uint8_t* pool, const int32_t* block_table_row, size_t ctx,
                                size_t block_size, size_t num_kv_heads, float* out) {
    for (size_t j = 0; j < ctx; ++j) {
        size_t slot = (size_t)block_table_row[j / block_size] * block_size + j % block_size;
        for (size_t h = 0; h < num_kv_heads; ++h)
            oracle_decode_turbo3_0_head(pool + (slot * num_kv_heads + h) * 56,
                                        out + (j * num_kv_heads + h) * 128);
    }
}

/* Ragged paged attention.  Per sequence: gather K/V (above), then for every
 * query token the SDPA arithmetic of crates/transformers/src/attention.rs:225-296
 * -- dot in fp32 (ascending d), times scale AFTER the dot, softmax_last_dim
 * over the visible keys, P.V in fp32 (ascending key) -- with the GQA map
 * q head h -> kv head h / groups (:366-382).  Visible keys of query token i
 * (n new tokens, context c): causal ? [0, c-n+i] : [0, c).  No visible key =>
 * zeros (softmax_last_dim over n = 0 columns).  Output rounded to fp16 once. */
static void paged_attn_core(const uint16_t* q, const void* k_pool_any, const void* v_pool_any,
                            int turbo3, const int32_t* block_tables, const int32_t* cu_seqlens_q,
                            const int32_t* context_lens, uint16_t* out, float* out_f32,
                            size_t num_seqs, size_t num_q_heads, size_t num_kv_heads,
                            size_t head_dim, size_t block_size, size_t max_blocks_per_seq,
                            float scale, int causal) {
    size_t groups = num_q_heads / num_kv_heads;
    size_t row = num_kv_heads * head_dim;
    const uint16_t* k_pool = (const uint16_t*)k_pool_any;
    const uint16_t* v_pool = (const uint16_t*)v_pool_any;
#pragma omp parallel for schedule(dynamic, 1)
    for (long s = 0; s < (long)num_seqs; ++s) {
        long ctx = context_lens[s];
        long t0 = cu_seqlens_q[s], t1 = cu_seqlens_q[s + 1];
        long n_new = t1 - t0;
        if (n_new <= 0) continue;
        size_t ctxu = ctx > 0 ? (size_t)ctx : 0;
        uint16_t* kh = (uint16_t*)malloc((ctxu ? ctxu : 1) * row * 2);
        uint16_t* vh = (uint16_t*)malloc((ctxu ? ctxu : 1) * row * 2);
        float* kf = (float*)malloc((ctxu ? ctxu : 1) * row * sizeof(float));
        float* vf = (float*)malloc((ctxu ? ctxu : 1) * row * sizeof(float));
        float* scores = (float*)malloc((ctxu ? ctxu : 1) * sizeof(float));
        float* probs = (float*)malloc((ctxu ? ctxu : 1) * sizeof(float));
        float* qf = (float*)malloc(head_dim * sizeof(float));
        float* of = (float*)malloc(head_dim * sizeof(float));
        const int32_t* bt = block_tables + (size_t)s * max_blocks_per_seq;
        if (turbo3) {
            oracle_paged_gather_turbo3((const uint8_t*)k_pool_any, bt, ctxu, block_size,
                                       num_kv_heads, kf);
            oracle_paged_gather_turbo3((const uint8_t*)v_pool_any, bt, ctxu, block_size,
                                       num_kv_heads, vf);
        } else {
            oracle_paged_gather_fp16(k_pool, bt, ctxu, block_size, row, kh);
            oracle_paged_gather_fp16(v_pool, bt, ctxu, block_size, row, vh);
            oracle_f16_to_f32_n(kh, kf, ctxu * row);
            oracle_f16_to_f32_n(vh, vf, ctxu * row);
        }
        for (long i = 0; i < n_new; ++i) {
            long vis = causal ? (ctx - n_new + i + 1) : ctx;
            if (vis < 0) vis = 0;
            if (vis > ctx) vis = ctx;
            for (size_t h = 0; h < num_q_heads; ++h) {
                size_t kvh = h / groups;
                size_t qoff = ((size_t)(t0 + i) * num_q_heads + h) * head_dim;
                oracle_f16_to_f32_n(q + qoff, qf, head_dim);
                for (long j = 0; j < vis; ++j) {
                    const float* kr = kf + (size_t)j * row + kvh * head_dim;
                    float acc = 0.0f;
                    for (size_t e = 0; e < head_dim; ++e) acc += qf[e] * kr[e];
                    scores[j] = acc * scale;
                }
                oracle_softmax_last_dim(scores, probs, 1, (size_t)vis);
                for (size_t e = 0; e < head_dim; ++e) of[e] = 0.0f;
                for (long j = 0; j < vis; ++j) {
                    const float* vr = vf + (size_t)j * row + kvh * head_dim;
                    float p = probs[j];
                    for (size_t e = 0; e < head_dim; ++e) of[e] += p * vr[e];
                }
                if (out_f32)
                    memcpy(out_f32 + qoff, of, head_dim * sizeof(float));
                else
                    oracle_f32_to_f16_n(of, out + qoff, head_dim);
            }
        }
        free(kh);
        free(vh);
        free(kf);
        free(vf);
        free(scores);
        free(probs);
        free(qf);
        free(of);
    }
}

void oracle_paged_attn_varlen_fp16(const uint16_t* q, const uint16_t* k_pool,
                                   const uint16_t* v_pool, const int32_t* block_tables,
                                   const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                   uint16_t* out, size_t num_seqs, size_t num_q_heads,
                                   size_t num_kv_heads, size_t head_dim, size_t block_size,
                                   size_t max_blocks_per_seq, float scale, int causal) {
    paged_attn_core(q, k_pool, v_pool, 0, block_tables, cu_seqlens_q, context_lens, out, NULL,
                    num_seqs, num_q_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq,
                    scale, causal);
}

/* The same attention with the fp32 result before its final rounding (the decode
 * step rounds it to bf16 once, for the o projection). */
void oracle_paged_attn_varlen_fp16_f32out(const uint16_t* q, const uint16_t* k_pool,
                                          const uint16_t* v_pool, const int32_t* block_tables,
                                          const int32_t* cu_seqlens_q,
                                          const int32_t* context_lens, float* out,
                                          size_t num_seqs, size_t num_q_heads,
                                          size_t num_kv_heads, size_t head_dim, size_t block_size,
                                          size_t max_blocks_per_seq, float scale, int causal) {
    paged_attn_core(q, k_pool, v_pool, 0, block_tables, cu_seqlens_q, context_lens, NULL, out,
                    num_seqs, num_q_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq,
                    scale, causal);
}

/* The same attention over turbo3 pools: every visible K / V head row is decoded with
 * `decode_turbo3_0_head` (f32) and then used exactly as the widened fp16 rows are above;
 * head_dim is 128. */
void oracle_paged_attn_varlen_turbo3(const uint16_t* q, const uint8_t* k_pool,
                                     const uint8_t* v_pool, const int32_t* block_tables,
                                     const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                     uint16_t* out, size_t num_seqs, size_t num_q_heads,
                                     size_t num_kv_heads, size_t block_size,
                                     size_t max_blocks_per_seq, float scale, int causal) {
    paged_attn_core(q, k_pool, v_pool, 1, block_tables, cu_seqlens_q, context_lens, out, NULL,
                    num_seqs, num_q_heads, num_kv_heads, 128, block_size, max_blocks_per_seq,
                    scale, causal);
}

/* The same with the fp32 result (what the decode step rounds once to bf16). */
void oracle_paged_attn_varlen_turbo3_f32out(const uint16_t* q, const uint8_t* k_pool,
                                            const uint8_t* v_pool, const int32_t* block_tables,
                                            const int32_t* cu_seqlens_q,
                                            const int32_t* context_lens, float* out,
                                            size_t num_seqs, size_t num_q_heads,
                                            size_t num_kv_heads, size_t block_size,
                                            size_t max_blocks_per_seq, float scale, int causal) {
    paged_attn_core(q, k_pool, v_pool, 1, block_tables, cu_seqlens_q, context_lens, NULL, out,
                    num_seqs, num_q_heads, num_kv_heads, 128, block_size, max_blocks_per_seq,
                    scale, causal);
}

/* ------------------------------------------------------------------ metric / threads */

/* crates/kernels/tests/matmul_parity.rs:83-99 -- max |g-c| and max |g-c| / max(|c|, 1e-3). */
void oracle_parity_metric_f32(const float* got, const float* want, size_t n, float* max_abs,
                              float* max_rel) {
    float ma = 0.0f, mr = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        float e = fabsf(got[i] - want[i]);
        if (!(e <= ma)) ma = e > ma || e != e ? e : ma;
        float den = fabsf(want[i]);
        if (den < 1e-3f) den = 1e-3f;
        float r = e / den;
        if (!(r <= mr)) mr = r > mr || r != r ? r : mr;
    }
    *max_abs = ma;
    *max_rel = mr;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
