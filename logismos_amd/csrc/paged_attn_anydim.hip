// Ragged paged attention for head widths other than 128 (fp16 KV, fp32 softmax): head_dim a
// multiple of 32 up to 256, GQA groups up to 16 heads.  Same semantics as the head_dim-128
// kernels (crates/kernels/src/cpu_f32/mod.rs:380-433 attention, :502-547 softmax; the GQA map
// of crates/transformers/src/attention.rs:233-260), not tuned to their degree: one kernel for
// every row of the ragged batch.
//
// One wave64 owns one (query token, KV head, KV partition) and serves the whole GQA group.
// Per tile of 16 keys (a tile never straddles a KV block: block_size % 16 == 0), with
// lane = (tg = lane / 16, c = lane % 16):
//   * scores on v_mfma_f32_16x16x32_f16: A = K (lane: key c, elements 32j + 8tg .. + 8 of
//     piece j, one 16-byte load per piece), B = the query group (column c = head c, same
//     pieces, kept in registers); head_dim / 32 MFMAs give 16 keys x 16 heads, lane (tg, c)
//     holding head c for the keys 4tg .. 4tg + 3.
//   * one running maximum per head shared by the four lane rows, sums per lane row.
//   * P.V on v_mfma_f32_16x16x16_f16: A = the probabilities as two fp16 terms (head c, keys
//     4tg + r: the layout the scores arrive in), B = V (lane: E = head_dim / 16 consecutive
//     elements E c .. E c + E - 1 of its keys 4tg + r, one load of 2E bytes per key; MFMA e
//     takes element e, so its output column c is element E c + e); lane (tg, c) ends up with
//     the heads 4tg + r at its E elements.
// Decode rows (one new token) are split into partitions of part_tokens keys whose partials
// (m, l, acc) the merge kernel combines; rows of sequences with several new tokens take their
// whole visible context in one wave.
//
// Algorithmic HBM bytes per (decode sequence, KV head): ctx * 4 * head_dim (K and V rows)
// + G * 4 * head_dim (q, out) + 4 * ceil(ctx / block_size).
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "paged_attn_params.hpp"

#include <math.h>

namespace lg {

namespace {

constexpr int kAnyTileKeys = 16;

template <int NJ>
struct AnyTile {
    half8_t k[NJ];
    _Float16 v[4][2 * NJ];
};

// E consecutive fp16 values; 2E bytes, aligned to 4 (E is even)
template <int E>
__device__ __forceinline__ void load_halves(const _Float16* src, _Float16 (&dst)[E]) {
    if constexpr (E % 8 == 0) {
#pragma unroll
        for (int i = 0; i < E / 8; ++i) {
            const half8_t x = *reinterpret_cast<const half8_t*>(src + 8 * i);
#pragma unroll
            for (int e = 0; e < 8; ++e) dst[8 * i + e] = x[e];
        }
    } else if constexpr (E % 4 == 0) {
#pragma unroll
        for (int i = 0; i < E / 4; ++i) {
            const half4_t x = *reinterpret_cast<const half4_t*>(src + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[4 * i + e] = x[e];
        }
    } else {
#pragma unroll
        for (int i = 0; i < E / 2; ++i) {
            const half2_t x = *reinterpret_cast<const half2_t*>(src + 2 * i);
            dst[2 * i] = x[0];
            dst[2 * i + 1] = x[1];
        }
    }
}

__device__ __forceinline__ float lane_read_f32(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane * 4, __float_as_int(v)));
}

// sequence of packed row t: the s with cu[s] <= t < cu[s + 1]
__device__ __forceinline__ int seq_of_row(const int32_t* cu, int num_seqs, int t) {
    int lo = 0, hi = num_seqs;  // cu[lo] <= t < cu[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu[mid] <= t) lo = mid;
        else hi = mid;
    }
    return lo;
}

template <int NJ>
__global__ __launch_bounds__(64) void paged_attn_anydim_kernel(const AttnParams p, int G,
                                                               int decode_rows) {
    constexpr int D = 32 * NJ;
    constexpr int E = 2 * NJ;
    const int lane = threadIdx.x;
    const int c = lane & 15, tg = lane >> 4;
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    // decode launch: grid.z walks the sequences and takes those with one new token;
    // the other launch walks the packed rows and takes those of the other sequences
    const int s = decode_rows ? (int)blockIdx.z : seq_of_row(p.cu_seqlens_q, p.num_seqs, blockIdx.z);
    const int row0 = p.cu_seqlens_q[s];
    const int n_new = p.cu_seqlens_q[s + 1] - row0;
    const int t = decode_rows ? row0 : (int)blockIdx.z;
    const int ctx = p.context_lens[s];
    const bool decode_row = n_new == 1;
    if (decode_row != (decode_rows != 0)) return;
    const int visible = p.causal ? ctx - n_new + (t - row0) + 1 : ctx;

    int key_begin = 0, key_end = visible;
    bool single = true;
    if (decode_row && p.num_splits > 1) {
        key_begin = split * p.part_tokens;
        key_end = min(visible, key_begin + p.part_tokens);
        single = visible <= p.part_tokens;
    } else if (split != 0) {
        return;
    }
    _Float16* out_row = p.out + ((int64_t)t * p.hq + (int64_t)kvh * G) * D;
    if (visible <= 0) {
        // no visible key: a row of zeros (written once)
        if (split == 0)
            for (int i = lane; i < G * D; i += 64) out_row[i] = (_Float16)0.0f;
        return;
    }
    if (key_begin >= key_end) return;

    // the query group as the B operand: column c = head c (zero beyond the group)
    half8_t qb[NJ];
    {
        const _Float16* qp = p.q + ((int64_t)t * p.hq + (int64_t)kvh * G + (c < G ? c : 0)) * D + 8 * tg;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            qb[j] = *reinterpret_cast<const half8_t*>(qp + 32 * j);
            if (c >= G) qb[j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }
    const int32_t* table = p.block_tables + (int64_t)s * p.max_blocks_per_seq;
    const int64_t row_halves = (int64_t)p.hkv * D;
    const int last_key = key_end - 1;

    auto load_tile = [&](int tile_begin, AnyTile<NJ>& tl) {
        const int block = table[tile_begin / p.block_size];
        const int64_t base = (int64_t)block * p.block_size + tile_begin % p.block_size;
        // keys past the end of the range read the last key of the range and are masked
        const int over = tile_begin + 15 - last_key;  // > 0: the tile runs past the range
        const int kk = (over > 0 && c > 15 - over) ? 15 - over : c;
        const _Float16* kp = p.k_pool + (base + kk) * row_halves + (int64_t)kvh * D + 8 * tg;
#pragma unroll
        for (int j = 0; j < NJ; ++j) tl.k[j] = *reinterpret_cast<const half8_t*>(kp + 32 * j);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int key = 4 * tg + r;
            const int vk = (over > 0 && key > 15 - over) ? 15 - over : key;
            load_halves<E>(p.v_pool + (base + vk) * row_halves + (int64_t)kvh * D + E * c, tl.v[r]);
        }
    };

    float m = -INFINITY, l = 0.0f;
    float4_t acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    auto compute_tile = [&](int tile_begin, const AnyTile<NJ>& tl) {
        float4_t sacc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(tl.k[j], qb[j], sacc, 0, 0, 0);
        float sc[4];
        float tmax = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            sc[r] = tile_begin + 4 * tg + r <= last_key ? sacc[r] * p.scale_log2e : -INFINITY;
            tmax = fmaxf(tmax, sc[r]);
        }
        tmax = fmaxf(tmax, lane_xor_f32<16>(tmax));
        tmax = fmaxf(tmax, lane_xor_f32<32>(tmax));
        const float m_new = fmaxf(m, tmax);  // finite: the first key of every tile is in range
        const float alpha = fast_exp2(m - m_new);
        m = m_new;
        half4_t pa, pb;
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float pr = fast_exp2(sc[r] - m_new);
            psum += pr;
            pa[r] = (_Float16)pr;
            pb[r] = (_Float16)(pr - (float)pa[r]);
        }
        l = l * alpha + psum;
        // the accumulators of lane row tg belong to the heads 4tg + r: their factors sit in
        // the lanes c = 4tg + r of this row
        float ar[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) ar[r] = lane_read_f32(alpha, (lane & 48) | (4 * tg + r));
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[e][r] *= ar[r];
            const half4_t vb = {tl.v[0][e], tl.v[1][e], tl.v[2][e], tl.v[3][e]};
            acc[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa, vb, acc[e], 0, 0, 0);
            acc[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(pb, vb, acc[e], 0, 0, 0);
        }
    };

    AnyTile<NJ> cur, nxt;
    load_tile(key_begin, cur);
    for (int tb = key_begin; tb < key_end; tb += kAnyTileKeys) {
        const bool more = tb + kAnyTileKeys < key_end;
        if (more) load_tile(tb + kAnyTileKeys, nxt);
        compute_tile(tb, cur);
        if (more) cur = nxt;
    }

    float lsum = l + lane_xor_f32<16>(l);
    lsum += lane_xor_f32<32>(lsum);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int h = 4 * tg + r;
        const float mh = lane_read_f32(m, (lane & 48) | h);
        const float lh = lane_read_f32(lsum, (lane & 48) | h);
        if (h >= G) continue;
        const int head = kvh * G + h;
        if (single) {
            const float inv = 1.0f / lh;
            unsigned short* dst =
                reinterpret_cast<unsigned short*>(p.out) + ((int64_t)t * p.hq + head) * D + E * c;
#pragma unroll
            for (int e = 0; e < E; e += 2) {
                const unsigned w = (unsigned)attn_out_elem(acc[e][r] * inv, p.out_bf16) |
                                   ((unsigned)attn_out_elem(acc[e + 1][r] * inv, p.out_bf16) << 16);
                *reinterpret_cast<unsigned*>(dst + e) = w;
            }
        } else {
            const int64_t idx = ((int64_t)s * p.num_splits + split) * p.hq + head;
            float* dst = p.ws_acc + idx * D + E * c;
#pragma unroll
            for (int e = 0; e < E; ++e) dst[e] = acc[e][r];
            if (c == 0) {
                p.ws_ml[idx * 2] = mh;
                p.ws_ml[idx * 2 + 1] = lh;
            }
        }
    }
}

// Decode rows with more than one partition: out = sum_p w_p acc_p / sum_p w_p l_p,
// w_p = 2^(m_p - max m).  grid (hq, num_seqs), one thread per element pair.
__global__ __launch_bounds__(128) void paged_attn_anydim_merge_kernel(const AttnParams p, int D) {
    const int head = blockIdx.x;
    const int s = blockIdx.y;
    const int t = p.cu_seqlens_q[s];
    if (p.cu_seqlens_q[s + 1] - t != 1) return;
    const int ctx = p.context_lens[s];
    if (ctx <= p.part_tokens) return;  // zero or one partition: already final
    const int parts = (ctx + p.part_tokens - 1) / p.part_tokens;
    const int64_t slot0 = (int64_t)s * p.num_splits;
    float mmax = -INFINITY;
    for (int q = 0; q < parts; ++q) mmax = fmaxf(mmax, p.ws_ml[((slot0 + q) * p.hq + head) * 2]);
    const int d = 2 * threadIdx.x;
    if (d >= D) return;
    float a0 = 0.0f, a1 = 0.0f, lt = 0.0f;
    for (int q = 0; q < parts; ++q) {
        const int64_t idx = (slot0 + q) * p.hq + head;
        const float w = fast_exp2(p.ws_ml[idx * 2] - mmax);
        lt += w * p.ws_ml[idx * 2 + 1];
        a0 += w * p.ws_acc[idx * D + d];
        a1 += w * p.ws_acc[idx * D + d + 1];
    }
    const float inv = 1.0f / lt;
    const unsigned w = (unsigned)attn_out_elem(a0 * inv, p.out_bf16) |
                       ((unsigned)attn_out_elem(a1 * inv, p.out_bf16) << 16);
    *reinterpret_cast<unsigned*>(reinterpret_cast<unsigned short*>(p.out) +
                                 ((int64_t)t * p.hq + head) * D + d) = w;
}

template <int NJ>
void launch_rows(const AttnParams& p, int total_tokens, int max_seqlen_q, int phases,
                 hipStream_t stream) {
    if (phases & LOGISMOS_ATTN_PHASE_DECODE) {
        dim3 grid(p.num_splits, p.hkv, p.num_seqs);
        paged_attn_anydim_kernel<NJ><<<grid, dim3(64), 0, stream>>>(p, p.hq / p.hkv, 1);
    }
    if ((phases & LOGISMOS_ATTN_PHASE_PREFILL) && max_seqlen_q > 1) {
        dim3 grid(1, p.hkv, total_tokens);
        paged_attn_anydim_kernel<NJ><<<grid, dim3(64), 0, stream>>>(p, p.hq / p.hkv, 0);
    }
}

}  // namespace

hipError_t paged_attn_anydim_launch(const AttnParams& p, int head_dim, int total_tokens,
                                    int max_seqlen_q, int phases, hipStream_t stream) {
    if (head_dim <= 0 || head_dim % 32 != 0 || head_dim > 256) return hipErrorInvalidValue;
    if (p.hq % p.hkv != 0 || p.hq / p.hkv > 16) return hipErrorInvalidValue;
    if (total_tokens > 65535 || p.num_seqs > 65535 || p.hkv > 65535) return hipErrorInvalidValue;
    if (p.out_bf16 != 0 && p.out_bf16 != 1) return hipErrorInvalidValue;
    if (phases & (LOGISMOS_ATTN_PHASE_DECODE | LOGISMOS_ATTN_PHASE_PREFILL)) {
        switch (head_dim / 32) {
            case 1: launch_rows<1>(p, total_tokens, max_seqlen_q, phases, stream); break;
            case 2: launch_rows<2>(p, total_tokens, max_seqlen_q, phases, stream); break;
            case 3: launch_rows<3>(p, total_tokens, max_seqlen_q, phases, stream); break;
            case 4: launch_rows<4>(p, total_tokens, max_seqlen_q, phases, stream); break;
            case 5: launch_rows<5>(p, total_tokens, max_seqlen_q, phases, stream); break;
            case 6: launch_rows<6>(p, total_tokens, max_seqlen_q, phases, stream); break;
            case 7: launch_rows<7>(p, total_tokens, max_seqlen_q, phases, stream); break;
            default: launch_rows<8>(p, total_tokens, max_seqlen_q, phases, stream); break;
        }
    }
    if ((phases & LOGISMOS_ATTN_PHASE_MERGE) && p.num_splits > 1) {
        dim3 grid(p.hq, p.num_seqs);
        paged_attn_anydim_merge_kernel<<<grid, dim3(128), 0, stream>>>(p, head_dim);
    }
    return hipGetLastError();
}

}  // namespace lg
