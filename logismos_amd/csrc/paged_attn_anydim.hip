// Ragged paged attention for head widths other than 128 (fp16 KV, fp32 softmax): head_dim a
// multiple of 32 up to 256, GQA groups up to 16 heads.  Same semantics as the head_dim-128
// kernels (crates/kernels/src/cpu_f32/mod.rs:380-433 attention, :502-547 softmax; the GQA map
// of crates/transformers/src/attention.rs:233-260); one body for every row of the ragged batch.
//
// One wave64 serves the whole GQA group of one KV head over 16-key tiles of one (query
// token, KV partition).  A workgroup of up to eight waves is (KV heads) x (tile phases): its
// waves of different heads read the same token rows, so the workgroup streams runs of whole
// rows (a wave alone reads one head's 2 * head_dim bytes out of every row); with fewer than
// eight KV heads the waves of a head take the partition's tiles in turn (phase f the tiles
// f, f + F, ...) and their (m, l, acc) states are combined through LDS at the end.
// Per tile of 16 keys (a tile never straddles a KV block: block_size % 16 == 0), with
// lane = (tg = lane / 16, c = lane % 16):
//   * scores on v_mfma_f32_16x16x32_f16: A = K (lane: key c, 8 elements per MFMA), B = the
//     query group (column c = head c, the same elements, kept in registers); head_dim / 32
//     MFMAs give 16 keys x 16 heads, lane (tg, c) holding head c for the keys 4tg .. 4tg + 3.
//     Which elements a lane contributes to which MFMA is free as long as K and q agree.
//     head_dim a multiple of 64 (head rows are whole 128-byte lines): a request covers 8 keys
//     x one line (lane (tg, c): 16-byte piece 2tg + c/8 of key c%8; keys 8..15 in a second
//     request), and the lanes c and c + 8 then swap halves (DPP row_ror:8), which leaves lane
//     (tg, c) with the pieces 2tg, 2tg + 1 of key c per line -- requests whose neighbouring
//     lanes read neighbouring bytes.  Other widths: lane (tg, c) loads the elements
//     32j + 8tg .. + 8 of key c directly (neighbouring lanes on different rows).
//   * one running maximum per head shared by the four lane rows, sums per lane row.
//   * P.V on v_mfma_f32_16x16x16_f16: A = the probabilities as two fp16 terms (head c, keys
//     4tg + r: the layout the scores arrive in), B = V (lane: E = head_dim / 16 elements of
//     its keys 4tg + r, in chunks of 8, 4 or 2 consecutive ones such that a request covers 16
//     lanes x one chunk = a run of consecutive bytes of the row, see v_chunk_pos; MFMA e takes
//     the lane's element e, so its output column c is that element's place in the row); lane
//     (tg, c) ends up with the heads 4tg + r at its E elements.
// Decode rows (one new token): a small batch is split into partitions of part_tokens keys, a
// large one evenly over one worker per CU (the balanced kernel below); the partials (m, l, acc)
// are combined by the merge kernel.  Rows of sequences with several new tokens: the 16
// columns of a score tile are (query token, head) pairs, 16 / G consecutive tokens of a chunk
// per wave, each column masked at its own token's visible length; such a wave takes the whole
// context its last token sees.
//
// Algorithmic HBM bytes per (decode sequence, KV head): ctx * 4 * head_dim (K and V rows)
// + G * 4 * head_dim (q, out) + 4 * ceil(ctx / block_size).
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "paged_attn_params.hpp"
#include "q4_common.hpp"

#include <math.h>

namespace lg {

constexpr int kAnyWaves = 8;           // waves of a workgroup: KV heads x tile phases
constexpr int kAnyLdsBytes = 48 * 1024;  // for the accumulators of the phases beyond the first
constexpr int kAnyWgHeads = 8;           // KV heads per workgroup at most
constexpr int kAnyPhases = 8;            // tile phases per head at most

// KV heads per workgroup: the largest divisor of hkv up to kAnyWgHeads
static int anydim_wg_heads(int hkv) {
    for (int w = kAnyWgHeads; w > 1; --w)
        if (hkv % w == 0) return w;
    return 1;
}

template <int NJ>
struct AnyTile {
    half8_t k[NJ];
    unsigned v[4][NJ];  // key 4tg + r: the lane's 2 NJ elements, two per dword
};

// A load that is (NT) or is not marked non-temporal: decode rows use every K/V byte once per
// launch, rows of chunks read theirs many times out of L2.
template <bool NT, typename T>
__device__ __forceinline__ T load_kv(const T* ptr) {
    if constexpr (NT) return __builtin_nontemporal_load(ptr);
    else return *ptr;
}

// Which of a head row's elements a lane holds for P.V: its E = head_dim / 16 elements come in
// chunks of 8, 4 or 2 (E = 14: 8 + 4 + 2), and chunk (eo, len) of lane c is the elements
// 16 eo + c len .. + len - 1 of the row -- so a request for one chunk of one row covers
// 16 lanes x len consecutive elements, whole 128-byte lines where len >= 4.
constexpr int v_chunk_len(int E, int eo) { return E - eo >= 8 ? 8 : (E - eo >= 4 ? 4 : 2); }
constexpr int v_chunk_start(int E, int e) {
    int eo = 0;
    while (e >= eo + v_chunk_len(E, eo)) eo += v_chunk_len(E, eo);
    return eo;
}
// first element of the chunk that holds the lane's element e, as a position in the row
__device__ __forceinline__ constexpr int v_chunk_pos(int E, int e, int c) {
    return 16 * v_chunk_start(E, e) + c * v_chunk_len(E, v_chunk_start(E, e));
}

// N consecutive dwords (N = 1, 2, 4: a chunk of V, aligned to its own size)
template <int N, bool NT>
__device__ __forceinline__ void load_dwords(const void* src, unsigned* dst) {
    static_assert(N == 1 || N == 2 || N == 4, "a chunk of 2, 4 or 8 elements");
    if constexpr (N == 4) {
        const uint4_t x = load_kv<NT>(static_cast<const uint4_t*>(src));
        dst[0] = x[0], dst[1] = x[1], dst[2] = x[2], dst[3] = x[3];
    } else if constexpr (N == 2) {
        const uint2_t x = load_kv<NT>(static_cast<const uint2_t*>(src));
        dst[0] = x[0], dst[1] = x[1];
    } else {
        dst[0] = load_kv<NT>(static_cast<const unsigned*>(src));
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

// The work of one workgroup on the keys [key_begin, key_end) (not empty) of sequence s for the
// ntok query tokens from packed row t on: scores, softmax, P.V, the merge of the tile phases,
// and either the finished rows (single) or the partial (m, l, acc) at workspace slot `slot`.
// Called by every wave of the workgroup (it holds two barriers).
template <int NJ, bool NT>
__device__ __forceinline__ void anydim_range(const AttnParams& p, int G, int wg_heads, int phases,
                                             int cols, int s, int t, int ntok, int vis_first,
                                             int visible, int key_begin, int key_end, bool single,
                                             int64_t slot, float (*sm_m)[16], float (*sm_l)[16],
                                             float* sm_acc) {
    constexpr int D = 32 * NJ;
    constexpr int E = 2 * NJ;
    constexpr bool kLines = NJ % 2 == 0;  // head rows are whole 128-byte lines
    // (the wave index as a scalar: tile positions and block ids stay in scalar registers, the
    // block table is read with scalar loads)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, tg = lane >> 4;
    const int wg_head = wave % wg_heads, phase = wave / wg_heads;
    const int kvh = blockIdx.y * wg_heads + wg_head;
    // columns of the score tile: (query token, head)
    const int ncols = ntok * G;
    const int ctok = c / G, chead = c - ctok * G;
    const int vis_c = (p.causal && c < ncols) ? vis_first + ctok : visible;

    // the queries as the B operand: column c = (token ctok, head chead), zero beyond ncols
    half8_t qb[NJ];
    {
        const bool cvalid = c < ncols;
        const _Float16* qp = p.q + ((int64_t)(t + (cvalid ? ctok : 0)) * p.hq + (int64_t)kvh * G +
                                    (cvalid ? chead : 0)) * D;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            // (the element order of the K operand, see load_tile / k_operand)
            const int off = kLines ? 64 * (j >> 1) + 16 * tg + 8 * (j & 1) : 32 * j + 8 * tg;
            qb[j] = *reinterpret_cast<const half8_t*>(qp + off);
            if (!cvalid) qb[j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }
    const int32_t* table = p.block_tables + (int64_t)s * p.max_blocks_per_seq;
    const int last_key = key_end - 1;
    // a column's keys end at lim_c; tiles that reach past the shortest column are masked
    const int lim_c = min(vis_c, key_end);
    const int mask_from = min(vis_first, key_end);
    // A tile's addresses: a scalar base (block, offset in the block, KV head) plus a 32-bit
    // lane offset (key of the tile x row bytes + the lane's bytes inside the head row).
    const unsigned row_bytes = (unsigned)p.hkv * D * 2;  // (hkv <= 65535: 16 rows < 2^31)
    const unsigned k_lane = kLines ? 32 * tg + 16 * (c >> 3) : 16 * tg;

    auto load_tile = [&](int tile_begin, int block, int off_in_block, AnyTile<NJ>& tl) {
        const int64_t row0_bytes =
            ((int64_t)block * p.block_size + off_in_block) * row_bytes + (int64_t)kvh * (D * 2);
        const char* kb = reinterpret_cast<const char*>(p.k_pool) + row0_bytes;
        const char* vb = reinterpret_cast<const char*>(p.v_pool) + row0_bytes;
        // keys past the end of the range read the last key of the range and are masked
        const int over = tile_begin + 15 - last_key;  // > 0: the tile runs past the range
        const int lim = over > 0 ? 15 - over : 15;
        if constexpr (kLines) {
            // k[2u + kh]: piece 2tg + c/8 of line u of key 8kh + c%8
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                const unsigned koff = (unsigned)min(8 * kh + (c & 7), lim) * row_bytes + k_lane;
#pragma unroll
                for (int u = 0; u < NJ / 2; ++u)
                    tl.k[2 * u + kh] =
                        load_kv<NT>(reinterpret_cast<const half8_t*>(kb + koff + 128 * u));
            }
        } else {
            const unsigned koff = (unsigned)min(c, lim) * row_bytes + k_lane;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                tl.k[j] = load_kv<NT>(reinterpret_cast<const half8_t*>(kb + koff + 64 * j));
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const unsigned voff = (unsigned)min(4 * tg + r, lim) * row_bytes;
            static_for<E>([&](auto ec) {
                constexpr int e = decltype(ec)::value;
                if constexpr (v_chunk_start(E, e) == e)  // one request per chunk
                    load_dwords<v_chunk_len(E, e) / 2, NT>(vb + voff + 2 * v_chunk_pos(E, e, c),
                                                           &tl.v[r][e / 2]);
            });
        }
    };

    float m = -INFINITY, l = 0.0f;
    float4_t acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    auto compute_tile = [&](int tile_begin, const AnyTile<NJ>& tl) {
        float4_t sacc = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (kLines) {
            // lane c < 8 holds (key c, key c + 8), lane c >= 8 (key c - 8, key c) of its
            // piece: each sends the one its partner c ^ 8 needs and keeps its own key's
#pragma unroll
            for (int u = 0; u < NJ / 2; ++u) {
                const uint4_t r0 = __builtin_bit_cast(uint4_t, tl.k[2 * u]);
                const uint4_t r1 = __builtin_bit_cast(uint4_t, tl.k[2 * u + 1]);
                uint4_t x0, x1;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // row_ror:8 written to the upper (lower) eight lanes of each row only
                    x0[i] = (unsigned)__builtin_amdgcn_update_dpp((int)r0[i], (int)r1[i],
                                                                  kDppRowRor + 8, 0xf, 0xc, false);
                    x1[i] = (unsigned)__builtin_amdgcn_update_dpp((int)r1[i], (int)r0[i],
                                                                  kDppRowRor + 8, 0xf, 0x3, false);
                }
                const half8_t a0 = __builtin_bit_cast(half8_t, x0);
                const half8_t a1 = __builtin_bit_cast(half8_t, x1);
                sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, qb[2 * u], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, qb[2 * u + 1], sacc, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(tl.k[j], qb[j], sacc, 0, 0, 0);
        }
        float sc[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) sc[r] = sacc[r] * p.scale_log2e;
        if (tile_begin + 16 > mask_from) {  // (a whole-wave branch) some column ends in the tile
#pragma unroll
            for (int r = 0; r < 4; ++r)
                sc[r] = tile_begin + 4 * tg + r < lim_c ? sc[r] : -INFINITY;
        }
        float tmax = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        tmax = fmaxf(tmax, lane_xor_f32<16>(tmax));
        tmax = fmaxf(tmax, lane_xor_f32<32>(tmax));
        // Only when some head's maximum grows (a whole-wave branch; rare once a few tiles are
        // in) are the sums and accumulators rescaled.  The accumulators of lane row tg belong
        // to the heads 4tg + r: their factors sit in the lanes c = 4tg + r of this row.
        // (A column none of whose keys has come yet -- a token of a chunk that sees nothing --
        // keeps m = -inf, l = 0: factors and probabilities are taken against 0 there.)
        if (NJ > 4 || __builtin_amdgcn_ballot_w64(tmax > m) != 0) {
            const float m_new = fmaxf(m, tmax);
            const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2(m - m_new);
            m = m_new;
            l *= alpha;
            float ar[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) ar[r] = lane_read_f32(alpha, (lane & 48) | (4 * tg + r));
#pragma unroll
            for (int e = 0; e < E; ++e)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[e][r] *= ar[r];
        }
        half4_t pa, pb;
        float psum = 0.0f;
        const float mref = m == -INFINITY ? 0.0f : m;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float pr = fast_exp2(sc[r] - mref);
            psum += pr;
            pa[r] = (_Float16)pr;
            pb[r] = (_Float16)(pr - (float)pa[r]);
        }
        l += psum;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            // B = element e of the lane's four keys: the low or high halves of their dwords e/2
            const unsigned sel = (e & 1) ? 0x07060302u : 0x05040100u;
            const uint2_t bw = {__builtin_amdgcn_perm(tl.v[1][e >> 1], tl.v[0][e >> 1], sel),
                                __builtin_amdgcn_perm(tl.v[3][e >> 1], tl.v[2][e >> 1], sel)};
            const half4_t vb = __builtin_bit_cast(half4_t, bw);
            acc[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa, vb, acc[e], 0, 0, 0);
            acc[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(pb, vb, acc[e], 0, 0, 0);
        }
    };

    {
        // Two tile buffers in turn, straight-line: the requests of one tile are in flight while
        // the other is consumed, and the block id of a tile is read (a scalar load) a tile
        // before its requests.  A position past the wave's last tile stays on the last tile:
        // every request is unconditional and reads memory the range owns; what was read twice
        // is not consumed.
        const int kStep = kTileKeys * phases;
        const int tb0 = key_begin + kTileKeys * phase;
        if (tb0 < key_end) {
            const int n_tiles = (key_end - tb0 + kStep - 1) / kStep;
            int tb = tb0, bi = tb0 / p.block_size, bo = tb0 - bi * p.block_size;
            auto advance = [&]() {
                if (tb + kStep < key_end) {
                    tb += kStep;
                    bo += kStep;
                    while (bo >= p.block_size) {
                        bo -= p.block_size;
                        ++bi;
                    }
                }
            };
            AnyTile<NJ> ta, tc;
            int tb_a = tb, bo_a = bo, id_a = table[bi];
            advance();
            int tb_c = tb, bo_c = bo, id_c = table[bi];
            load_tile(tb_a, id_a, bo_a, ta);
            for (int i = 0; i < n_tiles; i += 2) {
                load_tile(tb_c, id_c, bo_c, tc);
                advance();
                const int tb_a2 = tb, bo_a2 = bo, id_a2 = table[bi];
                compute_tile(tb_a, ta);
                load_tile(tb_a2, id_a2, bo_a2, ta);
                tb_a = tb_a2;
                advance();
                const int tb_c2 = tb, bo_c2 = bo, id_c2 = table[bi];
                if (i + 1 < n_tiles) compute_tile(tb_c, tc);
                tb_c = tb_c2, bo_c = bo_c2, id_c = id_c2;
            }
        }
    }

    // ---- the states of a head's phases into its phase 0: M = max m_f, factors 2^(m_f - M).
    // A wave without a tile has m = -inf, l = 0, acc = 0 and factor 0; phase 0 always has one.
    float lsum = l + lane_xor_f32<16>(l);
    lsum += lane_xor_f32<32>(lsum);
    if (tg == 0) {
        sm_m[wave][c] = m;
        sm_l[wave][c] = lsum;
    }
    __syncthreads();
    float mall = m, lall = 0.0f;
    for (int f = 0; f < phases; ++f) mall = fmaxf(mall, sm_m[f * wg_heads + wg_head][c]);
    const float mall_ref = mall == -INFINITY ? 0.0f : mall;
    for (int f = 0; f < phases; ++f)
        lall += fast_exp2(sm_m[f * wg_heads + wg_head][c] - mall_ref) *
                sm_l[f * wg_heads + wg_head][c];
    const float fown = fast_exp2(m - mall_ref);
    float fr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) fr[r] = lane_read_f32(fown, (lane & 48) | (4 * tg + r));
    if (phase > 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int h = 4 * tg + r;  // the column these accumulator rows belong to
            if (h >= ncols) continue;
            float* dst = sm_acc + (((phase - 1) * wg_heads + wg_head) * cols + h) * D + E * c;
#pragma unroll
            for (int e = 0; e < E; ++e) dst[e] = acc[e][r] * fr[r];
        }
    }
    __syncthreads();
    if (phase > 0) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int h = 4 * tg + r;
        const float mh = lane_read_f32(mall, (lane & 48) | h);
        const float lh = lane_read_f32(lall, (lane & 48) | h);
        if (h >= ncols) continue;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float a = acc[e][r] * fr[r];
            for (int f = 0; f < phases - 1; ++f)
                a += sm_acc[((f * wg_heads + wg_head) * cols + h) * D + E * c + e];
            acc[e][r] = a;
        }
        const int htok = h / G;
        const int head = kvh * G + (h - htok * G);
        if (single) {
            const float inv = lh > 0.0f ? 1.0f / lh : 0.0f;  // a token that sees no key: zeros
            unsigned short* dst = reinterpret_cast<unsigned short*>(p.out) +
                                  ((int64_t)(t + htok) * p.hq + head) * D;
            static_for<E / 2>([&](auto ec) {
                constexpr int e = 2 * decltype(ec)::value;
                const unsigned w = (unsigned)attn_out_elem(acc[e][r] * inv, p.out_bf16) |
                                   ((unsigned)attn_out_elem(acc[e + 1][r] * inv, p.out_bf16) << 16);
                *reinterpret_cast<unsigned*>(dst + v_chunk_pos(E, e, c) +
                                             (e - v_chunk_start(E, e))) = w;
            });
        } else {
            const int64_t idx = slot * p.hq + head;
            float* dst = p.ws_acc + idx * D;
            static_for<E>([&](auto ec) {
                constexpr int e = decltype(ec)::value;
                dst[v_chunk_pos(E, e, c) + (e - v_chunk_start(E, e))] = acc[e][r];
            });
            if (c == 0) {
                p.ws_ml[idx * 2] = mh;
                p.ws_ml[idx * 2 + 1] = lh;
            }
        }
    }
}

// Static split and rows of chunks: grid (partitions, KV-head groups, sequences or packed rows).
template <int NJ>
__global__ __launch_bounds__(64 * kAnyWaves) void paged_attn_anydim_kernel(const AttnParams p,
                                                                           int G,
                                                                           int decode_rows,
                                                                           int wg_heads,
                                                                           int phases, int cols) {
    constexpr int D = 32 * NJ;
    __shared__ float sm_m[kAnyWaves][16], sm_l[kAnyWaves][16];  // [phase * wg_heads + head]
    extern __shared__ float sm_acc[];  // [phases - 1][wg_heads][cols][D]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wg_head = wave % wg_heads, phase = wave / wg_heads;
    const int kvh = blockIdx.y * wg_heads + wg_head;
    // decode launch: grid.z walks the sequences and takes those with one new token;
    // the other launch walks the packed rows and takes those of the other sequences.  There a
    // workgroup serves 16 / G consecutive rows of a chunk and the workgroups of the other rows
    // leave at once: grid.z walks the rows with that stride (0, n, 2n, .., then 1, n + 1, ..),
    // so that the workgroups that stay are neighbours in launch order and spread over all
    // XCDs (walking row by row, every n-th workgroup stays: with n = 4, two XCDs of eight).
    const int tpw = decode_rows ? 1 : 16 / G;
    int row = blockIdx.z;
    if (!decode_rows) {
        const int nq = (p.out_rows + tpw - 1) / tpw;
        row = (row % nq) * tpw + row / nq;
        if (row >= p.out_rows) return;
    }
    const int s = decode_rows ? (int)blockIdx.z : seq_of_row(p.cu_seqlens_q, p.num_seqs, row);
    // Partition of this workgroup: rotated by the sequence index.  Workgroups are dealt to the
    // eight XCDs in launch order; with partition p of every sequence at x = p and a partition
    // count that is a multiple of 8, the first partitions (which every sequence has) would all
    // land on the same XCDs and the last ones (which only long sequences have) on others.
    const int split = decode_rows ? (int)((blockIdx.x + 5u * (unsigned)s) % gridDim.x) : 0;
    const int row0 = p.cu_seqlens_q[s];
    const int n_new = p.cu_seqlens_q[s + 1] - row0;
    const int t = decode_rows ? row0 : row;
    const int ctx = p.context_lens[s];
    const bool decode_row = n_new == 1;
    if (decode_row != (decode_rows != 0)) return;
    // columns of the score tile: (query token, head).  A decode row: its G heads.  A chunk:
    // 16 / G consecutive tokens, taken by the workgroup of the first of them.
    const int i0 = t - row0;
    if (i0 % tpw != 0) return;
    const int ntok = min(tpw, n_new - i0);
    // visible keys of the first and the last token of the group
    const int vis_first = p.causal ? ctx - n_new + i0 + 1 : ctx;
    const int visible = p.causal ? vis_first + ntok - 1 : ctx;

    int key_begin = 0, key_end = visible;
    bool single = true;
    if (decode_row && p.num_splits > 1) {
        key_begin = split * p.part_tokens;
        key_end = min(visible, key_begin + p.part_tokens);
        single = visible <= p.part_tokens;
    } else if (split != 0) {
        return;
    }
    if (visible <= 0) {
        // no visible key for any of the tokens: rows of zeros (written once)
        if (split == 0)
            for (int tq = 0; tq < ntok; ++tq) {
                _Float16* out_row = p.out + ((int64_t)(t + tq) * p.hq + (int64_t)kvh * G) * D;
                for (int i = lane + 64 * phase; i < G * D; i += 64 * phases)
                    out_row[i] = (_Float16)0.0f;
            }
        return;
    }
    if (key_begin >= key_end) return;

    // (plain loads: rows of chunks read their keys many times out of L2, and the short
    // partitions of a small decode batch measured slower with non-temporal ones, 10.2 vs 9.3 us)
    anydim_range<NJ, false>(p, G, wg_heads, phases, cols, s, t, ntok, vis_first, visible,
                            key_begin, key_end, single, (int64_t)s * p.num_splits + split, sm_m,
                            sm_l, sm_acc);
}

// Decode rows, balanced: the 16-key tiles of all decode sequences form one stream (each
// sequence preceded by kSeqStartUnits units for starting it); worker w (grid.x) takes the units
// [wR, (w + 1)R), R = ceil(total / workers), whichever sequences they belong to, so every
// workgroup does the same amount of work whatever the context lengths are.  Its piece of
// sequence s goes to workspace slot w + s (the pieces of a sequence get consecutive slots); a
// sequence inside one worker is finished there.  grid (workers, KV-head groups).
template <int NJ>
__global__ __launch_bounds__(64 * kAnyWaves) void paged_attn_anydim_balanced_kernel(
    const AttnParams p, int G, int wg_heads, int phases) {
    __shared__ int pt[kMaxBalancedSeqs + 1];  // exclusive prefix of the sequences' units
    __shared__ float sm_m[kAnyWaves][16], sm_l[kAnyWaves][16];
    extern __shared__ float sm_acc[];  // [phases - 1][wg_heads][G][D]
    const int lane = threadIdx.x & 63;
    const int S = p.num_seqs;
    if (threadIdx.x < 64) {
        const int per = (S + 63) / 64;
        int sum = 0;
        for (int i = 0; i < per; ++i) {
            const int s = lane * per + i;
            if (s < S) sum += decode_tiles(p, s);
        }
        int incl = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (lane >= off) incl += v;
        }
        int run = incl - sum;
        for (int i = 0; i < per; ++i) {
            const int s = lane * per + i;
            if (s < S) {
                pt[s] = run;
                run += decode_tiles(p, s);
            }
        }
        if (lane == 63) pt[S] = incl;
    }
    __syncthreads();
    // (LDS reads land in vector registers: wave-uniform values are made scalar again so that
    // block ids keep coming through scalar loads)
    const int total = __builtin_amdgcn_readfirstlane(pt[S]);
    const int w = blockIdx.x;
    const int R = worker_tiles(total, p.num_workers);
    const int64_t ub64 = (int64_t)w * R;
    if (ub64 >= total) return;
    const int ub = (int)ub64;
    const int ue = (int)min((int64_t)total, ub64 + R);
    int lo = 0, hi = S;  // the sequence holding unit ub: the largest s with pt[s] <= ub
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (__builtin_amdgcn_readfirstlane(pt[mid]) <= ub) lo = mid;
        else hi = mid;
    }
    int ucur = ub;
    for (int s = lo; ucur < ue; ++s) {
        const int seq_begin = __builtin_amdgcn_readfirstlane(pt[s]);
        const int seq_end = __builtin_amdgcn_readfirstlane(pt[s + 1]);
        if (seq_end <= ucur) continue;  // a sequence without decode tiles
        const int seg_end = min(ue, seq_end);
        // units -> tiles of the sequence: its first kSeqStartUnits units are the start-up cost
        const int tile_lo = max(ucur - seq_begin - kSeqStartUnits, 0);
        const int tile_hi = seg_end - seq_begin - kSeqStartUnits;
        if (tile_hi > tile_lo) {
            const int ctx = p.context_lens[s];
            const bool single = tile_lo == 0 && seg_end == seq_end;
            // (inlined: as a call the body needs its frame in scratch memory; four tile buffers
            // instead of two measured no faster at head_dim 64, 46.8 vs 45.6 us)
            // Non-temporal K/V loads where every request covers whole 128-byte lines: head_dim
            // a multiple of 64 (K requested line-wise, V in chunks of 4 or 8 elements per lane).
            // Config 5's batch: 41.9 vs 45.6 us at head_dim 64, 228-235 vs 240-248 us at 256.
            // Otherwise a line is split between requests and the later one, marked non-temporal,
            // fetches it again.
            anydim_range<NJ, NJ % 2 == 0>(p, G, wg_heads, phases, G, s, p.cu_seqlens_q[s], 1, ctx, ctx,
                             tile_lo * kTileKeys, min(ctx, tile_hi * kTileKeys), single,
                             (int64_t)w + s, sm_m, sm_l, sm_acc);
        }
        ucur = seg_end;
    }
}

// Decode rows with more than one partition: out = sum_p w_p acc_p / sum_p w_p l_p,
// w_p = 2^(m_p - max m).  grid (hq, num_seqs), 256 threads: thread = (stripe, element pair),
// stripe j sums the partitions j, j + S, ...; the stripes are added through LDS.
__global__ __launch_bounds__(256) void paged_attn_anydim_merge_kernel(const AttnParams p, int D) {
    __shared__ float sm_red[4];
    __shared__ float sm_a[256][2];
    __shared__ float sm_lt[128];
    const int head = blockIdx.x;
    const int s = blockIdx.y;
    const int t = p.cu_seqlens_q[s];
    if (p.cu_seqlens_q[s + 1] - t != 1) return;
    const int ctx = p.context_lens[s];
    const int tid = threadIdx.x;
    int parts;      // partials of this sequence
    int64_t slot0;  // of its first partial
    if (p.num_workers > 0) {
        // balanced split: where this sequence sits in the stream of units
        __shared__ int red[2][4];
        int before = 0, total = 0;
        for (int i = tid; i < p.num_seqs; i += 256) {
            const int nt = decode_tiles(p, i);
            total += nt;
            before += i < s ? nt : 0;
        }
#pragma unroll
        for (int mask = 32; mask >= 1; mask >>= 1) {
            total += __shfl_xor(total, mask, 64);
            before += __shfl_xor(before, mask, 64);
        }
        if ((tid & 63) == 0) {
            red[0][tid >> 6] = total;
            red[1][tid >> 6] = before;
        }
        __syncthreads();
        total = red[0][0] + red[0][1] + red[0][2] + red[0][3];
        before = red[1][0] + red[1][1] + red[1][2] + red[1][3];
        if (ctx <= 0) {
            // the stream has no tile of this row and nobody wrote it: a row of zeros
            if (2 * tid < D)
                *reinterpret_cast<unsigned*>(reinterpret_cast<unsigned short*>(p.out) +
                                             ((int64_t)t * p.hq + head) * D + 2 * tid) = 0u;
            return;
        }
        // its tiles are the units [before + kSeqStartUnits, before + nt)
        const int nt = (ctx + kTileKeys - 1) / kTileKeys + kSeqStartUnits;
        const int R = worker_tiles(total, p.num_workers);
        const int w_first = (before + kSeqStartUnits) / R;
        parts = (before + nt - 1) / R - w_first + 1;
        slot0 = (int64_t)w_first + s;
    } else {
        parts = ctx <= 0 ? 0 : (ctx + p.part_tokens - 1) / p.part_tokens;
        slot0 = (int64_t)s * p.num_splits;
    }
    if (parts <= 1) return;  // zero or one partial: already final
    float mmax = -INFINITY;
    for (int q = tid; q < parts; q += 256)
        mmax = fmaxf(mmax, p.ws_ml[((slot0 + q) * p.hq + head) * 2]);
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) mmax = fmaxf(mmax, shfl_xor_f32(mmax, o));
    if ((tid & 63) == 0) sm_red[tid >> 6] = mmax;
    __syncthreads();
    mmax = fmaxf(fmaxf(sm_red[0], sm_red[1]), fmaxf(sm_red[2], sm_red[3]));

    const int d2 = D / 2;
    const int stripes = 256 / d2;  // >= 2
    const int stripe = tid / d2, pair = tid - stripe * d2;
    float a0 = 0.0f, a1 = 0.0f, lt = 0.0f;
    if (stripe < stripes) {
        for (int q = stripe; q < parts; q += stripes) {
            const int64_t idx = (slot0 + q) * p.hq + head;
            const float w = fast_exp2(p.ws_ml[idx * 2] - mmax);
            lt += w * p.ws_ml[idx * 2 + 1];
            const float2 a = *reinterpret_cast<const float2*>(p.ws_acc + idx * D + 2 * pair);
            a0 += w * a.x;
            a1 += w * a.y;
        }
        sm_a[tid][0] = a0;
        sm_a[tid][1] = a1;
        if (pair == 0) sm_lt[stripe] = lt;
    }
    __syncthreads();
    if (stripe != 0) return;
    for (int j = 1; j < stripes; ++j) {
        a0 += sm_a[j * d2 + pair][0];
        a1 += sm_a[j * d2 + pair][1];
        lt += sm_lt[j];
    }
    const float inv = 1.0f / lt;
    const unsigned w = (unsigned)attn_out_elem(a0 * inv, p.out_bf16) |
                       ((unsigned)attn_out_elem(a1 * inv, p.out_bf16) << 16);
    *reinterpret_cast<unsigned*>(reinterpret_cast<unsigned short*>(p.out) +
                                 ((int64_t)t * p.hq + head) * D + 2 * pair) = w;
}

template <int NJ>
static void launch_rows(const AttnParams& p, int total_tokens, int max_seqlen_q, int phases,
                 hipStream_t stream) {
    const int g = p.hq / p.hkv;
    // waves of a workgroup: KV heads first, the rest as tile phases (a power of two) as far as
    // their accumulators fit the LDS budget
    const int wg_heads = anydim_wg_heads(p.hkv);
    // (cols: the columns a wave's accumulators cover -- a decode row's group, or the
    // 16 / G tokens of a chunk times the group)
    auto launch = [&](int grid_x, int grid_z, int decode_rows, int cols, int wg_heads) {
        const size_t phase_bytes = (size_t)wg_heads * cols * (32 * NJ) * sizeof(float);
        int tile_phases = 1;
        while (tile_phases * 2 <= kAnyPhases && tile_phases * 2 * wg_heads <= kAnyWaves &&
               (size_t)(tile_phases * 2 - 1) * phase_bytes <= (size_t)kAnyLdsBytes)
            tile_phases *= 2;
        const size_t lds = (size_t)(tile_phases - 1) * phase_bytes;
        paged_attn_anydim_kernel<NJ>
            <<<dim3(grid_x, p.hkv / wg_heads, grid_z), dim3(64 * wg_heads * tile_phases), lds,
               stream>>>(p, g, decode_rows, wg_heads, tile_phases, cols);
    };
    if (phases & LOGISMOS_ATTN_PHASE_DECODE) {
        if (p.num_workers > 0) {
            const size_t phase_bytes = (size_t)wg_heads * g * (32 * NJ) * sizeof(float);
            int tile_phases = 1;
            while (tile_phases * 2 <= kAnyPhases && tile_phases * 2 * wg_heads <= kAnyWaves &&
                   (size_t)(tile_phases * 2 - 1) * phase_bytes <= (size_t)kAnyLdsBytes)
                tile_phases *= 2;
            paged_attn_anydim_balanced_kernel<NJ>
                <<<dim3(p.num_workers, p.hkv / wg_heads), dim3(64 * wg_heads * tile_phases),
                   (size_t)(tile_phases - 1) * phase_bytes, stream>>>(p, g, wg_heads, tile_phases);
        } else {
            launch(p.num_splits, p.num_seqs, 1, g, wg_heads);
        }
    }
    // rows of chunks: a workgroup walks a whole context, most of it out of L2, and the longest
    // walk sets the time of the launch -- more tile phases per head, fewer heads together
    if ((phases & LOGISMOS_ATTN_PHASE_PREFILL) && max_seqlen_q > 1)
        launch(1, (total_tokens + 16 / g - 1) / (16 / g) * (16 / g), 0, (16 / g) * g,
               wg_heads % 2 == 0 ? 2 : 1);
}

// Workers of a balanced launch per group of KV heads: one workgroup per CU (narrow heads fit
// two, and measured slower with two: 62 vs 56 us at head_dim 64 on config 5's batch).
static int64_t anydim_resident_workgroups(int) { return (int64_t)device_cu_count(); }

// Workers of the balanced decode launch (0: static split -- one partition, a small batch, or
// more sequences than the prefix table holds): what is resident at once per group of KV heads,
// limited by the workspace the caller sized for num_splits partials per sequence (slots used:
// at most workers + num_seqs - 1).
static int anydim_workers(const AttnParams& p, int head_dim) {
    if (p.num_splits <= 1 || p.num_seqs > kMaxBalancedSeqs ||
        small_decode_batch(p.num_seqs, p.hkv, p.block_size, p.max_blocks_per_seq))
        return 0;
    int64_t target = anydim_resident_workgroups(head_dim) / (p.hkv / anydim_wg_heads(p.hkv));
    if (target < 1) target = 1;
    const int64_t cap = (int64_t)p.num_seqs * (p.num_splits - 1);
    return (int)(target < cap ? target : cap);
}

// Workgroups = partitions x groups of KV heads.  Narrow heads (two workgroups fit a CU) aim at
// two per CU, wide ones at half the CUs (one workgroup per CU and no second round even when
// the contexts run long), for contexts of half the longest on average; a partition keeps at
// least 128 keys.
int paged_attn_anydim_num_splits(int num_seqs, int num_kv_heads, int head_dim, int block_size,
                                 int max_blocks_per_seq) {
    if (num_seqs <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
        max_blocks_per_seq <= 0)
        return 1;
    const int64_t max_ctx = (int64_t)block_size * max_blocks_per_seq;
    const int64_t cus = device_cu_count();
    const int64_t target = head_dim <= 64 ? 2 * cus : cus / 2;
    const int64_t groups = (int64_t)num_seqs * (num_kv_heads / anydim_wg_heads(num_kv_heads));
    int64_t splits = (2 * target + groups - 1) / groups;
    const int64_t most = (max_ctx + 127) / 128;
    if (splits > most) splits = most;
    if (num_seqs <= kMaxBalancedSeqs &&
        !small_decode_batch(num_seqs, num_kv_heads, block_size, max_blocks_per_seq)) {
        // the balanced launch: slots for every resident workgroup (workers + num_seqs - 1)
        const int64_t workers =
            anydim_resident_workgroups(head_dim) / (num_kv_heads / anydim_wg_heads(num_kv_heads));
        const int64_t need = (workers + num_seqs - 1) / num_seqs + 1;
        if (splits < need) splits = need;
    }
    if (splits > 4096) splits = 4096;
    if (splits < 1) splits = 1;
    return (int)splits;
}

hipError_t paged_attn_anydim_launch(const AttnParams& params, int head_dim, int total_tokens,
                                    int max_seqlen_q, int phases, hipStream_t stream) {
    AttnParams p = params;
    p.num_workers = anydim_workers(p, head_dim);
    if (head_dim <= 0 || head_dim % 32 != 0 || head_dim > 256) return hipErrorInvalidValue;
    if (p.hq % p.hkv != 0 || p.hq / p.hkv > 16) return hipErrorInvalidValue;
    if (total_tokens > 65520 || p.num_seqs > 65535 || p.hkv > 65535) return hipErrorInvalidValue;
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
        paged_attn_anydim_merge_kernel<<<grid, dim3(256), 0, stream>>>(p, head_dim);
    }
    return hipGetLastError();
}

}  // namespace lg
