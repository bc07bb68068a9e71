// One continuous-batching decode step (one new token per live sequence) as a
// sequence of asynchronous launches on one stream: the executor the reference
// does not have yet (crates/decoders/src/lib.rs is a scaffold), written against
// the launchers of this library only.  Nothing is allocated, nothing
// synchronises; a caller may capture the whole step into a HIP graph.
#include "launch_common.hpp"

#include <math.h>

namespace {

constexpr int kChunkRows = 32;  // rows the prepared layout and the decode GEMMs hold

// A step with this many packed rows or more takes the projections on the tiled GEMM (plain bf16
// activations, fp32 products for the whole batch at once) instead of 32-row chunks.
constexpr int kTallRows = 97;

struct Workspace {
    char* xn;        // prepared activations of width hidden, one per 32-row chunk (input of qkv /
                     // gate_up; a chunk's buffer carries its normed rows from the end of one
                     // layer to the start of the next)
    char* qkv;       // f32  [Jqkv][rows][(hq+2hkv)*d]   split-K parts of one chunk
    char* q;         // f16  [T][hq*d]
    char* attn_b;    // prepared activations of width hq*d of one chunk (input of the o projection)
    char* attn_out;  // bf16 [T][hq*d]: attention output of a step that is not one chunk of
                     // decode rows (those go straight into attn_b)
    char* proj;      // f32  [max(Jo,Jdown)][rows][hidden]  (o projection, then down projection)
    char* gate_up;   // f32  [Jgu][rows][2*inter]
    char* act;       // prepared activations of width inter (input of the down projection)
    char* attn_ws;   // split-K workspace of the attention
    char* head_ws;   // per-workgroup candidates of the token selection (vocab > 0)
    // many-row steps (tall): plain buffers for all T rows
    char* t_xn;    // bf16 [T][hidden]
    char* t_qkv;   // f32  [T][(hq+2hkv)*d]
    char* t_proj;  // f32  [T][hidden]
    char* t_gu;    // f32  [T][2*inter]
    char* t_act;   // bf16 [T][inter] (or the down projection's own workspace, see carve)
    bool t_act_is_workspace;
    char* t_gemm;  // workspace of the tiled GEMM (its copy of x in unpack order + group sums)
    // tokens for the last row of every sequence (vocab > 0)
    char* norm_out;   // bf16 [T][hidden]: the normed rows when the caller takes none (chunked
                      // steps; a many-row step has t_xn free by then)
    char* last_rows;  // bf16 [num_seqs][hidden]: the normed last rows, gathered
    char* last_xn;    // prepared activations of one chunk of them
    bool tall;
    size_t xn_stride;
    int chunks, rows;  // rows: rows of a full chunk (= T when there is one chunk)
    int j_qkv, j_o, j_gu, j_down;
    size_t total;
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

Workspace carve(const logismos_decode_config_t& c, int num_seqs, int t, int num_splits,
                char* base) {
    Workspace w{};
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* p = base ? base + off : nullptr;
        off += align256(bytes);
        return p;
    };
    const size_t qd = (size_t)c.num_q_heads * c.head_dim;
    const size_t kvd = (size_t)c.num_kv_heads * c.head_dim;
    w.tall = t >= kTallRows;
    if (w.tall) {
        w.attn_ws = take(
            logismos_paged_attn_workspace_bytes(num_seqs, c.num_q_heads, c.head_dim, num_splits));
        w.t_xn = take((size_t)t * c.hidden * 2);
        w.t_qkv = take((size_t)t * (qd + 2 * kvd) * 4);
        w.q = take((size_t)t * qd * 2);
        w.attn_out = take((size_t)t * qd * 2);
        w.t_proj = take((size_t)t * c.hidden * 4);
        w.t_gu = take((size_t)t * 2 * c.intermediate * 4);
        // bf16 [T][inter], or (inter a multiple of 256) a whole workspace of the tiled GEMM over
        // K = inter: the gate/up projection then writes the down projection's operand there
        const size_t act_rows = (size_t)t * c.intermediate * 2;
        const size_t act_ws = c.intermediate % 256 == 0
                                  ? logismos_qgemm_q4g128_tall_workspace_bytes(t, c.intermediate)
                                  : 0;
        w.t_act_is_workspace = act_ws >= act_rows && act_ws > 0;
        w.t_act = take(w.t_act_is_workspace ? act_ws : act_rows);
        const int kmax = c.intermediate > (int)qd ? (c.intermediate > c.hidden ? c.intermediate : c.hidden)
                                                  : ((int)qd > c.hidden ? (int)qd : c.hidden);
        w.t_gemm = take(logismos_qgemm_q4g128_tall_workspace_bytes(t, kmax));
        if (c.vocab > 0) {
            w.last_rows = take((size_t)num_seqs * c.hidden * 2);
            w.last_xn = take(logismos_q4_xprep_bytes(kChunkRows, c.hidden));
            w.head_ws =
                take(logismos_qgemm_q4g128_greedy_workspace_bytes(kChunkRows, c.vocab, c.hidden));
        }
        w.total = off;
        return w;
    }
    w.chunks = (t + kChunkRows - 1) / kChunkRows;
    w.rows = t < kChunkRows ? t : kChunkRows;
    const int b = w.rows;
    // the number of K parts depends on the batch only through its tile height (<= 16 rows or
    // more), so a ragged last chunk of a long step may plan fewer parts than a full one: size
    // for the larger and let every launch use its own count
    auto parts = [&](int n, int k) {
        int j = logismos_qgemm_q4g128_splitk_xprep_parts(b, n, k);
        const int last = t - (w.chunks - 1) * kChunkRows;
        const int jl = logismos_qgemm_q4g128_splitk_xprep_parts(last, n, k);
        return j > jl ? j : jl;
    };
    w.j_qkv = parts((int)(qd + 2 * kvd), c.hidden);
    w.j_o = parts(c.hidden, (int)qd);
    w.j_gu = parts(2 * c.intermediate, c.hidden);
    w.j_down = parts(c.hidden, c.intermediate);
    const int j_proj = w.j_o > w.j_down ? w.j_o : w.j_down;
    w.xn_stride = align256(logismos_q4_xprep_bytes(b, c.hidden));
    w.xn = take(w.xn_stride * w.chunks);
    w.qkv = take((size_t)w.j_qkv * b * (qd + 2 * kvd) * 4);
    w.q = take((size_t)t * qd * 2);
    w.attn_b = take(logismos_q4_xprep_bytes(b, (int)qd));
    w.attn_out = take((size_t)t * qd * 2);
    w.proj = take((size_t)j_proj * b * c.hidden * 4);
    w.gate_up = take((size_t)w.j_gu * b * 2 * c.intermediate * 4);
    w.act = take(logismos_q4_xprep_bytes(b, c.intermediate));
    w.attn_ws =
        take(logismos_paged_attn_workspace_bytes(num_seqs, c.num_q_heads, c.head_dim, num_splits));
    if (c.vocab > 0) {
        const int hb = num_seqs < kChunkRows ? (b > num_seqs ? b : num_seqs) : kChunkRows;
        w.head_ws = take(logismos_qgemm_q4g128_greedy_workspace_bytes(hb, c.vocab, c.hidden));
        w.norm_out = take((size_t)t * c.hidden * 2);
        w.last_rows = take((size_t)num_seqs * c.hidden * 2);
        w.last_xn = take(logismos_q4_xprep_bytes(kChunkRows, c.hidden));
    }
    w.total = off;
    return w;
}

bool config_ok(const logismos_decode_config_t* c, int num_seqs, int t, int max_seqlen_q) {
    if (!c || num_seqs <= 0 || t < num_seqs || max_seqlen_q < 1 || max_seqlen_q > t) return false;
    if (num_seqs > 65535 || t > 65535) return false;
    if (c->num_layers <= 0 || c->hidden <= 0 || c->intermediate <= 0 || c->max_pos <= 0)
        return false;
    if (c->num_q_heads <= 0 || c->num_kv_heads <= 0) return false;
    // heads of 128 on the kernels built for them; other multiples of 32 up to 256 on the general
    // attention kernel (fp16 pools only: a turbo3 head row is 128 wide)
    if (c->head_dim <= 0 || c->head_dim % 32 != 0 || c->head_dim > 256) return false;
    if (c->head_dim != 128 && c->kv_turbo3) return false;
    // what the attention launcher accepts, checked here so that no step is launched in part:
    // GQA groups up to 8 (16 on the general kernel), whose packed rows end at 65520
    if (c->num_q_heads % c->num_kv_heads != 0 ||
        c->num_q_heads / c->num_kv_heads > (c->head_dim == 128 ? 8 : 16))
        return false;
    if (c->head_dim != 128 && t > 65520) return false;
    if (c->hidden % 128 != 0 || c->intermediate % 128 != 0) return false;
    if (((int64_t)c->num_q_heads * c->head_dim) % 128 != 0) return false;
    // every position a block table can hold must have a row in the RoPE tables
    if (c->block_size <= 0 || c->max_blocks_per_seq <= 0 ||
        (int64_t)c->max_pos < (int64_t)c->block_size * c->max_blocks_per_seq)
        return false;
    if ((int64_t)t * (c->num_q_heads + 2 * c->num_kv_heads) * c->head_dim > (int64_t)INT32_MAX ||
        (int64_t)t * c->hidden > (int64_t)INT32_MAX)
        return false;
    if (c->vocab < 0) return false;
    // tokens in / tokens out for every packed row is a decode-step feature: one chunk
    if (c->vocab > 0 && t <= kChunkRows &&
        logismos_check_qgemm_q4g128_greedy_shape(t, c->vocab, c->hidden, nullptr, 0))
        return false;
    const int b = t < kChunkRows ? t : kChunkRows;
    const int qd = c->num_q_heads * c->head_dim;
    const int kvd = c->num_kv_heads * c->head_dim;
    if (t >= kTallRows) {
        // the tiled GEMM's own limits (the products of the whole batch are held in fp32)
        const int64_t lim = INT32_MAX;
        const int64_t widest = 2 * (int64_t)c->intermediate > qd + 2 * kvd
                                   ? 2 * (int64_t)c->intermediate
                                   : (int64_t)qd + 2 * kvd;
        return (int64_t)t * widest <= lim && (int64_t)widest * c->hidden <= lim &&
               (int64_t)c->hidden * c->intermediate <= lim && c->hidden >= 128 && qd >= 128;
    }
    // every projection must have a plan for a full chunk of rows and for the ragged last chunk
    const int last = t - (t - 1) / kChunkRows * kChunkRows;
    for (const int rows : {b, last}) {
        if (logismos_qgemm_q4g128_splitk_xprep_parts(rows, qd + 2 * kvd, c->hidden) <= 0 ||
            logismos_qgemm_q4g128_splitk_xprep_parts(rows, c->hidden, qd) <= 0 ||
            logismos_qgemm_q4g128_splitk_xprep_parts(rows, 2 * c->intermediate, c->hidden) <= 0 ||
            logismos_qgemm_q4g128_splitk_xprep_parts(rows, c->hidden, c->intermediate) <= 0)
            return false;
    }
    return true;
}

// total_tokens / max_seqlen_q of a batch: 0 means "one new token per sequence"
int batch_tokens(const logismos_decode_batch_t* b) {
    return b->total_tokens > 0 ? b->total_tokens : b->num_seqs;
}
int batch_max_q(const logismos_decode_batch_t* b) {
    return b->max_seqlen_q > 0 ? b->max_seqlen_q : 1;
}

}  // namespace

extern "C" size_t logismos_decode_step_workspace_bytes(const logismos_decode_config_t* cfg,
                                                       int num_seqs, int num_splits) {
    return logismos_decode_step_workspace_bytes_tokens(cfg, num_seqs, num_seqs, num_splits);
}

extern "C" size_t logismos_decode_step_workspace_bytes_tokens(const logismos_decode_config_t* cfg,
                                                              int num_seqs, int total_tokens,
                                                              int num_splits) {
    if (!config_ok(cfg, num_seqs, total_tokens, 1) || num_splits <= 0) return 0;
    return carve(*cfg, num_seqs, total_tokens, num_splits, nullptr).total;
}

#define LG_TRY(call)                                  \
    do {                                              \
        logismos_status_t st__ = (call);              \
        if (st__ != 0) return st__;                   \
    } while (0)

extern "C" logismos_status_t logismos_launch_decode_step(const logismos_decode_config_t* cfg,
                                                         const logismos_decode_layer_t* layers,
                                                         const logismos_decode_batch_t* batch,
                                                         void* workspace,
                                                         logismos_stream_t stream) {
    if (!cfg || !layers || !batch || !workspace) return hipErrorInvalidValue;
    const int num_seqs = batch->num_seqs;
    const int t = batch_tokens(batch);
    const int max_q = batch_max_q(batch);
    if (!config_ok(cfg, num_seqs, t, max_q) || batch->num_splits <= 0) return hipErrorInvalidValue;
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return hipErrorInvalidValue;
    const logismos_decode_config_t& c = *cfg;
    const bool tokens_in = batch->token_ids != nullptr;
    const bool tokens_out = batch->lm_head != nullptr;
    if ((tokens_in || tokens_out) && c.vocab <= 0) return hipErrorInvalidValue;
    if (tokens_in && !batch->embed_table_bf16) return hipErrorInvalidValue;
    if (tokens_out && !batch->out_tokens_u32) return hipErrorInvalidValue;
    if (!tokens_out && !batch->out_bf16) return hipErrorInvalidValue;
    const bool last_only = tokens_out && batch->tokens_for_last_rows != 0;
    if (last_only) {
        // the sequences' last rows go through the vocabulary projection 32 at a time
        const int full = num_seqs < kChunkRows ? num_seqs : kChunkRows;
        const int rest = num_seqs % kChunkRows;
        for (const int rows : {full, rest ? rest : full})
            if (logismos_check_qgemm_q4g128_greedy_shape(rows, c.vocab, c.hidden, nullptr, 0))
                return hipErrorInvalidValue;
    }
    // the vocabulary projection with its token choice takes one chunk of rows: every packed
    // row of a step of up to 32, or (tokens_for_last_rows) the last row of every sequence
    if (tokens_out && !last_only && t > kChunkRows) return hipErrorInvalidValue;
    const Workspace w = carve(c, num_seqs, t, batch->num_splits, static_cast<char*>(workspace));
    const int qd = c.num_q_heads * c.head_dim;
    const int kvd = c.num_kv_heads * c.head_dim;
    const int width = qd + 2 * kvd;
    const float scale = 1.0f / sqrtf((float)c.head_dim);
    const bool one_chunk = w.chunks == 1;
    // tokens for last rows: the normed rows of the whole batch, in the caller's buffer or in
    // the workspace, are gathered afterwards
    char* const norm_dst = batch->out_bf16 ? static_cast<char*>(batch->out_bf16)
                                           : (w.tall ? w.t_xn : w.norm_out);
    auto project_last_rows = [&]() -> logismos_status_t {
        LG_TRY(lg::gather_last_rows_bf16_launch(norm_dst, batch->cu_seqlens, w.last_rows, num_seqs,
                                                c.hidden, static_cast<hipStream_t>(stream)));
        const logismos_q4_weight_t& H = *batch->lm_head;
        for (int s0 = 0; s0 < num_seqs; s0 += kChunkRows) {
            const int rows = num_seqs - s0 < kChunkRows ? num_seqs - s0 : kChunkRows;
            LG_TRY(logismos_launch_q4_prepare_x_bf16(w.last_rows + (size_t)s0 * c.hidden * 2,
                                                     w.last_xn, rows, c.hidden, stream));
            LG_TRY(logismos_launch_qgemm_q4g128_greedy_xprep(
                w.last_xn, H.qw, H.scale, H.zero,
                static_cast<uint32_t*>(batch->out_tokens_u32) + s0,
                batch->logits_f32 ? static_cast<float*>(batch->logits_f32) + (size_t)s0 * c.vocab
                                  : nullptr,
                w.head_ws, rows, c.vocab, c.hidden, stream));
        }
        return 0;
    };
    // attention writes the o projection's input (the prepared layout's groups of 128 are whole
    // heads only at head_dim 128)
    const bool direct = one_chunk && max_q == 1 && c.head_dim == 128;
    float* const h = static_cast<float*>(batch->hidden_f32);
    auto rows_of = [&](int ch) {
        const int r0 = ch * kChunkRows;
        return t - r0 < kChunkRows ? t - r0 : kChunkRows;
    };

    if (tokens_in)
        LG_TRY(logismos_launch_embed_lookup_bf16(batch->embed_table_bf16, batch->token_ids,
                                                 batch->hidden_f32, t, c.hidden, c.vocab, stream));
    if (w.tall) {
        // ---- many rows: every projection is one launch of the tiled GEMM over all T rows
        // (fp32 products, consumed un-rounded by the next operator as in the chunked path), the
        // small operators run over all rows at once
        hipStream_t st = static_cast<hipStream_t>(stream);
        auto gemm = [&](const void* x_bf16, const logismos_q4_weight_t& W, const void* bias,
                        void* y_f32, int n, int k) -> logismos_status_t {
            // K in pairs of groups: the kernel that takes x through a first pass into the
            // workspace; otherwise the one that stages x itself
            if (logismos_check_qgemm_q4g128_tall_shape(t, n, k, nullptr, 0) == 0)
                return logismos_launch_qgemm_q4g128_tall(x_bf16, W.qw, W.scale, W.zero, bias, y_f32,
                                                         1, w.t_gemm, t, n, k, stream);
            return lg::qgemm_q4_tall_f32_launch(x_bf16, W.qw, W.scale, W.zero,
                                                static_cast<const float*>(bias), y_f32, t, n, k, st);
        };
        // add + norm followed by a projection of the normed rows: where the tiled GEMM with a
        // workspace takes the shape, the normed rows go straight into its workspace in the
        // kernel's operand order (no first pass over them)
        auto norm_then_gemm = [&](int parts, const void* gains, const logismos_q4_weight_t& W,
                                  void* y_f32, int n) -> logismos_status_t {
            if (logismos_check_qgemm_q4g128_tall_shape(t, n, c.hidden, nullptr, 0) == 0 &&
                c.hidden <= 16384) {
                LG_TRY(logismos_launch_add_rms_norm_f32p_tall(
                    batch->hidden_f32, w.t_proj, parts, gains, w.t_gemm, t, c.hidden, c.rms_eps,
                    logismos_qgemm_q4g128_tall_pairs_per_load(c.hidden, W.scale, W.zero), stream));
                return logismos_launch_qgemm_q4g128_tall_prepared(W.qw, W.scale, W.zero, nullptr,
                                                                  y_f32, 1, w.t_gemm, t, n,
                                                                  c.hidden, stream);
            }
            LG_TRY(logismos_launch_add_rms_norm_f32p(batch->hidden_f32, w.t_proj, parts, gains,
                                                     w.t_xn, t, c.hidden, c.rms_eps, stream));
            return gemm(w.t_xn, W, nullptr, y_f32, n, c.hidden);
        };
        int res_parts = 0;
        for (int l = 0; l < c.num_layers; ++l) {
            const logismos_decode_layer_t& L = layers[l];
            LG_TRY(norm_then_gemm(res_parts, L.norm1_w_f32, L.qkv, w.t_qkv, width));
            const auto rope_kv_write = c.kv_turbo3 ? logismos_launch_rope_kv_write_f32p_turbo3_bias
                                                   : logismos_launch_rope_kv_write_f32p_bias;
            LG_TRY(rope_kv_write(w.t_qkv, 1, L.qkv_bias_f32, batch->positions, batch->rope_cos_f32,
                                 batch->rope_sin_f32, batch->slot_mapping, w.q, L.k_pool_f16,
                                 L.v_pool_f16, t, c.num_q_heads, c.num_kv_heads, c.head_dim,
                                 c.max_pos, stream));
            LG_TRY(lg::paged_attn_launch(
                w.q, L.k_pool_f16, L.v_pool_f16, batch->block_tables, batch->cu_seqlens,
                batch->context_lens, w.attn_out, w.attn_ws, num_seqs, t, max_q, c.num_q_heads,
                c.num_kv_heads, c.head_dim, c.block_size, c.max_blocks_per_seq, batch->num_splits,
                scale, 1, LOGISMOS_ATTN_PHASE_ALL, 1, c.kv_turbo3 ? 1 : 0, stream));
            LG_TRY(gemm(w.attn_out, L.o, nullptr, w.t_proj, c.hidden, qd));
            if (logismos_check_qgemm_q4g128_tall_shape(t, 2 * c.intermediate, c.hidden, nullptr, 0) ==
                    0 &&
                c.hidden <= 16384) {
                // the gate/up projection with the SwiGLU where its products are summed: the
                // fp32 gate and up products never go to memory
                LG_TRY(logismos_launch_add_rms_norm_f32p_tall(
                    batch->hidden_f32, w.t_proj, 1, L.norm2_w_f32, w.t_gemm, t, c.hidden, c.rms_eps,
                    logismos_qgemm_q4g128_tall_pairs_per_load(c.hidden, L.gate_up.scale,
                                                              L.gate_up.zero),
                    stream));
                if (w.t_act_is_workspace &&
                    logismos_check_qgemm_q4g128_tall_shape(t, c.hidden, c.intermediate, nullptr,
                                                           0) == 0) {
                    // ... and the activations written as the down projection's operand, in its
                    // own workspace: no bf16 rows in between, no first pass over them
                    LG_TRY(logismos_launch_qgemm_q4g128_tall_swiglu_operand(
                        L.gate_up.qw, L.gate_up.scale, L.gate_up.zero, w.t_act,
                        logismos_qgemm_q4g128_tall_pairs_per_load(c.intermediate, L.down.scale,
                                                                  L.down.zero),
                        w.t_gemm, t, c.intermediate, c.hidden, stream));
                    LG_TRY(logismos_launch_qgemm_q4g128_tall_prepared(
                        L.down.qw, L.down.scale, L.down.zero, nullptr, w.t_proj, 1, w.t_act, t,
                        c.hidden, c.intermediate, stream));
                } else {
                    LG_TRY(logismos_launch_qgemm_q4g128_tall_swiglu_prepared(
                        L.gate_up.qw, L.gate_up.scale, L.gate_up.zero, w.t_act, w.t_gemm, t,
                        c.intermediate, c.hidden, stream));
                    LG_TRY(gemm(w.t_act, L.down, nullptr, w.t_proj, c.hidden, c.intermediate));
                }
                res_parts = 1;
                continue;
            }
            LG_TRY(norm_then_gemm(1, L.norm2_w_f32, L.gate_up, w.t_gu, 2 * c.intermediate));
            if (logismos_check_qgemm_q4g128_tall_shape(t, c.hidden, c.intermediate, nullptr, 0) == 0) {
                // the activation goes straight into the down projection's workspace, in the
                // kernel's operand order: no first pass over it
                LG_TRY(logismos_launch_silu_mul_f32p_tall(
                    w.t_gu, 1, w.t_gemm, t, c.intermediate,
                    logismos_qgemm_q4g128_tall_pairs_per_load(c.intermediate, L.down.scale,
                                                              L.down.zero),
                    stream));
                LG_TRY(logismos_launch_qgemm_q4g128_tall_prepared(L.down.qw, L.down.scale, L.down.zero,
                                                                  nullptr, w.t_proj, 1, w.t_gemm, t,
                                                                  c.hidden, c.intermediate, stream));
            } else {
                LG_TRY(logismos_launch_silu_mul_f32p(w.t_gu, 1, w.t_act, t, c.intermediate, stream));
                LG_TRY(gemm(w.t_act, L.down, nullptr, w.t_proj, c.hidden, c.intermediate));
            }
            res_parts = 1;
        }
        LG_TRY(logismos_launch_add_rms_norm_f32p(batch->hidden_f32, w.t_proj, res_parts,
                                                 batch->final_norm_w_f32, norm_dst, t, c.hidden,
                                                 c.rms_eps, stream));
        return last_only ? project_last_rows() : 0;
    }
    // The normed input of a layer's first half is produced where the residual stream is
    // completed: before layer 0 here, afterwards by the add + norm that folds a chunk's down
    // projection into h (with the NEXT layer's gains).
    for (int ch = 0; ch < w.chunks; ++ch)
        LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(
            h + (int64_t)ch * kChunkRows * c.hidden, nullptr, 0, layers[0].norm1_w_f32,
            w.xn + ch * w.xn_stride, rows_of(ch), c.hidden, c.rms_eps, stream));
    int res_parts = 0;  // split-K parts of the last down projection not yet folded into h
    for (int l = 0; l < c.num_layers; ++l) {
        const logismos_decode_layer_t& L = layers[l];
        const bool last_layer = l + 1 == c.num_layers;
        // ---- first half, chunk by chunk: q/k/v projection, RoPE, K/V rows into the pools
        for (int ch = 0; ch < w.chunks; ++ch) {
            const int r0 = ch * kChunkRows, rows = rows_of(ch);
            LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(
                w.xn + ch * w.xn_stride, L.qkv.qw, L.qkv.scale, L.qkv.zero, w.qkv, rows, width,
                c.hidden, stream));
            const int j = logismos_qgemm_q4g128_splitk_xprep_parts(rows, width, c.hidden);
            const auto rope_kv_write = c.kv_turbo3 ? logismos_launch_rope_kv_write_f32p_turbo3_bias
                                                   : logismos_launch_rope_kv_write_f32p_bias;
            LG_TRY(rope_kv_write(w.qkv, j, L.qkv_bias_f32, batch->positions + r0,
                                 batch->rope_cos_f32, batch->rope_sin_f32,
                                 batch->slot_mapping + r0, w.q + (size_t)r0 * qd * 2, L.k_pool_f16,
                                 L.v_pool_f16, rows, c.num_q_heads, c.num_kv_heads, c.head_dim,
                                 c.max_pos, stream));
        }
        // ---- attention over the whole ragged batch.  One chunk of decode rows: the result
        // goes straight into the prepared layout of the o projection; otherwise bf16 rows that
        // each chunk prepares for itself.
        LG_TRY(lg::paged_attn_launch(
            w.q, L.k_pool_f16, L.v_pool_f16, batch->block_tables, batch->cu_seqlens,
            batch->context_lens, direct ? w.attn_b : w.attn_out,
            w.attn_ws, num_seqs, t, max_q, c.num_q_heads, c.num_kv_heads, c.head_dim, c.block_size,
            c.max_blocks_per_seq, batch->num_splits, scale, 1, LOGISMOS_ATTN_PHASE_ALL,
            direct ? 2 : 1, c.kv_turbo3 ? 1 : 0, stream));
        // ---- second half, chunk by chunk
        for (int ch = 0; ch < w.chunks; ++ch) {
            const int r0 = ch * kChunkRows, rows = rows_of(ch);
            float* hc = h + (int64_t)r0 * c.hidden;
            if (!direct)
                LG_TRY(logismos_launch_q4_prepare_x_bf16(w.attn_out + (size_t)r0 * qd * 2, w.attn_b,
                                                         rows, qd, stream));
            LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(
                w.attn_b, L.o.qw, L.o.scale, L.o.zero, w.proj, rows, c.hidden, qd, stream));
            LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(
                hc, w.proj, logismos_qgemm_q4g128_splitk_xprep_parts(rows, c.hidden, qd),
                L.norm2_w_f32, w.xn + ch * w.xn_stride, rows, c.hidden, c.rms_eps, stream));
            LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(
                w.xn + ch * w.xn_stride, L.gate_up.qw, L.gate_up.scale, L.gate_up.zero, w.gate_up,
                rows, 2 * c.intermediate, c.hidden, stream));
            LG_TRY(logismos_launch_silu_mul_f32p_xprep(
                w.gate_up,
                logismos_qgemm_q4g128_splitk_xprep_parts(rows, 2 * c.intermediate, c.hidden), w.act,
                rows, c.intermediate, stream));
            LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(
                w.act, L.down.qw, L.down.scale, L.down.zero, w.proj, rows, c.hidden, c.intermediate,
                stream));
            const int j_down =
                logismos_qgemm_q4g128_splitk_xprep_parts(rows, c.hidden, c.intermediate);
            if (!last_layer) {
                // fold the down projection into h and norm for the next layer's first half
                LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(
                    hc, w.proj, j_down, layers[l + 1].norm1_w_f32, w.xn + ch * w.xn_stride, rows,
                    c.hidden, c.rms_eps, stream));
            } else if (!one_chunk) {
                // last layer of a multi-chunk step: the final norm of this chunk's rows
                LG_TRY(logismos_launch_add_rms_norm_f32p(
                    hc, w.proj, j_down, batch->final_norm_w_f32,
                    norm_dst + (size_t)r0 * c.hidden * 2, rows, c.hidden, c.rms_eps, stream));
            } else {
                res_parts = j_down;
            }
        }
    }
    if (!one_chunk) return last_only ? project_last_rows() : 0;
    if (last_only) {
        LG_TRY(logismos_launch_add_rms_norm_f32p(batch->hidden_f32, w.proj, res_parts,
                                                 batch->final_norm_w_f32, norm_dst, t, c.hidden,
                                                 c.rms_eps, stream));
        return project_last_rows();
    }
    if (tokens_out) {
        // the normed state in the layout of the vocabulary projection, then the projection
        // with the token choice fused into it
        LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(batch->hidden_f32, w.proj, res_parts,
                                                       batch->final_norm_w_f32, w.xn, t, c.hidden,
                                                       c.rms_eps, stream));
        res_parts = 0;  // folded into h by the call above
        const logismos_q4_weight_t& H = *batch->lm_head;
        LG_TRY(logismos_launch_qgemm_q4g128_greedy_xprep(w.xn, H.qw, H.scale, H.zero,
                                                         batch->out_tokens_u32, batch->logits_f32,
                                                         w.head_ws, t, c.vocab, c.hidden, stream));
    }
    if (batch->out_bf16)
        LG_TRY(logismos_launch_add_rms_norm_f32p(batch->hidden_f32, w.proj, res_parts,
                                                 batch->final_norm_w_f32, batch->out_bf16, t,
                                                 c.hidden, c.rms_eps, stream));
    return 0;
}
