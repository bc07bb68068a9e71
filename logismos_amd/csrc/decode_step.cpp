// One continuous-batching decode step (one new token per live sequence) as a
// sequence of asynchronous launches on one stream: the executor the reference
// does not have yet (crates/decoders/src/lib.rs is a scaffold), written against
// the launchers of this library only.  Nothing is allocated, nothing
// synchronises; a caller may capture the whole step into a HIP graph.
#include "launch_common.hpp"

#include <math.h>

namespace {

struct Workspace {
    char* xn;        // prepared activations of width hidden (input of qkv / gate_up)
    char* qkv;       // f32  [Jqkv][B][(hq+2hkv)*d]   split-K parts
    char* q;         // f16  [B][hq*d]
    char* attn_b;    // prepared activations of width hq*d (input of the o projection)
    char* proj;      // f32  [max(Jo,Jdown)][B][hidden]  (o projection, then down projection)
    char* gate_up;   // f32  [Jgu][B][2*inter]
    char* act;       // prepared activations of width inter (input of the down projection)
    char* attn_ws;   // split-K workspace of the attention
    char* head_ws;   // per-workgroup candidates of the token selection (vocab > 0)
    int j_qkv, j_o, j_gu, j_down;
    size_t total;
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

Workspace carve(const logismos_decode_config_t& c, int b, int num_splits, char* base) {
    Workspace w{};
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* p = base ? base + off : nullptr;
        off += align256(bytes);
        return p;
    };
    const size_t qd = (size_t)c.num_q_heads * c.head_dim;
    const size_t kvd = (size_t)c.num_kv_heads * c.head_dim;
    w.j_qkv = logismos_qgemm_q4g128_splitk_xprep_parts(b, (int)(qd + 2 * kvd), c.hidden);
    w.j_o = logismos_qgemm_q4g128_splitk_xprep_parts(b, c.hidden, (int)qd);
    w.j_gu = logismos_qgemm_q4g128_splitk_xprep_parts(b, 2 * c.intermediate, c.hidden);
    w.j_down = logismos_qgemm_q4g128_splitk_xprep_parts(b, c.hidden, c.intermediate);
    const int j_proj = w.j_o > w.j_down ? w.j_o : w.j_down;
    w.xn = take(logismos_q4_xprep_bytes(b, c.hidden));
    w.qkv = take((size_t)w.j_qkv * b * (qd + 2 * kvd) * 4);
    w.q = take((size_t)b * qd * 2);
    w.attn_b = take(logismos_q4_xprep_bytes(b, (int)qd));
    w.proj = take((size_t)j_proj * b * c.hidden * 4);
    w.gate_up = take((size_t)w.j_gu * b * 2 * c.intermediate * 4);
    w.act = take(logismos_q4_xprep_bytes(b, c.intermediate));
    w.attn_ws = take(logismos_paged_attn_workspace_bytes(b, c.num_q_heads, c.head_dim, num_splits));
    w.head_ws = c.vocab > 0
                    ? take(logismos_qgemm_q4g128_greedy_workspace_bytes(b, c.vocab, c.hidden))
                    : nullptr;
    w.total = off;
    return w;
}

bool config_ok(const logismos_decode_config_t* c, int b) {
    if (!c || b <= 0 || b > 32) return false;
    if (c->num_layers <= 0 || c->hidden <= 0 || c->intermediate <= 0 || c->max_pos <= 0)
        return false;
    if (c->head_dim != 128 || c->num_q_heads <= 0 || c->num_kv_heads <= 0) return false;
    if (c->hidden % 128 != 0 || c->intermediate % 128 != 0) return false;
    if (((int64_t)c->num_q_heads * c->head_dim) % 128 != 0) return false;
    // every position a block table can hold must have a row in the RoPE tables
    if (c->block_size <= 0 || c->max_blocks_per_seq <= 0 ||
        (int64_t)c->max_pos < (int64_t)c->block_size * c->max_blocks_per_seq)
        return false;
    if (c->vocab < 0) return false;
    if (c->vocab > 0 && logismos_check_qgemm_q4g128_greedy_shape(b, c->vocab, c->hidden, nullptr, 0))
        return false;
    return true;
}

}  // namespace

extern "C" size_t logismos_decode_step_workspace_bytes(const logismos_decode_config_t* cfg,
                                                       int num_seqs, int num_splits) {
    if (!config_ok(cfg, num_seqs) || num_splits <= 0) return 0;
    return carve(*cfg, num_seqs, num_splits, nullptr).total;
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
    const int b = batch->num_seqs;
    if (!config_ok(cfg, b) || batch->num_splits <= 0) return hipErrorInvalidValue;
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return hipErrorInvalidValue;
    const logismos_decode_config_t& c = *cfg;
    const bool tokens_in = batch->token_ids != nullptr;
    const bool tokens_out = batch->lm_head != nullptr;
    if ((tokens_in || tokens_out) && c.vocab <= 0) return hipErrorInvalidValue;
    if (tokens_in && !batch->embed_table_bf16) return hipErrorInvalidValue;
    if (tokens_out && !batch->out_tokens_u32) return hipErrorInvalidValue;
    if (!tokens_out && !batch->out_bf16) return hipErrorInvalidValue;
    const Workspace w = carve(c, b, batch->num_splits, static_cast<char*>(workspace));
    const int qd = c.num_q_heads * c.head_dim;
    const int kvd = c.num_kv_heads * c.head_dim;
    const float scale = 1.0f / sqrtf((float)c.head_dim);

    if (tokens_in)
        LG_TRY(logismos_launch_embed_lookup_bf16(batch->embed_table_bf16, batch->token_ids,
                                                 batch->hidden_f32, b, c.hidden, c.vocab, stream));
    int res_parts = 0;  // split-K parts of the projection the next add_rms_norm folds into h
    for (int l = 0; l < c.num_layers; ++l) {
        const logismos_decode_layer_t& L = layers[l];
        LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(batch->hidden_f32, w.proj, res_parts,
                                                       L.norm1_w_f32, w.xn, b, c.hidden, c.rms_eps,
                                                       stream));
        LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(
            w.xn, L.qkv.qw, L.qkv.scale, L.qkv.zero, w.qkv, b, qd + 2 * kvd, c.hidden, stream));
        const auto rope_kv_write = c.kv_turbo3 ? logismos_launch_rope_kv_write_f32p_turbo3
                                               : logismos_launch_rope_kv_write_f32p;
        LG_TRY(rope_kv_write(w.qkv, w.j_qkv, batch->positions, batch->rope_cos_f32,
                             batch->rope_sin_f32, batch->slot_mapping, w.q, L.k_pool_f16,
                             L.v_pool_f16, b, c.num_q_heads, c.num_kv_heads, c.head_dim, c.max_pos,
                             stream));
        // attention writes the prepared layout directly: its output only feeds the o projection
        LG_TRY(lg::paged_attn_launch(
            w.q, L.k_pool_f16, L.v_pool_f16, batch->block_tables, batch->cu_seqlens,
            batch->context_lens, w.attn_b, w.attn_ws, b, b, 1, c.num_q_heads, c.num_kv_heads,
            c.head_dim, c.block_size, c.max_blocks_per_seq, batch->num_splits, scale, 1,
            LOGISMOS_ATTN_PHASE_ALL, 2, c.kv_turbo3 ? 1 : 0, stream));
        LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(w.attn_b, L.o.qw, L.o.scale, L.o.zero,
                                                             w.proj, b, c.hidden, qd, stream));
        LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(batch->hidden_f32, w.proj, w.j_o,
                                                       L.norm2_w_f32, w.xn, b, c.hidden, c.rms_eps,
                                                       stream));
        LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(w.xn, L.gate_up.qw, L.gate_up.scale,
                                                             L.gate_up.zero, w.gate_up, b,
                                                             2 * c.intermediate, c.hidden, stream));
        LG_TRY(logismos_launch_silu_mul_f32p_xprep(w.gate_up, w.j_gu, w.act, b, c.intermediate,
                                                   stream));
        LG_TRY(logismos_launch_qgemm_q4g128_f32_splitk_xprep(w.act, L.down.qw, L.down.scale,
                                                             L.down.zero, w.proj, b, c.hidden,
                                                             c.intermediate, stream));
        res_parts = w.j_down;
    }
    if (tokens_out) {
        // the normed state in the layout of the vocabulary projection, then the projection
        // with the token choice fused into it
        LG_TRY(logismos_launch_add_rms_norm_f32p_xprep(batch->hidden_f32, w.proj, res_parts,
                                                       batch->final_norm_w_f32, w.xn, b, c.hidden,
                                                       c.rms_eps, stream));
        res_parts = 0;  // folded into h by the call above
        const logismos_q4_weight_t& H = *batch->lm_head;
        LG_TRY(logismos_launch_qgemm_q4g128_greedy_xprep(w.xn, H.qw, H.scale, H.zero,
                                                         batch->out_tokens_u32, batch->logits_f32,
                                                         w.head_ws, b, c.vocab, c.hidden, stream));
    }
    if (batch->out_bf16)
        LG_TRY(logismos_launch_add_rms_norm_f32p(batch->hidden_f32, w.proj, res_parts,
                                                 batch->final_norm_w_f32, batch->out_bf16, b,
                                                 c.hidden, c.rms_eps, stream));
    return 0;
}
