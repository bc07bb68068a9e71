/*
 * logismos_oracle.h -- CPU oracle for the ragged-batch decode path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * CPU functions that define the arithmetic of the path, plus CPU definitions
 * of the contracts the reference does not have (paged KV, block tables,
 * ragged packing, Q8G32 / Q4G128 weights).  Only the test-suite, the smoke
 * check and the `cpu_baseline` leg of the benchmark may link or load it; the
 * shipped library never does.
 *
 * Every function names the reference file:line it follows.  How each one is
 * pinned (reference known-answer tests, closed forms, brute force) is listed
 * in tests/test_oracle_*.py; none is "parity unpinned".
 *
 * Deviation that cannot be closed here: `cpu_f32::linear` / `linear_t`
 * delegate the fp32 summation order to the third-party crate
 * `matrixmultiply` ("0.3", no lockfile, not vendored under the reference).
 * The oracle accumulates in ascending k like the reference's own
 * `matmul_fp16_ref`; parity at that boundary is tolerance-based, exactly as
 * in the reference's own tests (crates/kernels/src/cpu_f32/tests.rs:46-92).
 */
#ifndef LOGISMOS_ORACLE_H
#define LOGISMOS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar conversions (IEEE round-to-nearest-even, like half::f16::from_f32) */
uint16_t oracle_f32_to_f16(float x);
float oracle_f16_to_f32(uint16_t h);
uint16_t oracle_f32_to_bf16(float x);
float oracle_bf16_to_f32(uint16_t h);
void oracle_f32_to_f16_n(const float* x, uint16_t* y, size_t n);
void oracle_f16_to_f32_n(const uint16_t* x, float* y, size_t n);
void oracle_f32_to_bf16_n(const float* x, uint16_t* y, size_t n);
void oracle_bf16_to_f32_n(const uint16_t* x, float* y, size_t n);

/* ---- cpu_f32 op set (crates/kernels/src/cpu_f32/mod.rs) */
void oracle_embed_lookup(const float* weight, size_t hidden, size_t vocab, const uint32_t* ids,
                         size_t n_ids, float* out);
void oracle_rms_norm(const float* x, const float* weight, float* y, size_t rows, size_t n,
                     float eps);
void oracle_linear(const float* a, const float* b, const float* bias, float* c, size_t m, size_t n,
                   size_t k);
void oracle_linear_t(const float* a, const float* b, const float* bias, float* c, size_t m,
                     size_t n, size_t k);
void oracle_silu(const float* x, float* y, size_t n);
void oracle_hadamard(const float* a, const float* b, float* c, size_t n);
void oracle_softmax_last_dim(const float* x, float* y, size_t rows, size_t n);
int oracle_mask_additive_in_place(float* scores, const uint8_t* mask, size_t mask_len, size_t rows,
                                  size_t n);
void oracle_rope_halves_in_place(float* x, const float* cos, const float* sin, size_t rows,
                                 size_t head_dim);
void oracle_build_rope_table_f32(size_t seq, size_t head_dim, double theta, float* cos_out,
                                 float* sin_out);

/* ---- fp16-I/O references (crates/kernels/src/{matmul,softmax,rms_norm}/cpu.rs) */
void oracle_matmul_fp16_ref(const uint16_t* a, const uint16_t* b, uint16_t* d, size_t m, size_t n,
                            size_t k);
void oracle_softmax_fp16_ref(const uint16_t* x, uint16_t* y, size_t m, size_t n);
void oracle_rms_norm_fp16_ref(const uint16_t* x, const uint16_t* w, uint16_t* y, size_t m, size_t n,
                              float eps);
void oracle_build_cos_sin_table(size_t seq, size_t head_dim, float theta_base, float* table);
void oracle_rope_apply_fp16_ref(uint16_t* qk, const float* cos_sin, size_t batch, size_t seq,
                                size_t heads, size_t head_dim);

/* ---- attention pieces (crates/transformers/src/attention.rs) */
void oracle_transpose_seq_heads(const float* x, float* out, size_t seq, size_t heads, size_t d);
void oracle_merge_heads(const float* attn, float* out, size_t heads, size_t seq, size_t d);
void oracle_repeat_kv(const float* kv, float* out, size_t n_kv, size_t groups, size_t seq,
                      size_t d);
/* SDPA section of QwenAttention::forward: q [n_h,seq,d], k/v [n_kv,seq,d] (already roped),
 * mask [seq] (0 = padded key), out [n_h,seq,d]. */
void oracle_sdpa_f32(const float* q_hsd, const float* k_hsd, const float* v_hsd,
                     const uint8_t* mask, float* out_hsd, size_t n_h, size_t n_kv, size_t seq,
                     size_t d);

/* ---- decode::greedy (crates/decode/src/lib.rs:73-83) */
uint32_t oracle_greedy(const float* logits, size_t n);

/* ---- nibble order (crates/quant/src/lib.rs:272-301) */
int oracle_pack_nibbles(const uint8_t* idx, size_t n, uint8_t* packed);
void oracle_unpack_nibbles(const uint8_t* packed, size_t n, uint8_t* idx);

/* ---- Q8G32 (ggml Q8_0 arithmetic; planar and 34-byte block forms) */
void oracle_quantize_q8g32(const float* w, int8_t* qs, uint16_t* d, size_t n, size_t k);
void oracle_dequantize_q8g32(const int8_t* qs, const uint16_t* d, float* w, size_t n, size_t k);
void oracle_q8g32_to_q8_0_blocks(const int8_t* qs, const uint16_t* d, uint8_t* blocks, size_t n,
                                 size_t k);
void oracle_q8_0_blocks_to_q8g32(const uint8_t* blocks, int8_t* qs, uint16_t* d, size_t n,
                                 size_t k);
void oracle_qgemv_q8g32_f32(const float* x, const int8_t* qs, const uint16_t* d, float* y,
                            size_t n, size_t k);

/* ---- ggml Q4_0 / Q4_1 blocks (18 / 20 bytes per 32 values) and planar Q4G32 */
void oracle_quantize_q4_0_blocks(const float* w, uint8_t* blocks, size_t n, size_t k);
void oracle_quantize_q4_1_blocks(const float* w, uint8_t* blocks, size_t n, size_t k);
void oracle_dequantize_q4_0_blocks(const uint8_t* blocks, float* w, size_t n, size_t k);
void oracle_dequantize_q4_1_blocks(const uint8_t* blocks, float* w, size_t n, size_t k);
void oracle_q4_blocks_to_q4g32(const uint8_t* blocks, int has_min, uint8_t* qw, uint16_t* scale,
                               uint16_t* minv, size_t n, size_t k);
void oracle_dequantize_q4g32(const uint8_t* qw, const uint16_t* scale, const uint16_t* minv,
                             float* w, size_t n, size_t k);
void oracle_qgemv_q4g32_f32(const float* x, const uint8_t* qw, const uint16_t* scale,
                            const uint16_t* minv, float* y, size_t n, size_t k);

/* ---- Q4G128 */
void oracle_quantize_q4g128(const float* w, uint8_t* qw, uint16_t* scale, uint16_t* zero, size_t n,
                            size_t k);
void oracle_dequantize_q4g128(const uint8_t* qw, const uint16_t* scale, const uint16_t* zero,
                              float* w, size_t n, size_t k);
void oracle_qgemm_q4g128_bf16(const uint16_t* x_bf16, const uint8_t* qw, const uint16_t* scale,
                              const uint16_t* zero, uint16_t* y_bf16, size_t b, size_t n,
                              size_t k);

void oracle_qgemm_q4g128_f32(const uint16_t* x_bf16, const uint8_t* qw, const uint16_t* scale,
                             const uint16_t* zero, float* y_f32, size_t b, size_t n, size_t k);

/* ---- ragged packing / paged KV */
int oracle_pack_ragged(const int32_t* new_tokens, const int32_t* prior_ctx,
                       const int32_t* block_tables, int32_t* cu_seqlens, int64_t* slot_mapping,
                       int32_t* context_lens, size_t num_seqs, size_t block_size,
                       size_t max_blocks);
void oracle_kv_write_fp16(const uint16_t* k_new, const uint16_t* v_new, uint16_t* k_pool,
                          uint16_t* v_pool, const int64_t* slot_mapping, size_t total_tokens,
                          size_t row_elems);
void oracle_paged_gather_fp16(const uint16_t* pool, const int32_t* block_table_row, size_t ctx,
                              size_t block_size, size_t row_elems, uint16_t* out);
void oracle_paged_attn_varlen_fp16(const uint16_t* q, const uint16_t* k_pool,
                                   const uint16_t* v_pool, const int32_t* block_tables,
                                   const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                   uint16_t* out, size_t num_seqs, size_t num_q_heads,
                                   size_t num_kv_heads, size_t head_dim, size_t block_size,
                                   size_t max_blocks_per_seq, float scale, int causal);

void oracle_paged_attn_varlen_fp16_f32out(const uint16_t* q, const uint16_t* k_pool,
                                          const uint16_t* v_pool, const int32_t* block_tables,
                                          const int32_t* cu_seqlens_q,
                                          const int32_t* context_lens, float* out,
                                          size_t num_seqs, size_t num_q_heads,
                                          size_t num_kv_heads, size_t head_dim, size_t block_size,
                                          size_t max_blocks_per_seq, float scale, int causal);

/* ---- TurboQuant 3-bit KV codec (crates/quant/src/lib.rs) and attention over turbo3 pools */
void oracle_turbo3_codebook(float* out8);
void oracle_fwht_128(float* data);
int oracle_pack_turbo3_indices(const uint8_t* idx32, uint8_t* packed12);
void oracle_unpack_turbo3_indices(const uint8_t* packed12, uint8_t* idx32);
void oracle_encode_turbo3_0_head(const float* values128, uint8_t* out56);
void oracle_decode_turbo3_0_head(const uint8_t* in56, float* values128);
void oracle_kv_write_turbo3(const uint16_t* k_new, const uint16_t* v_new, uint8_t* k_pool,
                            uint8_t* v_pool, const int64_t* slot_mapping, size_t total_tokens,
                            size_t num_kv_heads);
void oracle_paged_gather_turbo3(const uint8_t* pool, const int32_t* block_table_row, size_t ctx,
                                size_t block_size, size_t num_kv_heads, float* out);
void oracle_paged_attn_varlen_turbo3(const uint16_t* q, const uint8_t* k_pool,
                                     const uint8_t* v_pool, const int32_t* block_tables,
                                     const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                     uint16_t* out, size_t num_seqs, size_t num_q_heads,
                                     size_t num_kv_heads, size_t block_size,
                                     size_t max_blocks_per_seq, float scale, int causal);
void oracle_paged_attn_varlen_turbo3_f32out(const uint16_t* q, const uint8_t* k_pool,
                                     const uint8_t* v_pool, const int32_t* block_tables,
                                     const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                     float* out, size_t num_seqs, size_t num_q_heads,
                                     size_t num_kv_heads, size_t block_size,
                                     size_t max_blocks_per_seq, float scale, int causal);

/* ---- parity metric of the reference's GPU tests (crates/kernels/tests/matmul_parity.rs:83-99) */
void oracle_parity_metric_f32(const float* got, const float* want, size_t n, float* max_abs,
                              float* max_rel);

/* threads the OpenMP loops will use (for the cpu_baseline report) */
int oracle_num_threads(void);
void oracle_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
