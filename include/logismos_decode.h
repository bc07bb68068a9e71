/*
 * logismos_decode.h -- C ABI of the MI355X (gfx950) ragged-batch decode path.
 *
 * Every launcher follows the convention of the reference's HIP launchers
 * (crates/kernels/src/matmul/hip/matmul_launchers.cpp:14-52,
 *  crates/kernels/src/rms_norm/hip/rms_norm.hip:58-84,
 *  crates/kernels/src/rope/hip/rope.hip:45-68):
 *
 *   - `extern "C"`, plain pointers and `int` dims, scalars by value, the
 *     stream last;
 *   - all pointers are caller-owned DEVICE memory, valid for the launch;
 *     outputs never alias inputs; the launcher allocates and frees nothing;
 *   - the launch is asynchronous on `stream`; nothing synchronises inside;
 *   - the return value is the raw HIP status (`hipError_t` as uint32_t,
 *     0 = success), the value the reference's Rust wrapper feeds to
 *     `hipcore::ErrorKind::from_raw` (crates/hipcore/src/error.rs:125-150,
 *     crates/kernels/src/matmul/mod.rs:140-186).  A shape the kernels cannot
 *     address is rejected on the host before any launch with
 *     hipErrorInvalidValue (1); nothing ever aborts;
 *   - index arithmetic inside the kernels is 64-bit
 *     (crates/kernels/src/matmul/hip/matmul_naive.hip:26-41).
 *
 * The library is re-entrant across streams (the reference's `Stream` is Send
 * but not Sync, crates/hipcore/src/stream.rs:21-25: one caller thread per
 * stream): no launch changes library state.  What it keeps are values computed
 * once per process and the same from whichever thread computes them first (the
 * device's CU count, kernel attribute opt-ins, the address of the static
 * workspace of the `_noalloc` entry point), for the device that is current at
 * that moment: one device per process.
 *
 * The reference defines none of the data contracts below (its `sched`,
 * paged `cache` and weight-`quant` crates are scaffolds); they extend the
 * conventions it does define, cited at each item.
 */
#ifndef LOGISMOS_DECODE_H
#define LOGISMOS_DECODE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Opaque stream handle: a `hipStream_t` (what `hipcore::Stream::raw()`
 * yields, crates/hipcore/src/stream.rs).  NULL is the default stream. */
typedef void* logismos_stream_t;

/* Raw HIP status code. */
typedef uint32_t logismos_status_t;

/* ------------------------------------------------------------------------
 * Data contracts
 * ------------------------------------------------------------------------
 *
 * Paged KV pool.  K and V live in separate pools (the reference keeps K and
 * V in separate per-layer buffers, crates/cache/src/flat.rs:84-89).  A pool
 * is `[num_blocks][block_size][num_kv_heads][head_dim]` fp16, little-endian;
 * one token row is `[num_kv_heads][head_dim]` contiguous, exactly a
 * `FlatKvCache` row (`CacheLayout::row_elems`, crates/cache/src/flat.rs:36-69),
 * and a block is `block_size` consecutive such rows.
 *
 * Block table.  int32, row-major `[num_seqs][max_blocks_per_seq]`; entry j of
 * row s is the physical block that holds tokens [j*block_size,(j+1)*block_size)
 * of sequence s.  Entries past ceil(context_len/block_size) are never read.
 *
 * Slot.  `slot = block_table[s][pos / block_size] * block_size + pos % block_size`
 * (int64): the row index of token `pos` of sequence s inside a pool viewed as
 * `[num_blocks*block_size][num_kv_heads*head_dim]`.
 *
 * cu_seqlens.  int32 exclusive prefix sum over the per-sequence number of NEW
 * (query) tokens, leading 0, length num_seqs+1
 * (research/14-gdn-aiter-preflight.md:338 is the only place the reference
 * shows one: `[0,512,1536,2048]`).
 *
 * context_lens.  int32 `[num_seqs]`: tokens of the sequence visible to its
 * LAST query token = prior context + new tokens.
 *
 * GQA.  Query head h reads KV head h / (num_q_heads / num_kv_heads)
 * (`repeat_kv`, crates/transformers/src/attention.rs:366-382).
 *
 * Q8G32 weights (8-bit symmetric, group 32 along K; value-identical to ggml
 * Q8_0, type id 8 in crates/loader/src/gguf.rs:57-78).  Device layout is
 * planar: `qs` int8 `[N][K]` row-major and `d` fp16 `[N][K/32]`;
 * w[n][k] = f16_to_f32(d[n][k/32]) * qs[n][k].
 * `logismos_launch_repack_q8_0` converts ggml's 34-byte
 * `{f16 d; int8 qs[32]}` blocks into it.
 *
 * Q4G32 weights (4-bit, group 32 along K: the arithmetic of ggml Q4_1, type id
 * 3, and of Q4_0, id 2, in crates/loader/src/gguf.rs:57-78).  Planar: `qw`
 * uint8 `[N][K/2]`, element k in the low (k even) or high (k odd) nibble of
 * byte k/2 (the nibble order of `pack_turbo4_indices`,
 * crates/quant/src/lib.rs:272-285); `scale` fp16 `[N][K/32]`, `min` fp16
 * `[N][K/32]`; w[n][k] = q * scale + min.  `logismos_launch_repack_q4_1`
 * converts ggml's 20-byte `{f16 d; f16 m; u8 qs[16]}` blocks (scale = d,
 * min = m) and `logismos_launch_repack_q4_0` its 18-byte `{f16 d; u8 qs[16]}`
 * blocks (scale = d, min = -8 d, so that q*d + min = (q - 8)*d); ggml keeps
 * value j in the low and value j + 16 in the high nibble of byte j.
 *
 * Q4G128 weights (4-bit asymmetric, group 128 along K).  `qw` uint8
 * `[N][K/2]`, element 2j in the low nibble of byte j and 2j+1 in the high
 * nibble (index i at bit 4*i of a little-endian integer, the reference's
 * only nibble convention: `pack_turbo4_indices`,
 * crates/quant/src/lib.rs:272-285); `scale` fp16 `[N][K/128]`, `zero` fp16
 * `[N][K/128]`; w[n][k] = (q - zero) * scale, q in [0,15].
 */

#define LOGISMOS_Q8_GROUP 32
#define LOGISMOS_Q4_GROUP 128
#define LOGISMOS_Q8_0_BLOCK_BYTES 34

/* ------------------------------------------------------------------------
 * Library identity / host-side shape guards (no device access; safe to call
 * without a GPU).  The guards are the C counterpart of the reference's
 * `check_matmul_shape` / `check_rope_shape` (crates/kernels/src/matmul/mod.rs:89-121,
 * crates/kernels/src/rope/mod.rs:79-140): positive dims and every
 * element-index product <= INT32_MAX.  They return 0 when the shape is
 * accepted and hipErrorInvalidValue (1) otherwise; when `msg` is non-NULL a
 * NUL-terminated reason is written into it (at most `msg_cap` bytes).
 * ------------------------------------------------------------------------ */

/* ABI version of this header; bumped on any signature change. */
int logismos_decode_abi_version(void);

/* The gfx target the kernels in this library were compiled for ("gfx950"). */
const char* logismos_decode_offload_arch(void);

logismos_status_t logismos_check_qgemv_q8g32_shape(int n, int k, char* msg, size_t msg_cap);

logismos_status_t logismos_check_paged_attn_shape(int num_seqs, int total_tokens, int max_seqlen_q,
                                                  int num_q_heads, int num_kv_heads, int head_dim,
                                                  int block_size, int max_blocks_per_seq,
                                                  int num_splits, char* msg, size_t msg_cap);

/* ------------------------------------------------------------------------
 * Quantized row-GEMV / GEMM
 * ------------------------------------------------------------------------ */

/* y[n] = sum_k x[k] * w[n][k], w in planar Q8G32.  x f32[K], y f32[N], fp32
 * accumulation.  The quantized counterpart of `cpu_f32::linear_t` at m = 1
 * (crates/kernels/src/cpu_f32/mod.rs:271-345: weight is `[out,in]`
 * row-major).  Requires k % 32 == 0.  qs must be 16-byte aligned. */
logismos_status_t logismos_launch_qgemv_q8g32_f32(const void* x_f32, const void* qs_i8,
                                                  const void* d_f16, void* y_f32, int n, int k,
                                                  logismos_stream_t stream);
/* ... `+ bias[n]` (fp32 `[N]`, NULL: none), added to the finished fp32 sum as
 * `linear_t` adds it (crates/kernels/src/cpu_f32/mod.rs:336-343; the q/k/v
 * projections of Qwen2 carry one, crates/transformers/src/attention.rs:49-57). */
logismos_status_t logismos_launch_qgemv_q8g32_f32_bias(const void* x_f32, const void* qs_i8,
                                                       const void* d_f16, const void* bias_f32,
                                                       void* y_f32, int n, int k,
                                                       logismos_stream_t stream);

/* y[b][n] = sum_k x[b][k] * w[n][k], w in Q4G128.  x bf16 `[B][K]`, y bf16
 * `[B][N]`, fp32 accumulation, one rounding at the end: `cpu_f32::linear_t`
 * (crates/kernels/src/cpu_f32/mod.rs:271-345) over the dequantised matrix with
 * m = B.  Batch 1..2 runs the bandwidth-bound VALU GEMV (in-register nibble
 * unpack, v_dot2), batch >= 3 the MFMA kernels (measured crossover on MI355X);
 * more than 32 rows (the prefill chunks of a mixed batch) are taken 32 at a
 * time, each pass streaming the weights once.  Requires k % 128 == 0; x and qw
 * 16-byte aligned. */
logismos_status_t logismos_check_qgemm_q4g128_shape(int b, int n, int k, char* msg, size_t msg_cap);
logismos_status_t logismos_launch_qgemm_q4g128_bf16(const void* x_bf16, const void* qw_u8,
                                                    const void* scale_f16, const void* zero_f16,
                                                    void* y_bf16, int b, int n, int k,
                                                    logismos_stream_t stream);
/* ... `+ bias[n]` (fp32 `[N]`, NULL: none) on the fp32 sum before the one
 * rounding to bf16 (`linear_t`'s bias, crates/kernels/src/cpu_f32/mod.rs:336-343). */
logismos_status_t logismos_launch_qgemm_q4g128_bf16_bias(const void* x_bf16, const void* qw_u8,
                                                         const void* scale_f16,
                                                         const void* zero_f16,
                                                         const void* bias_f32, void* y_bf16, int b,
                                                         int n, int k, logismos_stream_t stream);

/* The same product forced onto the MFMA kernel for any batch 1..32 (the default
 * launcher uses it from batch 3): lets a caller or a benchmark compare the two
 * paths on identical inputs. */
logismos_status_t logismos_launch_qgemm_q4g128_bf16_mfma(const void* x_bf16, const void* qw_u8,
                                                         const void* scale_f16,
                                                         const void* zero_f16, void* y_bf16, int b,
                                                         int n, int k, logismos_stream_t stream);

/* `linear_t` over many rows of x (the prefill chunks of a mixed batch: hundreds to thousands
 * of rows, crates/transformers/src/mlp.rs:104-111) with a workspace: a first pass copies x
 * into the element order the kernel's nibble unpack produces and takes every row's sum over
 * each group of 128 columns, the tiled matrix-core kernel then moves that copy straight into
 * LDS and takes the zero-point term as a small product of its own.  Any m >= 1 (built for
 * m >= ~100), K a multiple of 256, y bf16 `[m][N]` or, with y_is_f32, fp32 (what the step
 * executor keeps between operators); bias fp32 `[N]` or NULL.  The workspace
 * (`..._workspace_bytes(m, k)`, 16-byte aligned, caller-owned: the copy of x, its group sums
 * and 64 MiB for fp32 partial tiles -- the tiles of a last, partial round of workgroups are
 * split over K and summed by a small kernel) is scratch: nothing in it matters before or
 * after the call.  Scales and zeros 16-byte aligned with K a multiple of 1024 take the
 * fastest path (8-byte aligned and a multiple of 512 the next).  The entry points above
 * serve the same product without a workspace (slower from about a hundred rows on). */
logismos_status_t logismos_check_qgemm_q4g128_tall_shape(int m, int n, int k, char* msg,
                                                         size_t msg_cap);
size_t logismos_qgemm_q4g128_tall_workspace_bytes(int m, int k);
/* The two halves of the launch below for a caller whose producer writes x where the kernel
 * wants it: `..._tall_prepared` is the product alone over a workspace that already holds x in
 * the kernel's operand order with its group sums (the first `m_pad*K*2` bytes and the sums
 * behind them, as `logismos_launch_silu_mul_f32p_tall` and
 * `logismos_launch_add_rms_norm_f32p_tall` write them), `..._pairs_per_load` the
 * one parameter of that layout that depends on the weights (how many pairs of groups of K the
 * kernel loads scales and zeros for at once: 4, 2 or 1 by K and their alignment).  No
 * counterpart in the reference: `linear_t` takes plain rows. */
int logismos_qgemm_q4g128_tall_pairs_per_load(int k, const void* scale_f16, const void* zero_f16);
logismos_status_t logismos_launch_qgemm_q4g128_tall_prepared(
    const void* qw_u8, const void* scale_f16, const void* zero_f16, const void* bias_f32, void* y,
    int y_is_f32, void* workspace, int m, int n, int k, logismos_stream_t stream);
/* The gate/up projection of a SwiGLU MLP with the activation applied where the products are
 * summed (crates/transformers/src/mlp.rs:104-111: down(silu(gate(x)) * up(x))): weights
 * `[2*inter][K]`, gate rows first; `act_bf16 [m][inter] = bf16(silu(x.gate^T) * (x.up^T))`, the
 * fp32 products rounded once, as `logismos_launch_silu_mul_f32p` rounds them.  Over a prepared
 * workspace like `..._tall_prepared`. */
logismos_status_t logismos_launch_qgemm_q4g128_tall_swiglu_prepared(
    const void* gate_up_qw_u8, const void* scale_f16, const void* zero_f16, void* act_bf16,
    void* workspace, int m, int inter, int k, logismos_stream_t stream);
/* The same, with the activations written as the operand of the product that follows (the
 * down projection, K = inter): `next_workspace` is that product's workspace
 * (`logismos_qgemm_q4g128_tall_workspace_bytes(m, inter)` bytes, not the one this launch
 * reads), and receives what `logismos_launch_silu_mul_f32p_tall` would write there from the
 * fp32 gate/up products, bit for bit -- the bf16 activations in the kernel's operand order,
 * zero rows up to the padded row count, and the group sums in the layout for
 * `next_pairs_per_load` (`..._pairs_per_load` of the following product's K and weights).
 * inter a multiple of 256 * next_pairs_per_load. */
logismos_status_t logismos_launch_qgemm_q4g128_tall_swiglu_operand(
    const void* gate_up_qw_u8, const void* scale_f16, const void* zero_f16, void* next_workspace,
    int next_pairs_per_load, void* workspace, int m, int inter, int k, logismos_stream_t stream);
logismos_status_t logismos_launch_qgemm_q4g128_tall(const void* x_bf16, const void* qw_u8,
                                                    const void* scale_f16, const void* zero_f16,
                                                    const void* bias_f32, void* y, int y_is_f32,
                                                    void* workspace, int m, int n, int k,
                                                    logismos_stream_t stream);

/* Split-K form for a decode batch (b <= 32): fp32 partial products
 *   parts[j][b][n] = sum over K part j of x[b][k] * w[n][k],  j < J,
 * whose sum over j is the product.  Workgroups are tall (up to 256 weight rows
 * by a short K part) so that the x each one needs is small next to its weights;
 * the J parts are added by the consumer (the `_f32p` operators below), which
 * keeps the result deterministic and un-rounded.  J depends on (b, n, k) only:
 * `logismos_qgemm_q4g128_splitk_parts` returns it (0 for a rejected shape);
 * `parts_f32` needs J*b*n*4 bytes. */
int logismos_qgemm_q4g128_splitk_parts(int b, int n, int k);
logismos_status_t logismos_launch_qgemm_q4g128_f32_splitk(const void* x_bf16, const void* qw_u8,
                                                          const void* scale_f16,
                                                          const void* zero_f16, void* parts_f32,
                                                          int b, int n, int k,
                                                          logismos_stream_t stream);

/* Prepared activations.  The MFMA kernels want x in "pair order" with per-group
 * sums; a producer that writes x in that form once saves every GEMM workgroup
 * from rebuilding it.  Layout (b <= 32 rows, BP = 16 for b <= 16 else 32):
 *   uint4 xp[K/8][BP]    8 consecutive bf16 x0..x7 of row r, chunk c, stored as
 *                        the pairs (x0,x4) (x1,x5) (x2,x6) (x3,x7)
 *   float xg[K/128][BP]  sum of the bf16 values of each group of 128, after xp.
 * `logismos_q4_xprep_bytes` sizes the buffer, `logismos_launch_q4_prepare_x_bf16`
 * converts a plain bf16 `[b][K]` matrix, `..._splitk_xprep` consumes it.  The
 * step operators below can emit it directly (`out_prepared != 0`).  With x
 * prepared, other kernels become possible (x held in registers, a workgroup
 * covering 2048 or 4096 columns of K), so the number of parts of this entry
 * point is its own: `logismos_qgemm_q4g128_splitk_xprep_parts`. */
size_t logismos_q4_xprep_bytes(int b, int k);
int logismos_qgemm_q4g128_splitk_xprep_parts(int b, int n, int k);
logismos_status_t logismos_launch_q4_prepare_x_bf16(const void* x_bf16, void* x_prepared, int b,
                                                    int k, logismos_stream_t stream);
logismos_status_t logismos_launch_qgemm_q4g128_f32_splitk_xprep(
    const void* x_prepared, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* parts_f32, int b, int n, int k, logismos_stream_t stream);

/* y[n] = sum_k x[k] * (q[n][k] * scale[n][k/32] + min[n][k/32]): `linear_t` at m = 1
 * (crates/kernels/src/cpu_f32/mod.rs:271-345) over Q4G32 weights; x, y fp32;
 * K % 32 == 0, N*K <= i32::MAX; qw and x 16-byte aligned. */
logismos_status_t logismos_check_qgemv_q4g32_shape(int n, int k, char* msg, size_t msg_cap);
logismos_status_t logismos_launch_qgemv_q4g32_f32(const void* x_f32, const void* qw_u8,
                                                  const void* scale_f16, const void* min_f16,
                                                  void* y_f32, int n, int k,
                                                  logismos_stream_t stream);
logismos_status_t logismos_launch_qgemv_q4g32_f32_bias(const void* x_f32, const void* qw_u8,
                                                       const void* scale_f16, const void* min_f16,
                                                       const void* bias_f32, void* y_f32, int n,
                                                       int k, logismos_stream_t stream);

/* y[b][n] = bf16(sum_k x[b][k] * (q[n][k] * scale[n][k/32] + min[n][k/32])): `linear_t` at
 * m = batch (crates/kernels/src/cpu_f32/mod.rs:271-345) over the same Q4G32 weights, x and y
 * bf16 like those of the Q4G128 GEMM, fp32 accumulation on the matrix cores.  More than 32
 * rows are taken 32 at a time.  K % 128 == 0, N*K <= i32::MAX; qw and x 16-byte aligned, scale and min 8-byte aligned. */
logismos_status_t logismos_check_qgemm_q4g32_shape(int b, int n, int k, char* msg, size_t msg_cap);
logismos_status_t logismos_launch_qgemm_q4g32_bf16(const void* x_bf16, const void* qw_u8,
                                                   const void* scale_f16, const void* min_f16,
                                                   void* y_bf16, int b, int n, int k,
                                                   logismos_stream_t stream);
logismos_status_t logismos_launch_qgemm_q4g32_bf16_bias(const void* x_bf16, const void* qw_u8,
                                                        const void* scale_f16, const void* min_f16,
                                                        const void* bias_f32, void* y_bf16, int b,
                                                        int n, int k, logismos_stream_t stream);

/* ggml Q4_0 / Q4_1 block streams `[N][K/32]` (the tensors the loader rejects today,
 * crates/loader/src/gguf.rs:127-145,397-406) -> planar Q4G32.  blocks 2-byte aligned. */
logismos_status_t logismos_launch_repack_q4_0(const void* blocks_q4_0, void* qw_u8,
                                              void* scale_f16, void* min_f16, int n, int k,
                                              logismos_stream_t stream);
logismos_status_t logismos_launch_repack_q4_1(const void* blocks_q4_1, void* qw_u8,
                                              void* scale_f16, void* min_f16, int n, int k,
                                              logismos_stream_t stream);

/* ggml Q8_0 block stream `[N][K/32]{f16 d; int8 qs[32]}` -> planar Q8G32. */
logismos_status_t logismos_launch_repack_q8_0(const void* blocks_q8_0, void* qs_i8, void* d_f16,
                                              int n, int k, logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * Paged attention (ragged batch: decode rows and chunked-prefill rows)
 * ------------------------------------------------------------------------ */

/* Number of KV partitions ("splits") the decode kernel should use for this
 * problem size; pure host arithmetic, deterministic.  Pass the result both to
 * the workspace query and to the launcher. */
int logismos_paged_attn_num_splits(int num_seqs, int num_kv_heads, int block_size,
                                   int max_blocks_per_seq);

/* The same for a given head width.  head_dim 128: what the function above returns.  Other
 * widths (multiples of 32 up to 256, `crates/transformers/src/attention.rs:97-127` is
 * generic in head_dim) run on a general kernel with a static split, whose partition count
 * this sizes for its workgroups (one per partition and group of up to 8 KV heads). */
int logismos_paged_attn_num_splits_hd(int num_seqs, int num_kv_heads, int head_dim,
                                      int block_size, int max_blocks_per_seq);

/* Bytes of split-K workspace the launcher needs for these arguments. */
size_t logismos_paged_attn_workspace_bytes(int num_seqs, int num_q_heads, int head_dim,
                                           int num_splits);

/* out[t][h][:] = softmax_j( (q[t][h] . k[j][h/g]) * scale ) . v[j][h/g]
 * over the keys j visible to query token t.
 *
 *   q, out          fp16 `[total_tokens][num_q_heads][head_dim]`
 *   k_pool, v_pool  paged pools as described above
 *   block_tables    int32 `[num_seqs][max_blocks_per_seq]`
 *   cu_seqlens_q    int32 `[num_seqs+1]`; sequence s owns query tokens
 *                   [cu[s], cu[s+1])
 *   context_lens    int32 `[num_seqs]`
 *   total_tokens    cu_seqlens_q[num_seqs]; max_seqlen_q: the largest number of
 *                   new tokens of any sequence (both known to the host-side
 *                   scheduler; 1 for a pure decode step)
 *   num_splits      partial results the workspace can hold per decode sequence
 *                   (>= 1), e.g. from `logismos_paged_attn_num_splits`.  1: every
 *                   sequence is one partition.  Small batches: each context is
 *                   cut into num_splits static partitions.  Otherwise the key
 *                   tiles of all decode sequences are split evenly over one
 *                   worker per CU (at most num_seqs*(num_splits-1) workers), so
 *                   the work per CU does not depend on how the context lengths
 *                   are distributed; the result does not depend on num_splits
 *                   beyond fp32 summation order
 *   workspace       `logismos_paged_attn_workspace_bytes(...)` bytes, contents
 *                   don't matter on entry; must not be shared by launches that
 *                   can overlap in time
 *   causal != 0     query token i (0-based) of a sequence with n new tokens
 *                   and context c sees keys [0, c - n + i]; causal == 0: all c
 *                   keys.  For n == 1 both coincide.
 *
 * The scale multiplies the dot product (it is not folded into q), as in
 * `QwenAttention::forward` (crates/transformers/src/attention.rs:225-241);
 * the softmax is fp32 and max-subtracted
 * (`softmax_last_dim`, crates/kernels/src/cpu_f32/mod.rs:380-433); a query
 * with no visible key yields zeros.  `scale` must be finite and > 0 (else
 * hipErrorInvalidValue).  Requires block_size % 16 == 0,
 * num_q_heads % num_kv_heads == 0 and head_dim == 128 with a group size
 * num_q_heads/num_kv_heads <= 8 (the kernels the decode step of the headline
 * configuration runs on), or any other head_dim that is a multiple of 32 up to
 * 256 with a group size <= 16 and total_tokens <= 65520 (a general kernel:
 * decode rows on a static split, every row of a chunk over its whole visible
 * context; `QwenAttention` is generic in head_dim,
 * crates/transformers/src/attention.rs:97-127). */
logismos_status_t logismos_launch_paged_attn_varlen_fp16(
    const void* q_f16, const void* k_pool_f16, const void* v_pool_f16, const int32_t* block_tables,
    const int32_t* cu_seqlens_q, const int32_t* context_lens, void* out_f16, void* workspace,
    int num_seqs, int total_tokens, int max_seqlen_q, int num_q_heads, int num_kv_heads,
    int head_dim, int block_size, int max_blocks_per_seq, int num_splits, float scale, int causal,
    logismos_stream_t stream);

/* The same launch restricted to some of its phases (bitmask).  The full
 * launcher runs, in order: the decode kernel (sequences with one new token,
 * KV partitions in parallel), the prefill kernel (sequences with more than one
 * new token; skipped when max_seqlen_q <= 1) and the merge of the decode
 * partitions (skipped when num_splits == 1).  For callers that place the
 * phases on different streams, and for per-kernel timing. */
#define LOGISMOS_ATTN_PHASE_DECODE 1
#define LOGISMOS_ATTN_PHASE_PREFILL 2
#define LOGISMOS_ATTN_PHASE_MERGE 4
#define LOGISMOS_ATTN_PHASE_ALL 7
logismos_status_t logismos_launch_paged_attn_varlen_fp16_phases(
    const void* q_f16, const void* k_pool_f16, const void* v_pool_f16, const int32_t* block_tables,
    const int32_t* cu_seqlens_q, const int32_t* context_lens, void* out_f16, void* workspace,
    int num_seqs, int total_tokens, int max_seqlen_q, int num_q_heads, int num_kv_heads,
    int head_dim, int block_size, int max_blocks_per_seq, int num_splits, float scale, int causal,
    int phases, logismos_stream_t stream);

/* The full launch above without a workspace argument and without any allocation.
 * No counterpart in the reference: it is for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * it).  The split-K partials go to a static device array of
 * LOGISMOS_PAGED_ATTN_STATIC_WORKSPACE_BYTES bytes that every device the library
 * runs on holds until the process ends; a launch whose
 * `logismos_paged_attn_workspace_bytes(...)` exceeds it is refused with
 * hipErrorInvalidValue (choose a smaller num_splits).  All calls on a device share
 * that device's array: launches that can overlap in time (two streams, two
 * threads) race on it and must be ordered by the caller.  The array needs no
 * clearing between calls (its contents never matter on entry).  Results are
 * identical to `logismos_launch_paged_attn_varlen_fp16` with the same arguments.
 * `logismos_paged_attn_noalloc_init()`: call it once per device at set-up, with that
 * device current and outside any region that must not allocate: it resolves the
 * array's device address (the look-up makes the runtime load the library's code
 * object and place the array) and the device's CU count.  Without it the first
 * launch on a device does that work itself, and only the later ones allocate
 * nothing. */
#define LOGISMOS_PAGED_ATTN_STATIC_WORKSPACE_BYTES (16u << 20)
size_t logismos_paged_attn_static_workspace_bytes(void);
logismos_status_t logismos_paged_attn_noalloc_init(void);
logismos_status_t logismos_launch_paged_attn_varlen_fp16_noalloc(
    const void* q_f16, const void* k_pool_f16, const void* v_pool_f16, const int32_t* block_tables,
    const int32_t* cu_seqlens_q, const int32_t* context_lens, void* out_f16, int num_seqs,
    int total_tokens, int max_seqlen_q, int num_q_heads, int num_kv_heads, int head_dim,
    int block_size, int max_blocks_per_seq, int num_splits, float scale, int causal,
    logismos_stream_t stream);

/* Decode rows only (one new token per sequence: total_tokens == num_seqs,
 * cu_seqlens_q = 0,1,2,...), the bf16-rounded result written in the prepared
 * layout of a following Q4G128 GEMM over K = num_q_heads*head_dim
 * (`logismos_q4_xprep_bytes(num_seqs, num_q_heads*head_dim)` bytes; rows
 * num_seqs..BP-1 of the layout are left as they are): what the step executor
 * launches in front of its o projection (`merge_heads` then `wo`,
 * crates/transformers/src/attention.rs:296-302).  num_seqs <= 32, head_dim 128 (a group
 * of 128 of the layout is one head). */
logismos_status_t logismos_launch_paged_attn_decode_fp16_xprep(
    const void* q_f16, const void* k_pool_f16, const void* v_pool_f16, const int32_t* block_tables,
    const int32_t* cu_seqlens_q, const int32_t* context_lens, void* out_prepared, void* workspace,
    int num_seqs, int num_q_heads, int num_kv_heads, int head_dim, int block_size,
    int max_blocks_per_seq, int num_splits, float scale, logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * Ragged packing and KV writes
 * ------------------------------------------------------------------------ */

/* From per-sequence counts to the packed-batch index buffers, on the GPU:
 *   cu_seqlens[0] = 0, cu_seqlens[s+1] = cu_seqlens[s] + new_tokens[s]
 *   context_lens[s] = min(prior_ctx[s] + new_tokens[s], block_size * max_blocks)
 *   slot_mapping[cu_seqlens[s] + i] = slot of position prior_ctx[s] + i of sequence s, or
 *                                     -1 when that position lies past max_blocks or its
 *                                     table entry names no block (negative, or
 *                                     >= LOGISMOS_BLOCK_ID_LIMIT: the mark of an entry
 *                                     that never had one)
 * new_tokens, prior_ctx int32 `[num_seqs]` (negative values count as 0);
 * slot_mapping int64 `[sum new_tokens]`.  The host never needs the total.
 * A sequence that outgrows its table row is the reference cache's
 * `Error::LenOverflow` (crates/cache/src/flat.rs:180-255); a kernel cannot
 * refuse, so the rows past the capacity get slot -1 (every writer skips them)
 * and the context stops at the capacity (the attention never walks past the
 * row); the scheduler is expected to have checked the length on the host. */
#define LOGISMOS_BLOCK_ID_LIMIT 0x3FFFFFF
logismos_status_t logismos_check_pack_ragged_shape(int num_seqs, int block_size, int max_blocks,
                                                   char* msg, size_t msg_cap);
logismos_status_t logismos_launch_pack_ragged(const int32_t* new_tokens, const int32_t* prior_ctx,
                                              const int32_t* block_tables, int32_t* cu_seqlens,
                                              int64_t* slot_mapping, int32_t* context_lens,
                                              int num_seqs, int block_size, int max_blocks,
                                              logismos_stream_t stream);

/* Row t of k_new / v_new (fp16 `[total_tokens][num_kv_heads*head_dim]`, the rows
 * `KvCache::put` takes, crates/cache/src/lib.rs:57-64) is written to pool row
 * slot_mapping[t]; negative slots are skipped.  num_kv_heads*head_dim % 8 == 0. */
logismos_status_t logismos_launch_kv_write_fp16(const void* k_new_f16, const void* v_new_f16,
                                                void* k_pool_f16, void* v_pool_f16,
                                                const int64_t* slot_mapping, int total_tokens,
                                                int num_kv_heads, int head_dim,
                                                logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * Small operators of the decode step (gfx950 versions of the reference's
 * cpu_f32 contracts, crates/kernels/src/cpu_f32/mod.rs)
 * ------------------------------------------------------------------------ */

/* h[r][:] += y[r][:] (skipped when y_bf16 == NULL), then
 * out[r][:] = bf16( h * (1/sqrt(mean(h^2)+eps)) * w ): the pre-norm residual
 * step of a layer (crates/encoders/src/stella.rs:190-206) over `rms_norm`
 * (crates/kernels/src/cpu_f32/mod.rs:137-159).  h fp32 `[rows][n]` in place,
 * w fp32 `[n]`. */
logismos_status_t logismos_launch_add_rms_norm_bf16(void* h_f32, const void* y_bf16,
                                                    const void* w_f32, void* out_bf16, int rows,
                                                    int n, float eps, logismos_stream_t stream);

/* Splits qkv (bf16 `[T][(hq+2*hkv)*128]`, q heads, then k heads, then v heads),
 * applies RoPE in the halves convention (`rope_halves_in_place`,
 * crates/kernels/src/cpu_f32/mod.rs:502-547) to q and k with the token's
 * position, and writes q as fp16 `[T][hq][head_dim]`, k and
 * v as fp16 rows of the paged pools at slot_mapping[t] (negative: skipped).
 * cos / sin: fp32 `[max_pos][head_dim/2]` (`build_rope_table_f32`, :599-619);
 * head_dim even, at most 1024 (the turbo3 forms below: 128).  The caller
 * guarantees 0 <= positions[t] < max_pos (`RopeTable::gather` fails on a position past the
 * table); the kernel only keeps an out-of-range position from reading outside the tables
 * (it uses the nearest table row) and the result for such a token is unspecified. */
logismos_status_t logismos_launch_rope_kv_write_fp16(
    const void* qkv_bf16, const int32_t* positions, const void* cos_f32, const void* sin_f32,
    const int64_t* slot_mapping, void* q_out_f16, void* k_pool_f16, void* v_pool_f16,
    int total_tokens, int num_q_heads, int num_kv_heads, int head_dim, int max_pos,
    logismos_stream_t stream);

/* out[t][j] = bf16( silu(gate) * up ), gate_up bf16 `[rows][2*inter]` = gate | up
 * (`SwiGluMlp::forward`, crates/transformers/src/mlp.rs:82-125; `silu`,
 * `hadamard`, crates/kernels/src/cpu_f32/mod.rs:349-374). */
logismos_status_t logismos_launch_silu_mul_bf16(const void* gate_up_bf16, void* out_bf16, int rows,
                                                int inter, logismos_stream_t stream);

logismos_status_t logismos_launch_cast_f16_bf16(const void* in_f16, void* out_bf16, size_t count,
                                                logismos_stream_t stream);

/* The same three operators reading the fp32 split-K parts of the preceding GEMM
 * (`parts[j]` is a whole `[rows][width]` matrix; the operator adds the
 * num_parts of them in order, without intermediate rounding). */
logismos_status_t logismos_launch_add_rms_norm_f32p(void* h_f32, const void* parts_f32,
                                                    int num_parts, const void* w_f32,
                                                    void* out_bf16, int rows, int n, float eps,
                                                    logismos_stream_t stream);
logismos_status_t logismos_launch_rope_kv_write_f32p(
    const void* qkv_parts_f32, int num_parts, const int32_t* positions, const void* cos_f32,
    const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16, void* k_pool_f16,
    void* v_pool_f16, int total_tokens, int num_q_heads, int num_kv_heads, int head_dim,
    int max_pos, logismos_stream_t stream);
/* The same with turbo3 pools (see the TurboQuant section below): the rotated k and the v of
 * every new token are rounded to fp16, as the fp16 pools would hold them, and encoded with
 * `encode_turbo3_0_head` (crates/quant/src/lib.rs:316-353) into the 56-byte head rows at the
 * token's slot. */
logismos_status_t logismos_launch_rope_kv_write_f32p_turbo3(
    const void* qkv_parts_f32, int num_parts, const int32_t* positions, const void* cos_f32,
    const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16, void* k_pool_t3,
    void* v_pool_t3, int total_tokens, int num_q_heads, int num_kv_heads, int head_dim,
    int max_pos, logismos_stream_t stream);
/* The two launchers above with the projection's bias (fp32 `[(hq+2*hkv)*128]`, NULL: none)
 * added to the summed parts before the rotation: `linear_t`'s bias
 * (crates/kernels/src/cpu_f32/mod.rs:336-343) of the q/k/v projections
 * (crates/transformers/src/attention.rs:49-57). */
logismos_status_t logismos_launch_rope_kv_write_f32p_bias(
    const void* qkv_parts_f32, int num_parts, const void* bias_f32, const int32_t* positions,
    const void* cos_f32, const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16,
    void* k_pool_f16, void* v_pool_f16, int total_tokens, int num_q_heads, int num_kv_heads,
    int head_dim, int max_pos, logismos_stream_t stream);
logismos_status_t logismos_launch_rope_kv_write_f32p_turbo3_bias(
    const void* qkv_parts_f32, int num_parts, const void* bias_f32, const int32_t* positions,
    const void* cos_f32, const void* sin_f32, const int64_t* slot_mapping, void* q_out_f16,
    void* k_pool_t3, void* v_pool_t3, int total_tokens, int num_q_heads, int num_kv_heads,
    int head_dim, int max_pos, logismos_stream_t stream);
logismos_status_t logismos_launch_silu_mul_f32p(const void* parts_f32, int num_parts,
                                                void* out_bf16, int rows, int inter,
                                                logismos_stream_t stream);

/* h += sum of the fp32 parts, then the RMS-normed row times its gains written as the operand
 * of the many-row GEMM (see the SwiGLU form below; K = n a multiple of 256 * pairs_per_load,
 * n <= 16384).  The arithmetic is that of `logismos_launch_add_rms_norm_f32p_xprep`. */
logismos_status_t logismos_launch_add_rms_norm_f32p_tall(void* h_f32, const void* parts_f32,
                                                         int num_parts, const void* w_f32,
                                                         void* workspace, int rows, int n,
                                                         float eps, int pairs_per_load,
                                                         logismos_stream_t stream);

/* SwiGLU over the fp32 parts with the result written as the operand of the many-row GEMM
 * (`logismos_launch_qgemm_q4g128_tall_prepared` over the same workspace, K = inter a multiple
 * of 256 * pairs_per_load): x in the kernel's order, rows padded with zeros to its 128-row
 * tiles, the group sums behind it. */
logismos_status_t logismos_launch_silu_mul_f32p_tall(const void* parts_f32, int num_parts,
                                                     void* workspace, int rows, int inter,
                                                     int pairs_per_load,
                                                     logismos_stream_t stream);

/* The same with the result in the prepared layout of the next GEMM (rows <= 32,
 * width % 128 == 0; see `logismos_q4_xprep_bytes`). */
logismos_status_t logismos_launch_add_rms_norm_f32p_xprep(void* h_f32, const void* parts_f32,
                                                          int num_parts, const void* w_f32,
                                                          void* x_prepared, int rows, int n,
                                                          float eps, logismos_stream_t stream);
logismos_status_t logismos_launch_silu_mul_f32p_xprep(const void* parts_f32, int num_parts,
                                                      void* x_prepared, int rows, int inter,
                                                      logismos_stream_t stream);

/* out[r] = first index of the maximum of logits[r][:] (`decode::greedy`,
 * crates/decode/src/lib.rs:73-83: strict >, the first maximum wins). */
logismos_status_t logismos_launch_greedy_f32(const void* logits_f32, void* out_u32, int rows, int n,
                                             logismos_stream_t stream);

/* Vocabulary projection and token selection in one pass: logits = x . W^T over Q4G128
 * weights `[n][k]` (x in the prepared layout, rows = b <= 32, k % 1024 == 0), then
 * out_tokens[r] = `decode::greedy` of row r (crates/decode/src/lib.rs:73-83: strict >, the
 * first maximum wins; a row with no value above -inf gives 0).  The logits never go to
 * memory unless `logits_f32` (`[b][n]`, may be NULL) asks for them.  `workspace`:
 * logismos_qgemm_q4g128_greedy_workspace_bytes() bytes, 4-byte aligned, contents don't matter. */
logismos_status_t logismos_check_qgemm_q4g128_greedy_shape(int b, int n, int k, char* msg,
                                                           size_t msg_cap);
size_t logismos_qgemm_q4g128_greedy_workspace_bytes(int b, int n, int k);
logismos_status_t logismos_launch_qgemm_q4g128_greedy_xprep(
    const void* x_prepared, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    void* out_tokens_u32, void* logits_f32, void* workspace, int b, int n, int k,
    logismos_stream_t stream);

/* out[r][:] = table[ids[r]][:] as fp32, table `[vocab][hidden]` fp32 or bf16; an id >= vocab
 * gives a zero row (`embed_lookup`, crates/kernels/src/cpu_f32/mod.rs:106-127). */
logismos_status_t logismos_launch_embed_lookup_f32(const void* table_f32, const void* ids_u32,
                                                   void* out_f32, int rows, int hidden,
                                                   long long vocab, logismos_stream_t stream);
logismos_status_t logismos_launch_embed_lookup_bf16(const void* table_bf16, const void* ids_u32,
                                                    void* out_f32, int rows, int hidden,
                                                    long long vocab, logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * The launchers the reference already has (built there for gfx1100), for gfx950
 * ------------------------------------------------------------------------
 * Same symbols, argument lists and meaning as the reference's own, so its private
 * `extern "C"` blocks (crates/kernels/src/{rms_norm,softmax,rope,matmul}/mod.rs) link
 * against this archive unchanged and `praxis::{rms_norm, softmax, rope_apply, matmul}` run
 * on MI355X.  fp16 in and out, fp32 inside, one rounding at the output; results as the
 * CPU references define them (crates/kernels/src/{rms_norm,softmax,rope,matmul}/cpu.rs). */

/* crates/kernels/src/rms_norm/hip/rms_norm.hip:58-84: y[m][n] = x * inv_rms(row) * w[n]. */
logismos_status_t logismos_launch_rms_norm_fp16(const void* x_fp16, const void* w_fp16,
                                                void* y_fp16, int m, int n, float eps,
                                                logismos_stream_t stream);
/* crates/kernels/src/softmax/hip/softmax.hip:66-87: row softmax of x[m][n]; a row of -inf
 * becomes uniform 1/n as in `softmax_fp16_ref` (crates/kernels/src/softmax/cpu.rs:40-59). */
logismos_status_t logismos_launch_softmax_fp16(const void* x_fp16, void* y_fp16, int m, int n,
                                               logismos_stream_t stream);
/* `cpu_f32::mask_additive_in_place` (crates/kernels/src/cpu_f32/mod.rs:451-486) on device
 * scores: scores[r][c] becomes -inf where mask[r / repeat][c] == 0, with
 * mask_rows = mask_len / n and repeat = rows / mask_rows (one mask row -- a batch row's
 * key-padding mask -- serves the `repeat` consecutive score rows of its heads).  Like the
 * reference: nothing to do (success) when n, rows or mask_len is 0 or the mask is shorter
 * than a row; where the reference panics -- rows not a multiple of mask_rows -- and where
 * its debug assertion fires -- a mask that is not whole rows -- InvalidValue and nothing
 * launched.  `_f32` is the reference's own type; `_fp16` masks the fp16 scores that
 * `logismos_launch_matmul_*_fp16` produce and `logismos_launch_softmax_fp16` consumes (a row
 * masked everywhere then comes out uniform, as in the reference).  The fused paged attention
 * masks by context length and causality only; a padded batch goes through these. */
logismos_status_t logismos_launch_mask_additive_f32(void* scores_f32, const void* mask_u8,
                                                    size_t mask_len, size_t rows, size_t n,
                                                    logismos_stream_t stream);
logismos_status_t logismos_launch_mask_additive_fp16(void* scores_fp16, const void* mask_u8,
                                                     size_t mask_len, size_t rows, size_t n,
                                                     logismos_stream_t stream);
/* crates/kernels/src/rope/hip/rope.hip:45-68: in place on (batch, seq, heads, head_dim),
 * interleaved pairs (2i, 2i+1), table f32 `[seq][head_dim]` with cos at 2i and sin at 2i+1
 * (`build_cos_sin_table`, crates/kernels/src/rope/cpu.rs:19-40).  Shape guard of
 * `check_rope_shape` (crates/kernels/src/rope/mod.rs:79-130).  qk 4-byte, table 8-byte
 * aligned. */
logismos_status_t logismos_launch_rope_fp16(void* qk_fp16, const void* cos_sin_f32, int batch,
                                            int seq, int heads, int head_dim,
                                            logismos_stream_t stream);
/* crates/kernels/src/matmul/hip/matmul_launchers.cpp:14-52: D[M,N] = A[M,K] . B[K,N],
 * row-major, fp32 accumulation.  `naive`: one thread per element, ascending k, bit-identical
 * to `matmul_fp16_ref` (crates/kernels/src/matmul/cpu.rs:12-30).  `wmma`: the matrix-core
 * version (CDNA4 MFMA here; any M, N, K; a and b 16-byte aligned).  Shape guard of
 * `check_matmul_shape` (crates/kernels/src/matmul/mod.rs:89-117). */
logismos_status_t logismos_launch_matmul_naive_fp16(const void* a_fp16, const void* b_fp16,
                                                    void* d_fp16, int m, int n, int k,
                                                    logismos_stream_t stream);
logismos_status_t logismos_launch_matmul_wmma_fp16(const void* a_fp16, const void* b_fp16,
                                                   void* d_fp16, int m, int n, int k,
                                                   logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * Decode step: one new token for each of num_seqs <= 32 live sequences through
 * num_layers pre-norm layers (`StellaLayer::forward` order,
 * crates/encoders/src/stella.rs:190-206; attention and SwiGLU arithmetic of
 * crates/transformers/src/{attention,mlp}.rs) with Q4G128 weights and the paged
 * fp16 KV cache.  The reference has no decoder yet (crates/decoders/src/lib.rs).
 *
 * Per layer: h += previous projection; xn = RMSNorm(h); qkv = xn.Wqkv^T;
 * RoPE(q,k), K/V appended at slot_mapping; paged attention; h += attn.Wo^T;
 * xn = RMSNorm(h); act = silu(xn.Wgate^T) * (xn.Wup^T); down projection.
 * Wqkv stacks the q, k and v projections (rows: hq*128, hkv*128, hkv*128),
 * Wgate_up stacks gate and up (intermediate rows each).  After the last layer
 * out = bf16(RMSNorm(h) * final_norm_w).
 *
 * Tokens in, tokens out (both optional, cfg->vocab > 0): with `token_ids` the step first
 * fills hidden_f32 from `embed_table_bf16` (`embed_lookup`,
 * crates/kernels/src/cpu_f32/mod.rs:106-127: an id outside the vocabulary is a zero row);
 * with `lm_head` it ends with the vocabulary projection of the normed state and
 * `decode::greedy` per sequence (crates/decode/src/lib.rs:73-83) into `out_tokens_u32`
 * (and the fp32 logits into `logits_f32` if that is not NULL); `out_bf16` may then be NULL.
 *
 * With cfg->kv_turbo3 the KV cache is TurboQuant 3-bit: new K/V rows are encoded as they
 * are written and the attention decodes inside its gather (the entry points of the
 * TurboQuant section below), everything else unchanged.
 *
 * All launches are asynchronous on `stream`; `workspace` needs
 * logismos_decode_step_workspace_bytes() bytes, 256-byte aligned, contents don't matter.
 * ------------------------------------------------------------------------ */
typedef struct {
    const void* qw;    /* uint8 [N][K/2] */
    const void* scale; /* fp16  [N][K/128] */
    const void* zero;  /* fp16  [N][K/128] */
} logismos_q4_weight_t;

typedef struct {
    int num_layers, hidden, num_q_heads, num_kv_heads, head_dim, intermediate;
    /* head_dim: 128, or (fp16 pools only) another multiple of 32 up to 256;
       hidden, intermediate and num_q_heads*head_dim multiples of 128 */
    float rms_eps;
    int block_size, max_blocks_per_seq;
    int max_pos; /* rows of the RoPE tables; >= block_size * max_blocks_per_seq, so that no
                    position a block table can hold lies past the table (else rejected) */
    int vocab;     /* rows of the embedding table and of lm_head; 0 when neither is used */
    int kv_turbo3; /* != 0: the layers' pools are turbo3 pools (56 bytes per head row) */
} logismos_decode_config_t;

typedef struct {
    const void* norm1_w_f32; /* [hidden] */
    const void* norm2_w_f32; /* [hidden] */
    logismos_q4_weight_t qkv, o, gate_up, down;
    void* k_pool_f16; /* this layer's paged pools (turbo3 pools with cfg->kv_turbo3) */
    void* v_pool_f16;
    const void* qkv_bias_f32; /* [(hq+2*hkv)*head_dim] or NULL: the q/k/v projection's bias
                                 (crates/transformers/src/attention.rs:49-57), added to the
                                 projection's fp32 result before RoPE */
} logismos_decode_layer_t;

typedef struct {
    void* hidden_f32;             /* [num_seqs][hidden], in: embeddings, out: last residual */
    void* out_bf16;               /* [num_seqs][hidden] */
    const void* final_norm_w_f32; /* [hidden] */
    const int32_t* block_tables;  /* [num_seqs][max_blocks_per_seq] */
    const int32_t* cu_seqlens;    /* [num_seqs+1] = 0,1,2,... */
    const int32_t* context_lens;  /* [num_seqs], including the new token */
    const int32_t* positions;     /* [num_seqs] = context_lens - 1 */
    const int64_t* slot_mapping;  /* [num_seqs] */
    const void* rope_cos_f32;     /* [max_pos][head_dim/2] */
    const void* rope_sin_f32;
    int num_seqs;
    int num_splits;
    const uint32_t* token_ids;           /* [num_seqs] or NULL: hidden_f32 is the input */
    const void* embed_table_bf16;        /* [vocab][hidden], with token_ids */
    const logismos_q4_weight_t* lm_head; /* [vocab][hidden] Q4G128 (host pointer) or NULL */
    void* out_tokens_u32;                /* [num_seqs], with lm_head */
    void* logits_f32;                    /* [num_seqs][vocab] or NULL */
    /* A mixed batch (chunked prefill + decode): total_tokens = cu_seqlens[num_seqs] packed
     * rows and the largest number of new tokens of a sequence; 0 / 0 means one new token per
     * sequence.  Every per-row array above (hidden_f32, out_bf16, positions, slot_mapping) then
     * has total_tokens rows, in packed order.  Up to 96 rows go through the projections 32 at
     * a time, every pass streaming the layer's weights once; from 97 rows on every projection
     * is one launch of the tiled matrix-core GEMM over all rows (`linear_t` over `seq` rows,
     * crates/transformers/src/mlp.rs:104-111).  The attention takes the whole ragged batch in
     * one launch either way.  token_ids takes any number of rows; lm_head, as described
     * above (a token for every packed row), needs total_tokens <= 32. */
    int total_tokens;
    int max_seqlen_q;
    /* != 0, with lm_head: the vocabulary projection and the token choice are made for the LAST
     * packed row of every sequence only (row cu_seqlens[s + 1] - 1: the row whose choice is the
     * sequence's next token; every sequence must have a new token), for any total_tokens.
     * out_tokens_u32 and logits_f32 then have num_seqs rows, in sequence order.  out_bf16 may
     * still be given (all packed rows) or NULL. */
    int tokens_for_last_rows;
} logismos_decode_batch_t;

size_t logismos_decode_step_workspace_bytes(const logismos_decode_config_t* cfg, int num_seqs,
                                            int num_splits);
/* ... for a mixed batch of total_tokens packed rows */
size_t logismos_decode_step_workspace_bytes_tokens(const logismos_decode_config_t* cfg,
                                                   int num_seqs, int total_tokens, int num_splits);
logismos_status_t logismos_launch_decode_step(const logismos_decode_config_t* cfg,
                                              const logismos_decode_layer_t* layers,
                                              const logismos_decode_batch_t* batch, void* workspace,
                                              logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * Paged KV cache (host object over device pools)
 * ------------------------------------------------------------------------ */

/* Rows [start_pos, start_pos + n_tokens) of ONE sequence, contiguous fp16
 * `[n_tokens][num_kv_heads*head_dim]`, to / from the pools through the
 * sequence's block-table row (device int32): the device side of
 * `KvCache::put` and `KvCache::get` (crates/cache/src/lib.rs:57-68; row order
 * and bytes as `FlatKvCache`, crates/cache/src/flat.rs:180-304). */
logismos_status_t logismos_launch_kv_append_fp16(const void* k_new_f16, const void* v_new_f16,
                                                 void* k_pool_f16, void* v_pool_f16,
                                                 const int32_t* block_table_row, int start_pos,
                                                 int n_tokens, int num_kv_heads, int head_dim,
                                                 int block_size, logismos_stream_t stream);
logismos_status_t logismos_launch_kv_gather_fp16(const void* k_pool_f16, const void* v_pool_f16,
                                                 const int32_t* block_table_row, void* k_out_f16,
                                                 void* v_out_f16, int start_pos, int n_tokens,
                                                 int num_kv_heads, int head_dim, int block_size,
                                                 logismos_stream_t stream);

/* `CacheLayout` (crates/cache/src/flat.rs:36-69) for a paged cache: max_seq_len
 * = block_size * max_blocks_per_seq; dtype is fp16. */
typedef struct {
    int num_layers;
    int num_kv_heads;
    int head_dim;
    int block_size;         /* rows per block, multiple of 16 */
    int num_blocks;         /* blocks in every layer's K pool and V pool */
    int max_seqs;           /* sequence slots */
    int max_blocks_per_seq; /* width of the block table */
} logismos_paged_kv_layout_t;

typedef struct logismos_paged_kv_cache logismos_paged_kv_cache_t;

/* Results: the variants of the reference's cache `Error`
 * (crates/cache/src/error.rs) that apply, plus the pool-specific ones. */
enum {
    LOGISMOS_KV_OK = 0,
    LOGISMOS_KV_LAYER_OUT_OF_RANGE = 1,   /* Error::LayerOutOfRange */
    LOGISMOS_KV_LEN_OVERFLOW = 2,         /* Error::LenOverflow */
    LOGISMOS_KV_READ_BEYOND_WRITTEN = 3,  /* Error::ReadBeyondWritten */
    LOGISMOS_KV_SHAPE_MISMATCH = 4,       /* Error::ShapeMismatch */
    LOGISMOS_KV_BAD_SEQ = 5,              /* sequence id not open */
    LOGISMOS_KV_OUT_OF_BLOCKS = 6,        /* free list exhausted */
    LOGISMOS_KV_OUT_OF_SEQS = 7,          /* no free sequence slot */
    LOGISMOS_KV_HIP_ERROR = 8             /* allocation, copy or launch failed */
};

/* The paged implementation the `KvCache` trait was left open for
 * (crates/cache/src/lib.rs:9-13,51-82), one instance per device; create and
 * destroy allocate and free device memory (the current device), nothing else does.
 * put / get / len_of / num_layers / reset keep the trait's meaning per sequence:
 *   put     appends n_tokens rows to (seq, layer); refuses LayerOutOfRange and
 *           LenOverflow like FlatKvCache::put (crates/cache/src/flat.rs:180-255);
 *           takes blocks from the free list as the sequence grows
 *   get     gathers the first len rows into contiguous buffers; refuses
 *           ReadBeyondWritten like FlatKvCache::get (:257-304)
 *   len_of  written rows, or -1 where the trait returns None
 *   reset   every open sequence back to length zero, its blocks freed
 * open_seq / close_seq admit and retire a sequence; reserve makes the block
 * table cover total_rows rows ahead of a step whose kernels write the rows
 * themselves (`logismos_launch_rope_kv_write_*`), and advance then records
 * those rows as written.  k_pool / v_pool / block_tables return the device
 * pointers the attention and packing entry points take (block table row of
 * sequence s at `block_tables + s * max_blocks_per_seq`; entries that never
 * had a block hold 0x3FFFFFFF, entries of a retired sequence keep their last
 * value).  Copies and launches go to `stream`; one caller thread at a time per
 * cache.  close_seq and reset do not wait for the device: on the stream that
 * carried the sequence's copies and launches its blocks may be handed out
 * again at once (what the next owner writes is ordered behind them); work on
 * any other stream has to be ordered by the caller.  Table updates are copied
 * to the device from staging memory that is not reused before the copy has
 * run, never from the host table itself, so closing a sequence and reopening
 * and growing its slot cannot change what an earlier, still queued update
 * delivers (a reserve or put waits only if 32 such updates are all still
 * queued). */
int logismos_paged_kv_cache_create(const logismos_paged_kv_layout_t* layout,
                                   logismos_paged_kv_cache_t** out);
void logismos_paged_kv_cache_destroy(logismos_paged_kv_cache_t* cache);
int logismos_paged_kv_cache_open_seq(logismos_paged_kv_cache_t* cache, int* seq_id);
int logismos_paged_kv_cache_close_seq(logismos_paged_kv_cache_t* cache, int seq_id);
int logismos_paged_kv_cache_reserve(logismos_paged_kv_cache_t* cache, int seq_id,
                                    int64_t total_rows, logismos_stream_t stream);
int logismos_paged_kv_cache_advance(logismos_paged_kv_cache_t* cache, int seq_id, int layer_idx,
                                    int n_tokens);
int logismos_paged_kv_cache_put(logismos_paged_kv_cache_t* cache, int seq_id, int layer_idx,
                                const void* k_f16, const void* v_f16, int n_tokens,
                                logismos_stream_t stream);
int logismos_paged_kv_cache_get(const logismos_paged_kv_cache_t* cache, int seq_id, int layer_idx,
                                int64_t len, void* k_out_f16, void* v_out_f16,
                                logismos_stream_t stream);
int64_t logismos_paged_kv_cache_len_of(const logismos_paged_kv_cache_t* cache, int seq_id,
                                       int layer_idx);
int logismos_paged_kv_cache_num_layers(const logismos_paged_kv_cache_t* cache);
void logismos_paged_kv_cache_reset(logismos_paged_kv_cache_t* cache);
int logismos_paged_kv_cache_free_blocks(const logismos_paged_kv_cache_t* cache);
void* logismos_paged_kv_cache_k_pool(const logismos_paged_kv_cache_t* cache, int layer_idx);
void* logismos_paged_kv_cache_v_pool(const logismos_paged_kv_cache_t* cache, int layer_idx);
const int32_t* logismos_paged_kv_cache_block_tables(const logismos_paged_kv_cache_t* cache);
const int32_t* logismos_paged_kv_cache_block_tables_host(const logismos_paged_kv_cache_t* cache);

/* ------------------------------------------------------------------------
 * TurboQuant 3-bit KV (`turbo3_0`, crates/quant/src/lib.rs)
 * ------------------------------------------------------------------------
 * turbo3 pools hold every 128-value head row as four 14-byte blocks
 * `{norm_f16_le[2], packed_indices[12]}` (`Turbo3Block`, crates/quant/src/lib.rs:129-172;
 * 56 bytes per head, 4.57x smaller than fp16): `[num_blocks][block_size][num_kv_heads][56]`
 * bytes, 2-byte aligned, with the slots and block tables of the fp16 pools.
 * head_dim is 128 (`TURBOQUANT_HEAD_DIM`). */

/* `encode_turbo3_0_head` (crates/quant/src/lib.rs:316-353) of every head of row t of
 * k_new / v_new (fp16 `[total_tokens][num_kv_heads][128]`, 16-byte aligned, widened to f32),
 * written to pool row slot_mapping[t] (negative: skipped).  Bytes identical to the reference
 * function's. */
logismos_status_t logismos_launch_kv_write_turbo3(const void* k_new_f16, const void* v_new_f16,
                                                  void* k_pool_t3, void* v_pool_t3,
                                                  const int64_t* slot_mapping, int total_tokens,
                                                  int num_kv_heads, logismos_stream_t stream);

/* `decode_turbo3_0_head` (crates/quant/src/lib.rs:376-413) of rows
 * [start_pos, start_pos + n_tokens) of one sequence (block_table_row: device int32) into
 * f32 `[n_tokens][num_kv_heads][128]`; values identical to the reference function's. */
logismos_status_t logismos_launch_kv_gather_turbo3_f32(const void* k_pool_t3,
                                                       const void* v_pool_t3,
                                                       const int32_t* block_table_row,
                                                       void* k_out_f32, void* v_out_f32,
                                                       int start_pos, int n_tokens,
                                                       int num_kv_heads, int block_size,
                                                       logismos_stream_t stream);

/* `logismos_launch_paged_attn_varlen_fp16` over turbo3 pools (decode rows and
 * chunked-prefill rows of one packed batch): out = softmax(q . K^T * scale) . V with K and
 * V the rows `decode_turbo3_0_head` (crates/quant/src/lib.rs:376-413) would return.  The
 * decode is fused into the gather: since a decoded row is norm * H c with H the orthonormal,
 * symmetric transform of `fwht_128` (:88-113), the kernels transform each query once,
 * multiply with the centroid values c (as fp16) and transform each output once; nothing is
 * decoded to memory.  The new tokens' rows must already be in the pools
 * (`logismos_launch_kv_write_turbo3`).  Same workspace, num_splits and block tables as the
 * fp16 entry point; head_dim is 128; fp16 q and out. */
logismos_status_t logismos_launch_paged_attn_varlen_turbo3(
    const void* q_f16, const void* k_pool_t3, const void* v_pool_t3, const int32_t* block_tables,
    const int32_t* cu_seqlens_q, const int32_t* context_lens, void* out_f16, void* workspace,
    int num_seqs, int total_tokens, int max_seqlen_q, int num_q_heads, int num_kv_heads,
    int block_size, int max_blocks_per_seq, int num_splits, float scale,
    logismos_stream_t stream);

/* ------------------------------------------------------------------------
 * Memory-system probes (measurement aids; the reference has no counterpart,
 * its only timing helper is the hipEvent pair of
 * crates/kernels/examples/gemm_bench.rs:120-128).  A plain copy and a plain
 * read of `bytes` bytes (multiple of 16, 16-byte aligned): the achievable HBM
 * ceiling of the box, and the calibration for FETCH_SIZE / WRITE_SIZE.
 * `_read_ex` takes flags: non-temporal loads (what the decode attention reads
 * K and V with), and 256 resident workgroups taking chunks in turn instead of
 * 2048 workgroups with a slab each; the read ceiling at a size is the best of
 * the four.
 * ------------------------------------------------------------------------ */
#define LOGISMOS_PROBE_NON_TEMPORAL 1
#define LOGISMOS_PROBE_STRIDED 2
logismos_status_t logismos_launch_probe_copy(const void* src, void* dst, size_t bytes,
                                             logismos_stream_t stream);
logismos_status_t logismos_launch_probe_read(const void* src, void* sink_u32, size_t bytes,
                                             logismos_stream_t stream);
logismos_status_t logismos_launch_probe_read_ex(const void* src, void* sink_u32, size_t bytes,
                                                int flags, logismos_stream_t stream);

/* The matrix-core counterpart (no counterpart in the reference): 256 workgroups of
 * eight waves issue nothing but v_mfma_f32_32x32x16 (fp16, or bf16 with
 * LOGISMOS_PROBE_MFMA_BF16) on four accumulators, `iters` x 4 per wave; with
 * LOGISMOS_PROBE_MFMA_CHANGING both operands are rewritten between the MFMAs, as
 * they are on real data.  The rate of the second form is the matrix-core ceiling
 * the MFMA-bound kernels are measured against beside the datasheet peak: the part
 * holds the pipes back when their inputs toggle.  `_flops` is the work of one
 * launch.  `sink_f32` (4 bytes) is practically never written. */
#define LOGISMOS_PROBE_MFMA_CHANGING 1
#define LOGISMOS_PROBE_MFMA_BF16 2
logismos_status_t logismos_launch_probe_mfma(void* sink_f32, int iters, int flags,
                                             logismos_stream_t stream);
double logismos_probe_mfma_flops(int iters);

#ifdef __cplusplus
}
#endif
#endif /* LOGISMOS_DECODE_H */
