// Kernel parameters of the ragged paged attention, shared by the head_dim-128 kernels
// (paged_attn.hip) and the kernel for the other head widths (paged_attn_anydim.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lg {

struct AttnParams {
    const _Float16* q;
    const _Float16* k_pool;
    const _Float16* v_pool;
    const int32_t* block_tables;
    const int32_t* cu_seqlens_q;
    const int32_t* context_lens;
    _Float16* out;
    float* ws_acc;  // [slot][hq][head_dim], slot < num_seqs * num_splits
    float* ws_ml;   // [slot][hq][2]
    int num_seqs;
    int hq;
    int hkv;
    int block_size;
    int max_blocks_per_seq;
    int num_splits;
    int part_tokens;  // keys per partition (multiple of 16), static split only
    int num_workers;  // > 0: balanced decode (see paged_attn_balanced_kernel), else static split
    float scale_log2e;
    int causal;
    // 0: fp16 [T][hq][head_dim]; 1: bf16, same shape; 2: the prepared layout of the following
    // Q4G128 GEMM (x = [out_rows][hq*128], see q4_common.hpp) -- what the step executor uses
    // at head_dim 128
    int out_bf16;
    int out_rows;
};

__device__ __forceinline__ unsigned short attn_out_elem(float v, int out_bf16) {
    if (out_bf16) {
        unsigned u = __float_as_uint(v);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (unsigned short)(u >> 16);
    }
    const _Float16 hv = (_Float16)v;
    return __builtin_bit_cast(unsigned short, hv);
}

// ---- the balanced split of decode rows (both kernel families) -------------------------
constexpr int kTileKeys = 16;

// Units sequence s contributes to the decode stream: its 16-key tiles plus kSeqStartUnits for
// starting it.  A worker that finishes one sequence and starts the next pays for a second
// prologue (queries, first tiles with nothing in flight) and epilogue (row merge, partial
// write): with equal tile counts such workers ended 3 us after the others and set the
// duration of the launch.  With that cost in the stream they get fewer tiles (a tile of the
// head_dim-128 kernel takes about 2.3 us); 3 to 5 units measured alike, 0 and 1 worse.
constexpr int kSeqStartUnits = 4;
__device__ __forceinline__ int decode_tiles(const AttnParams& p, int s) {
    const int n_new = p.cu_seqlens_q[s + 1] - p.cu_seqlens_q[s];
    const int ctx = p.context_lens[s];
    return (n_new == 1 && ctx > 0) ? (ctx + kTileKeys - 1) / kTileKeys + kSeqStartUnits : 0;
}

constexpr int kMaxBalancedSeqs = 2048;  // prefix table held in LDS
constexpr int kMinWorkerTiles = 8;      // a worker streams at least 128 keys

__device__ __forceinline__ int worker_tiles(int total_tiles, int num_workers) {
    const int r = (total_tiles + num_workers - 1) / num_workers;
    return r < kMinWorkerTiles ? kMinWorkerTiles : r;
}

// Small batches stay on the static split: when every partition of every sequence is
// resident at once there is no second round to balance away, and the balanced kernel's
// prologue (prefix table, search) costs more than it saves (config 2: 12.7 vs 18 us).
// The bound is on what the block tables could hold, the only size the host knows.
inline bool small_decode_batch(int num_seqs, int num_kv_heads, int block_size,
                               int max_blocks_per_seq) {
    return (int64_t)num_seqs * num_kv_heads * block_size * max_blocks_per_seq <= 200000;
}

// The kernel for head widths other than 128 (multiples of 32 up to 256, GQA groups up to 16):
// decode rows on the static split, rows of sequences with several new tokens over their whole
// visible context, then the merge of the decode partitions.  `phases` as in the public launcher.
hipError_t paged_attn_anydim_launch(const AttnParams& p, int head_dim, int total_tokens,
                                    int max_seqlen_q, int phases, hipStream_t stream);

// Partition count for that kernel (pure host arithmetic).
int paged_attn_anydim_num_splits(int num_seqs, int num_kv_heads, int head_dim, int block_size,
                                 int max_blocks_per_seq);

}  // namespace lg
