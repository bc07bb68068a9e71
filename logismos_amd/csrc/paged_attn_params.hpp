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

// The kernel for head widths other than 128 (multiples of 32 up to 256, GQA groups up to 16):
// decode rows on the static split, rows of sequences with several new tokens over their whole
// visible context, then the merge of the decode partitions.  `phases` as in the public launcher.
hipError_t paged_attn_anydim_launch(const AttnParams& p, int head_dim, int total_tokens,
                                    int max_seqlen_q, int phases, hipStream_t stream);

// Partition count for that kernel (pure host arithmetic).
int paged_attn_anydim_num_splits(int num_seqs, int num_kv_heads, int head_dim, int block_size,
                                 int max_blocks_per_seq);

}  // namespace lg
