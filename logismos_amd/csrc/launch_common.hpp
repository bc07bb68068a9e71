// Host-side helpers shared by the launchers: status type, rejection messages.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/logismos_decode.h"

namespace lg {

// Writes the reason (if the caller wants one) and returns hipErrorInvalidValue.
inline logismos_status_t reject(char* msg, size_t cap, const char* fmt, ...) {
    if (msg && cap) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(msg, cap, fmt, ap);
        va_end(ap);
    }
    return static_cast<logismos_status_t>(hipErrorInvalidValue);
}

// Library-internal form of the paged-attention launcher: the public one with the
// output element type selectable (fp16, or bf16 for the step executor) and the pools either
// fp16 or turbo3 (kv_turbo3 != 0).
logismos_status_t paged_attn_launch(
    const void* q_f16, const void* k_pool_f16, const void* v_pool_f16, const int32_t* block_tables,
    const int32_t* cu_seqlens_q, const int32_t* context_lens, void* out, void* workspace,
    int num_seqs, int total_tokens, int max_seqlen_q, int num_q_heads, int num_kv_heads,
    int head_dim, int block_size, int max_blocks_per_seq, int num_splits, float scale, int causal,
    int phases, int out_bf16, int kv_turbo3, logismos_stream_t stream);

// Streaming Q4G128 GEMM over prepared activations (qgemm_q4_stream.hip): steps per worker
// for this shape (0: not applicable, use the split-K kernel) and the launch.  K parts are
// 8 groups there, so a shape it applies to has K/1024 parts.
int stream_steps(int b, int n, int k);
hipError_t qgemm_q4_stream_launch(const void* xprep, const void* qw, const void* scale,
                                  const void* zero, void* part, int b, int n, int k, int steps,
                                  hipStream_t stream);

// Q4G128 GEMM with x in registers and the weights streamed through LDS
// (qgemm_q4_regx.hip): the plan for a shape (parts == 0: not applicable) and the launch.
struct RegxPlan {
    int rows;   // weight rows per tile: 16 (up to 16 batch rows) or 32
    int gs;     // groups per wave slice; a workgroup covers 8 * gs groups of K
    int tpw;    // tiles per workgroup
    int ring;   // tiles a wave keeps in flight
    int parts;  // K parts = (K / 128) / (8 * gs)
};
RegxPlan regx_plan(int b, int n, int k);
// ... and for x as a plain bf16 [b][K] matrix with the bf16 product as output (one part)
RegxPlan regx_plain_plan(int b, int n, int k);
hipError_t qgemm_q4_regx_plain_launch(const RegxPlan& plan, const void* x_bf16, const void* qw,
                                      const void* scale, const void* zero, void* y_bf16,
                                      const float* bias, int b, int n, int k,
                                      hipStream_t stream);
hipError_t qgemm_q4_regx_launch(const RegxPlan& plan, const void* xprep, const void* qw,
                                const void* scale, const void* zero, void* part, int b, int n,
                                int k, hipStream_t stream);

// Q4G128 GEMM for a tall x (qgemm_q4_tall.hip): 128 x 128 output tiles, x through LDS, the
// matrix cores as the bound.  x bf16 [b][K], y bf16 [b][N], bias fp32 [N] or null.
bool qgemm_q4_tall_applies(int b, int n, int k);
hipError_t qgemm_q4_tall_launch(const void* x_bf16, const void* qw, const void* scale,
                                const void* zero, const float* bias, void* y_bf16, int b, int n,
                                int k, hipStream_t stream);
// ... with the fp32 product as output (the step executor keeps projections un-rounded)
hipError_t qgemm_q4_tall_f32_launch(const void* x_bf16, const void* qw, const void* scale,
                                    const void* zero, const float* bias, void* y_f32, int b,
                                    int n, int k, hipStream_t stream);

// dst[s][:] = src[cu_seqlens[s + 1] - 1][:], bf16 rows of `hidden` elements (step_ops.hip): the
// last packed row of every sequence of a ragged batch.
hipError_t gather_last_rows_bf16_launch(const void* src_bf16, const int32_t* cu_seqlens,
                                        void* dst_bf16, int num_seqs, int hidden,
                                        hipStream_t stream);

}  // namespace lg
