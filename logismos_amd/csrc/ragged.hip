// Ragged-batch bookkeeping on the GPU: packing per-sequence token counts into
// cu_seqlens / slot_mapping / context_lens, and writing new K/V rows into the
// paged pools by slot.  Integer work, bit-exact against the CPU definition.
#include "device_utils.hpp"
#include "launch_common.hpp"

namespace lg {

// One workgroup per sequence.  The exclusive prefix of new_tokens is
// recomputed per workgroup (num_seqs is small next to the token count), so one
// launch suffices and the host never needs the total.
__global__ __launch_bounds__(256) void pack_ragged_kernel(
    const int32_t* __restrict__ new_tokens, const int32_t* __restrict__ prior_ctx,
    const int32_t* __restrict__ block_tables, int32_t* __restrict__ cu_seqlens,
    int64_t* __restrict__ slot_mapping, int32_t* __restrict__ context_lens, int num_seqs,
    int block_size, int max_blocks) {
    (void)num_seqs;  // the grid has one workgroup per sequence
    const int s = blockIdx.x;
    __shared__ int partial[4];
    int sum = 0;
    for (int i = threadIdx.x; i < s; i += 256) {
        const int v = new_tokens[i];
        sum += v > 0 ? v : 0;
    }
    // integer wave reduction, then across the four waves
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, kWave);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
    __syncthreads();
    const int start = partial[0] + partial[1] + partial[2] + partial[3];
    int n_new = new_tokens[s];
    n_new = n_new > 0 ? n_new : 0;
    int prior = prior_ctx[s];
    prior = prior > 0 ? prior : 0;
    if (threadIdx.x == 0) {
        if (s == 0) cu_seqlens[0] = 0;
        cu_seqlens[s + 1] = start + n_new;
        // a context never exceeds what the block table can hold: the attention kernels walk
        // the table row by context_lens
        const int64_t cap = (int64_t)block_size * max_blocks;
        const int64_t ctx = (int64_t)prior + n_new;
        context_lens[s] = (int32_t)(ctx < cap ? ctx : cap);
    }
    const int32_t* bt = block_tables + (int64_t)s * max_blocks;
    for (int i = threadIdx.x; i < n_new; i += 256) {
        const int64_t pos = (int64_t)prior + i;
        const int64_t blk = pos / block_size;
        int64_t slot = -1;
        if (blk < max_blocks) {
            // an entry that names no block (negative, or the "unmapped" mark and above) gives
            // no slot: the row is skipped by the writers instead of landing outside the pool
            const int32_t id = bt[blk];
            if (id >= 0 && id < LOGISMOS_BLOCK_ID_LIMIT)
                slot = (int64_t)id * block_size + (pos - blk * block_size);
        }
        slot_mapping[(int64_t)start + i] = slot;
    }
}

// Row t of k_new / v_new -> pool row slot_mapping[t]; 16 bytes per lane.
__global__ __launch_bounds__(256) void kv_write_kernel(const uint4_t* __restrict__ k_new,
                                                       const uint4_t* __restrict__ v_new,
                                                       uint4_t* __restrict__ k_pool,
                                                       uint4_t* __restrict__ v_pool,
                                                       const int64_t* __restrict__ slot_mapping,
                                                       int total_tokens, int row_vec) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)total_tokens * row_vec) return;
    const int64_t t = idx / row_vec;
    const int64_t j = idx - t * row_vec;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    k_pool[slot * row_vec + j] = k_new[idx];
    v_pool[slot * row_vec + j] = v_new[idx];
}

// One sequence's rows [start_pos, start_pos + n_tokens) <-> contiguous rows, through the
// sequence's block-table row.  TO_POOL: contiguous -> pool (append); else pool -> contiguous
// (gather).  16 bytes per lane.
template <bool TO_POOL>
__global__ __launch_bounds__(256) void kv_seq_copy_kernel(uint4_t* __restrict__ k_flat,
                                                          uint4_t* __restrict__ v_flat,
                                                          uint4_t* __restrict__ k_pool,
                                                          uint4_t* __restrict__ v_pool,
                                                          const int32_t* __restrict__ bt_row,
                                                          int start_pos, int n_tokens, int row_vec,
                                                          int block_size) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)n_tokens * row_vec) return;
    const int t = (int)(idx / row_vec);
    const int64_t j = idx - (int64_t)t * row_vec;
    const int pos = start_pos + t;
    const int bi = pos / block_size;
    const int64_t slot = (int64_t)bt_row[bi] * block_size + (pos - bi * block_size);
    if (TO_POOL) {
        k_pool[slot * row_vec + j] = k_flat[idx];
        v_pool[slot * row_vec + j] = v_flat[idx];
    } else {
        k_flat[idx] = k_pool[slot * row_vec + j];
        v_flat[idx] = v_pool[slot * row_vec + j];
    }
}

}  // namespace lg

static logismos_status_t kv_seq_copy(bool to_pool, void* k_flat, void* v_flat, void* k_pool,
                                     void* v_pool, const int32_t* bt_row, int start_pos,
                                     int n_tokens, int num_kv_heads, int head_dim, int block_size,
                                     logismos_stream_t stream) {
    if (start_pos < 0 || n_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0)
        return hipErrorInvalidValue;
    const int64_t row_elems = (int64_t)num_kv_heads * head_dim;
    if (row_elems % 8 != 0 || row_elems > INT32_MAX) return hipErrorInvalidValue;
    if ((int64_t)start_pos + n_tokens > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (n_tokens == 0) return hipSuccess;
    if (!k_flat || !v_flat || !k_pool || !v_pool || !bt_row) return hipErrorInvalidValue;
    const int row_vec = (int)(row_elems / 8);
    const int64_t items = (int64_t)n_tokens * row_vec;
    const dim3 grid((unsigned)((items + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto* kf = static_cast<lg::uint4_t*>(k_flat);
    auto* vf = static_cast<lg::uint4_t*>(v_flat);
    auto* kp = static_cast<lg::uint4_t*>(k_pool);
    auto* vp = static_cast<lg::uint4_t*>(v_pool);
    if (to_pool)
        lg::kv_seq_copy_kernel<true><<<grid, dim3(256), 0, st>>>(kf, vf, kp, vp, bt_row, start_pos,
                                                                 n_tokens, row_vec, block_size);
    else
        lg::kv_seq_copy_kernel<false><<<grid, dim3(256), 0, st>>>(kf, vf, kp, vp, bt_row, start_pos,
                                                                  n_tokens, row_vec, block_size);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_kv_append_fp16(
    const void* k_new_f16, const void* v_new_f16, void* k_pool_f16, void* v_pool_f16,
    const int32_t* block_table_row, int start_pos, int n_tokens, int num_kv_heads, int head_dim,
    int block_size, logismos_stream_t stream) {
    return kv_seq_copy(true, const_cast<void*>(k_new_f16), const_cast<void*>(v_new_f16), k_pool_f16,
                       v_pool_f16, block_table_row, start_pos, n_tokens, num_kv_heads, head_dim,
                       block_size, stream);
}

extern "C" logismos_status_t logismos_launch_kv_gather_fp16(
    const void* k_pool_f16, const void* v_pool_f16, const int32_t* block_table_row, void* k_out_f16,
    void* v_out_f16, int start_pos, int n_tokens, int num_kv_heads, int head_dim, int block_size,
    logismos_stream_t stream) {
    return kv_seq_copy(false, k_out_f16, v_out_f16, const_cast<void*>(k_pool_f16),
                       const_cast<void*>(v_pool_f16), block_table_row, start_pos, n_tokens,
                       num_kv_heads, head_dim, block_size, stream);
}

extern "C" logismos_status_t logismos_check_pack_ragged_shape(int num_seqs, int block_size,
                                                              int max_blocks, char* msg,
                                                              size_t msg_cap) {
    if (num_seqs <= 0)
        return lg::reject(msg, msg_cap, "pack_ragged: num_seqs must be positive, got %d", num_seqs);
    if (block_size <= 0)
        return lg::reject(msg, msg_cap, "pack_ragged: block_size must be positive, got %d",
                          block_size);
    if (max_blocks <= 0)
        return lg::reject(msg, msg_cap, "pack_ragged: max_blocks must be positive, got %d",
                          max_blocks);
    if ((int64_t)num_seqs * max_blocks > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "pack_ragged: num_seqs*max_blocks exceeds i32::MAX");
    if ((int64_t)block_size * max_blocks > (int64_t)INT32_MAX)
        return lg::reject(msg, msg_cap, "pack_ragged: block_size*max_blocks exceeds i32::MAX");
    return 0;
}

extern "C" logismos_status_t logismos_launch_pack_ragged(
    const int32_t* new_tokens, const int32_t* prior_ctx, const int32_t* block_tables,
    int32_t* cu_seqlens, int64_t* slot_mapping, int32_t* context_lens, int num_seqs,
    int block_size, int max_blocks, logismos_stream_t stream) {
    if (logismos_check_pack_ragged_shape(num_seqs, block_size, max_blocks, nullptr, 0) != 0)
        return hipErrorInvalidValue;
    if (!new_tokens || !prior_ctx || !block_tables || !cu_seqlens || !slot_mapping || !context_lens)
        return hipErrorInvalidValue;
    lg::pack_ragged_kernel<<<dim3(num_seqs), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        new_tokens, prior_ctx, block_tables, cu_seqlens, slot_mapping, context_lens, num_seqs,
        block_size, max_blocks);
    return hipGetLastError();
}

extern "C" logismos_status_t logismos_launch_kv_write_fp16(
    const void* k_new_f16, const void* v_new_f16, void* k_pool_f16, void* v_pool_f16,
    const int64_t* slot_mapping, int total_tokens, int num_kv_heads, int head_dim,
    logismos_stream_t stream) {
    if (total_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0) return hipErrorInvalidValue;
    const int64_t row_elems = (int64_t)num_kv_heads * head_dim;
    if (row_elems % 8 != 0 || row_elems > INT32_MAX) return hipErrorInvalidValue;
    if ((int64_t)total_tokens * row_elems > (int64_t)INT32_MAX) return hipErrorInvalidValue;
    if (total_tokens == 0) return hipSuccess;
    if (!k_new_f16 || !v_new_f16 || !k_pool_f16 || !v_pool_f16 || !slot_mapping)
        return hipErrorInvalidValue;
    const int row_vec = (int)(row_elems / 8);
    const int64_t items = (int64_t)total_tokens * row_vec;
    lg::kv_write_kernel<<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                          static_cast<hipStream_t>(stream)>>>(
        static_cast<const lg::uint4_t*>(k_new_f16), static_cast<const lg::uint4_t*>(v_new_f16),
        static_cast<lg::uint4_t*>(k_pool_f16), static_cast<lg::uint4_t*>(v_pool_f16), slot_mapping,
        total_tokens, row_vec);
    return hipGetLastError();
}
