// Paged KV cache: the host object that owns the per-layer K/V pools and the block
// tables the ragged attention kernels read.
//
// It keeps the contract of the reference's `KvCache` trait
// (crates/cache/src/lib.rs:57-82: put / get / len_of / num_layers / reset) and the
// checks of its one implementation, `FlatKvCache` (crates/cache/src/flat.rs:180-304:
// layer range, overflow of max_seq_len, read beyond the written length), per sequence:
// a cache holds up to max_seqs independent sequences, each with its own written length
// per layer, and every layer's pool uses the same logical -> physical block mapping of a
// sequence (one block table serves all layers).  Storage is device memory: rows are
// fp16 `[num_kv_heads][head_dim]`, little-endian, in token order inside a block
// (`CacheLayout`, crates/cache/src/flat.rs:36-69).
//
// Blocks come from a free list (most recently freed first).  The host keeps the block
// tables as bookkeeping; whenever a sequence gains blocks the new entries are mirrored to
// the device with an asynchronous copy on the caller's stream, so a put or a reserve
// followed by a launch on the same stream sees them.  The source of such a copy is never
// the bookkeeping row itself (a row is rewritten when its sequence slot is closed, reopened
// and grown again, possibly before an earlier copy of it has run) but a slot of a ring of
// pinned staging rows, reused only after an event recorded behind its copy has completed.
// One thread at a time per cache.
#include "launch_common.hpp"
#include "staging_ring.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <new>
#include <vector>

namespace {

constexpr int kStagingSlots = 32;

// Fence of the staging ring: one HIP event per slot, recorded behind the slot's copy.
struct EventFence {
    hipEvent_t* events = nullptr;
    void record(int slot, hipStream_t stream) { (void)hipEventRecord(events[slot], stream); }
    void wait(int slot) { (void)hipEventSynchronize(events[slot]); }
};

}  // namespace

struct logismos_paged_kv_cache {
    logismos_paged_kv_layout_t layout{};
    int device = 0;
    std::vector<void*> k_pools, v_pools;  // per layer, device
    int32_t* bt_host = nullptr;           // pinned, [max_seqs][max_blocks_per_seq]; bookkeeping
    int32_t* bt_dev = nullptr;
    int32_t* staging_mem = nullptr;       // pinned, [kStagingSlots][max_blocks_per_seq]
    hipEvent_t staging_events[kStagingSlots] = {};
    int staging_events_made = 0;
    lg::StagingRing<EventFence, hipStream_t> staging;
    std::vector<int32_t> free_blocks;     // stack of physical block ids
    std::vector<uint8_t> seq_open;
    std::vector<int32_t> seq_blocks;      // blocks held by each sequence
    std::vector<int64_t> lens;            // [max_seqs][num_layers] written rows
    std::vector<int32_t> free_seqs;

    int64_t row_elems() const { return (int64_t)layout.num_kv_heads * layout.head_dim; }
    int64_t max_seq_len() const { return (int64_t)layout.block_size * layout.max_blocks_per_seq; }
    int64_t& len(int seq, int layer) { return lens[(size_t)seq * layout.num_layers + layer]; }
    int32_t* row(int seq) { return bt_host + (size_t)seq * layout.max_blocks_per_seq; }
    const int32_t* row_dev(int seq) const {
        return bt_dev + (size_t)seq * layout.max_blocks_per_seq;
    }
};

namespace {

constexpr int32_t kUnmapped = 0x3FFFFFFF;  // poison for table entries without a block

bool seq_ok(const logismos_paged_kv_cache* c, int seq) {
    return c && seq >= 0 && seq < c->layout.max_seqs && c->seq_open[(size_t)seq];
}

// Makes sure `seq` owns blocks for rows [0, rows); mirrors the new entries to the device.
int ensure_blocks(logismos_paged_kv_cache* c, int seq, int64_t rows, hipStream_t stream) {
    const int bs = c->layout.block_size;
    const int need = (int)((rows + bs - 1) / bs);
    const int have = c->seq_blocks[(size_t)seq];
    if (need <= have) return LOGISMOS_KV_OK;
    if ((size_t)(need - have) > c->free_blocks.size()) return LOGISMOS_KV_OUT_OF_BLOCKS;
    int32_t* r = c->row(seq);
    for (int b = have; b < need; ++b) {
        r[b] = c->free_blocks.back();
        c->free_blocks.pop_back();
    }
    c->seq_blocks[(size_t)seq] = need;
    // the copy reads its source when it runs: stage the entries, never copy from `r`
    int32_t* staged = nullptr;
    const int slot = c->staging.stage(r + have, need - have, &staged);
    const hipError_t e =
        hipMemcpyAsync(c->bt_dev + (size_t)seq * c->layout.max_blocks_per_seq + have, staged,
                       sizeof(int32_t) * (size_t)(need - have), hipMemcpyHostToDevice, stream);
    c->staging.queued(slot, stream);
    return e == hipSuccess ? LOGISMOS_KV_OK : LOGISMOS_KV_HIP_ERROR;
}

// Copies to the device that an earlier reserve or put queued may not have run yet; they read
// their staging slots, so the bookkeeping row is free to be rewritten by the next owner of
// this sequence slot.  (On one stream a freed block is safe to hand out at once: whatever the
// next owner writes is ordered after the launches that still use it.)
void release_blocks(logismos_paged_kv_cache* c, int seq) {
    const int32_t* r = c->row(seq);
    for (int b = c->seq_blocks[(size_t)seq] - 1; b >= 0; --b) c->free_blocks.push_back(r[b]);
    c->seq_blocks[(size_t)seq] = 0;
    for (int l = 0; l < c->layout.num_layers; ++l) c->len(seq, l) = 0;
}

}  // namespace

extern "C" int logismos_paged_kv_cache_create(const logismos_paged_kv_layout_t* layout,
                                              logismos_paged_kv_cache_t** out) {
    if (!layout || !out) return LOGISMOS_KV_SHAPE_MISMATCH;
    *out = nullptr;
    const logismos_paged_kv_layout_t& L = *layout;
    if (L.num_layers <= 0 || L.num_kv_heads <= 0 || L.head_dim <= 0 || L.block_size <= 0 ||
        L.num_blocks <= 0 || L.max_seqs <= 0 || L.max_blocks_per_seq <= 0)
        return LOGISMOS_KV_SHAPE_MISMATCH;
    const int64_t row_elems = (int64_t)L.num_kv_heads * L.head_dim;
    if (row_elems % 8 != 0 || L.block_size % 16 != 0) return LOGISMOS_KV_SHAPE_MISMATCH;
    if ((int64_t)L.block_size * L.max_blocks_per_seq > INT32_MAX ||
        (int64_t)L.max_seqs * L.max_blocks_per_seq > INT32_MAX ||
        (int64_t)L.block_size * row_elems > INT32_MAX || L.num_blocks > LOGISMOS_BLOCK_ID_LIMIT)
        return LOGISMOS_KV_SHAPE_MISMATCH;

    auto* c = new (std::nothrow) logismos_paged_kv_cache;
    if (!c) return LOGISMOS_KV_HIP_ERROR;
    c->layout = L;
    if (hipGetDevice(&c->device) != hipSuccess) {
        delete c;
        return LOGISMOS_KV_HIP_ERROR;
    }
    const size_t pool_bytes = (size_t)L.num_blocks * L.block_size * (size_t)row_elems * 2;
    const size_t bt_bytes = sizeof(int32_t) * (size_t)L.max_seqs * L.max_blocks_per_seq;
    bool ok = true;
    for (int l = 0; ok && l < L.num_layers; ++l) {
        void *k = nullptr, *v = nullptr;
        ok = hipMalloc(&k, pool_bytes) == hipSuccess;
        if (ok) c->k_pools.push_back(k);
        ok = ok && hipMalloc(&v, pool_bytes) == hipSuccess;
        if (ok) c->v_pools.push_back(v);
    }
    ok = ok && hipHostMalloc(reinterpret_cast<void**>(&c->bt_host), bt_bytes, hipHostMallocDefault) ==
                   hipSuccess;
    ok = ok && hipMalloc(reinterpret_cast<void**>(&c->bt_dev), bt_bytes) == hipSuccess;
    ok = ok && hipHostMalloc(reinterpret_cast<void**>(&c->staging_mem),
                             sizeof(int32_t) * (size_t)kStagingSlots * L.max_blocks_per_seq,
                             hipHostMallocDefault) == hipSuccess;
    for (int i = 0; ok && i < kStagingSlots; ++i) {
        ok = hipEventCreateWithFlags(&c->staging_events[i], hipEventDisableTiming) == hipSuccess;
        if (ok) c->staging_events_made = i + 1;
    }
    if (ok)
        c->staging.init(c->staging_mem, kStagingSlots, L.max_blocks_per_seq,
                        EventFence{c->staging_events});
    if (ok) {
        for (size_t i = 0; i < bt_bytes / sizeof(int32_t); ++i) c->bt_host[i] = kUnmapped;
        ok = hipMemcpy(c->bt_dev, c->bt_host, bt_bytes, hipMemcpyHostToDevice) == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        logismos_paged_kv_cache_destroy(c);
        return LOGISMOS_KV_HIP_ERROR;
    }
    c->free_blocks.resize((size_t)L.num_blocks);
    for (int b = 0; b < L.num_blocks; ++b) c->free_blocks[(size_t)b] = L.num_blocks - 1 - b;
    c->seq_open.assign((size_t)L.max_seqs, 0);
    c->seq_blocks.assign((size_t)L.max_seqs, 0);
    c->lens.assign((size_t)L.max_seqs * L.num_layers, 0);
    c->free_seqs.resize((size_t)L.max_seqs);
    for (int s = 0; s < L.max_seqs; ++s) c->free_seqs[(size_t)s] = L.max_seqs - 1 - s;
    *out = c;
    return LOGISMOS_KV_OK;
}

extern "C" void logismos_paged_kv_cache_destroy(logismos_paged_kv_cache_t* c) {
    if (!c) return;
    if (c->staging.slots() > 0) c->staging.drain();
    for (int i = 0; i < c->staging_events_made; ++i) (void)hipEventDestroy(c->staging_events[i]);
    if (c->staging_mem) (void)hipHostFree(c->staging_mem);
    for (void* p : c->k_pools) (void)hipFree(p);
    for (void* p : c->v_pools) (void)hipFree(p);
    if (c->bt_dev) (void)hipFree(c->bt_dev);
    if (c->bt_host) (void)hipHostFree(c->bt_host);
    delete c;
}

extern "C" int logismos_paged_kv_cache_open_seq(logismos_paged_kv_cache_t* c, int* seq_id) {
    if (!c || !seq_id) return LOGISMOS_KV_SHAPE_MISMATCH;
    if (c->free_seqs.empty()) return LOGISMOS_KV_OUT_OF_SEQS;
    const int s = c->free_seqs.back();
    c->free_seqs.pop_back();
    c->seq_open[(size_t)s] = 1;
    *seq_id = s;
    return LOGISMOS_KV_OK;
}

extern "C" int logismos_paged_kv_cache_close_seq(logismos_paged_kv_cache_t* c, int seq_id) {
    if (!seq_ok(c, seq_id)) return LOGISMOS_KV_BAD_SEQ;
    release_blocks(c, seq_id);
    c->seq_open[(size_t)seq_id] = 0;
    c->free_seqs.push_back(seq_id);
    return LOGISMOS_KV_OK;
}

extern "C" int logismos_paged_kv_cache_reserve(logismos_paged_kv_cache_t* c, int seq_id,
                                               int64_t total_rows, logismos_stream_t stream) {
    if (!seq_ok(c, seq_id)) return LOGISMOS_KV_BAD_SEQ;
    if (total_rows < 0) return LOGISMOS_KV_SHAPE_MISMATCH;
    if (total_rows > c->max_seq_len()) return LOGISMOS_KV_LEN_OVERFLOW;
    return ensure_blocks(c, seq_id, total_rows, static_cast<hipStream_t>(stream));
}

extern "C" int logismos_paged_kv_cache_put(logismos_paged_kv_cache_t* c, int seq_id, int layer_idx,
                                           const void* k_f16, const void* v_f16, int n_tokens,
                                           logismos_stream_t stream) {
    if (!seq_ok(c, seq_id)) return LOGISMOS_KV_BAD_SEQ;
    if (layer_idx < 0 || layer_idx >= c->layout.num_layers) return LOGISMOS_KV_LAYER_OUT_OF_RANGE;
    if (n_tokens < 0 || (n_tokens > 0 && (!k_f16 || !v_f16))) return LOGISMOS_KV_SHAPE_MISMATCH;
    const int64_t current = c->len(seq_id, layer_idx);
    if (current + n_tokens > c->max_seq_len()) return LOGISMOS_KV_LEN_OVERFLOW;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int rc = ensure_blocks(c, seq_id, current + n_tokens, st);
    if (rc != LOGISMOS_KV_OK) return rc;
    const logismos_status_t e = logismos_launch_kv_append_fp16(
        k_f16, v_f16, c->k_pools[(size_t)layer_idx], c->v_pools[(size_t)layer_idx],
        c->row_dev(seq_id), (int)current, n_tokens, c->layout.num_kv_heads, c->layout.head_dim,
        c->layout.block_size, stream);
    if (e != 0) return LOGISMOS_KV_HIP_ERROR;
    c->len(seq_id, layer_idx) = current + n_tokens;
    return LOGISMOS_KV_OK;
}

extern "C" int logismos_paged_kv_cache_advance(logismos_paged_kv_cache_t* c, int seq_id,
                                               int layer_idx, int n_tokens) {
    if (!seq_ok(c, seq_id)) return LOGISMOS_KV_BAD_SEQ;
    if (layer_idx < 0 || layer_idx >= c->layout.num_layers) return LOGISMOS_KV_LAYER_OUT_OF_RANGE;
    if (n_tokens < 0) return LOGISMOS_KV_SHAPE_MISMATCH;
    const int64_t current = c->len(seq_id, layer_idx);
    if (current + n_tokens > (int64_t)c->seq_blocks[(size_t)seq_id] * c->layout.block_size)
        return LOGISMOS_KV_LEN_OVERFLOW;
    c->len(seq_id, layer_idx) = current + n_tokens;
    return LOGISMOS_KV_OK;
}

extern "C" int logismos_paged_kv_cache_get(const logismos_paged_kv_cache_t* c, int seq_id,
                                           int layer_idx, int64_t len, void* k_out_f16,
                                           void* v_out_f16, logismos_stream_t stream) {
    if (!seq_ok(c, seq_id)) return LOGISMOS_KV_BAD_SEQ;
    if (layer_idx < 0 || layer_idx >= c->layout.num_layers) return LOGISMOS_KV_LAYER_OUT_OF_RANGE;
    if (len < 0 || (len > 0 && (!k_out_f16 || !v_out_f16))) return LOGISMOS_KV_SHAPE_MISMATCH;
    const int64_t current = c->lens[(size_t)seq_id * c->layout.num_layers + layer_idx];
    if (len > current) return LOGISMOS_KV_READ_BEYOND_WRITTEN;
    const logismos_status_t e = logismos_launch_kv_gather_fp16(
        c->k_pools[(size_t)layer_idx], c->v_pools[(size_t)layer_idx], c->row_dev(seq_id), k_out_f16,
        v_out_f16, 0, (int)len, c->layout.num_kv_heads, c->layout.head_dim, c->layout.block_size,
        stream);
    return e == 0 ? LOGISMOS_KV_OK : LOGISMOS_KV_HIP_ERROR;
}

extern "C" int64_t logismos_paged_kv_cache_len_of(const logismos_paged_kv_cache_t* c, int seq_id,
                                                  int layer_idx) {
    if (!seq_ok(c, seq_id) || layer_idx < 0 || layer_idx >= c->layout.num_layers) return -1;
    return c->lens[(size_t)seq_id * c->layout.num_layers + layer_idx];
}

extern "C" int logismos_paged_kv_cache_num_layers(const logismos_paged_kv_cache_t* c) {
    return c ? c->layout.num_layers : 0;
}

extern "C" void logismos_paged_kv_cache_reset(logismos_paged_kv_cache_t* c) {
    if (!c) return;
    for (int s = 0; s < c->layout.max_seqs; ++s)
        if (c->seq_open[(size_t)s]) release_blocks(c, s);
}

extern "C" int logismos_paged_kv_cache_free_blocks(const logismos_paged_kv_cache_t* c) {
    return c ? (int)c->free_blocks.size() : 0;
}

extern "C" void* logismos_paged_kv_cache_k_pool(const logismos_paged_kv_cache_t* c, int layer_idx) {
    return (c && layer_idx >= 0 && layer_idx < c->layout.num_layers) ? c->k_pools[(size_t)layer_idx]
                                                                      : nullptr;
}

extern "C" void* logismos_paged_kv_cache_v_pool(const logismos_paged_kv_cache_t* c, int layer_idx) {
    return (c && layer_idx >= 0 && layer_idx < c->layout.num_layers) ? c->v_pools[(size_t)layer_idx]
                                                                      : nullptr;
}

extern "C" const int32_t* logismos_paged_kv_cache_block_tables(const logismos_paged_kv_cache_t* c) {
    return c ? c->bt_dev : nullptr;
}

extern "C" const int32_t* logismos_paged_kv_cache_block_tables_host(
    const logismos_paged_kv_cache_t* c) {
    return c ? c->bt_host : nullptr;
}
