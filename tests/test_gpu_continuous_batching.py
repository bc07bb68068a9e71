"""A continuous-batching decode loop on the GPU, through the C ABI: the churn of the
baseline's full-step workload (one sequence finishing and one admitted per step) with the
paged cache driving the block tables.

Every step: the oldest live sequence is closed and a new one opened in its slot
(`logismos_paged_kv_cache_{close_seq,open_seq}`: its blocks go back to the free list and are
handed out again), the admitted prompt's K/V rows are `put` (its prefill is not part of a
decode step), every live sequence `reserve`s one more row, `logismos_launch_pack_ragged`
builds cu_seqlens / slot mapping / context lengths on the device from the cache's own block
tables, `logismos_launch_decode_step` runs token ids -> token ids (embedding lookup, the
layers with their K/V append, vocabulary projection + greedy), the chosen tokens stay on the
device as the next step's input, and `advance` records the appended rows.

The CPU oracle runs the same schedule over its own pools laid out by the cache's host block
table.  The chain mirrors the reference's integration test of cache put/get/reset with greedy
decode (crates/logismos/tests/phase_2_pipeline.rs:54-182) over the `KvCache` trait
(crates/cache/src/lib.rs:57-82).
"""
import copy
import ctypes as C

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from logismos_amd import hip, kernels
from logismos_amd.paged_kv_cache import PagedKvCache
from tests import workloads
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu

LAYERS, HIDDEN, HQ, HKV, D, INTER, BS, VOCAB = 2, 1024, 4, 2, 128, 1024, 16, 1000
SEQS, STEPS, MAX_BLOCKS, NUM_BLOCKS = 6, 5, 8, 40


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _dev(a):
    return hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _memset(ptr, nbytes):
    hip.check(hip._runtime().hipMemset(ptr, C.c_int(0), C.c_size_t(nbytes)), "hipMemset")


def test_five_steps_with_one_sequence_retired_and_one_admitted_per_step():
    rng = np.random.default_rng(77)
    row = HKV * D
    pool_rows = NUM_BLOCKS * BS
    # weights, embedding, lm_head: one decode-step problem's worth (its batch part is unused)
    cfg, layers, proto = workloads.decode_step_problem(
        rng, num_layers=LAYERS, hidden=HIDDEN, hq=HQ, hkv=HKV, inter=INTER, ctx=[1] * SEQS,
        vocab=VOCAB, max_pos=BS * MAX_BLOCKS)
    cos, sin = proto["cos"], proto["sin"]
    max_pos = cos.size // (D // 2)
    assert max_pos >= BS * MAX_BLOCKS

    # ---- device side: the cache owns pools and block tables
    cache = PagedKvCache(LAYERS, HKV, D, BS, NUM_BLOCKS, SEQS, MAX_BLOCKS)
    stream = hip.Stream()
    for l in range(LAYERS):
        _memset(cache.k_pool(l), pool_rows * row * 2)
        _memset(cache.v_pool(l), pool_rows * row * 2)
    keep = []

    def w3(t):
        bufs = [_dev(t[0]), _dev(np.ascontiguousarray(t[1]).view(np.uint16)),
                _dev(np.ascontiguousarray(t[2]).view(np.uint16))]
        keep.extend(bufs)
        return kernels.Q4Weight(*[b.ptr.value for b in bufs])

    d_layers = (kernels.DecodeLayer * LAYERS)()
    for l, L in enumerate(layers):
        n1, n2 = _dev(L["norm1"]), _dev(L["norm2"])
        keep += [n1, n2]
        d_layers[l].norm1_w_f32, d_layers[l].norm2_w_f32 = n1.ptr.value, n2.ptr.value
        for name in ("qkv", "o", "gate_up", "down"):
            setattr(d_layers[l], name, w3(L[name]))
        d_layers[l].k_pool_f16 = cache.k_pool(l).value
        d_layers[l].v_pool_f16 = cache.v_pool(l).value
    head = w3(proto["lm_head"])
    d_embed = _dev(proto["embed_table"])
    d_cfg = kernels.DecodeConfig(LAYERS, HIDDEN, HQ, HKV, D, INTER, cfg["eps"], BS, MAX_BLOCKS,
                                 max_pos, VOCAB, 0)
    num_splits = 3
    d_h = hip.DeviceBuffer(SEQS * HIDDEN * 4)
    d_out = hip.DeviceBuffer(SEQS * HIDDEN * 2)
    d_logits = hip.DeviceBuffer(SEQS * VOCAB * 4)
    d_tok = hip.DeviceBuffer(SEQS * 4)          # input of a step, overwritten by its output
    d_ones = _dev(np.ones(SEQS, np.int32))
    d_prior = hip.DeviceBuffer(SEQS * 4)        # prior context = position of the new token
    d_cu, d_ctx = hip.DeviceBuffer((SEQS + 1) * 4), hip.DeviceBuffer(SEQS * 4)
    d_slots = hip.DeviceBuffer(SEQS * 8)
    d_cos, d_sin, d_fnorm = _dev(cos), _dev(sin), _dev(proto["final_norm"])
    ws_bytes = kernels.decode_step_workspace_bytes(d_cfg, SEQS, num_splits)
    assert ws_bytes > 0   # 0: a geometry the step executor refuses
    d_ws = hip.DeviceBuffer(ws_bytes)
    d_batch = kernels.DecodeBatch(
        d_h.ptr.value, d_out.ptr.value, d_fnorm.ptr.value, cache.block_tables().value,
        d_cu.ptr.value, d_ctx.ptr.value, d_prior.ptr.value, d_slots.ptr.value, d_cos.ptr.value,
        d_sin.ptr.value, SEQS, num_splits)
    d_batch.token_ids = d_tok.ptr.value
    d_batch.embed_table_bf16 = d_embed.ptr.value
    d_batch.lm_head = C.pointer(head)
    d_batch.out_tokens_u32 = d_tok.ptr.value
    d_batch.logits_f32 = d_logits.ptr.value

    # ---- oracle side: its own pools, addressed through the cache's host block table
    o_layers = copy.deepcopy(layers)
    for L in o_layers:
        L["k_pool"] = np.zeros((pool_rows, row), np.float16)
        L["v_pool"] = np.zeros((pool_rows, row), np.float16)
    exact = np.zeros((LAYERS, pool_rows), bool)   # rows last written by a `put`: bit-exact
    approx = np.zeros((LAYERS, pool_rows), bool)  # rows last written by a step's K/V append

    def slots_of(seq, start, n):
        bt = cache.block_tables_host()[seq]
        pos = np.arange(start, start + n)
        return bt[pos // BS].astype(np.int64) * BS + pos % BS

    def admit(prompt_len):
        """open a sequence, put its prompt's K/V rows (device and oracle), return its id"""
        s = cache.open_seq()
        for l in range(LAYERS):
            k = rng.standard_normal((prompt_len, row), np.float32).astype(np.float16)
            v = rng.standard_normal((prompt_len, row), np.float32).astype(np.float16)
            dk, dv = _dev(k), _dev(v)
            keep.extend([dk, dv])
            cache.put(s, l, dk, dv, prompt_len, stream)
            sl = slots_of(s, 0, prompt_len)
            o_layers[l]["k_pool"][sl], o_layers[l]["v_pool"][sl] = k, v
            exact[l, sl], approx[l, sl] = True, False
        return s

    prompts = [5, 40, 17, 63, 100, 31]
    seqs = [admit(p) for p in prompts]
    assert seqs == list(range(SEQS))  # batch row s reads block-table row s
    tokens = rng.integers(0, VOCAB, size=SEQS, dtype=np.uint32)
    d_tok.copy_from_host(tokens)
    lens = list(prompts)
    free_after_admission = cache.free_blocks()
    assert free_after_admission == NUM_BLOCKS - sum(-(-p // BS) for p in prompts)
    clear_total = 0

    for step in range(STEPS):
        # ---- churn: the sequence in slot `step` finishes, a new one is admitted in its place
        retire = step % SEQS
        held = -(-lens[retire] // BS)
        free0 = cache.free_blocks()
        cache.close_seq(retire)
        assert cache.free_blocks() == free0 + held and cache.len_of(retire, 0) is None
        new_len = int(rng.integers(3, 70))
        assert admit(new_len) == retire      # the freed slot, and blocks from the free list
        lens[retire] = new_len
        first = np.array([rng.integers(0, VOCAB)], np.uint32)
        stream.synchronize()                 # (the step before wrote d_tok on this stream)
        d_tok.copy_from_host(first, dst_offset=4 * retire)

        # ---- the step on the device
        for s in range(SEQS):
            cache.reserve(s, lens[s] + 1, stream)
            assert cache.len_of(s, 0) == lens[s] == cache.len_of(s, LAYERS - 1)
        d_prior.copy_from_host(np.asarray(lens, np.int32))
        tok_in = d_tok.to_numpy(np.uint32, (SEQS,))   # what the step's embedding lookup reads
        kernels.launch_pack_ragged(d_ones, d_prior, cache.block_tables(), d_cu, d_slots, d_ctx,
                                   SEQS, BS, MAX_BLOCKS, stream)
        kernels.launch_decode_step(d_cfg, d_layers, d_batch, d_ws, stream)
        stream.synchronize()
        for s in range(SEQS):
            for l in range(LAYERS):
                cache.advance(s, l, 1)

        # ---- the same step on the oracle, from the same input tokens
        bt = cache.block_tables_host()[:SEQS]
        prior = np.asarray(lens, np.int32)
        cu, slots, ctx_lens, _ = O.pack_ragged(np.ones(SEQS, np.int32), prior, bt, BS)
        # packing is integer work: bit-exact
        assert np.array_equal(d_cu.to_numpy(np.int32, (SEQS + 1,)), cu)
        assert np.array_equal(d_slots.to_numpy(np.int64, (SEQS,)), slots)
        assert np.array_equal(d_ctx.to_numpy(np.int32, (SEQS,)), ctx_lens)
        assert np.array_equal(slots, [slots_of(s, lens[s], 1)[0] for s in range(SEQS)])
        batch = dict(h=np.zeros((SEQS, HIDDEN), np.float32), block_tables=bt, cu_seqlens=cu,
                     context_lens=ctx_lens, positions=prior, slots=slots, cos=cos, sin=sin,
                     final_norm=proto["final_norm"], token_ids=tok_in,
                     embed_table=proto["embed_table"], lm_head=proto["lm_head"])
        want_out = O.bf16_bits_to_f32(OS.decode_step(cfg, o_layers, batch))
        for l in range(LAYERS):
            exact[l, slots], approx[l, slots] = False, True

        got_out = O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (SEQS, HIDDEN)))
        assert _rel_l2(got_out, want_out) < 5e-3, step
        assert np.all(np.abs(got_out - want_out) <= 2e-2 + 3e-2 * np.abs(want_out)), step
        logits = d_logits.to_numpy(np.float32, (SEQS, VOCAB))
        assert _rel_l2(logits, batch["logits"]) < 6e-3, step
        tok_out = d_tok.to_numpy(np.uint32, (SEQS,))
        # the selection rule exactly, on the logits the step stored ...
        assert np.array_equal(tok_out, np.array([O.greedy(x) for x in logits], np.uint32))
        # ... and the oracle's token wherever its winner is clear of the logit error
        err = float(np.abs(logits - batch["logits"]).max())
        top2 = np.sort(batch["logits"], axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 4 * err
        clear_total += int(clear.sum())
        assert np.array_equal(tok_out[clear], batch["tokens"][clear]), step
        lens = [n + 1 for n in lens]
        for s in range(SEQS):
            assert cache.len_of(s, 0) == lens[s]

    assert clear_total >= STEPS * SEQS // 2
    # ---- the pools after the loop: rows nobody wrote are still zero and rows last written by
    # a put hold the put's bytes (integer work, bit-exact); rows appended by the steps agree
    # with the oracle's to the fp16 tolerance of the step
    for l in range(LAYERS):
        for name, ptr in (("k_pool", cache.k_pool(l)), ("v_pool", cache.v_pool(l))):
            got = hip.DevicePtrView(ptr, pool_rows * row * 2).to_numpy(np.float16, (pool_rows, row))
            want = o_layers[l][name]
            still = ~(exact[l] | approx[l])
            assert still.any() and not got[still].view(np.uint16).any()
            assert np.array_equal(got[exact[l]].view(np.uint16), want[exact[l]].view(np.uint16))
            assert approx[l].sum() >= SEQS
            assert_parity(got[approx[l]], want[approx[l]], max_abs=4e-3, max_rel=1e-2,
                          what=f"layer {l} {name}: rows appended by the steps")
    # blocks: every live sequence holds ceil(len / block) of them, the rest are free
    assert cache.free_blocks() == NUM_BLOCKS - sum(-(-n // BS) for n in lens)
    cache.reset()
    assert cache.free_blocks() == NUM_BLOCKS and cache.len_of(0, 0) == 0
    cache.close()
