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

A second loop has the step itself take the admitted prompt: its tokens are a chunk of the
packed batch next to the other sequences' single tokens (a mixed chunked-prefill + decode
batch), and its K/V rows are appended by the step's layers instead of being `put`.

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


class _Rig:
    """Device side (cache, weights, step buffers for up to `max_tokens` packed rows) and oracle
    side (its own pools, addressed through the cache's host block table) of one loop."""

    def __init__(self, rng, max_tokens):
        self.rng = rng
        self.row = row = HKV * D
        self.pool_rows = pool_rows = NUM_BLOCKS * BS
        self.T = max_tokens
        # weights, embedding, lm_head: one decode-step problem's worth (its batch part is unused)
        self.cfg, self.layers, self.proto = cfg, layers, proto = workloads.decode_step_problem(
            rng, num_layers=LAYERS, hidden=HIDDEN, hq=HQ, hkv=HKV, inter=INTER, ctx=[1] * SEQS,
            vocab=VOCAB, max_pos=BS * MAX_BLOCKS)
        self.cos, self.sin = proto["cos"], proto["sin"]
        max_pos = self.cos.size // (D // 2)
        assert max_pos >= BS * MAX_BLOCKS

        # ---- device side: the cache owns pools and block tables
        self.cache = cache = PagedKvCache(LAYERS, HKV, D, BS, NUM_BLOCKS, SEQS, MAX_BLOCKS)
        self.stream = hip.Stream()
        for l in range(LAYERS):
            _memset(cache.k_pool(l), pool_rows * row * 2)
            _memset(cache.v_pool(l), pool_rows * row * 2)
        self.keep = keep = []

        def w3(t):
            bufs = [_dev(t[0]), _dev(np.ascontiguousarray(t[1]).view(np.uint16)),
                    _dev(np.ascontiguousarray(t[2]).view(np.uint16))]
            keep.extend(bufs)
            return kernels.Q4Weight(*[b.ptr.value for b in bufs])

        self.d_layers = d_layers = (kernels.DecodeLayer * LAYERS)()
        for l, L in enumerate(layers):
            n1, n2 = _dev(L["norm1"]), _dev(L["norm2"])
            keep += [n1, n2]
            d_layers[l].norm1_w_f32, d_layers[l].norm2_w_f32 = n1.ptr.value, n2.ptr.value
            for name in ("qkv", "o", "gate_up", "down"):
                setattr(d_layers[l], name, w3(L[name]))
            d_layers[l].k_pool_f16 = cache.k_pool(l).value
            d_layers[l].v_pool_f16 = cache.v_pool(l).value
        self.head = w3(proto["lm_head"])
        self.d_embed = _dev(proto["embed_table"])
        self.d_cfg = kernels.DecodeConfig(LAYERS, HIDDEN, HQ, HKV, D, INTER, cfg["eps"], BS,
                                          MAX_BLOCKS, max_pos, VOCAB, 0)
        self.num_splits = 3
        T = max_tokens
        self.d_h = hip.DeviceBuffer(T * HIDDEN * 4)
        self.d_out = hip.DeviceBuffer(T * HIDDEN * 2)
        self.d_logits = hip.DeviceBuffer(T * VOCAB * 4)
        self.d_tok = hip.DeviceBuffer(T * 4)     # input of a step, overwritten by its output
        self.d_new = hip.DeviceBuffer(SEQS * 4)  # new tokens per sequence
        self.d_prior = hip.DeviceBuffer(SEQS * 4)
        self.d_pos = hip.DeviceBuffer(T * 4)     # position of every packed row
        self.d_cu, self.d_ctx = hip.DeviceBuffer((SEQS + 1) * 4), hip.DeviceBuffer(SEQS * 4)
        self.d_slots = hip.DeviceBuffer(T * 8)
        self.d_cos, self.d_sin = _dev(self.cos), _dev(self.sin)
        self.d_fnorm = _dev(proto["final_norm"])

        # ---- oracle side
        self.o_layers = copy.deepcopy(layers)
        for L in self.o_layers:
            L["k_pool"] = np.zeros((pool_rows, row), np.float16)
            L["v_pool"] = np.zeros((pool_rows, row), np.float16)
        self.exact = np.zeros((LAYERS, pool_rows), bool)   # rows last written by a `put`
        self.approx = np.zeros((LAYERS, pool_rows), bool)  # rows last written by a step
        self.clear_total = 0

    def slots_of(self, seq, start, n):
        bt = self.cache.block_tables_host()[seq]
        pos = np.arange(start, start + n)
        return bt[pos // BS].astype(np.int64) * BS + pos % BS

    def admit(self, prompt_len):
        """open a sequence, put its prompt's K/V rows (device and oracle), return its id"""
        s = self.cache.open_seq()
        for l in range(LAYERS):
            k = self.rng.standard_normal((prompt_len, self.row), np.float32).astype(np.float16)
            v = self.rng.standard_normal((prompt_len, self.row), np.float32).astype(np.float16)
            dk, dv = _dev(k), _dev(v)
            self.keep.extend([dk, dv])
            self.cache.put(s, l, dk, dv, prompt_len, self.stream)
            sl = self.slots_of(s, 0, prompt_len)
            self.o_layers[l]["k_pool"][sl], self.o_layers[l]["v_pool"][sl] = k, v
            self.exact[l, sl], self.approx[l, sl] = True, False
        return s

    def step(self, lens, new, tok_in, what):
        """One step on the device and on the oracle: sequence s has lens[s] cached rows and
        new[s] new tokens (ids tok_in, packed).  Checks packing (bit-exact), states, logits and
        the token choice; returns the tokens the step chose for every packed row."""
        cache, stream = self.cache, self.stream
        new = np.asarray(new, np.int32)
        prior = np.asarray(lens, np.int32)
        t = int(new.sum())
        assert t <= self.T and len(tok_in) == t
        for s in range(SEQS):
            cache.reserve(s, lens[s] + int(new[s]), stream)
            assert cache.len_of(s, 0) == lens[s] == cache.len_of(s, LAYERS - 1)
        positions = np.concatenate([np.arange(p, p + n) for p, n in zip(prior, new)]).astype(np.int32)
        self.d_new.copy_from_host(new)
        self.d_prior.copy_from_host(prior)
        self.d_pos.copy_from_host(positions)
        self.d_tok.copy_from_host(np.asarray(tok_in, np.uint32))
        kernels.launch_pack_ragged(self.d_new, self.d_prior, cache.block_tables(), self.d_cu,
                                   self.d_slots, self.d_ctx, SEQS, BS, MAX_BLOCKS, stream)
        ws_bytes = kernels.decode_step_workspace_bytes_tokens(self.d_cfg, SEQS, t,
                                                              self.num_splits)
        assert ws_bytes > 0   # 0: a geometry the step executor refuses
        d_ws = hip.DeviceBuffer(ws_bytes)
        b = kernels.DecodeBatch(
            self.d_h.ptr.value, self.d_out.ptr.value, self.d_fnorm.ptr.value,
            cache.block_tables().value, self.d_cu.ptr.value, self.d_ctx.ptr.value,
            self.d_pos.ptr.value, self.d_slots.ptr.value, self.d_cos.ptr.value,
            self.d_sin.ptr.value, SEQS, self.num_splits)
        b.token_ids = self.d_tok.ptr.value
        b.embed_table_bf16 = self.d_embed.ptr.value
        b.lm_head = C.pointer(self.head)
        b.out_tokens_u32 = self.d_tok.ptr.value
        b.logits_f32 = self.d_logits.ptr.value
        if t != SEQS:
            b.total_tokens, b.max_seqlen_q = t, int(new.max())
        kernels.launch_decode_step(self.d_cfg, self.d_layers, b, d_ws, stream)
        stream.synchronize()
        for s in range(SEQS):
            for l in range(LAYERS):
                cache.advance(s, l, int(new[s]))

        # ---- the same step on the oracle, from the same input tokens
        bt = cache.block_tables_host()[:SEQS]
        cu, slots, ctx_lens, _ = O.pack_ragged(new, prior, bt, BS)
        # packing is integer work: bit-exact
        assert np.array_equal(self.d_cu.to_numpy(np.int32, (SEQS + 1,)), cu)
        assert np.array_equal(self.d_slots.to_numpy(np.int64, (t,)), slots)
        assert np.array_equal(self.d_ctx.to_numpy(np.int32, (SEQS,)), ctx_lens)
        assert np.array_equal(slots, np.concatenate(
            [self.slots_of(s, lens[s], int(new[s])) for s in range(SEQS)]))
        batch = dict(h=np.zeros((t, HIDDEN), np.float32), block_tables=bt, cu_seqlens=cu,
                     context_lens=ctx_lens, positions=positions, slots=slots, cos=self.cos,
                     sin=self.sin, final_norm=self.proto["final_norm"],
                     token_ids=np.asarray(tok_in, np.uint32),
                     embed_table=self.proto["embed_table"], lm_head=self.proto["lm_head"])
        want_out = O.bf16_bits_to_f32(OS.decode_step(self.cfg, self.o_layers, batch))
        for l in range(LAYERS):
            self.exact[l, slots], self.approx[l, slots] = False, True

        got_out = O.bf16_bits_to_f32(self.d_out.to_numpy(np.uint16, (t, HIDDEN)))
        assert _rel_l2(got_out, want_out) < 5e-3, what
        assert np.all(np.abs(got_out - want_out) <= 2e-2 + 3e-2 * np.abs(want_out)), what
        logits = self.d_logits.to_numpy(np.float32, (t, VOCAB))
        assert _rel_l2(logits, batch["logits"]) < 6e-3, what
        tok_out = self.d_tok.to_numpy(np.uint32, (t,))
        # the selection rule exactly, on the logits the step stored ...
        assert np.array_equal(tok_out, np.array([O.greedy(x) for x in logits], np.uint32))
        # ... and the oracle's token wherever its winner is clear of the logit error
        err = float(np.abs(logits - batch["logits"]).max())
        top2 = np.sort(batch["logits"], axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 4 * err
        self.clear_total += int(clear.sum())
        assert np.array_equal(tok_out[clear], batch["tokens"][clear]), what
        return tok_out, cu

    def check_pools_and_blocks(self, lens):
        """rows nobody wrote are still zero and rows last written by a put hold the put's
        bytes (integer work, bit-exact); rows appended by the steps agree with the oracle's to
        the fp16 tolerance of the step; every live sequence holds ceil(len / block) blocks"""
        cache, pool_rows, row = self.cache, self.pool_rows, self.row
        for l in range(LAYERS):
            for name, ptr in (("k_pool", cache.k_pool(l)), ("v_pool", cache.v_pool(l))):
                got = hip.DevicePtrView(ptr, pool_rows * row * 2).to_numpy(np.float16,
                                                                          (pool_rows, row))
                want = self.o_layers[l][name]
                exact, approx = self.exact[l], self.approx[l]
                still = ~(exact | approx)
                assert still.any() and not got[still].view(np.uint16).any()
                assert np.array_equal(got[exact].view(np.uint16), want[exact].view(np.uint16))
                assert approx.sum() >= SEQS
                assert_parity(got[approx], want[approx], max_abs=4e-3, max_rel=1e-2,
                              what=f"layer {l} {name}: rows appended by the steps")
        assert cache.free_blocks() == NUM_BLOCKS - sum(-(-n // BS) for n in lens)
        cache.reset()
        assert cache.free_blocks() == NUM_BLOCKS and cache.len_of(0, 0) == 0
        cache.close()


def test_five_steps_with_one_sequence_retired_and_one_admitted_per_step():
    rng = np.random.default_rng(77)
    rig = _Rig(rng, SEQS)
    cache = rig.cache
    prompts = [5, 40, 17, 63, 100, 31]
    seqs = [rig.admit(p) for p in prompts]
    assert seqs == list(range(SEQS))  # batch row s reads block-table row s
    tokens = rng.integers(0, VOCAB, size=SEQS, dtype=np.uint32)
    lens = list(prompts)
    assert cache.free_blocks() == NUM_BLOCKS - sum(-(-p // BS) for p in prompts)

    for step in range(STEPS):
        # ---- churn: the sequence in slot `step` finishes, a new one is admitted in its place
        retire = step % SEQS
        held = -(-lens[retire] // BS)
        free0 = cache.free_blocks()
        cache.close_seq(retire)
        assert cache.free_blocks() == free0 + held and cache.len_of(retire, 0) is None
        new_len = int(rng.integers(3, 70))
        assert rig.admit(new_len) == retire  # the freed slot, and blocks from the free list
        lens[retire] = new_len
        tokens[retire] = rng.integers(0, VOCAB)
        # the chosen tokens are the next step's input
        tokens, _ = rig.step(lens, [1] * SEQS, tokens, f"step {step}")
        lens = [n + 1 for n in lens]
        for s in range(SEQS):
            assert cache.len_of(s, 0) == lens[s]

    assert rig.clear_total >= STEPS * SEQS // 2
    rig.check_pools_and_blocks(lens)


def test_steps_that_take_the_admitted_prompt_as_a_chunk_of_the_batch():
    """The same churn with the admitted sequence's prompt processed BY the step: its tokens
    are a chunk of the packed batch next to the other sequences' single tokens (a mixed
    chunked-prefill + decode batch, causal inside the chunk), its K/V rows are appended by the
    step's layers, and its last row's choice is its first generated token."""
    rng = np.random.default_rng(78)
    rig = _Rig(rng, 32)
    cache = rig.cache
    prompts = [9, 33, 17, 50, 70, 21]
    assert [rig.admit(p) for p in prompts] == list(range(SEQS))
    lens = list(prompts)
    last = rng.integers(0, VOCAB, size=SEQS, dtype=np.uint32)  # each sequence's latest token
    for step in range(4):
        retire = (2 * step + 1) % SEQS
        cache.close_seq(retire)
        assert cache.open_seq() == retire and cache.len_of(retire, 0) == 0
        lens[retire] = 0
        chunk = int(rng.integers(2, 32 - (SEQS - 1) + 1))      # 2 .. 27 prompt tokens
        prompt = rng.integers(0, VOCAB, size=chunk, dtype=np.uint32)
        new = [1] * SEQS
        new[retire] = chunk
        tok_in = np.concatenate([prompt if s == retire else last[s:s + 1] for s in range(SEQS)])
        tok_out, cu = rig.step(lens, new, tok_in, f"step {step}, chunk of {chunk}")
        last = tok_out[cu[1:] - 1]                              # the last row of every sequence
        lens = [n + k for n, k in zip(lens, new)]
        for s in range(SEQS):
            assert cache.len_of(s, 0) == lens[s]
    assert rig.clear_total >= 20
    rig.check_pools_and_blocks(lens)


def test_twelve_steps_of_random_churn():
    """A longer loop with the schedule drawn: every step retires none, one or two sequences
    (always one that would outgrow its block table), and admits each replacement either with
    its prompt `put` beforehand or as a chunk of the step's own batch; the blocks a retired
    sequence held go back to the free list and out again many times over."""
    rng = np.random.default_rng(79)
    rig = _Rig(rng, 32)
    cache = rig.cache
    prompts = [12, 45, 3, 60, 28, 16]
    assert [rig.admit(p) for p in prompts] == list(range(SEQS))
    lens = list(prompts)
    last = rng.integers(0, VOCAB, size=SEQS, dtype=np.uint32)
    retired = 0
    for step in range(12):
        out = [s for s in range(SEQS) if lens[s] + 1 > 80]          # would outgrow 6 blocks
        extra = [int(s) for s in rng.permutation(SEQS)[:int(rng.integers(0, 3))]]
        out = list(dict.fromkeys(out + extra))[:3]
        new = [1] * SEQS
        tok = {s: last[s:s + 1] for s in range(SEQS)}
        room = 32 - SEQS                                            # rows left for chunks
        for s in out:
            held = -(-lens[s] // BS)
            free0 = cache.free_blocks()
            cache.close_seq(s)
            assert cache.free_blocks() == free0 + held
            retired += 1
            if room >= 2 and rng.integers(0, 2):
                # the step takes the prompt itself: a chunk of its batch
                assert cache.open_seq() == s and cache.len_of(s, 0) == 0
                chunk = int(rng.integers(2, min(room, 20) + 1))
                room -= chunk - 1
                lens[s], new[s] = 0, chunk
                tok[s] = rng.integers(0, VOCAB, size=chunk, dtype=np.uint32)
            else:
                plen = int(rng.integers(3, 50))
                assert rig.admit(plen) == s
                lens[s] = plen
                tok[s] = rng.integers(0, VOCAB, size=1, dtype=np.uint32)
        tok_in = np.concatenate([tok[s] for s in range(SEQS)])
        tok_out, cu = rig.step(lens, new, tok_in, f"step {step}, retired {out}, new {new}")
        last = tok_out[cu[1:] - 1]
        lens = [n + k for n, k in zip(lens, new)]
        for s in range(SEQS):
            assert cache.len_of(s, 0) == lens[s]
        assert cache.free_blocks() == NUM_BLOCKS - sum(-(-n // BS) for n in lens)
    assert retired >= 8 and rig.clear_total >= 50
    rig.check_pools_and_blocks(lens)
