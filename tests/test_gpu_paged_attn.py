"""GPU parity: ragged paged attention vs the CPU oracle, through the C ABI.

Tolerance (fp16 outputs, fp32 accumulation): 2e-3 max-abs or 1e-2 relative.
"""
import numpy as np
import pytest

import oracle as O
from tests import workloads
from tests.gpu_harness import PagedAttnRunner, assert_parity

pytestmark = pytest.mark.gpu


def _oracle(c, causal=True):
    return O.paged_attn_varlen_fp16(c["q"], c["k_pool"], c["v_pool"], c["block_tables"],
                                    c["cu_seqlens"], c["context_lens"], c["hq"], c["hkv"], c["d"],
                                    c["block_size"], c["scale"], causal)


def _check(c, num_splits=None, causal=True, what=""):
    r = PagedAttnRunner(c, num_splits=num_splits, causal=causal)
    r.launch()
    got = r.result()
    return assert_parity(got, _oracle(c, causal), what=what)


def test_config2_ragged_decode_matches_oracle():
    c = workloads.config2()
    _check(c, what="config 2")


@pytest.mark.parametrize("num_splits", [1, 2, 3, 8, 128])
def test_result_is_invariant_to_the_number_of_splits(num_splits):
    c = workloads.config2(seed=77)
    _check(c, num_splits=num_splits, what=f"config 2, {num_splits} splits")


def test_split_count_changes_nothing_beyond_rounding():
    c = workloads.config2(seed=78)
    outs = []
    for ns in (1, 2, 8):
        r = PagedAttnRunner(c, num_splits=ns)
        r.launch()
        outs.append(r.result().astype(np.float32))
    assert np.abs(outs[0] - outs[1]).max() <= 2e-3
    assert np.abs(outs[0] - outs[2]).max() <= 2e-3


@pytest.mark.parametrize("hq,hkv", [(1, 1), (2, 2), (4, 2), (12, 2), (12, 4), (32, 8), (8, 1),
                                    (5, 1), (14, 2)])
def test_gqa_group_sizes(hq, hkv):
    rng = np.random.default_rng(hq * 100 + hkv)
    ctx = np.array([1, 2, 15, 16, 17, 31, 33, 100, 257])
    c = workloads.paged_case(rng, np.ones(len(ctx), np.int32), ctx - 1, hq=hq, hkv=hkv)
    _check(c, what=f"gqa {hq}/{hkv}")
    _check(c, num_splits=4, what=f"gqa {hq}/{hkv} split 4")


@pytest.mark.parametrize("block_size", [16, 32, 64])
def test_block_sizes(block_size):
    rng = np.random.default_rng(block_size)
    ctx = np.array([1, 16, 17, 63, 64, 65, 200, 511])
    c = workloads.paged_case(rng, np.ones(len(ctx), np.int32), ctx - 1, hq=8, hkv=2,
                             block_size=block_size)
    _check(c, what=f"block_size {block_size}")
    _check(c, num_splits=5, what=f"block_size {block_size} split 5")


def test_special_cases():
    rng = np.random.default_rng(3)
    # ctx = 1: out = v of the only key, exactly
    c = workloads.paged_case(rng, [1, 1], [0, 0], hq=4, hkv=2)
    r = PagedAttnRunner(c)
    r.launch()
    got = r.result()
    for s in range(2):
        v0 = c["v_pool"][c["block_tables"][s, 0] * 16].reshape(2, 128)
        assert np.array_equal(got[s], v0[[0, 0, 1, 1]])
    # all keys equal: out = mean(v)
    c = workloads.paged_case(rng, [1], [99], hq=4, hkv=2)
    c["k_pool"][:] = c["k_pool"][0]
    _check(c, what="equal keys")
    # long context with a peaked softmax (large scale): argmax behaviour survives splitting
    c = workloads.paged_case(rng, [1], [4999], hq=8, hkv=2)
    c["scale"] = 4.0
    _check(c, num_splits=16, what="peaked softmax")


def test_mixed_chunked_prefill_and_decode_small():
    rng = np.random.default_rng(4)
    new = [1, 5, 1, 33, 16, 1, 2]
    prior = [300, 0, 0, 40, 16, 17, 1000]
    c = workloads.paged_case(rng, new, prior, hq=8, hkv=2)
    _check(c, causal=True, what="mixed causal")
    _check(c, causal=False, what="mixed non-causal")
    _check(c, causal=True, num_splits=7, what="mixed causal split 7")


@pytest.mark.parametrize("hq,hkv", [(4, 4), (4, 2), (12, 4), (8, 2), (10, 2), (12, 2), (14, 2),
                                    (16, 2), (32, 8)])
def test_chunked_prefill_gqa_group_sizes(hq, hkv):
    # chunk lengths on both sides of the query-tile and key-tile edges, with and
    # without prior context, next to decode rows
    rng = np.random.default_rng(40 + hq + hkv)
    new = [31, 1, 32, 33, 2, 64, 65, 129, 7]
    prior = [0, 77, 5, 100, 31, 0, 333, 17, 1]
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv)
    _check(c, causal=True, what=f"prefill causal {hq}/{hkv}")
    _check(c, causal=False, what=f"prefill non-causal {hq}/{hkv}")


@pytest.mark.parametrize("block_size", [16, 32, 128])
def test_chunked_prefill_block_sizes(block_size):
    rng = np.random.default_rng(50 + block_size)
    c = workloads.paged_case(rng, [100, 1, 40], [300, 50, 0], hq=8, hkv=2, block_size=block_size)
    _check(c, what=f"prefill block {block_size}")


def test_chunked_prefill_512_token_chunks_with_prior_context():
    # config-4 chunk shape at Qwen3-8B head geometry, contexts the oracle finishes quickly
    rng = np.random.default_rng(41)
    c = workloads.paged_case(rng, [512, 1, 512, 200, 1], [0, 700, 1000, 77, 12], hq=32, hkv=8)
    _check(c, what="512-token chunks")


def test_chunked_prefill_with_a_block_table_wider_than_the_kernels_lds_copy():
    # the prefill kernel keeps 8192 entries of a sequence's block-table row in LDS; the keys
    # of the blocks beyond that (here the last 3 of 8195) take the ids from memory.  Pools
    # repeat 5003 random rows (a 131 k-key pool takes a while to draw), which a wrong block
    # id does not survive: the new tokens see all 131 k keys.
    rng = np.random.default_rng(43)
    c = workloads.paged_case(rng, [8, 1], [8192 * 16 + 40, 9], hq=1, hkv=1,
                             pool_period_rows=5003, spare_frac=0.0)
    assert c["max_blocks"] > 8192
    _check(c, what="block table wider than 8192 entries")


def test_chunked_prefill_peaked_softmax():
    rng = np.random.default_rng(42)
    c = workloads.paged_case(rng, [96, 1], [200, 10], hq=8, hkv=2)
    c["scale"] = 4.0
    _check(c, what="prefill peaked softmax")


def test_config4_prefill_rows_agree_with_decode_rows_at_full_size():
    # Size-independent property at config 4's full size: under the causal mask, new
    # token i of a chunk attends to exactly the keys a decode row with context
    # prior + i + 1 would, so the prefill kernel must reproduce what the (oracle-checked)
    # decode kernel gives for the same query over the same block table.
    c = workloads.config4()
    r = PagedAttnRunner(c)
    r.launch()
    got = r.result()
    assert np.isfinite(got.astype(np.float32)).all()
    rng = np.random.default_rng(43)
    pre = [s for s in range(len(c["new_tokens"])) if c["new_tokens"][s] > 1]
    picks = [(s, int(i)) for s in pre for i in rng.choice(int(c["new_tokens"][s]), 3, replace=False)]
    picks += [(pre[0], 0), (pre[-1], int(c["new_tokens"][pre[-1]]) - 1)]
    d = dict(c)
    d["q"] = np.stack([c["q"][c["cu_seqlens"][s] + i] for s, i in picks])
    d["block_tables"] = np.stack([c["block_tables"][s] for s, _ in picks])
    d["new_tokens"] = np.ones(len(picks), np.int32)
    d["context_lens"] = np.array([c["prior_ctx"][s] + i + 1 for s, i in picks], np.int32)
    d["prior_ctx"] = d["context_lens"] - 1
    d["cu_seqlens"] = np.arange(len(picks) + 1, dtype=np.int32)
    rd = PagedAttnRunner(d)
    rd.launch()
    want = rd.result()
    rows = np.stack([got[c["cu_seqlens"][s] + i] for s, i in picks])
    assert_parity(rows, want, what="config 4 prefill rows vs decode rows")
    # and the decode rows of the mixed batch against the oracle on a reduced copy
    dec = [s for s in range(len(c["new_tokens"])) if c["new_tokens"][s] == 1][:6]
    e = dict(c)
    e["q"] = np.stack([c["q"][c["cu_seqlens"][s]] for s in dec])
    e["block_tables"] = np.stack([c["block_tables"][s] for s in dec])
    e["new_tokens"] = np.ones(len(dec), np.int32)
    e["context_lens"] = c["context_lens"][dec]
    e["prior_ctx"] = e["context_lens"] - 1
    e["cu_seqlens"] = np.arange(len(dec) + 1, dtype=np.int32)
    want_dec = _oracle(e)
    rows_dec = np.stack([got[c["cu_seqlens"][s]] for s in dec])
    assert_parity(rows_dec, want_dec, what="config 4 decode rows vs oracle")


def test_config4_prefill_chunk_at_full_size_against_the_oracle():
    # one chunk of config 4 at its largest: 512 new tokens behind 8 100 tokens of prior context
    # (the config draws priors from 0..8192), 32 query / 8 KV heads, next to a decode row; pools
    # of distinct random rows, the whole chunk against the CPU oracle
    rng = np.random.default_rng(44)
    c = workloads.paged_case(rng, [512, 1], [8100, 8611], hq=32, hkv=8)
    _check(c, what="512-token chunk, prior 8100")


def test_config5_attention_at_full_size_with_distinct_pool_rows():
    # the decode step's attention at its own size (32 sequences, contexts U[256, 8192], 32 / 8
    # heads) over pools in which no two rows are alike: a gather that is off by any number of
    # rows reads different values
    c = workloads.config5_attention()
    assert int(c["context_lens"].sum()) > 100_000
    _check(c, what="config 5 attention, distinct rows")


@pytest.mark.parametrize("hq,hkv", [(1, 1), (4, 2), (12, 2), (12, 4), (32, 8), (8, 1), (16, 16),
                                    (14, 2)])
def test_balanced_decode_kernel_gqa_group_sizes(hq, hkv):
    # wide block tables put even a small batch on the balanced decode kernel (one stream of
    # key tiles split evenly over the workers): ragged contexts around the tile and worker
    # edges, rows with one visible key, a zero-context row, prefill rows in between
    rng = np.random.default_rng(60 + hq + hkv)
    new = [1, 1, 1, 9, 1, 1, 1, 0, 1, 1]
    prior = [0, 15, 16, 40, 127, 128, 1000, 5, 2047, 333]
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv, min_max_blocks=8192)
    c["context_lens"][9] = 0
    for ns in (2, 5, 64):
        _check(c, num_splits=ns, what=f"balanced {hq}/{hkv} splits {ns}")
    r = PagedAttnRunner(c)
    r.launch()
    got = r.result()
    t = int(c["cu_seqlens"][9])
    assert (got[t] == 0).all()


def test_balanced_decode_kernel_many_short_sequences():
    # more sequences than workers' worth of tiles: most workers cross several sequences
    rng = np.random.default_rng(61)
    n = 300
    prior = rng.integers(0, 40, size=n)
    c = workloads.paged_case(rng, np.ones(n, np.int32), prior, hq=8, hkv=2, min_max_blocks=512)
    _check(c, what="300 short sequences")
    _check(c, num_splits=2, what="300 short sequences, 2 splits")


@pytest.mark.parametrize("seed", [70, 71, 72, 73, 74, 75])
def test_balanced_decode_kernel_random_batches(seed):
    # The balanced kernel splits a stream in which every sequence is preceded by a few units of
    # start-up cost: random batches (2..40 sequences, 1..5000 visible keys) put worker edges on
    # start-up units, on first and last tiles and inside sequences, and give sequences one, two
    # or many pieces to merge
    rng = np.random.default_rng(seed)
    n = int(rng.integers(2, 41))
    prior = np.where(rng.random(n) < 0.3, rng.integers(0, 48, size=n), rng.integers(0, 5000, size=n))
    c = workloads.paged_case(rng, np.ones(n, np.int32), prior, hq=8, hkv=2, min_max_blocks=2048)
    _check(c, what=f"random batch, seed {seed}")
    _check(c, num_splits=3, what=f"random batch, seed {seed}, 3 splits")


def test_zero_context_and_empty_sequences():
    rng = np.random.default_rng(5)
    c = workloads.paged_case(rng, [1, 0, 1, 3], [0, 5, 40, 0], hq=4, hkv=2)
    c["context_lens"][0] = 0  # a decode row with nothing visible
    r = PagedAttnRunner(c)
    r.launch()
    got = r.result()
    want = _oracle(c)
    assert (got[0] == 0).all() and (want[0] == 0).all()
    assert_parity(got, want, what="zero ctx")


def test_long_context_32k_single_sequence():
    # size-independent property at config-4's longest decode context: with all
    # keys equal the output is the mean of V whatever the partitioning
    rng = np.random.default_rng(6)
    c = workloads.paged_case(rng, [1, 1], [32767, 127], hq=32, hkv=8)
    _check(c, what="32k context")


def test_chunked_prefill_sequence_order_ties_and_many_sequences():
    # The prefill kernel takes sequences longest first (ranked inside the kernel): equal
    # contexts must still give each workgroup a different sequence, decode rows and empty
    # chunks rank last, and with more sequences than the ranking handles it falls back to
    # grid order.
    rng = np.random.default_rng(61)
    new = [40] * 12 + [1, 1, 3, 3]
    prior = [60] * 12 + [100, 5, 0, 0]
    c = workloads.paged_case(rng, new, prior, hq=8, hkv=2)
    _check(c, what="prefill, equal contexts")
    n = 530
    new = np.where(np.arange(n) % 3 == 0, 1, 2 + (np.arange(n) % 5)).astype(np.int32)
    prior = (np.arange(n) * 7 % 40).astype(np.int32)
    c = workloads.paged_case(rng, new, prior, hq=4, hkv=2)
    _check(c, what="prefill, 530 sequences")
