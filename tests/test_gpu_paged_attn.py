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
