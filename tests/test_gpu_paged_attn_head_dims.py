"""GPU parity: ragged paged attention at head widths other than 128 vs the CPU oracle,
through the C ABI (the reference's attention is generic in head_dim,
crates/transformers/src/attention.rs:97-127; its encoders use 64 as well as 128,
crates/transformers/src/modernbert.rs:406).

Tolerance (fp16 outputs, fp32 accumulation): 2e-3 max-abs or 1e-2 relative.
"""
import numpy as np
import pytest

import oracle as O
from logismos_amd import kernels
from tests import workloads
from tests.gpu_harness import PagedAttnRunner, assert_parity

pytestmark = pytest.mark.gpu

HEAD_DIMS = [32, 64, 96, 160, 192, 224, 256]


def _oracle(c, causal=True):
    return O.paged_attn_varlen_fp16(c["q"], c["k_pool"], c["v_pool"], c["block_tables"],
                                    c["cu_seqlens"], c["context_lens"], c["hq"], c["hkv"], c["d"],
                                    c["block_size"], c["scale"], causal)


def _check(c, num_splits=None, causal=True, what=""):
    r = PagedAttnRunner(c, num_splits=num_splits, causal=causal)
    r.launch()
    return assert_parity(r.result(), _oracle(c, causal), what=what)


@pytest.mark.parametrize("d", HEAD_DIMS)
def test_ragged_decode_at_every_head_dim(d):
    rng = np.random.default_rng(1000 + d)
    ctx = np.array([1, 2, 15, 16, 17, 31, 33, 100, 257, 1000])
    c = workloads.paged_case(rng, np.ones(len(ctx), np.int32), ctx - 1, hq=6, hkv=2, d=d)
    _check(c, what=f"d={d}")
    _check(c, num_splits=1, what=f"d={d}, one partition")
    _check(c, num_splits=4, what=f"d={d}, 4 splits")
    _check(c, num_splits=63, what=f"d={d}, 63 splits")


@pytest.mark.parametrize("hq,hkv", [(1, 1), (2, 2), (14, 2), (9, 1), (16, 1), (32, 2), (12, 4),
                                    (16, 8), (12, 6), (9, 3), (20, 10), (7, 7)])
def test_gqa_group_sizes_at_head_dim_64(hq, hkv):
    rng = np.random.default_rng(hq * 100 + hkv)
    ctx = np.array([1, 16, 17, 63, 64, 65, 200, 511])
    c = workloads.paged_case(rng, np.ones(len(ctx), np.int32), ctx - 1, hq=hq, hkv=hkv, d=64)
    _check(c, what=f"gqa {hq}/{hkv}")
    _check(c, num_splits=5, what=f"gqa {hq}/{hkv}, 5 splits")


def test_decode_at_qwen2_05b_head_geometry():
    # 14 query / 2 KV heads of 64, 16 sequences with contexts U{64..2048}: config 2's batch
    # at the head geometry of the family's smallest model
    rng = np.random.default_rng(7)
    ctx = rng.integers(64, 2049, size=16)
    c = workloads.paged_case(rng, np.ones(16, np.int32), ctx - 1, hq=14, hkv=2, d=64)
    _check(c, what="14/2 x 64")


@pytest.mark.parametrize("d", [64, 96, 256])
@pytest.mark.parametrize("block_size", [16, 64])
def test_mixed_chunked_prefill_and_decode(d, block_size):
    rng = np.random.default_rng(d + block_size)
    new = [1, 5, 1, 33, 16, 1, 2, 70]
    prior = [300, 0, 0, 40, 16, 17, 600, 3]
    c = workloads.paged_case(rng, new, prior, hq=8, hkv=2, d=d, block_size=block_size)
    _check(c, causal=True, what=f"mixed causal d={d}")
    _check(c, causal=False, what=f"mixed non-causal d={d}")
    _check(c, causal=True, num_splits=7, what=f"mixed causal d={d}, 7 splits")


def test_zero_context_empty_sequences_and_single_key():
    rng = np.random.default_rng(5)
    c = workloads.paged_case(rng, [1, 0, 1, 3, 1], [0, 5, 40, 0, 0], hq=4, hkv=2, d=64)
    c["context_lens"][0] = 0  # a decode row with nothing visible
    for ns in (1, 3):
        r = PagedAttnRunner(c, num_splits=ns)
        r.launch()
        got = r.result()
        want = _oracle(c)
        assert (got[0] == 0).all() and (want[0] == 0).all()
        assert_parity(got, want, what="zero ctx")
        # one visible key: the output is that key's value row, exactly
        v0 = c["v_pool"][c["block_tables"][4, 0] * 16].reshape(2, 64)
        assert np.array_equal(got[5], v0[[0, 0, 1, 1]])


def test_peaked_softmax_and_equal_keys():
    rng = np.random.default_rng(8)
    c = workloads.paged_case(rng, [1], [99], hq=4, hkv=2, d=64)
    c["k_pool"][:] = c["k_pool"][0]
    _check(c, what="equal keys: mean of V")
    c = workloads.paged_case(rng, [1, 40], [4999, 300], hq=8, hkv=2, d=64)
    c["scale"] = 4.0
    _check(c, num_splits=16, what="peaked softmax")


def test_phases_and_rejections():
    rng = np.random.default_rng(9)
    c = workloads.paged_case(rng, [1, 20, 1], [500, 30, 90], hq=4, hkv=2, d=64)
    want = _oracle(c)
    r = PagedAttnRunner(c, num_splits=4)
    # the three phases one after another give what the single call gives
    for ph in (kernels.ATTN_PHASE_DECODE, kernels.ATTN_PHASE_PREFILL, kernels.ATTN_PHASE_MERGE):
        r.launch(phases=ph)
    assert_parity(r.result(), want, what="phases")
    # turbo3 head rows and GQA groups beyond 16 stay with head_dim 128 / are refused
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_paged_attn_shape(3, 22, 20, 34, 2, 64, 16, 64, 4)
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_paged_attn_shape(3, 22, 20, 4, 2, 80, 16, 64, 4)


def _random_case(rng, d, max_group):
    hkv = int(rng.choice([1, 2, 3, 4, 8]))
    g = int(rng.integers(1, max_group + 1))
    block_size = int(rng.choice([16, 32, 48, 64]))
    n = int(rng.integers(1, 10))
    # a mix of decode rows, chunks and (sometimes) empty sequences
    kind = rng.integers(0, 4, size=n)
    new = np.where(kind == 0, 0, np.where(kind == 1, 1, rng.integers(2, 45, size=n)))
    prior = rng.integers(0, 500, size=n) * (rng.random(n) < 0.8)
    if new.sum() == 0:
        new[0] = 1
    c = workloads.paged_case(rng, new.astype(np.int32), prior.astype(np.int32), hq=g * hkv,
                             hkv=hkv, d=d, block_size=block_size)
    return c, f"d={d} heads {g * hkv}/{hkv} block {block_size} new {new.tolist()} prior {prior.tolist()}"


@pytest.mark.parametrize("seed", range(24))
def test_randomized_ragged_batches(seed):
    # random geometry, batch mix and partition count, every supported width in turn (128:
    # the kernels built for it, groups up to 8)
    rng = np.random.default_rng(9000 + seed)
    d = [32, 64, 96, 128, 160, 192, 224, 256][seed % 8]
    c, what = _random_case(rng, d, 8 if d == 128 else 16)
    causal = bool(rng.integers(0, 2))
    ns = [None, 1, int(rng.integers(2, 40))][seed % 3]
    _check(c, num_splits=ns, causal=causal, what=f"{what} causal={causal} splits={ns}")


@pytest.mark.parametrize("d,hq,hkv", [(64, 32, 8), (64, 14, 2), (96, 12, 4), (256, 8, 8), (32, 16, 1)])
def test_balanced_split_of_large_batches(d, hq, hkv):
    # block tables wide enough that the launch takes the balanced split (its size test looks at
    # what the tables could hold): the tiles of all sequences dealt evenly to the workers,
    # sequences that start and end inside a worker, a row without context, single keys
    rng = np.random.default_rng(7000 + d + hq)
    ctx = np.array([1, 3000, 17, 1, 640, 5000, 33, 2, 900, 128, 129, 4097, 16, 15, 700, 31])
    c = workloads.paged_case(rng, np.ones(len(ctx), np.int32), ctx - 1, hq=hq, hkv=hkv, d=d,
                             min_max_blocks=2048)
    c["context_lens"][3] = 0
    _check(c, what=f"balanced d={d} {hq}/{hkv}")
    _check(c, num_splits=2, what=f"balanced d={d} {hq}/{hkv}, 2 splits (few workers)")
    _check(c, num_splits=40, what=f"balanced d={d} {hq}/{hkv}, 40 splits")
    # a mixed batch on the same wide tables: chunks beside balanced decode rows
    new = [1, 40, 1, 1, 7, 1, 1, 130]
    prior = [2000, 100, 0, 4000, 0, 777, 15, 300]
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv, d=d, min_max_blocks=2048)
    _check(c, what=f"balanced mixed d={d} {hq}/{hkv}")
    _check(c, causal=False, num_splits=9, what=f"balanced mixed non-causal d={d} {hq}/{hkv}")


@pytest.mark.parametrize("d", [64, 128])
def test_more_decode_sequences_than_the_balanced_split_holds(d):
    # 2100 decode sequences: past the prefix table of the balanced launches (2048 entries), so
    # both kernel families fall back to the static split; also a batch of 2048, the last that
    # takes the balanced one
    for n in (2100, 2048):
        rng = np.random.default_rng(d + n)
        ctx = rng.integers(1, 60, size=n)
        c = workloads.paged_case(rng, np.ones(n, np.int32), ctx - 1, hq=4, hkv=2, d=d,
                                 min_max_blocks=8)
        _check(c, what=f"{n} sequences, d={d}")
        _check(c, num_splits=3, what=f"{n} sequences, d={d}, 3 splits")
