"""GPU parity (bit-exact): ragged packing, KV writes by slot, and the
write -> paged-attention round trip, through the C ABI."""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip, kernels
from tests import workloads
from tests.gpu_harness import PagedAttnRunner, assert_parity

pytestmark = pytest.mark.gpu


def _pack_gpu(new, prior, bt, block_size):
    new = np.ascontiguousarray(new, np.int32)
    prior = np.ascontiguousarray(prior, np.int32)
    bt = np.ascontiguousarray(bt, np.int32)
    s = len(new)
    total = int(new.sum())
    d_new, d_prior, d_bt = (hip.DeviceBuffer.from_numpy(a) for a in (new, prior, bt))
    d_cu, d_ctx = hip.DeviceBuffer(4 * (s + 1)), hip.DeviceBuffer(4 * s)
    d_slots = hip.DeviceBuffer(max(8 * total, 8))
    for b in (d_cu, d_ctx, d_slots):
        b.fill(0xEE)
    kernels.launch_pack_ragged(d_new, d_prior, d_bt, d_cu, d_slots, d_ctx, s, block_size,
                               bt.shape[1])
    hip.synchronize()
    return (d_cu.to_numpy(np.int32, (s + 1,)), d_slots.to_numpy(np.int64, (total,)),
            d_ctx.to_numpy(np.int32, (s,)))


def _check_pack(new, prior, bt, block_size):
    cu, slots, ctx = _pack_gpu(new, prior, bt, block_size)
    cu_o, slots_o, ctx_o, _ = O.pack_ragged(new, prior, bt, block_size)
    assert np.array_equal(cu, cu_o)
    assert np.array_equal(ctx, ctx_o)
    assert np.array_equal(slots, slots_o)


def test_config4_mixed_batch_packing_is_bit_exact():
    rng = np.random.default_rng(workloads.SEED + 4)
    # 48 decode rows (1 token, ctx log-uniform 128..32768) + 16 prefill chunks of 512 tokens
    dec_ctx = np.exp(rng.uniform(np.log(128), np.log(32768), size=48)).astype(np.int64)
    new = np.concatenate([np.ones(48, np.int64), np.full(16, 512)])
    prior = np.concatenate([dec_ctx - 1, rng.integers(0, 8193, size=16)])
    order = rng.permutation(64)
    new, prior = new[order], prior[order]
    max_blocks = int(((new + prior + 15) // 16).max())
    bt = rng.permutation(64 * max_blocks).astype(np.int32).reshape(64, max_blocks)
    _check_pack(new, prior, bt, 16)


def test_overflowing_and_unmapped_positions_get_no_slot():
    # past the table row: slot -1 and the context capped; entries that name no block
    # (negative, the cache's 0x3FFFFFFF mark, anything from LOGISMOS_BLOCK_ID_LIMIT up): -1
    bt = np.array([[1, 0, 7, 7, 7], [5, 0x3FFFFFFF, -3, 0x3FFFFFF, 0x3FFFFFE]], np.int32)
    new, prior = [60, 80], [30, 0]
    cu, slots, ctx = _pack_gpu(new, prior, bt, 16)
    cu_o, slots_o, ctx_o, bad = O.pack_ragged(new, prior, bt, 16)
    assert np.array_equal(cu, cu_o) and np.array_equal(ctx, ctx_o)
    assert np.array_equal(slots, slots_o)
    assert ctx.tolist() == [80, 80] and bad == 10 + 48
    assert (slots[50:60] == -1).all() and (slots[60 + 16:60 + 64] == -1).all()


@pytest.mark.parametrize("s", [1, 2, 63, 64, 65, 257, 1000, 5000])
def test_sequence_counts(s):
    rng = np.random.default_rng(s)
    new = rng.integers(0, 9, size=s)
    prior = rng.integers(0, 300, size=s)
    bt = rng.integers(0, 1 << 20, size=(s, 20)).astype(np.int32)
    _check_pack(new, prior, bt, 16)


def test_edge_cases_empty_rows_overflow_and_block_sizes():
    bt = np.arange(8, dtype=np.int32).reshape(2, 4)
    _check_pack([0, 0], [5, 0], bt, 16)                    # nothing to pack
    _check_pack([3, 70], [62, 0], bt, 16)                  # both run past max_blocks -> -1
    _check_pack([5, 1], [0, 127], bt, 32)
    cu, slots, _ = _pack_gpu([3], [62], bt[:1], 16)
    assert slots.tolist() == [3 * 16 + 14, 3 * 16 + 15, -1] and cu.tolist() == [0, 3]


def test_reference_cu_seqlens_example():
    """research/14-gdn-aiter-preflight.md:338"""
    bt = np.arange(3 * 64, dtype=np.int32).reshape(3, 64)
    cu, _, _ = _pack_gpu([512, 1024, 512], [0, 0, 0], bt, 16)
    assert cu.tolist() == [0, 512, 1536, 2048]


def test_kv_write_is_bit_exact_and_skips_negative_slots():
    rng = np.random.default_rng(11)
    hkv, d, bs, nblk = 8, 128, 16, 40
    new, prior = [1, 37, 1, 512 - 20], [100, 3, 0, 20]
    max_blocks = 33
    bt = rng.permutation(4 * max_blocks).astype(np.int32).reshape(4, max_blocks) % nblk
    # make the block ids of different sequences distinct so writes do not collide
    bt = (np.arange(4 * max_blocks, dtype=np.int32).reshape(4, max_blocks) * 7) % (4 * max_blocks)
    nblk = 4 * max_blocks
    cu, slots, ctx, _ = O.pack_ragged(new, prior, bt, bs)
    slots[5] = -1
    t = len(slots)
    k_new = rng.standard_normal((t, hkv * d), np.float32).astype(np.float16)
    v_new = rng.standard_normal((t, hkv * d), np.float32).astype(np.float16)
    k_pool = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    v_pool = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    d_kp, d_vp = hip.DeviceBuffer.from_numpy(k_pool), hip.DeviceBuffer.from_numpy(v_pool)
    kernels.launch_kv_write_fp16(hip.DeviceBuffer.from_numpy(k_new),
                                 hip.DeviceBuffer.from_numpy(v_new), d_kp, d_vp,
                                 hip.DeviceBuffer.from_numpy(slots), t, hkv, d)
    hip.synchronize()
    O.kv_write_fp16(k_new, v_new, k_pool, v_pool, slots, hkv * d)
    assert np.array_equal(d_kp.to_numpy(np.float16, k_pool.shape).view(np.uint16),
                          k_pool.view(np.uint16))
    assert np.array_equal(d_vp.to_numpy(np.float16, v_pool.shape).view(np.uint16),
                          v_pool.view(np.uint16))


def test_pack_write_attend_round_trip():
    # GPU packer -> GPU kv_write of the new tokens -> GPU attention == oracle on the same pools
    rng = np.random.default_rng(12)
    c = workloads.paged_case(rng, [1, 9, 1, 40], [70, 0, 15, 24], hq=8, hkv=2)
    cu, slots, ctx = _pack_gpu(c["new_tokens"], c["prior_ctx"], c["block_tables"], 16)
    assert np.array_equal(cu, c["cu_seqlens"]) and np.array_equal(ctx, c["context_lens"])
    t = len(slots)
    k_new = rng.standard_normal((t, 2 * 128), np.float32).astype(np.float16)
    v_new = rng.standard_normal((t, 2 * 128), np.float32).astype(np.float16)
    r = PagedAttnRunner(c)
    kernels.launch_kv_write_fp16(hip.DeviceBuffer.from_numpy(k_new),
                                 hip.DeviceBuffer.from_numpy(v_new), r.k_pool, r.v_pool,
                                 hip.DeviceBuffer.from_numpy(slots), t, 2, 128)
    r.launch()
    got = r.result()
    O.kv_write_fp16(k_new, v_new, c["k_pool"], c["v_pool"], slots, 2 * 128)
    want = O.paged_attn_varlen_fp16(c["q"], c["k_pool"], c["v_pool"], c["block_tables"],
                                    c["cu_seqlens"], c["context_lens"], 8, 2, 128, 16, c["scale"])
    assert_parity(got, want, what="round trip")
