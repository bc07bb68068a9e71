"""GPU tests of the paged KV cache object, through the C ABI.

The first group restates the reference's `FlatKvCache` tests
(crates/cache/src/flat_tests.rs) on the paged implementation of the same trait; byte-exact
(the cache only moves fp16 rows).  The second group covers what paging adds: several
sequences, block reuse, and attention over the cache's own pools and block tables.
"""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip, kernels
from logismos_amd.paged_kv_cache import CacheError, PagedKvCache
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu


def small(**kw):
    # flat_tests.rs:7-15 layout_small (4 layers, 2 kv heads; max_seq_len 8 there), with the
    # head width and block size this build's kernels need
    args = dict(num_layers=4, num_kv_heads=2, head_dim=8, block_size=16, num_blocks=8, max_seqs=3,
                max_blocks_per_seq=2)
    args.update(kw)
    return PagedKvCache(**args)


def rows(val, n, c):
    return np.full((n, c.layout.num_kv_heads * c.layout.head_dim), val, np.float16)


def dev(a):
    return hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def test_put_then_get_round_trip_f16():
    # flat_tests.rs:52-86
    c = small()
    s = c.open_seq()
    c.put(s, 0, dev(rows(1.5, 1, c)), dev(rows(2.5, 1, c)), 1)
    assert c.len_of(s, 0) == 1
    k, v = c.get(s, 0, 1)
    assert k.shape == (1, 16) and (k == np.float16(1.5)).all() and (v == np.float16(2.5)).all()


def test_grows_monotonically_across_layers():
    # flat_tests.rs:234-248
    c = small()
    s = c.open_seq()
    for _ in range(3):
        for layer in range(c.num_layers()):
            c.put(s, layer, dev(rows(0.1, 1, c)), dev(rows(0.2, 1, c)), 1)
    assert [c.len_of(s, layer) for layer in range(4)] == [3, 3, 3, 3]


def test_reset_zeros_lengths():
    # flat_tests.rs:251-265
    c = small()
    s = c.open_seq()
    k = dev(rows(1.0, 1, c))
    c.put(s, 0, k, k, 1)
    c.put(s, 1, k, k, 1)
    free_before = c.free_blocks()
    c.reset()
    assert c.len_of(s, 0) == 0 and c.len_of(s, 1) == 0
    assert c.free_blocks() == free_before + 1 == 8
    c.put(s, 0, k, k, 1)
    assert c.len_of(s, 0) == 1


def test_overflow_errors_cleanly():
    # flat_tests.rs:268-284: max_seq_len rows fit, one more is LenOverflow and changes nothing
    c = small(num_layers=1, max_blocks_per_seq=1)
    s = c.open_seq()
    k = dev(rows(1.0, 16, c))
    c.put(s, 0, k, k, 16)
    with pytest.raises(CacheError) as e:
        c.put(s, 0, k, k, 1)
    assert e.value.kind == "LenOverflow" and c.len_of(s, 0) == 16


def test_read_beyond_written_errors():
    # flat_tests.rs:287-292
    c = small()
    s = c.open_seq()
    with pytest.raises(CacheError) as e:
        c.get(s, 0, 1)
    assert e.value.kind == "ReadBeyondWritten"


def test_layer_out_of_range_errors():
    # flat_tests.rs:295-300
    c = small()
    s = c.open_seq()
    with pytest.raises(CacheError) as e:
        c.get(s, 99, 0)
    assert e.value.kind == "LayerOutOfRange"
    with pytest.raises(CacheError) as e:
        c.put(s, 4, dev(rows(1, 1, c)), dev(rows(1, 1, c)), 1)
    assert e.value.kind == "LayerOutOfRange"


def test_put_multi_token_batch_verifies_values():
    # flat_tests.rs:307-330: rows come back in put order, across block boundaries
    c = small()
    s = c.open_seq()
    rng = np.random.default_rng(1)
    kd = rng.standard_normal((27, 16)).astype(np.float16)
    vd = rng.standard_normal((27, 16)).astype(np.float16)
    c.put(s, 0, dev(kd[:5]), dev(vd[:5]), 5)
    c.put(s, 0, dev(kd[5:20]), dev(vd[5:20]), 15)
    c.put(s, 0, dev(kd[20:]), dev(vd[20:]), 7)
    assert c.len_of(s, 0) == 27
    k, v = c.get(s, 0, 27)
    assert np.array_equal(k.view(np.uint16), kd.view(np.uint16))
    assert np.array_equal(v.view(np.uint16), vd.view(np.uint16))
    k, v = c.get(s, 0, 9)   # a prefix
    assert np.array_equal(k.view(np.uint16), kd[:9].view(np.uint16))


def test_get_zero_len_returns_empty():
    # flat_tests.rs:333-346
    c = small()
    s = c.open_seq()
    k, v = c.get(s, 0, 0)
    assert k.shape == (0, 16) and v.shape == (0, 16)


def test_len_of_distinguishes_out_of_range_from_unwritten():
    # flat_tests.rs:349-360
    c = small()
    s = c.open_seq()
    assert c.len_of(s, 0) == 0
    assert c.len_of(s, c.num_layers()) is None
    assert c.len_of(s, 9999) is None
    assert c.len_of(s + 1, 0) is None    # a sequence that was never opened


def test_little_endian_f16_rows_in_the_pool():
    # flat_tests.rs:376-404 pins f16 1.0 -> 00 3C; the pool holds the same bytes
    c = small()
    s = c.open_seq()
    c.put(s, 0, dev(rows(1.0, 1, c)), dev(rows(1.0, 1, c)), 1)
    hip.synchronize()
    blk = int(c.block_tables_host()[s, 0])
    pool = hip.DevicePtrView(c.k_pool(0), 8 * 16 * 16 * 2).to_numpy(np.uint8)
    row0 = pool[blk * 16 * 16 * 2: blk * 16 * 16 * 2 + 4]
    assert row0.tolist() == [0x00, 0x3C, 0x00, 0x3C]


def test_sequences_are_independent_and_blocks_are_reused():
    c = small(num_blocks=4, max_blocks_per_seq=3)
    rng = np.random.default_rng(2)
    a, b = c.open_seq(), c.open_seq()
    da = rng.standard_normal((20, 16)).astype(np.float16)
    db = rng.standard_normal((17, 16)).astype(np.float16)
    c.put(a, 1, dev(da[:10]), dev(da[:10]), 10)
    c.put(b, 1, dev(db), dev(db), 17)
    c.put(a, 1, dev(da[10:]), dev(da[10:]), 10)
    assert c.free_blocks() == 0
    bt = c.block_tables_host()
    used = sorted(bt[a, :2].tolist() + bt[b, :2].tolist())
    assert used == [0, 1, 2, 3] and bt[a, 2] == 0x3FFFFFFF
    assert np.array_equal(c.get(a, 1, 20)[0].view(np.uint16), da.view(np.uint16))
    assert np.array_equal(c.get(b, 1, 17)[1].view(np.uint16), db.view(np.uint16))
    d = c.open_seq()
    with pytest.raises(CacheError) as e:
        c.put(d, 0, dev(da[:1]), dev(da[:1]), 1)
    assert e.value.kind == "OutOfBlocks" and c.len_of(d, 0) == 0
    c.close_seq(b)
    assert c.free_blocks() == 2 and c.len_of(b, 1) is None
    c.put(d, 0, dev(db), dev(db), 17)          # takes b's blocks
    assert np.array_equal(c.get(d, 0, 17)[0].view(np.uint16), db.view(np.uint16))
    assert np.array_equal(c.get(a, 1, 20)[0].view(np.uint16), da.view(np.uint16))
    with pytest.raises(CacheError) as e:
        c.open_seq(); c.open_seq()
    assert e.value.kind == "OutOfSeqs"


def test_attention_over_the_caches_pools_matches_the_oracle_on_contiguous_rows():
    # pack -> put -> attend round trip: the cache's pools and block tables go straight into
    # the ragged attention entry point; the oracle sees the same rows through an identity table
    hq, hkv, d, bs, L = 8, 2, 128, 16, 2
    c = PagedKvCache(num_layers=L, num_kv_heads=hkv, head_dim=d, block_size=bs, num_blocks=40,
                     max_seqs=4, max_blocks_per_seq=12)
    rng = np.random.default_rng(3)
    ctx = [150, 33, 1, 77]
    seqs = [c.open_seq() for _ in ctx]
    data = {}
    order = [(0, 100), (1, 33), (2, 1), (0, 50), (3, 77)]    # interleaved growth
    for layer in range(L):
        for s in range(4):
            data[(s, layer)] = (rng.standard_normal((ctx[s], hkv * d)).astype(np.float16),
                                rng.standard_normal((ctx[s], hkv * d)).astype(np.float16))
        done = [0] * 4
        for s, n in order:
            k, v = data[(s, layer)]
            c.put(seqs[s], layer, dev(k[done[s]:done[s] + n]), dev(v[done[s]:done[s] + n]), n)
            done[s] += n
    hip.synchronize()
    layer = 1
    q = rng.standard_normal((4, hq, d)).astype(np.float16)
    cu = np.arange(5, dtype=np.int32)
    ctx_a = np.asarray(ctx, np.int32)
    out = hip.DeviceBuffer(q.nbytes)
    ns = 4
    ws = hip.DeviceBuffer(max(16, kernels.paged_attn_workspace_bytes(4, hq, d, ns)))
    assert seqs == [0, 1, 2, 3]   # block-table rows of the batch are the first four
    kernels.launch_paged_attn_varlen_fp16(
        dev(q), c.k_pool(layer), c.v_pool(layer), c.block_tables(), dev(cu), dev(ctx_a), out, ws,
        4, 4, 1, hq, hkv, d, bs, 12, ns, 1.0 / np.sqrt(d), True)
    hip.synchronize()
    got = out.to_numpy(np.float16, q.shape)
    # oracle over contiguous rows: one block table of consecutive ids per sequence
    nblk = [(x + bs - 1) // bs for x in ctx]
    bt = np.zeros((4, 12), np.int32)
    kp = np.zeros((sum(nblk) * bs, hkv * d), np.float16)
    vp = np.zeros_like(kp)
    o = 0
    for s in range(4):
        bt[s, :nblk[s]] = np.arange(o, o + nblk[s])
        kp[o * bs:o * bs + ctx[s]] = data[(s, layer)][0]
        vp[o * bs:o * bs + ctx[s]] = data[(s, layer)][1]
        o += nblk[s]
    want = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx_a, hq, hkv, d, bs, 1.0 / np.sqrt(d),
                                    True)
    assert_parity(got, want, what="attention over PagedKvCache")


def test_reserve_and_advance_cover_rows_written_by_the_step_kernels():
    c = small()
    s = c.open_seq()
    c.reserve(s, 20)
    assert c.free_blocks() == 6 and c.len_of(s, 0) == 0
    c.advance(s, 0, 20)
    assert c.len_of(s, 0) == 20
    with pytest.raises(CacheError) as e:
        c.advance(s, 0, 13)      # beyond the reserved blocks
    assert e.value.kind == "LenOverflow"
    with pytest.raises(CacheError) as e:
        c.reserve(s, 33)         # beyond max_seq_len = 32
    assert e.value.kind == "LenOverflow"


def test_retiring_a_sequence_does_not_disturb_a_queued_table_copy():
    # reserve queues the copy of the new table entries on a stream; closing the sequence
    # right away must not change what that copy delivers (the launches queued behind it
    # still read through those entries)
    c = small(num_blocks=6, max_blocks_per_seq=3)
    st = hip.Stream()
    s = c.open_seq()
    c.reserve(s, 40, st)
    want = c.block_tables_host()[s, :3].copy()
    c.close_seq(s)
    st.synchronize()
    got = hip.DevicePtrView(c.block_tables(), 4 * c.layout.max_seqs * 3).to_numpy(np.int32)
    assert sorted(want.tolist()) == sorted(set(want.tolist())) and (want < 6).all()
    assert np.array_equal(got.reshape(-1, 3)[s], want)
    assert c.free_blocks() == 6


def test_reopened_slot_does_not_change_a_queued_table_update():
    """A sequence retires and its slot is reopened and grown while the stream is still busy:
    the table update queued for the first owner must deliver the first owner's block ids (the
    cache stages every update; it does not copy from the host table, which the second owner
    rewrites).  The gather queued between the two owners reads the device table when it runs."""
    c = small(num_layers=1, num_kv_heads=1, head_dim=8, num_blocks=8, max_seqs=2,
              max_blocks_per_seq=4)
    row = 8
    nrows = 8 * 16
    # pool row r holds the value r in every element
    pool = np.repeat(np.arange(nrows, dtype=np.float16)[:, None], row, axis=1)
    d_pool = hip.DeviceBuffer.from_numpy(pool)
    view_k = hip.DevicePtrView(c.k_pool(0), pool.nbytes)
    view_v = hip.DevicePtrView(c.v_pool(0), pool.nbytes)
    for view in (view_k, view_v):
        hip.check(hip._runtime().hipMemcpy(view.ptr, d_pool.ptr, pool.nbytes, 3), "hipMemcpy")
    stream = hip.Stream()
    busy = hip.DeviceBuffer(1 << 30)
    a = c.open_seq()
    other = c.open_seq()
    # keep the stream busy so that the copies below are still queued while the host goes on
    for _ in range(4):
        kernels.launch_probe_copy(busy, busy.offset(1 << 29), 1 << 29, stream)
    c.reserve(a, 32, stream)
    first_owner = c.block_tables_host()[a, :2].copy()
    c.advance(a, 0, 32)
    k_out = hip.DeviceBuffer(32 * row * 2)
    v_out = hip.DeviceBuffer(32 * row * 2)
    _check = c._lib.logismos_paged_kv_cache_get(c._h, a, 0, 32, k_out.ptr, v_out.ptr, stream.raw)
    assert _check == 0
    c.close_seq(a)
    c.reserve(other, 16, stream)           # takes the block the first owner freed last
    b = c.open_seq()
    assert b == a                          # the slot is handed out again
    c.reserve(b, 48, stream)
    second_owner = c.block_tables_host()[b, :3].copy()
    assert not np.array_equal(second_owner[:2], first_owner)
    stream.synchronize()
    want = np.concatenate([np.arange(16) + 16 * int(blk) for blk in first_owner])
    got = k_out.to_numpy(np.float16, (32, row))
    assert np.array_equal(got[:, 0].astype(np.int64), want)
    # and the device table ends up with the second owner's ids
    bt = hip.DevicePtrView(c.block_tables(), 2 * 4 * 4).to_numpy(np.int32, (2, 4))
    assert np.array_equal(bt[b, :3], second_owner)
