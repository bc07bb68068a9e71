"""GPU parity of the TurboQuant 3-bit KV path vs the CPU oracle, through the C ABI.

Encoding and decoding are bit-exact (the kernels follow the reference's operation order);
attention over turbo3 pools is held to the fp16-output tolerance."""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip, kernels
from tests import workloads
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu


def _dev(a):
    return hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _encode_gpu(k, v, slots, rows, hkv):
    kp = hip.DeviceBuffer(rows * hkv * 56)
    vp = hip.DeviceBuffer(rows * hkv * 56)
    kp.fill(0xAA)
    vp.fill(0xAA)
    kernels.launch_kv_write_turbo3(_dev(k), _dev(v), kp, vp, _dev(slots), len(slots), hkv)
    hip.synchronize()
    return kp, vp


@pytest.mark.parametrize("hkv,scale", [(1, 1.0), (2, 0.02), (8, 30.0)])
def test_encode_is_bit_exact(hkv, scale):
    rng = np.random.default_rng(hkv)
    T, rows = 37, 64
    k = (rng.standard_normal((T, hkv * 128)) * scale).astype(np.float16)
    v = (rng.standard_normal((T, hkv * 128)) * scale).astype(np.float16)
    slots = rng.permutation(rows)[:T].astype(np.int64)
    slots[5] = -1
    kp, vp = _encode_gpu(k, v, slots, rows, hkv)
    want_k = np.full((rows, hkv * 56), 0xAA, np.uint8)
    want_v = np.full((rows, hkv * 56), 0xAA, np.uint8)
    O.kv_write_turbo3(k, v, want_k, want_v, slots, hkv)
    assert np.array_equal(kp.to_numpy(np.uint8, (rows, hkv * 56)), want_k)
    assert np.array_equal(vp.to_numpy(np.uint8, (rows, hkv * 56)), want_v)


def test_encode_special_rows():
    # zero row (norm 0 -> indices of the centroid nearest 0), a one-hot row, tiny and large
    # magnitudes, the reference's own round-trip signal
    i = np.arange(128, dtype=np.float32)
    rows = np.zeros((6, 128), np.float32)
    rows[1, 17] = 1.0
    rows[2] = 1e-4
    rows[3] = 300.0 * np.sign(np.sin(i))
    rows[4] = np.sin(i * np.float32(0.1)) * np.float32(0.1) + np.cos(i * np.float32(0.03)) * np.float32(0.1)
    rows[5] = 6e-8      # fp16 subnormal
    k = rows.astype(np.float16)
    slots = np.arange(6, dtype=np.int64)
    kp, vp = _encode_gpu(k, k, slots, 6, 1)
    want = np.zeros((6, 56), np.uint8)
    want2 = np.zeros((6, 56), np.uint8)
    O.kv_write_turbo3(k, k, want, want2, slots, 1)
    assert np.array_equal(kp.to_numpy(np.uint8, (6, 56)), want)
    assert np.array_equal(vp.to_numpy(np.uint8, (6, 56)), want2)


@pytest.mark.parametrize("block_size", [16, 64])
def test_decode_gather_is_bit_exact(block_size):
    rng = np.random.default_rng(7)
    hkv, ctx = 4, 100
    nblk = (ctx + block_size - 1) // block_size
    total = nblk + 3
    bt = rng.permutation(total)[:nblk].astype(np.int32)
    pool_rows = total * block_size
    # arbitrary payload bits and finite norms, not only what the encoder emits
    kp = rng.integers(0, 256, size=(pool_rows, hkv * 56), dtype=np.uint8)
    vp = rng.integers(0, 256, size=(pool_rows, hkv * 56), dtype=np.uint8)
    for p in (kp, vp):
        p.reshape(pool_rows, hkv, 4, 14)[:, :, :, 1] &= 0x7B
    k_out = hip.DeviceBuffer(ctx * hkv * 128 * 4)
    v_out = hip.DeviceBuffer(ctx * hkv * 128 * 4)
    kernels.launch_kv_gather_turbo3_f32(_dev(kp), _dev(vp), _dev(bt), k_out, v_out, 0, ctx, hkv,
                                        block_size)
    hip.synchronize()
    want_k = O.paged_gather_turbo3(kp, bt, ctx, block_size, hkv)
    want_v = O.paged_gather_turbo3(vp, bt, ctx, block_size, hkv)
    assert np.array_equal(k_out.to_numpy(np.float32, (ctx, hkv * 128)), want_k)
    assert np.array_equal(v_out.to_numpy(np.float32, (ctx, hkv * 128)), want_v)
    # a window in the middle
    kernels.launch_kv_gather_turbo3_f32(_dev(kp), _dev(vp), _dev(bt), k_out, v_out, 33, 20, hkv,
                                        block_size)
    hip.synchronize()
    assert np.array_equal(k_out.to_numpy(np.float32, (20, hkv * 128)), want_k[33:53])


def test_encode_then_decode_round_trip_on_the_gpu():
    # put -> get through the codec: equals the CPU encode -> decode, and stays within the
    # codebook's quantisation error of the input
    rng = np.random.default_rng(8)
    hkv, T = 2, 48
    k = rng.standard_normal((T, hkv * 128)).astype(np.float16)
    slots = np.arange(T, dtype=np.int64)
    kp, vp = _encode_gpu(k, k, slots, T, hkv)
    bt = np.arange(T // 16, dtype=np.int32)
    k_out = hip.DeviceBuffer(T * hkv * 128 * 4)
    v_out = hip.DeviceBuffer(T * hkv * 128 * 4)
    kernels.launch_kv_gather_turbo3_f32(kp, vp, _dev(bt), k_out, v_out, 0, T, hkv, 16)
    hip.synchronize()
    got = k_out.to_numpy(np.float32, (T, hkv, 128))
    kf = k.astype(np.float32).reshape(T, hkv, 128)
    for t in range(0, T, 7):
        for h in range(hkv):
            assert np.array_equal(got[t, h], O.decode_turbo3_0_head(O.encode_turbo3_0_head(kf[t, h])))
    rel = np.linalg.norm(got - kf, axis=2) / np.linalg.norm(kf, axis=2)
    assert rel.max() < 0.25


# ------------------------------------------------------------------ attention over turbo3 pools
def _turbo3_pools(c):
    """Encodes the fp16 pools of a paged case row by row (on the CPU oracle)."""
    rows, hkv = c["k_pool"].shape[0], c["hkv"]
    kp = np.zeros((rows, hkv * 56), np.uint8)
    vp = np.zeros((rows, hkv * 56), np.uint8)
    O.kv_write_turbo3(c["k_pool"], c["v_pool"], kp, vp, np.arange(rows, dtype=np.int64), hkv)
    return kp, vp


def _attn_turbo3(c, kp, vp, num_splits=None):
    S = len(c["context_lens"])
    T = int(c["cu_seqlens"][-1])
    ns = num_splits or kernels.paged_attn_num_splits(S, c["hkv"], c["block_size"], c["max_blocks"])
    out = hip.DeviceBuffer(max(16, c["q"].nbytes))
    out.fill(0xFF)
    ws = hip.DeviceBuffer(max(16, kernels.paged_attn_workspace_bytes(S, c["hq"], 128, ns)))
    ws.fill(0xFF)
    kernels.launch_paged_attn_varlen_turbo3(
        _dev(c["q"]), _dev(kp), _dev(vp), _dev(c["block_tables"]), _dev(c["cu_seqlens"]),
        _dev(c["context_lens"]), out, ws, S, T, int(c["new_tokens"].max()), c["hq"], c["hkv"],
        c["block_size"], c["max_blocks"], ns, c["scale"])
    hip.synchronize()
    return out.to_numpy(np.float16, c["q"].shape)


def _oracle_t3(c, kp, vp):
    return O.paged_attn_varlen_turbo3(c["q"], kp, vp, c["block_tables"], c["cu_seqlens"],
                                      c["context_lens"], c["hq"], c["hkv"], c["block_size"],
                                      c["scale"], True)


@pytest.mark.parametrize("hq,hkv", [(1, 1), (4, 2), (12, 2), (32, 8), (8, 1), (14, 2)])
def test_turbo3_attention_gqa_group_sizes(hq, hkv):
    rng = np.random.default_rng(70 + hq + hkv)
    new = [1, 1, 1, 1, 1, 0, 1]
    prior = [0, 15, 16, 127, 1000, 5, 333]
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv)
    kp, vp = _turbo3_pools(c)
    want = _oracle_t3(c, kp, vp)
    for ns in (1, 3, 16):
        assert_parity(_attn_turbo3(c, kp, vp, ns), want, what=f"turbo3 {hq}/{hkv} splits {ns}")


@pytest.mark.parametrize("hq,hkv", [(8, 2), (16, 2), (32, 8), (7, 1), (3, 1)])
def test_turbo3_attention_balanced_kernel_and_zero_context(hq, hkv):
    # group sizes on both sides of four (a lane row of the P.V accumulators holds four heads),
    # one to eight waves sharing the workgroup's centroid table, odd and even tile counts
    rng = np.random.default_rng(71 + hq)
    new = np.ones(12, np.int32)
    prior = [0, 40, 2047, 16, 511, 300, 1, 999, 64, 65, 129, 700]
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv, min_max_blocks=8192)
    c["context_lens"][3] = 0
    kp, vp = _turbo3_pools(c)
    want = _oracle_t3(c, kp, vp)
    got = _attn_turbo3(c, kp, vp)
    assert (got[3] == 0).all() and (want[3] == 0).all()
    assert_parity(got, want, what="turbo3 balanced")
    assert_parity(_attn_turbo3(c, kp, vp, 5), want, what="turbo3 balanced, 5 splits")


def test_turbo3_attention_tracks_fp16_attention_over_the_same_rows():
    # the codec's error, not the kernel's: turbo3 attention stays close to fp16 attention
    # over the rows it was encoded from (loose bound; values ~N(0,1), outputs ~0.1..1)
    rng = np.random.default_rng(72)
    c = workloads.paged_case(rng, [1, 1], [600, 90], hq=8, hkv=2)
    kp, vp = _turbo3_pools(c)
    got = _attn_turbo3(c, kp, vp).astype(np.float32)
    ref = O.paged_attn_varlen_fp16(c["q"], c["k_pool"], c["v_pool"], c["block_tables"],
                                   c["cu_seqlens"], c["context_lens"], 8, 2, 128, 16, c["scale"],
                                   True).astype(np.float32)
    assert np.abs(got - ref).max() < 0.35 and np.corrcoef(got.ravel(), ref.ravel())[0, 1] > 0.8


@pytest.mark.parametrize("hq,hkv", [(4, 4), (8, 2), (12, 2), (32, 8), (14, 2)])
def test_turbo3_chunked_prefill_rows(hq, hkv):
    # chunks on both sides of the query-tile and key-tile edges, with and without prior
    # context, next to decode rows: the movers decode turbo3 rows into the K / V^T tiles
    rng = np.random.default_rng(75 + hq + hkv)
    new = [31, 1, 32, 33, 2, 64, 65, 129, 7]
    prior = [0, 77, 5, 100, 31, 0, 333, 17, 1]
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv)
    kp, vp = _turbo3_pools(c)
    want = _oracle_t3(c, kp, vp)
    assert_parity(_attn_turbo3(c, kp, vp), want, what=f"turbo3 prefill {hq}/{hkv}")


def test_turbo3_prefill_512_token_chunks_and_block_sizes():
    rng = np.random.default_rng(76)
    c = workloads.paged_case(rng, [512, 1, 200, 1], [0, 700, 1000, 12], hq=32, hkv=8)
    kp, vp = _turbo3_pools(c)
    assert_parity(_attn_turbo3(c, kp, vp), _oracle_t3(c, kp, vp), what="turbo3 512-token chunks")
    for bs in (32, 128):
        c = workloads.paged_case(rng, [100, 1, 40], [300, 50, 0], hq=8, hkv=2, block_size=bs)
        kp, vp = _turbo3_pools(c)
        assert_parity(_attn_turbo3(c, kp, vp), _oracle_t3(c, kp, vp),
                      what=f"turbo3 prefill block {bs}")


def test_turbo3_prefill_chunk_of_one_row_agrees_with_the_decode_kernel():
    # the same (query, visible keys) through both kernels: a 2-token chunk's last row against
    # a decode row over the same context
    rng = np.random.default_rng(77)
    c2 = workloads.paged_case(rng, [2], [300], hq=8, hkv=2)
    kp, vp = _turbo3_pools(c2)
    got2 = _attn_turbo3(c2, kp, vp).astype(np.float32)
    c1 = dict(c2, new_tokens=np.array([1], np.int32), cu_seqlens=np.array([0, 1], np.int32),
              q=np.ascontiguousarray(c2["q"][1:2]))
    got1 = _attn_turbo3(c1, kp, vp).astype(np.float32)
    assert_parity(got2[1:2], got1, what="turbo3 prefill row vs decode row")


def test_put_encode_then_attend_round_trip_on_the_gpu():
    # new rows encoded by the GPU writer into turbo3 pools, then attended to: the same
    # bytes and the same result as the CPU path end to end
    rng = np.random.default_rng(74)
    c = workloads.paged_case(rng, np.ones(3, np.int32), [70, 5, 300], hq=8, hkv=2)
    rows = c["k_pool"].shape[0]
    kp, vp = _encode_gpu(c["k_pool"], c["v_pool"], np.arange(rows, dtype=np.int64), rows, 2)
    kp_h, vp_h = _turbo3_pools(c)
    assert np.array_equal(kp.to_numpy(np.uint8, kp_h.shape), kp_h)
    got = _attn_turbo3(c, kp_h, vp_h)
    assert_parity(got, _oracle_t3(c, kp_h, vp_h), what="turbo3 put -> attend")


def test_turbo3_attention_at_config5_contexts():
    """The decode step's own attention shape (32 sequences, contexts U{256..8192}, 32 query /
    8 KV heads: the balanced kernel, eight waves per workgroup, partitions that start and end
    inside sequences) over turbo3 pools, every row against the oracle."""
    rng = np.random.default_rng(workloads.SEED + 5)
    ctx = rng.integers(256, 8193, size=32)
    # (pools that repeat 4099 random rows: drawing 150 k distinct rows takes a quarter minute)
    c = workloads.paged_case(rng, np.ones(32, np.int32), ctx - 1, hq=32, hkv=8, spare_frac=0.05,
                             pool_period_rows=4099)
    kp, vp = _turbo3_pools(c)
    want = _oracle_t3(c, kp, vp)
    assert_parity(_attn_turbo3(c, kp, vp), want, what="turbo3 attention, config-5 contexts")
