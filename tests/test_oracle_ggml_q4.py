"""Pins of the oracle's ggml Q4_0 / Q4_1 restatement and of the planar Q4G32 format.

The reference parses the two type ids and rejects the tensors (crates/loader/src/gguf.rs:
57-78,127-145); it holds no struct, arithmetic or vector for them.  What pins the oracle
here: hand-built blocks decoded by the published formulas (w = (q - 8) d, w = q d + m, value
j / j + 16 in the low / high nibble of byte j), independent numpy restatements of decode and
of the reference quantisers, their closed-form error bounds, and a float64 brute force of
the GEMV.  A dropped `- 8`, swapped nibbles, a wrong byte offset of `m` or a transposed
planar order each fail one of them.
"""
import numpy as np
import pytest

import oracle as O


def _blocks_np(blocks, n, k, has_min):
    bs = 20 if has_min else 18
    b = np.asarray(blocks, np.uint8).reshape(n, k // 32, bs)
    d = b[:, :, 0:2].copy().view(np.float16)[..., 0].astype(np.float32)
    m = b[:, :, 2:4].copy().view(np.float16)[..., 0].astype(np.float32) if has_min else None
    qs = b[:, :, (4 if has_min else 2):]
    q = np.concatenate([qs & 0x0F, qs >> 4], axis=2).astype(np.float32)  # values 0..15, 16..31
    return d, m, q


def test_hand_built_q4_0_block_decodes_by_the_published_formula():
    # d = 0.5; byte j = j | (15 - j) << 4: value j -> (j - 8)/2, value j + 16 -> (7 - j)/2
    blk = np.zeros(18, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    for j in range(16):
        blk[2 + j] = j | ((15 - j) << 4)
    w = O.dequantize_q4_blocks(blk, 1, 32, False)[0]
    assert w[:16].tolist() == [(j - 8) * 0.5 for j in range(16)]
    assert w[16:].tolist() == [(7 - j) * 0.5 for j in range(16)]


def test_hand_built_q4_1_block_decodes_by_the_published_formula():
    blk = np.zeros(20, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(-1.5).tobytes(), np.uint8)
    for j in range(16):
        blk[4 + j] = (15 - j) | (j << 4)
    w = O.dequantize_q4_blocks(blk, 1, 32, True)[0]
    assert w[:16].tolist() == [(15 - j) * 0.25 - 1.5 for j in range(16)]
    assert w[16:].tolist() == [j * 0.25 - 1.5 for j in range(16)]


@pytest.mark.parametrize("has_min", [False, True])
def test_decode_matches_an_independent_numpy_restatement(has_min):
    rng = np.random.default_rng(7)
    n, k = 9, 160
    bs = 20 if has_min else 18
    blocks = rng.integers(0, 256, size=n * (k // 32) * bs, dtype=np.uint8)
    # keep the fp16 fields finite
    b = blocks.reshape(-1, bs)
    b[:, 1] &= 0x3B
    if has_min:
        b[:, 3] &= 0xBB
    d, m, q = _blocks_np(blocks, n, k, has_min)
    want = (q * d[..., None] + m[..., None]) if has_min else ((q - 8.0) * d[..., None])
    got = O.dequantize_q4_blocks(blocks, n, k, has_min)
    assert np.array_equal(got, want.reshape(n, k).astype(np.float32))


def test_q4_0_quantiser_follows_the_reference_rule_and_bound():
    rng = np.random.default_rng(8)
    n, k = 16, 256
    w = rng.standard_normal((n, k)).astype(np.float32)
    blocks = O.quantize_q4_blocks(w, n, k, False)
    d, _, q = _blocks_np(blocks, n, k, False)
    g = w.reshape(n, k // 32, 32)
    idx = np.abs(g).argmax(axis=2)
    mx = np.take_along_axis(g, idx[..., None], axis=2)[..., 0]      # signed value of max |x|
    assert np.array_equal(d, (mx / np.float32(-8.0)).astype(np.float16).astype(np.float32))
    # the value of largest magnitude lands on q = 0 (w = -8 d): exact up to the fp16 rounding of d
    assert (np.take_along_axis(q, np.where(idx < 16, idx, idx)[..., None], axis=2)[..., 0] == 0).all()
    deq = O.dequantize_q4_blocks(blocks, n, k, False).reshape(n, k // 32, 32)
    dd = np.abs(mx / -8.0)
    err = np.abs(deq - g)
    # inside the grid half a step; the positive side clips at q = 15 (7 d), one more step
    assert (err <= dd[..., None] * 1.0 + 1e-3 * np.abs(g) + 1e-6).all()
    assert (err[np.sign(g) == np.sign(mx)[..., None]] <= (dd[..., None] * 0.5 * np.ones_like(g) +
            2e-3 * np.abs(g) + 1e-6)[np.sign(g) == np.sign(mx)[..., None]]).all()


def test_q4_1_quantiser_follows_the_reference_rule_and_bound():
    rng = np.random.default_rng(9)
    n, k = 16, 256
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = O.quantize_q4_blocks(w, n, k, True)
    d, m, q = _blocks_np(blocks, n, k, True)
    g = w.reshape(n, k // 32, 32)
    mn, mx = g.min(axis=2), g.max(axis=2)
    assert np.array_equal(m, mn.astype(np.float16).astype(np.float32))
    assert np.array_equal(d, ((mx - mn) / np.float32(15.0)).astype(np.float16).astype(np.float32))
    assert q.min() == 0 and q.max() == 15
    deq = O.dequantize_q4_blocks(blocks, n, k, True).reshape(n, k // 32, 32)
    step = (mx - mn) / 15.0
    # half a step, plus what rounding d and m to fp16 moves the grid (15 steps of 2^-11 relative)
    assert (np.abs(deq - g) <= step[..., None] * 0.5 + 15 * step[..., None] * 2.0 ** -10 +
            np.abs(mn)[..., None] * 2.0 ** -10 + 1e-8).all()


def test_constant_and_zero_groups():
    w = np.zeros((1, 64), np.float32)
    w[0, 32:] = 0.75
    for has_min in (False, True):
        blocks = O.quantize_q4_blocks(w, 1, 64, has_min)
        deq = O.dequantize_q4_blocks(blocks, 1, 64, has_min)
        assert np.array_equal(deq, w)           # 0 -> d = 0; constant -> exact


@pytest.mark.parametrize("has_min", [False, True])
def test_planar_q4g32_keeps_every_value_and_uses_k_order_low_nibble_first(has_min):
    rng = np.random.default_rng(10)
    n, k = 5, 96
    w = rng.standard_normal((n, k)).astype(np.float32)
    blocks = O.quantize_q4_blocks(w, n, k, has_min)
    qw, scale, minv = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
    d, m, q = _blocks_np(blocks, n, k, has_min)
    qk = q.reshape(n, k).astype(np.uint8)                       # nibble of element k
    assert np.array_equal(qw & 0x0F, qk[:, 0::2]) and np.array_equal(qw >> 4, qk[:, 1::2])
    assert np.array_equal(scale.astype(np.float32), d)
    want_min = m if has_min else (-8.0 * d)
    assert np.array_equal(minv.astype(np.float32), want_min.astype(np.float32))
    # dequantising the planar form gives the block decode (Q4_0: (q-8)d == qd - 8d here
    # because both products are exact in fp32 for 4-bit q and fp16 d)
    assert np.array_equal(O.dequantize_q4g32(qw, scale, minv, n, k),
                          O.dequantize_q4_blocks(blocks, n, k, has_min))


@pytest.mark.parametrize("has_min", [False, True])
def test_qgemv_q4g32_matches_float64_bruteforce_and_orientation(has_min):
    rng = np.random.default_rng(11)
    n, k = 37, 224
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    blocks = O.quantize_q4_blocks(w, n, k, has_min)
    qw, scale, minv = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
    deq = O.dequantize_q4_blocks(blocks, n, k, has_min).astype(np.float64)
    want = deq @ x.astype(np.float64)
    got = O.qgemv_q4g32_f32(x, qw, scale, minv, n, k)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(deq).sum(axis=1).max()
    # one-hot x reads back one dequantised column (weight is [out, in])
    e = np.zeros(k, np.float32)
    e[45] = 1.0
    assert np.array_equal(O.qgemv_q4g32_f32(e, qw, scale, minv, n, k), deq[:, 45].astype(np.float32))


@pytest.mark.parametrize("has_min", [False, True])
def test_qgemm_q4g32_is_the_float64_product_row_by_row(has_min):
    rng = np.random.default_rng(12)
    b, n, k = 5, 19, 256
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    xbits = O.f32_to_bf16_bits(rng.standard_normal((b, k)).astype(np.float32))
    x = O.bf16_bits_to_f32(xbits).astype(np.float64)
    blocks = O.quantize_q4_blocks(w, n, k, has_min)
    qw, scale, minv = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
    deq = O.dequantize_q4_blocks(blocks, n, k, has_min).astype(np.float64)
    want = x @ deq.T                                            # [b, n]: weight is [out, in]
    got = O.qgemm_q4g32_f32(xbits, qw, scale, minv, b, n, k)
    assert got.shape == (b, n)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(deq).sum(axis=1).max() * np.abs(x).max()
    # the bf16 form is that sum rounded once, to nearest even
    bits = O.qgemm_q4g32_bf16(xbits, qw, scale, minv, b, n, k)
    back = O.bf16_bits_to_f32(bits)
    assert np.abs(back - got).max() <= np.abs(got).max() * 2.0 ** -8
    assert np.array_equal(bits, O.f32_to_bf16_bits(got))
