"""Pins the parts of the oracle the reference does not define.

Conversions are checked against numpy/torch (independent implementations);
quantisers against closed-form invariants; GEMV/GEMM against float64 brute
force over the dequantised matrix; ragged packing, the paged gather and paged
attention against closed forms, brute force and special cases chosen so that
a dropped term, a wrong index or a transposed operand fails.
"""
import math

import numpy as np
import pytest

import oracle as O


# ------------------------------------------------------------------ conversions
def test_f16_roundtrip_all_65536_patterns_match_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    f = O.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(f), nan)
    assert np.array_equal(f[~nan].view(np.uint32), want[~nan].view(np.uint32))
    back = O.f32_to_f16_bits(f)
    assert np.array_equal(back[~nan], bits[~nan])


def test_f32_to_f16_rounding_matches_numpy_rne():
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.normal(size=200_000).astype(np.float32),
        (rng.normal(size=100_000) * 1e-6).astype(np.float32),   # subnormal halves
        (rng.normal(size=100_000) * 3e4).astype(np.float32),    # near overflow
        np.array([65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001,
                  0.0, -0.0, np.inf, -np.inf, 1.0 + 2.0**-11, 1.0 + 3 * 2.0**-11], np.float32),
    ])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16_bits(x), want)


def test_bf16_matches_torch_rne():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(8)
    x = np.concatenate([rng.normal(size=100_000).astype(np.float32) * 10,
                        np.array([1.0, 1.0 + 2.0**-8, 1.0 + 3 * 2.0**-8, 3.3895e38, np.inf, -0.0],
                                 np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.f32_to_bf16_bits(x)
    assert np.array_equal(got, want)
    assert np.array_equal(O.bf16_bits_to_f32(got).view(np.uint32), got.astype(np.uint32) << 16)


# ------------------------------------------------------------------ Q8G32
def test_q8g32_closed_form_and_error_bound():
    rng = np.random.default_rng(11)
    n, k = 7, 96
    w = rng.normal(0, 0.02, size=(n, k)).astype(np.float32)
    qs, d = O.quantize_q8g32(w, n, k)
    g = w.reshape(n, k // 32, 32)
    amax = np.abs(g).max(axis=2)
    d32 = (amax / np.float32(127.0)).astype(np.float32)
    assert np.array_equal(d.view(np.uint16), d32.astype(np.float16).view(np.uint16))
    inv = np.where(d32 != 0, np.float32(1.0) / d32, 0).astype(np.float32)
    x = g * inv[..., None]
    q_want = np.clip(np.sign(x) * np.floor(np.abs(x) + np.float32(0.5)), -127, 127)
    assert np.array_equal(qs.reshape(g.shape), q_want.astype(np.int8))
    # |w - d*q| <= d/2 (+ the f16 rounding of d: |q| * d * 2^-11)
    wh = O.dequantize_q8g32(qs, d, n, k).reshape(g.shape)
    bound = d32[..., None] * (0.5 + 127 * 2.0**-11) + 1e-9
    assert (np.abs(wh - g) <= bound).all()
    # the element with the largest magnitude maps to +-127
    assert (np.abs(qs.reshape(g.shape)).max(axis=2) == 127).all()


def test_q8g32_zero_group_and_all_equal_group():
    w = np.zeros((1, 64), np.float32)
    w[0, 32:] = 0.5
    qs, d = O.quantize_q8g32(w, 1, 64)
    assert (qs[0, :32] == 0).all() and float(d[0, 0]) == 0.0
    assert (qs[0, 32:] == 127).all()
    wh = O.dequantize_q8g32(qs, d, 1, 64)
    assert np.abs(wh[0, 32:] - 0.5).max() <= 0.5 * 2.0**-11 * 1.01
    assert (wh[0, :32] == 0).all()


def test_q8_0_block_stream_layout_and_roundtrip():
    rng = np.random.default_rng(12)
    n, k = 3, 64
    qs, d = O.quantize_q8g32(rng.normal(size=(n, k)).astype(np.float32), n, k)
    blocks = O.q8g32_to_q8_0_blocks(qs, d, n, k)
    assert blocks.size == n * (k // 32) * 34
    b = blocks.reshape(n, k // 32, 34)
    # {f16 d little-endian; int8 qs[32]}
    assert np.array_equal(b[:, :, 0].astype(np.uint16) | (b[:, :, 1].astype(np.uint16) << 8),
                          d.view(np.uint16))
    assert np.array_equal(b[:, :, 2:].reshape(n, k).view(np.int8), qs)
    qs2, d2 = O.q8_0_blocks_to_q8g32(blocks, n, k)
    assert np.array_equal(qs2, qs) and np.array_equal(d2.view(np.uint16), d.view(np.uint16))


def test_qgemv_q8_equals_linear_t_over_dequantised_matrix():
    rng = np.random.default_rng(13)
    n, k = 33, 160
    w = rng.normal(0, 0.02, size=(n, k)).astype(np.float32)
    x = rng.normal(size=k).astype(np.float32)
    qs, d = O.quantize_q8g32(w, n, k)
    y = O.qgemv_q8g32_f32(x, qs, d, n, k)
    wd = O.dequantize_q8g32(qs, d, n, k)
    # same ascending-k fp32 arithmetic as linear_t at m = 1: bit-identical
    assert np.array_equal(y, O.linear_t(x, wd, None, 1, n, k))
    # float64 brute force
    y64 = wd.astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - y64).max() < 1e-5
    # orientation: row r of W produces y[r] (a transposed operand fails here)
    x1 = np.zeros(k, np.float32)
    x1[5] = 1.0
    assert np.array_equal(O.qgemv_q8g32_f32(x1, qs, d, n, k), wd[:, 5])


# ------------------------------------------------------------------ Q4G128
def test_q4g128_invariants():
    rng = np.random.default_rng(21)
    n, k = 5, 256
    w = rng.normal(0, 0.02, size=(n, k)).astype(np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    assert qw.shape == (n, k // 2) and s.shape == (n, 2) and z.shape == (n, 2)
    g = w.reshape(n, 2, 128)
    s_want = ((g.max(axis=2) - g.min(axis=2)) / np.float32(15.0)).astype(np.float16)
    assert np.array_equal(s.view(np.uint16), s_want.view(np.uint16))
    sf = s.astype(np.float32)
    z_want = (-g.min(axis=2) / sf).astype(np.float32).astype(np.float16)
    assert np.array_equal(z.view(np.uint16), z_want.view(np.uint16))
    idx = O.unpack_nibbles(qw.ravel(), n * k).reshape(n, 2, 128)
    assert idx.min() == 0 and idx.max() == 15
    wh = O.dequantize_q4g128(qw, s, z, n, k).reshape(n, 2, 128)
    # |w - w^| <= s/2 plus the error of the rounded zero point (|z| * 2^-11 * s)
    zf = z.astype(np.float32)
    bound = sf[..., None] * (0.5 + np.abs(zf[..., None]) * 2.0**-11) + 1e-7
    assert (np.abs(wh - g) <= bound).all()
    # dequantisation closed form
    assert np.array_equal(wh, (idx.astype(np.float32) - zf[..., None]) * sf[..., None])


def test_q4g128_nibble_order_low_first():
    w = np.zeros((1, 128), np.float32)
    w[0, 0] = 0.0
    w[0, 1] = 15.0  # scale = 1, zero = 0 -> q = w
    w[0, 2] = 3.0
    qw, s, z = O.quantize_q4g128(w, 1, 128)
    assert float(s[0, 0]) == 1.0 and float(z[0, 0]) == 0.0
    assert qw[0, 0] == 0xF0 and qw[0, 1] == 0x03


def test_q4g128_constant_group_is_exact():
    w = np.full((1, 128), 0.375, np.float32)
    qw, s, z = O.quantize_q4g128(w, 1, 128)
    assert np.array_equal(O.dequantize_q4g128(qw, s, z, 1, 128), w)


def test_qgemm_q4_matches_float64_bruteforce():
    rng = np.random.default_rng(22)
    b, n, k = 3, 17, 256
    w = rng.normal(0, 0.02, size=(n, k)).astype(np.float32)
    x_bits = O.f32_to_bf16_bits(rng.normal(size=(b, k)).astype(np.float32))
    qw, s, z = O.quantize_q4g128(w, n, k)
    y = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(x_bits, qw, s, z, b, n, k))
    wd = O.dequantize_q4g128(qw, s, z, n, k).astype(np.float64)
    y64 = O.bf16_bits_to_f32(x_bits).astype(np.float64) @ wd.T
    assert y.shape == (b, n)
    # one bf16 rounding of an fp32 sum: relative 2^-9
    assert (np.abs(y - y64) <= np.abs(y64) * 2.0**-8 + 1e-6).all()


def test_quantized_products_with_bias_equal_linear_t_with_bias():
    """`linear_t(a, b, Some(bias), m, n, k)` (crates/kernels/src/cpu_f32/mod.rs:271-345, pinned
    by cpu_f32/tests.rs:46-63,84-92 on the oracle's linear_t): the quantized products with a
    bias are that function over the dequantised matrix -- the bias is added to the finished
    fp32 sum, once per output, the same vector for every row."""
    rng = np.random.default_rng(23)
    b, n, k = 3, 19, 256
    w = rng.normal(0, 0.02, size=(n, k)).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    x = rng.normal(size=(b, k)).astype(np.float32)
    # Q8G32, m = 1: bit-identical to linear_t with the bias (same ascending-k sum, one add)
    qs, d = O.quantize_q8g32(w, n, k)
    wd8 = O.dequantize_q8g32(qs, d, n, k)
    assert np.array_equal(O.qgemv_q8g32_f32(x[0], qs, d, n, k, bias),
                          O.linear_t(x[0], wd8, bias, 1, n, k))
    # the reference's hand-computed case (tests.rs:84-92) through the quantized path: weights
    # that Q8G32 holds exactly
    w_exact = np.zeros((2, 32), np.float32)
    w_exact[0, 0] = 1.0
    w_exact[1, 1] = w_exact[1, 2] = 1.0
    qe, de = O.quantize_q8g32(w_exact, 2, 32)
    xe = np.zeros(32, np.float32)
    xe[:3] = [1.0, 2.0, 3.0]
    ye = O.qgemv_q8g32_f32(xe, qe, de, 2, 32, [10.0, 20.0])
    assert abs(ye[0] - 11.0) < 1e-2 and abs(ye[1] - 25.0) < 1e-2  # d = 1/127 in fp16
    # Q4G128 and Q4G32, m = 3: float64 brute force, bias before the bf16 rounding
    x_bits = O.f32_to_bf16_bits(x)
    xb = O.bf16_bits_to_f32(x_bits).astype(np.float64)
    qw, s, z = O.quantize_q4g128(w, n, k)
    wd4 = O.dequantize_q4g128(qw, s, z, n, k).astype(np.float64)
    y64 = xb @ wd4.T + bias.astype(np.float64)
    yf = O.qgemm_q4g128_f32(x_bits, qw, s, z, b, n, k, bias)
    assert np.abs(yf - y64).max() < 2e-5
    yb = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(x_bits, qw, s, z, b, n, k, bias))
    assert (np.abs(yb - y64) <= np.abs(y64) * 2.0**-8 + 1e-6).all()
    # without a bias nothing changes, and the bias is not applied twice or per group
    assert np.array_equal(O.qgemm_q4g128_f32(x_bits, qw, s, z, b, n, k, None),
                          O.qgemm_q4g128_f32(x_bits, qw, s, z, b, n, k))
    assert np.abs((yf - O.qgemm_q4g128_f32(x_bits, qw, s, z, b, n, k)) - bias).max() < 1e-6
    blocks = O.quantize_q4_blocks(w, n, k, True)
    q32, s32, m32 = O.q4_blocks_to_q4g32(blocks, n, k, True)
    wd32 = O.dequantize_q4g32(q32, s32, m32, n, k).astype(np.float64)
    y32 = O.qgemm_q4g32_f32(x_bits, q32, s32, m32, b, n, k, bias)
    assert np.abs(y32 - (xb @ wd32.T + bias)).max() < 2e-5


# ------------------------------------------------------------------ ragged packing
def test_pack_ragged_closed_forms():
    rng = np.random.default_rng(31)
    s, bs, max_blocks = 9, 16, 40
    new = rng.integers(0, 70, size=s).astype(np.int32)
    new[3] = 0
    prior = rng.integers(0, 500, size=s).astype(np.int32)
    bt = rng.permutation(s * max_blocks).astype(np.int32).reshape(s, max_blocks)
    cu, slots, ctx, bad = O.pack_ragged(new, prior, bt, bs)
    assert bad == 0
    assert cu[0] == 0 and np.array_equal(cu[1:], np.cumsum(new))
    assert np.array_equal(ctx, prior + new)
    t = 0
    for i in range(s):
        for j in range(new[i]):
            pos = prior[i] + j
            assert slots[t] == int(bt[i, pos // bs]) * bs + pos % bs
            t += 1
    assert t == slots.size


def test_pack_ragged_reference_cu_seqlens_example():
    """research/14-gdn-aiter-preflight.md:338 -- [0, 512, 1536, 2048]"""
    bt = np.arange(3 * 64, dtype=np.int32).reshape(3, 64)
    cu, _, _, _ = O.pack_ragged([512, 1024, 512], [0, 0, 0], bt, 16)
    assert cu.tolist() == [0, 512, 1536, 2048]


def test_pack_ragged_overflowing_position_gets_minus_one():
    bt = np.arange(2, dtype=np.int32).reshape(1, 2)
    cu, slots, ctx, bad = O.pack_ragged([3], [30], bt, 16)
    assert bad == 1 and slots.tolist() == [1 * 16 + 14, 1 * 16 + 15, -1]
    assert ctx.tolist() == [32]  # capped at what the table row holds (LenOverflow upstream)
    with pytest.raises(ValueError):
        O.pack_ragged([-1], [0], bt, 16)


def test_pack_ragged_entries_that_name_no_block_give_no_slot():
    # the cache marks never-mapped entries 0x3FFFFFFF; the workloads poison with 0x3FFFFFF;
    # a negative id is no block either
    bt = np.array([[5, 0x3FFFFFFF, -3, 0x3FFFFFF, 0x3FFFFFE]], np.int32)
    cu, slots, ctx, bad = O.pack_ragged([80], [0], bt, 16)
    assert bad == 48 and ctx.tolist() == [80]
    assert slots[:16].tolist() == [5 * 16 + i for i in range(16)]
    assert (slots[16:64] == -1).all()
    assert slots[64:].tolist() == [0x3FFFFFE * 16 + i for i in range(16)]


def test_kv_write_then_gather_is_identity_through_a_permutation():
    rng = np.random.default_rng(32)
    bs, row, nblk = 16, 2 * 8, 12
    ctx = 150
    perm = rng.permutation(nblk).astype(np.int32)
    bt = perm[: math.ceil(ctx / bs)][None, :]
    k_new = rng.normal(size=(ctx, row)).astype(np.float16)
    v_new = rng.normal(size=(ctx, row)).astype(np.float16)
    _, slots, _, _ = O.pack_ragged([ctx], [0], bt, bs)
    k_pool = np.zeros((nblk * bs, row), np.float16)
    v_pool = np.zeros((nblk * bs, row), np.float16)
    O.kv_write_fp16(k_new, v_new, k_pool, v_pool, slots, row)
    assert np.array_equal(O.paged_gather_fp16(k_pool, bt[0], ctx, bs, row), k_new)
    assert np.array_equal(O.paged_gather_fp16(v_pool, bt[0], ctx, bs, row), v_new)
    # independent scatter in numpy
    ref = np.zeros_like(k_pool)
    for p in range(ctx):
        ref[perm[p // bs] * bs + p % bs] = k_new[p]
    assert np.array_equal(ref, k_pool)


def test_identity_block_table_is_flat_cache_row_order():
    """With block_table = [0,1,2,..] the pool IS a FlatKvCache buffer: rows in token
    order, row = [kv_heads][head_dim] (crates/cache/src/flat.rs:180-252)."""
    ctx, row = 40, 6
    flat = np.arange(48 * row, dtype=np.float32).astype(np.float16).reshape(48, row)
    bt = np.arange(3, dtype=np.int32)
    assert np.array_equal(O.paged_gather_fp16(flat, bt, ctx, 16, row), flat[:ctx])


# ------------------------------------------------------------------ paged attention
def _brute_paged_attn(q, k_pool, v_pool, bt, cu, ctx_lens, hq, hkv, d, bs, scale, causal):
    out = np.zeros(q.shape, np.float64)
    g = hq // hkv
    kp = k_pool.astype(np.float64).reshape(-1, hkv, d)
    vp = v_pool.astype(np.float64).reshape(-1, hkv, d)
    for s in range(len(ctx_lens)):
        c = int(ctx_lens[s])
        n = int(cu[s + 1] - cu[s])
        rows = [int(bt[s, p // bs]) * bs + p % bs for p in range(c)]
        for i in range(n):
            vis = c - n + i + 1 if causal else c
            for h in range(hq):
                if vis <= 0:
                    continue
                kk = kp[rows[:vis], h // g]
                vv = vp[rows[:vis], h // g]
                sc = (kk @ q[cu[s] + i, h].astype(np.float64)) * scale
                p = np.exp(sc - sc.max())
                p /= p.sum()
                out[cu[s] + i, h] = p @ vv
    return out


def _make_paged_case(rng, new, prior, hq, hkv, d, bs, spare=3):
    new = np.asarray(new, np.int32)
    prior = np.asarray(prior, np.int32)
    ctx = new + prior
    nblk_seq = [(int(c) + bs - 1) // bs for c in ctx]
    total_blocks = sum(nblk_seq) + spare
    perm = rng.permutation(total_blocks).astype(np.int32)
    max_blocks = max(max(nblk_seq), 1) + 1
    bt = np.full((len(new), max_blocks), -7, np.int32)  # unread entries are poison
    o = 0
    for s, nb in enumerate(nblk_seq):
        bt[s, :nb] = perm[o:o + nb]
        o += nb
    k_pool = rng.normal(size=(total_blocks * bs, hkv * d)).astype(np.float16)
    v_pool = rng.normal(size=(total_blocks * bs, hkv * d)).astype(np.float16)
    cu = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    q = rng.normal(size=(int(cu[-1]), hq, d)).astype(np.float16)
    return q, k_pool, v_pool, bt, cu, ctx.astype(np.int32)


@pytest.mark.parametrize("causal", [True, False])
def test_paged_attn_matches_float64_bruteforce(causal):
    rng = np.random.default_rng(41)
    hq, hkv, d, bs = 6, 2, 32, 16
    q, kp, vp, bt, cu, ctx = _make_paged_case(rng, [1, 5, 1, 17], [37, 0, 0, 23], hq, hkv, d, bs)
    scale = 1.0 / math.sqrt(d)
    got = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, scale, causal)
    want = _brute_paged_attn(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, scale, causal)
    assert np.abs(got.astype(np.float64) - want).max() < 2e-3
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16)) or \
        np.abs(got.astype(np.float64) - want).max() <= np.abs(want).max() * 2.0**-10


def test_paged_attn_identity_table_equals_reference_sdpa():
    """One sequence, identity block table, non-causal, every query sees every key:
    exactly the SDPA section of QwenAttention::forward on contiguous K/V."""
    rng = np.random.default_rng(42)
    hq, hkv, d, bs, seq = 4, 2, 16, 16, 32
    k = rng.normal(size=(seq, hkv, d)).astype(np.float16)
    v = rng.normal(size=(seq, hkv, d)).astype(np.float16)
    q = rng.normal(size=(seq, hq, d)).astype(np.float16)
    bt = np.arange(2, dtype=np.int32)[None, :]
    got = O.paged_attn_varlen_fp16(q, k.reshape(seq, -1), v.reshape(seq, -1), bt, [0, seq], [seq],
                                   hq, hkv, d, bs, 1.0 / math.sqrt(d), causal=False)
    f = lambda a, h: O.transpose_seq_heads(a.astype(np.float32), seq, h, d)
    ref = O.sdpa_f32(f(q, hq), f(k, hkv), f(v, hkv), np.ones(seq, np.uint8), hq, hkv, seq, d)
    ref = O.merge_heads(ref, hq, seq, d).reshape(seq, hq, d)
    assert np.array_equal(got, ref.astype(np.float16))


def test_paged_attn_special_cases():
    rng = np.random.default_rng(43)
    hq, hkv, d, bs = 4, 2, 8, 16
    # ctx = 1: out = v0 of the mapped kv head
    q, kp, vp, bt, cu, ctx = _make_paged_case(rng, [1], [0], hq, hkv, d, bs)
    got = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, 0.3)
    v0 = vp[bt[0, 0] * bs].reshape(hkv, d)
    assert np.array_equal(got[0], v0[[0, 0, 1, 1]])
    # all keys equal: softmax is uniform, out = mean(v)
    q, kp, vp, bt, cu, ctx = _make_paged_case(rng, [1], [40], hq, hkv, d, bs)
    kp[:] = kp[0]
    got = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, 0.3).astype(np.float32)
    rows = [bt[0, p // bs] * bs + p % bs for p in range(41)]
    mean = vp[rows].astype(np.float32).reshape(41, hkv, d).mean(axis=0)
    assert np.abs(got[0] - mean[[0, 0, 1, 1]]).max() < 2e-3
    # chunk of length 1 with causal masking equals plain decode
    a = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, 0.3, causal=True)
    b = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, 0.3, causal=False)
    assert np.array_equal(a, b)
    # empty sequence and zero context: nothing written, zeros
    out = O.paged_attn_varlen_fp16(q, kp, vp, bt, [0, 1], [0], hq, hkv, d, bs, 0.3)
    assert (out == 0).all()


def test_paged_attn_scale_multiplies_the_dot_product():
    rng = np.random.default_rng(44)
    hq, hkv, d, bs = 2, 1, 16, 16
    q, kp, vp, bt, cu, ctx = _make_paged_case(rng, [1], [30], hq, hkv, d, bs)
    hot = O.paged_attn_varlen_fp16(q, kp, vp, bt, cu, ctx, hq, hkv, d, bs, 50.0).astype(np.float32)
    # a huge scale turns softmax into argmax: out = v[argmax q.k]
    rows = [bt[0, p // bs] * bs + p % bs for p in range(31)]
    for h in range(hq):
        j = int(np.argmax(kp[rows].astype(np.float32) @ q[0, h].astype(np.float32)))
        assert np.abs(hot[0, h] - vp[rows[j]].astype(np.float32)).max() < 2e-2
