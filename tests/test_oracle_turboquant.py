"""Pins of the oracle's TurboQuant 3-bit KV codec against the reference's own tests and
constants (crates/quant/src/lib.rs), and of the attention over turbo3 pools against an
independent numpy restatement."""
import numpy as np
import pytest

import oracle as O


def _cyclic(n, period):
    return (np.arange(n) % period).astype(np.uint8)


def test_block_sizes_match_the_upstream_contract():
    # turbo3_block_layout_matches_upstream_contract (lib.rs:492-498): 14-byte blocks, 56 / head
    assert O.TURBO3_BYTES_PER_HEAD == 56
    assert O.encode_turbo3_0_head(np.zeros(128, np.float32)).size == 4 * 14


def test_turbo3_pack_matches_golden_pattern():
    # lib.rs:536-549
    idx = _cyclic(32, 8)
    expected = np.array([0x88, 0xC6, 0xFA] * 4, np.uint8)
    assert np.array_equal(O.pack_turbo3_indices(idx), expected)
    assert np.array_equal(O.unpack_turbo3_indices(expected), idx)


def test_turbo3_pack_rejects_out_of_range_index():
    # lib.rs:566-581: position 5, value 8
    idx = np.zeros(32, np.uint8)
    idx[5] = 8
    with pytest.raises(ValueError, match="position 5"):
        O.pack_turbo3_indices(idx)


def test_pack_unpack_roundtrip_random_and_bit_positions():
    rng = np.random.default_rng(0)
    for _ in range(50):
        idx = rng.integers(0, 8, 32).astype(np.uint8)
        p = O.pack_turbo3_indices(idx)
        assert np.array_equal(O.unpack_turbo3_indices(p), idx)
        # index i lives at bits [3i, 3i+3) of the little-endian integer
        big = int.from_bytes(p.tobytes(), "little")
        assert all(((big >> (3 * i)) & 7) == idx[i] for i in range(32))


def test_codebook_is_the_upstream_table():
    # lib.rs:66-80
    want = np.array([-0.1883972972, -0.1181399059, -0.0665857641, -0.0216044751,
                     0.0216041461, 0.0665854520, 0.1181396281, 0.1883970748], np.float32)
    assert np.array_equal(O.turbo3_codebook(), want)


def test_fwht_128_identity():
    # lib.rs:660-668
    data = (np.sin(np.arange(128, dtype=np.float32)) * np.float32(0.5)).astype(np.float32)
    twice = O.fwht_128(O.fwht_128(data))
    assert np.abs(twice - data).max() < 1e-5


def test_fwht_128_orthonormal():
    # lib.rs:671-682
    data = (np.cos(np.arange(128, dtype=np.float32)) * np.float32(0.3)).astype(np.float32)
    t = O.fwht_128(data)
    assert abs(np.sqrt((data * data).sum()) - np.sqrt((t * t).sum())) < 1e-5


def test_fwht_128_is_the_sylvester_hadamard_matrix():
    # closed form: H[i][j] = (-1)^popcount(i & j) / sqrt(128) (natural order)
    i = np.arange(128)
    h = np.array([[(-1.0) ** bin(a & b).count("1") for b in i] for a in i]) / np.sqrt(128.0)
    rng = np.random.default_rng(1)
    x = rng.standard_normal(128).astype(np.float32)
    assert np.abs(O.fwht_128(x) - h @ x.astype(np.float64)).max() < 1e-5
    e = np.zeros(128, np.float32)
    e[37] = 1.0
    assert np.allclose(O.fwht_128(e), h[:, 37], atol=1e-7)


def test_encode_decode_turbo3_roundtrip():
    # lib.rs:685-699: same data, same bound
    i = np.arange(128, dtype=np.float32)
    src = (np.sin(i * np.float32(0.1)) * np.float32(0.1) +
           np.cos(i * np.float32(0.03)) * np.float32(0.1)).astype(np.float32)
    dec = O.decode_turbo3_0_head(O.encode_turbo3_0_head(src))
    assert ((src - dec) ** 2).sum() / 128.0 < 0.05


def test_encode_rejects_wrong_head_dim_and_decode_wrong_block_count():
    # lib.rs:598-609, 702-712, 625-637
    with pytest.raises(ValueError):
        O.encode_turbo3_0_head(np.zeros(0, np.float32))
    with pytest.raises(ValueError):
        O.decode_turbo3_0_head(np.zeros(0, np.uint8))


def test_encode_follows_the_reference_steps():
    # an independent numpy restatement of encode (lib.rs:316-353) and decode (:376-413)
    rng = np.random.default_rng(2)
    cb = O.turbo3_codebook()
    for _ in range(20):
        v = (rng.standard_normal(128) * rng.uniform(0.01, 30)).astype(np.float32)
        enc = O.encode_turbo3_0_head(v)
        ss = np.float32(0.0)
        for x in v:
            ss = np.float32(ss + np.float32(x * x))
        norm = np.sqrt(ss, dtype=np.float32)
        t = O.fwht_128((v / norm).astype(np.float32))
        idx = np.abs(t[:, None] - cb[None, :]).argmin(axis=1).astype(np.uint8)   # first minimum
        for b in range(4):
            blk = enc[14 * b:14 * b + 14]
            assert blk[:2].tobytes() == np.float16(norm).tobytes()          # norm in every block
            assert np.array_equal(O.unpack_turbo3_indices(blk[2:]), idx[32 * b:32 * b + 32])
        dec = O.decode_turbo3_0_head(enc)
        want = O.fwht_128(cb[idx]) * np.float32(np.float16(norm))
        assert np.array_equal(dec, want)


def test_zero_vector_and_norm_from_the_first_block():
    enc = O.encode_turbo3_0_head(np.zeros(128, np.float32))
    assert (enc.reshape(4, 14)[:, :2] == 0).all()
    assert (O.decode_turbo3_0_head(enc) == 0).all()
    # decode scales by the FIRST block's norm (lib.rs:398-411)
    v = np.linspace(-1, 1, 128, dtype=np.float32)
    enc = O.encode_turbo3_0_head(v)
    base = O.decode_turbo3_0_head(enc)
    enc2 = enc.copy()
    enc2[14:16] = np.frombuffer(np.float16(123.0).tobytes(), np.uint8)    # block 1's norm: ignored
    assert np.array_equal(O.decode_turbo3_0_head(enc2), base)
    enc2[0:2] = np.frombuffer(np.float16(2.0).tobytes(), np.uint8)
    n0 = np.float32(np.frombuffer(enc[0:2].tobytes(), np.float16)[0])
    assert np.allclose(O.decode_turbo3_0_head(enc2), base / n0 * np.float32(2.0), rtol=1e-6)


def test_quantisation_error_is_that_of_the_codebook():
    # after normalisation the coefficients have unit norm; the decode error relative to the
    # input norm is the codebook's quantisation error (< 0.25 for Gaussian-like data)
    rng = np.random.default_rng(3)
    for _ in range(10):
        v = rng.standard_normal(128).astype(np.float32)
        dec = O.decode_turbo3_0_head(O.encode_turbo3_0_head(v))
        assert np.linalg.norm(dec - v) / np.linalg.norm(v) < 0.25


def _turbo3_case(rng, new, prior, hq, hkv, bs=16):
    from tests import workloads
    c = workloads.paged_case(rng, new, prior, hq=hq, hkv=hkv, block_size=bs)
    rows = c["k_pool"].shape[0]
    kp = np.zeros((rows, hkv * 56), np.uint8)
    vp = np.zeros((rows, hkv * 56), np.uint8)
    slots = np.arange(rows, dtype=np.int64)
    O.kv_write_turbo3(c["k_pool"], c["v_pool"], kp, vp, slots, hkv)
    return c, kp, vp


def test_kv_write_turbo3_encodes_each_head_row_at_its_slot():
    rng = np.random.default_rng(4)
    k = rng.standard_normal((5, 2 * 128)).astype(np.float16)
    v = rng.standard_normal((5, 2 * 128)).astype(np.float16)
    kp = np.full((8, 2 * 56), 0xAA, np.uint8)
    vp = np.full((8, 2 * 56), 0xAA, np.uint8)
    slots = np.array([3, -1, 0, 7, 5], np.int64)
    O.kv_write_turbo3(k, v, kp, vp, slots, 2)
    for t, s in enumerate(slots):
        if s < 0:
            continue
        for h in range(2):
            assert np.array_equal(kp[s, 56 * h:56 * h + 56],
                                  O.encode_turbo3_0_head(k[t, 128 * h:128 * h + 128].astype(np.float32)))
            assert np.array_equal(vp[s, 56 * h:56 * h + 56],
                                  O.encode_turbo3_0_head(v[t, 128 * h:128 * h + 128].astype(np.float32)))
    untouched = [1, 2, 4, 6]
    assert (kp[untouched] == 0xAA).all() and (vp[untouched] == 0xAA).all()


@pytest.mark.parametrize("causal", [True, False])
def test_attention_over_turbo3_pools_equals_sdpa_over_the_decoded_rows(causal):
    rng = np.random.default_rng(5)
    new, prior = [1, 3, 1], [20, 5, 0]
    hq, hkv = 4, 2
    c, kp, vp = _turbo3_case(rng, new, prior, hq, hkv)
    got = O.paged_attn_varlen_turbo3(c["q"], kp, vp, c["block_tables"], c["cu_seqlens"],
                                     c["context_lens"], hq, hkv, 16, c["scale"], causal)
    want = np.zeros(c["q"].shape, np.float64)
    for s in range(3):
        ctx = int(c["context_lens"][s])
        kf = O.paged_gather_turbo3(kp, c["block_tables"][s], ctx, 16, hkv).astype(np.float64)
        vf = O.paged_gather_turbo3(vp, c["block_tables"][s], ctx, 16, hkv).astype(np.float64)
        for i in range(new[s]):
            t = int(c["cu_seqlens"][s]) + i
            vis = ctx - new[s] + i + 1 if causal else ctx
            for h in range(hq):
                kh = kf[:vis, (h // 2) * 128:(h // 2) * 128 + 128]
                vh = vf[:vis, (h // 2) * 128:(h // 2) * 128 + 128]
                sc = kh @ c["q"][t, h].astype(np.float64) * c["scale"]
                p = np.exp(sc - sc.max())
                want[t, h] = (p / p.sum()) @ vh
    assert np.abs(got.astype(np.float64) - want).max() < 2e-3
