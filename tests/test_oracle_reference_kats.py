"""Pins the CPU oracle to the reference's own known-answer tests.

Each test restates one test of the reference (file:line in the docstring) with
the same inputs and the same expected values, so the oracle's restatement of
`cpu_f32`, the fp16 refs, the attention helpers, `greedy` and the nibble order
is checked against numbers the reference itself holds.
"""
import math

import numpy as np
import pytest

import oracle as O


def test_embed_lookup_in_range_copies_rows():
    """crates/kernels/src/cpu_f32/tests.rs:5-13"""
    w = [1.0, 2.0, 10.0, 20.0, 100.0, 200.0]
    out = O.embed_lookup(w, 2, 3, [1, 0, 2])
    assert out.tolist() == [10.0, 20.0, 1.0, 2.0, 100.0, 200.0]


def test_embed_lookup_out_of_range_id_yields_zero_row():
    """crates/kernels/src/cpu_f32/tests.rs:16-31"""
    out = O.embed_lookup([1.0, 2.0, 10.0, 20.0], 2, 2, [0, 5])
    assert out.tolist() == [1.0, 2.0, 0.0, 0.0]


def test_rms_norm_matches_manual():
    """crates/kernels/src/cpu_f32/tests.rs:34-43"""
    y = O.rms_norm([1.0, 2.0, 3.0, 4.0], [1.0] * 4, 1, 4, 1e-6)
    inv = np.float32(1.0) / np.sqrt(np.float32((1.0 + 4.0 + 9.0 + 16.0) / 4.0) + np.float32(1e-6))
    want = np.array([1.0, 2.0, 3.0, 4.0], np.float32) * inv
    assert np.abs(y - want).max() < 1e-6


def test_linear_matches_hand_computed():
    """crates/kernels/src/cpu_f32/tests.rs:46-63"""
    a = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    b = [1.0, 0.0, 0.0, 1.0, 1.0, 1.0]
    y = O.linear(a, b, [100.0, 200.0], 2, 2, 3)
    assert np.abs(y - np.array([104.0, 205.0, 110.0, 211.0])).max() < 1e-5


def test_linear_matches_linear_t_with_transposed_weight():
    """crates/kernels/src/cpu_f32/tests.rs:66-81"""
    a = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    b = [1.0, 0.0, 0.0, 1.0, 1.0, 1.0]
    b_t = [1.0, 0.0, 1.0, 0.0, 1.0, 1.0]
    assert np.abs(O.linear(a, b, None, 2, 2, 3) - O.linear_t(a, b_t, None, 2, 2, 3)).max() < 1e-5


def test_linear_t_matches_naive():
    """crates/kernels/src/cpu_f32/tests.rs:84-92"""
    y = O.linear_t([1.0, 2.0, 3.0], [1.0, 0.0, 0.0, 0.0, 1.0, 1.0], [10.0, 20.0], 1, 2, 3)
    assert abs(y[0] - 11.0) < 1e-6 and abs(y[1] - 25.0) < 1e-6


@pytest.mark.parametrize("fn,a,b,bias", [
    ("linear", [1.0] * 5, [1.0] * 6, None),      # tests.rs:94-111  a too short
    ("linear", [1.0] * 6, [1.0] * 5, None),      # tests.rs:113-119 b too short
    ("linear", [1.0] * 6, [1.0] * 6, [1.0]),     # tests.rs:121-... bias too short
    ("linear_t", [1.0] * 5, [1.0] * 6, None),
    ("linear_t", [1.0] * 6, [1.0] * 5, None),
])
def test_linear_shape_guards_are_real(fn, a, b, bias):
    """crates/kernels/src/cpu_f32/tests.rs:94-224 -- the reference panics; the binding raises."""
    with pytest.raises(ValueError):
        getattr(O, fn)(a, b, bias, 2, 2, 3)


def test_softmax_rows_sum_to_one():
    """crates/kernels/src/cpu_f32/tests.rs:227-234"""
    y = O.softmax_last_dim([0.0, 1.0, 2.0, -1.0, 0.0, 1.0], 2, 3).reshape(2, 3)
    assert np.abs(y.sum(axis=1) - 1.0).max() < 1e-6


def test_softmax_fully_masked_row_is_uniform_not_nan():
    """crates/kernels/src/cpu_f32/tests.rs:237-250"""
    y = O.softmax_last_dim([-np.inf] * 4, 1, 4)
    assert np.isfinite(y).all()
    assert abs(y.sum() - 1.0) < 1e-6
    assert np.abs(y - 0.25).max() < 1e-6


def test_softmax_mixed_masked_and_unmasked_rows_both_finite():
    """crates/kernels/src/cpu_f32/tests.rs:253-274"""
    y = O.softmax_last_dim([-np.inf, -np.inf, -np.inf, 0.0, 1.0, 2.0], 2, 3).reshape(2, 3)
    assert np.isfinite(y).all()
    assert np.abs(y.sum(axis=1) - 1.0).max() < 1e-6


def test_softmax_matches_float64_closed_form():
    rng = np.random.default_rng(3)
    x = rng.normal(size=(5, 37)).astype(np.float32) * 4
    y = O.softmax_last_dim(x, 5, 37).reshape(5, 37)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    assert np.abs(y - e / e.sum(axis=1, keepdims=True)).max() < 1e-6


def test_rope_zero_pos_identity_halves():
    """crates/kernels/src/cpu_f32/tests.rs:277-282"""
    x = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    cos, sin = O.build_rope_table_f32(1, 4, 1_000_000.0)
    O.rope_halves_in_place(x, cos, sin, 1, 4)
    assert x.tolist() == [1.0, 2.0, 3.0, 4.0]


def test_rope_table_nonzero_position_matches_hand_computed_angles():
    """crates/kernels/src/cpu_f32/tests.rs:285-327"""
    cos, sin = O.build_rope_table_f32(2, 4, 10_000.0)
    half = 2
    assert abs(cos[half] - math.cos(1.0)) < 1e-5 and abs(sin[half] - math.sin(1.0)) < 1e-5
    assert abs(cos[half + 1] - math.cos(0.01)) < 1e-5
    assert abs(sin[half + 1] - math.sin(0.01)) < 1e-5


def test_rope_rotation_is_inverse():
    """crates/kernels/src/cpu_f32/tests.rs:330-343"""
    x = np.array([1.0, 2.0], np.float32)
    c = np.array([math.sqrt(0.5)], np.float32)
    O.rope_halves_in_place(x, c, c, 1, 2)
    O.rope_halves_in_place(x, c, -c, 1, 2)
    assert np.abs(x - [1.0, 2.0]).max() < 1e-5


def test_rope_halves_pairs_i_with_i_plus_half():
    # the halves convention (not interleaved pairs): element i rotates with i + d/2
    x = np.array([1.0, 0.0, 0.0, 0.0], np.float32)
    cos = np.array([0.0, 1.0], np.float32)
    sin = np.array([1.0, 0.0], np.float32)
    O.rope_halves_in_place(x, cos, sin, 1, 4)
    assert x.tolist() == [0.0, 0.0, 1.0, 0.0]


def test_mask_additive_broadcasts_across_heads():
    """crates/kernels/src/cpu_f32/tests.rs:380-391 -- same inputs, same assertions"""
    s = np.ones(12, np.float32)                     # 4 rows, 3 cols
    mask = np.array([1, 0, 1, 1, 1, 1], np.uint8)   # 2 mask rows
    O.mask_additive_in_place(s, mask, 4, 3)
    # rows 0 + 1 see mask row 0 [1,0,1]; rows 2 + 3 see mask row 1 [1,1,1]
    assert np.isfinite(s[0]) and np.isneginf(s[1]) and np.isfinite(s[2])
    assert np.isneginf(s[4])
    assert np.isfinite(s[6:]).all()


def test_mask_additive_rejects_non_dividing_rows():
    """crates/kernels/src/cpu_f32/mod.rs:463-466 (the reference panics)"""
    with pytest.raises(ValueError):
        O.mask_additive_in_place(np.zeros(6, np.float32), np.ones(4, np.uint8), 3, 2)


def test_silu_known_values():
    """crates/kernels/src/cpu_f32/tests.rs:466-471 (+ one large argument)"""
    y = O.silu([0.0, 1.0, -1.0, 10.0])
    want = [0.0, 1 / (1 + math.exp(-1)), -1 / (1 + math.exp(1)), 10 / (1 + math.exp(-10))]
    assert np.abs(y - np.array(want)).max() < 1e-6


def test_hadamard_and_guard():
    assert O.hadamard([1.0, 2.0, 3.0], [4.0, 5.0, 6.0]).tolist() == [4.0, 10.0, 18.0]
    with pytest.raises(ValueError):
        O.hadamard([1.0, 2.0], [1.0])


def test_matmul_fp16_identity():
    """crates/kernels/src/matmul/cpu.rs:70-89"""
    a = np.array([1.0, 0.0, 0.0, 1.0], np.float16)
    b = np.array([1.0, 2.0, 3.0, 4.0, 5.0, 6.0], np.float16)
    assert O.matmul_fp16_ref(a, b, 2, 3, 2).tolist() == b.tolist()


def test_matmul_fp16_accumulates_in_fp32_and_rounds_once():
    # 2048 + 1 + 1: a running fp16 sum would stay at 2048; fp32 accumulation gives 2050.
    a = np.array([[2048.0, 1.0, 1.0]], np.float16)
    b = np.ones((3, 1), np.float16)
    assert float(O.matmul_fp16_ref(a, b, 1, 1, 3)[0]) == 2050.0


def test_softmax_fp16_ref_rows_and_masked_row():
    """crates/kernels/src/softmax/cpu.rs:84-96,118-137"""
    x = np.array([0.0, 1.0, 2.0, 3.0], np.float16)
    y = O.softmax_fp16_ref(x, 1, 4).astype(np.float32)
    assert abs(y.sum() - 1.0) < 2e-3
    y = O.softmax_fp16_ref(np.full(4, -np.inf, np.float16), 1, 4).astype(np.float32)
    assert np.isfinite(y).all() and np.abs(y - 0.25).max() < 1e-3
    with pytest.raises(ValueError):
        O.softmax_fp16_ref(x, 2, 4)


def test_rms_norm_fp16_ref_unit_weight():
    """crates/kernels/src/rms_norm/cpu.rs:52-67"""
    x = np.array([1.0, 2.0, 3.0, 4.0], np.float16)
    y = O.rms_norm_fp16_ref(x, np.ones(4, np.float16), 1, 4, 1e-6).astype(np.float32)
    inv = 1.0 / math.sqrt(30.0 / 4.0 + 1e-6)
    assert np.abs(y - np.array([1, 2, 3, 4]) * inv).max() < 2e-3


def test_transpose_roundtrips():
    """crates/transformers/src/attention.rs:430-438"""
    x = np.arange(3 * 2 * 2, dtype=np.float32)
    t = O.transpose_seq_heads(x, 3, 2, 2)
    assert O.merge_heads(t, 2, 3, 2).tolist() == x.tolist()
    assert t.reshape(2, 3, 2).tolist() == x.reshape(3, 2, 2).transpose(1, 0, 2).tolist()


def test_repeat_kv_basic():
    """crates/transformers/src/attention.rs:441-454 -- heads [kv0,kv0,kv0,kv1,kv1,kv1]"""
    rep = O.repeat_kv([1.0, 2.0, 10.0, 20.0], 2, 3, 1, 2)
    assert rep.tolist() == [1.0, 2.0, 1.0, 2.0, 1.0, 2.0, 10.0, 20.0, 10.0, 20.0, 10.0, 20.0]


def test_sdpa_fully_masked_is_finite():
    """crates/transformers/src/attention.rs:487-520 -- every key padded => finite output"""
    rng = np.random.default_rng(0)
    n_h, n_kv, seq, d = 2, 1, 3, 4
    q = rng.normal(size=(n_h, seq, d)).astype(np.float32)
    k = rng.normal(size=(n_kv, seq, d)).astype(np.float32)
    v = rng.normal(size=(n_kv, seq, d)).astype(np.float32)
    out = O.sdpa_f32(q, k, v, np.zeros(seq, np.uint8), n_h, n_kv, seq, d).reshape(n_h, seq, d)
    assert np.isfinite(out).all()
    # uniform weights => every row is the mean of v
    assert np.abs(out - v[0].mean(axis=0)).max() < 1e-6


def test_sdpa_matches_float64_textbook():
    rng = np.random.default_rng(1)
    n_h, n_kv, seq, d = 6, 2, 9, 16
    q = rng.normal(size=(n_h, seq, d)).astype(np.float32)
    k = rng.normal(size=(n_kv, seq, d)).astype(np.float32)
    v = rng.normal(size=(n_kv, seq, d)).astype(np.float32)
    mask = np.array([1, 1, 0, 1, 1, 1, 0, 1, 1], np.uint8)
    out = O.sdpa_f32(q, k, v, mask, n_h, n_kv, seq, d).reshape(n_h, seq, d)
    for h in range(n_h):
        kv = h // (n_h // n_kv)
        s = q[h].astype(np.float64) @ k[kv].astype(np.float64).T / math.sqrt(d)
        s[:, mask == 0] = -np.inf
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        assert np.abs(out[h] - p @ v[kv].astype(np.float64)).max() < 2e-6


def test_greedy_returns_first_max_index():
    """crates/decode/src/lib.rs:90-92"""
    assert O.greedy([0.0, 2.0, 2.0]) == 1
    assert O.greedy([-np.inf, -np.inf]) == 0


def test_turbo4_pack_matches_golden_pattern():
    """crates/quant/src/lib.rs:552-564 -- cyclic indices 0..15 pack to 10 32 54 76 98 BA DC FE"""
    idx = np.arange(32, dtype=np.uint8) % 16
    expected = bytes([0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE] * 2)
    assert O.pack_nibbles(idx).tobytes() == expected
    assert O.unpack_nibbles(np.frombuffer(expected, np.uint8), 32).tolist() == idx.tolist()


def test_pack_nibbles_rejects_out_of_range_index():
    """crates/quant/src/lib.rs:566-... (Error::IndexOutOfRange)"""
    idx = np.zeros(32, np.uint8)
    idx[5] = 16
    with pytest.raises(ValueError):
        O.pack_nibbles(idx)


def test_little_endian_element_pins():
    """crates/cache/src/flat_tests.rs:376-404 -- f16 1.0 = 00 3C, bf16 1.0 = 80 3F"""
    assert O.f32_to_f16_bits([1.0]).tobytes() == bytes([0x00, 0x3C])
    assert O.f32_to_bf16_bits([1.0]).tobytes() == bytes([0x80, 0x3F])


def test_parity_metric_matches_reference_definition():
    """crates/kernels/tests/matmul_parity.rs:83-99"""
    ma, mr = O.parity_metric([1.0, 0.0005, -2.0], [1.1, 0.0, -2.0])
    assert abs(ma - 0.1) < 1e-6
    assert abs(mr - max(0.1 / 1.1, 0.0005 / 1e-3)) < 1e-5


def test_rope_fp16_zero_positions_are_identity():
    """crates/kernels/src/rope/cpu.rs:133-158"""
    table = O.build_cos_sin_table(1, 4, 10_000.0)
    for i, v in enumerate(table):
        assert abs(v - (1.0 if i % 2 == 0 else 0.0)) < 1e-6
    orig = np.array([1.0, 2.0, 3.0, 4.0], np.float16)
    out = O.rope_apply_fp16_ref(orig, table, 1, 1, 1, 4)
    assert np.array_equal(out.view(np.uint16), orig.view(np.uint16))


def test_rope_fp16_table_length_mismatch_is_rejected():
    """crates/kernels/src/rope/cpu.rs:160-183"""
    short_table = np.zeros(4, np.float32)  # seq*head_dim = 8, only 4 present
    qk = np.ones(1 * 2 * 1 * 4, np.float16)
    with pytest.raises(ValueError, match="cos_sin.len"):
        O.rope_apply_fp16_ref(qk, short_table, 1, 2, 1, 4)


def test_rope_fp16_rotates_interleaved_pairs_by_the_table_angles():
    # what the reference leaves open, fixed by the mathematics: pair (2i, 2i+1) at position
    # pos is rotated by pos * theta^(-2i/d); a quarter turn maps (1, 0) to (0, 1); rotating
    # by the table and by its transpose-in-sign (sin -> -sin) returns the input
    d, seq = 8, 5
    table = O.build_cos_sin_table(seq, d, 10_000.0).reshape(seq, d)
    for pos in range(seq):
        for i in range(d // 2):
            ang = pos * 10_000.0 ** (-2.0 * i / d)
            assert abs(table[pos, 2 * i] - math.cos(ang)) < 1e-5
            assert abs(table[pos, 2 * i + 1] - math.sin(ang)) < 1e-5
    quarter = np.zeros((1, 2), np.float32)
    quarter[0] = [0.0, 1.0]  # cos = 0, sin = 1
    out = O.rope_apply_fp16_ref(np.array([1.0, 0.0], np.float16), quarter, 1, 1, 1, 2)
    assert out.tolist() == [0.0, 1.0]
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, seq, 3, d)).astype(np.float16)
    fwd = O.rope_apply_fp16_ref(x, table, 2, seq, 3, d)
    inv = table.copy()
    inv[:, 1::2] *= -1
    back = O.rope_apply_fp16_ref(fwd, inv, 2, seq, 3, d).astype(np.float32)
    assert np.abs(back.ravel() - x.ravel().astype(np.float32)).max() < 4e-3
