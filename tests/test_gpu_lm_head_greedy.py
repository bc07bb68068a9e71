"""GPU parity: vocabulary projection fused with greedy token selection, and the embedding
lookup, through the C ABI.

Logits (fp32, fp32 accumulation over bf16 x and 4-bit weights) are compared with the CPU
oracle's Q4G128 GEMM within 2e-4 max-abs or 1e-3 relative.  Token selection is integer work
and is checked exactly: the tokens must be `decode::greedy` (first maximum wins) of the very
logits the kernel stored, and must agree with the oracle's choice wherever the oracle's top
two logits are further apart than the logit tolerance.  The embedding lookup is a copy and
is compared bit for bit.
"""
import numpy as np
import pytest

import oracle as O
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu


def _first_argmax(rows):
    return np.array([O.greedy(r) for r in rows], np.uint32)


def _run(xb, qw, s, z, b, n, k, want_logits=True):
    from logismos_amd import hip, kernels
    d_x = hip.DeviceBuffer.from_numpy(xb)
    d_xp = hip.DeviceBuffer(kernels.q4_xprep_bytes(b, k))
    d_xp.fill(0xFF)  # padding rows are NaN: they must not reach a token or a stored logit
    kernels.launch_q4_prepare_x_bf16(d_x, d_xp, b, k)
    d_ws = hip.DeviceBuffer(kernels.qgemm_q4g128_greedy_workspace_bytes(b, n, k))
    d_ws.fill(0xFF)
    d_tok = hip.DeviceBuffer(b * 4)
    d_tok.fill(0xFF)
    d_logits = None
    if want_logits:
        d_logits = hip.DeviceBuffer(b * n * 4)
        d_logits.fill(0xFF)
    kernels.launch_qgemm_q4g128_greedy_xprep(
        d_xp, hip.DeviceBuffer.from_numpy(np.ascontiguousarray(qw)),
        hip.DeviceBuffer.from_numpy(np.ascontiguousarray(s).view(np.uint16)),
        hip.DeviceBuffer.from_numpy(np.ascontiguousarray(z).view(np.uint16)),
        d_tok, d_logits, d_ws, b, n, k)
    hip.synchronize()
    tokens = d_tok.to_numpy(np.uint32, (b,))
    logits = d_logits.to_numpy(np.float32, (b, n)) if want_logits else None
    return tokens, logits


def _case(b, n, k, seed):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    return O.f32_to_bf16_bits(x), qw, s, z


@pytest.mark.parametrize("b,n,k", [(32, 5000, 1024), (7, 1000, 1024), (16, 4099, 4096),
                                   (17, 50, 1024), (1, 16, 2048), (32, 20000, 2048),
                                   (3, 33000, 1024), (32, 170000, 1024)])
def test_logits_and_tokens_match_oracle(b, n, k):
    xb, qw, s, z = _case(b, n, k, b * 7919 + n * 13 + k)
    tokens, logits = _run(xb, qw, s, z, b, n, k)
    want = O.qgemm_q4g128_f32(xb, qw, s, z, b, n, k)
    max_abs, _ = assert_parity(logits, want, max_abs=2e-4, max_rel=1e-3,
                               what=f"lm_head logits {b}x{n}x{k}")
    # the selection rule, exactly, on the kernel's own logits
    assert np.array_equal(tokens, _first_argmax(logits))
    # and the oracle's tokens wherever its winner is clear of the tolerance
    want_tokens = _first_argmax(want)
    top2 = np.sort(want, axis=1)[:, -2:] if n > 1 else None
    for r in range(b):
        if top2 is None or top2[r, 1] - top2[r, 0] > 4 * max(max_abs, 1e-6):
            assert tokens[r] == want_tokens[r], (r, tokens[r], want_tokens[r])


def test_tokens_without_logits_are_the_same():
    b, n, k = 32, 9000, 1024
    xb, qw, s, z = _case(b, n, k, 5)
    with_logits, _ = _run(xb, qw, s, z, b, n, k)
    without, none = _run(xb, qw, s, z, b, n, k, want_logits=False)
    assert none is None
    assert np.array_equal(with_logits, without)


def test_first_of_equal_maxima_wins_across_tiles_and_workgroups():
    # the winning weight row of batch row 0 is copied to a lower and to a much higher index:
    # identical rows give bit-identical logits wherever they sit, and the lowest index wins
    b, n, k = 32, 60000, 1024
    xb, qw, s, z = _case(b, n, k, 11)
    qw, s, z = qw.copy(), s.copy(), z.copy()
    ref = O.qgemm_q4g128_f32(xb, qw, s, z, b, n, k)
    a = int(np.argmax(ref[0]))
    lo, hi = 3, n - 2
    if a <= lo:
        a = int(np.argsort(ref[0])[-2])
    for dst in (lo, hi):
        qw[dst], s[dst], z[dst] = qw[a], s[a], z[a]
    tokens, logits = _run(xb, qw, s, z, b, n, k)
    assert logits[0, lo].tobytes() == logits[0, a].tobytes() == logits[0, hi].tobytes()
    assert tokens[0] == lo
    assert np.array_equal(tokens, _first_argmax(logits))


def test_row_without_a_value_above_minus_infinity_gives_token_zero():
    # NaN activations make every logit of that row NaN: `v > best` never holds, index 0
    b, n, k = 4, 3000, 1024
    xb, qw, s, z = _case(b, n, k, 3)
    xb = xb.copy().reshape(b, k)
    xb[2, :] = 0x7FC0  # bf16 quiet NaN
    tokens, logits = _run(xb, qw, s, z, b, n, k)
    assert np.isnan(logits[2]).all()
    assert tokens[2] == 0
    keep = [0, 1, 3]
    assert np.array_equal(tokens[keep], _first_argmax(logits[keep]))


def test_shape_guards():
    from logismos_amd import kernels
    for bad in [(0, 100, 1024), (33, 100, 1024), (4, 0, 1024), (4, 100, 1152), (4, 100, 0),
                (4, 3_000_000, 1024)]:
        with pytest.raises(kernels.UnsupportedShape):
            kernels.check_qgemm_q4g128_greedy_shape(*bad)
        assert kernels.qgemm_q4g128_greedy_workspace_bytes(*bad) == 0
    kernels.check_qgemm_q4g128_greedy_shape(32, 151936, 4096)
    assert kernels.qgemm_q4g128_greedy_workspace_bytes(32, 151936, 4096) > 0


@pytest.mark.parametrize("bf16", [False, True])
def test_embed_lookup_matches_oracle(bf16):
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(21)
    vocab, hidden = 1000, 4096
    table = rng.standard_normal((vocab, hidden), np.float32)
    ids = np.array([0, 999, 5, 5, 1000, 0xFFFFFFFF, 17, 123456], np.uint32)
    if bf16:
        bits = O.f32_to_bf16_bits(table)
        table = O.bf16_bits_to_f32(bits).reshape(vocab, hidden)
        d_table = hip.DeviceBuffer.from_numpy(bits)
    else:
        d_table = hip.DeviceBuffer.from_numpy(table)
    d_out = hip.DeviceBuffer(ids.size * hidden * 4)
    d_out.fill(0xFF)
    kernels.launch_embed_lookup(d_table, hip.DeviceBuffer.from_numpy(ids), d_out, ids.size, hidden,
                                vocab, bf16)
    hip.synchronize()
    got = d_out.to_numpy(np.float32, (ids.size, hidden))
    want = O.embed_lookup(table, hidden, vocab, ids).reshape(ids.size, hidden)
    assert got.tobytes() == want.tobytes()
    assert not got[4].any() and not got[5].any() and not got[7].any()
