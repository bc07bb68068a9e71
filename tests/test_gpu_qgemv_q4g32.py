"""GPU parity: ggml Q4_0 / Q4_1 repack (bit-exact) and the Q4G32 GEMV (fp32 tolerance) vs the
CPU oracle, through the C ABI."""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip, kernels
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu


def _dev(a):
    return hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _repack_gpu(blocks, n, k, has_min):
    qw = hip.DeviceBuffer(n * k // 2)
    sc = hip.DeviceBuffer(n * (k // 32) * 2)
    mn = hip.DeviceBuffer(n * (k // 32) * 2)
    for b in (qw, sc, mn):
        b.fill(0xEE)
    kernels.launch_repack_q4_blocks(_dev(blocks), qw, sc, mn, n, k, has_min)
    hip.synchronize()
    return qw, sc, mn


@pytest.mark.parametrize("has_min", [False, True])
@pytest.mark.parametrize("n,k", [(1, 32), (3, 96), (130, 2048), (1536, 8960)])
def test_repack_is_bit_exact(n, k, has_min):
    rng = np.random.default_rng(n * 31 + k + has_min)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    blocks = O.quantize_q4_blocks(w, n, k, has_min)
    qw, sc, mn = _repack_gpu(blocks, n, k, has_min)
    want_qw, want_sc, want_mn = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
    assert np.array_equal(qw.to_numpy(np.uint8, (n, k // 2)), want_qw)
    assert np.array_equal(sc.to_numpy(np.uint16, (n, k // 32)), want_sc.view(np.uint16))
    assert np.array_equal(mn.to_numpy(np.uint16, (n, k // 32)), want_mn.view(np.uint16))


def test_repack_of_arbitrary_block_bytes_is_bit_exact():
    # every nibble pattern and odd fp16 fields, not only what the quantiser emits
    rng = np.random.default_rng(3)
    n, k = 64, 512
    for has_min in (False, True):
        bs = 20 if has_min else 18
        blocks = rng.integers(0, 256, size=n * (k // 32) * bs, dtype=np.uint8)
        blocks.reshape(-1, bs)[:, 1] &= 0x7B   # finite d (the Q4_0 min is computed from it)
        qw, sc, mn = _repack_gpu(blocks, n, k, has_min)
        want_qw, want_sc, want_mn = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
        assert np.array_equal(qw.to_numpy(np.uint8, (n, k // 2)), want_qw)
        assert np.array_equal(sc.to_numpy(np.uint16, (n, k // 32)), want_sc.view(np.uint16))
        assert np.array_equal(mn.to_numpy(np.uint16, (n, k // 32)), want_mn.view(np.uint16))


def _gemv(x, qw, sc, mn, n, k):
    y = hip.DeviceBuffer(n * 4)
    y.fill(0xFF)
    kernels.launch_qgemv_q4g32_f32(_dev(np.asarray(x, np.float32)), qw, sc, mn, y, n, k)
    hip.synchronize()
    return y.to_numpy(np.float32, (n,))


@pytest.mark.parametrize("has_min", [False, True])
@pytest.mark.parametrize("n,k", [(1, 32), (3, 64), (5, 1024), (7, 1056), (257, 8960),
                                 (12288, 4096)])
def test_block_stream_to_gemv_matches_oracle(n, k, has_min):
    # the whole row f3 describes: ggml blocks -> device repack -> dequant-fused GEMV
    rng = np.random.default_rng(n * 7919 + k + has_min)
    x = rng.standard_normal(k, np.float32)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    blocks = O.quantize_q4_blocks(w, n, k, has_min)
    qw, sc, mn = _repack_gpu(blocks, n, k, has_min)
    got = _gemv(x, qw, sc, mn, n, k)
    pq, ps, pm = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
    want = O.qgemv_q4g32_f32(x, pq, ps, pm, n, k)
    # fp32 in, fp32 accumulate, fp32 out: only the summation order differs
    assert_parity(got, want, max_abs=5e-5, max_rel=2e-4, what=f"qgemv_q4g32 {n}x{k}")
    # and against ggml's own decode of the blocks (Q4_0: (q - 8) d)
    ref = O.dequantize_q4_blocks(blocks, n, k, has_min).astype(np.float64) @ x.astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())


def test_orientation_with_a_one_hot_x():
    rng = np.random.default_rng(5)
    n, k = 64, 256
    w = rng.standard_normal((n, k), np.float32)
    blocks = O.quantize_q4_blocks(w, n, k, True)
    qw, sc, mn = _repack_gpu(blocks, n, k, True)
    x = np.zeros(k, np.float32)
    x[37] = 1.0
    got = _gemv(x, qw, sc, mn, n, k)
    pq, ps, pm = O.q4_blocks_to_q4g32(blocks, n, k, True)
    d = ps.astype(np.float32)[:, 37 // 32]
    m = pm.astype(np.float32)[:, 37 // 32]
    q = ((pq[:, 37 // 2] >> 4) & 0x0F).astype(np.float32)      # 37 is odd: high nibble
    # one product and the min term per row: fma(x_sum = 1, m, q * d) in fp32
    assert_parity(got, q * d + m, max_abs=1e-7, max_rel=1e-6, what="one-hot column")


def test_linearity_at_full_size():
    # size-independent property at the config-3 matrix size
    rng = np.random.default_rng(9)
    n, k = 12288, 4096
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    blocks = O.quantize_q4_blocks(w, n, k, False)
    qw, sc, mn = _repack_gpu(blocks, n, k, False)
    x1 = rng.standard_normal(k, np.float32)
    x2 = rng.standard_normal(k, np.float32)
    y1, y2 = _gemv(x1, qw, sc, mn, n, k), _gemv(x2, qw, sc, mn, n, k)
    y3 = _gemv(np.float32(0.5) * x1 + x2, qw, sc, mn, n, k)
    assert_parity(y3, np.float32(0.5) * y1 + y2, max_abs=2e-5, max_rel=2e-4, what="linearity")


def test_shape_guards():
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_qgemv_q4g32_shape(4, 48)
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_qgemv_q4g32_shape(0, 64)
