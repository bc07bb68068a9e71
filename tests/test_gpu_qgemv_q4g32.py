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
                                 (12288, 4096),
                                 # several rows per wave with a ragged last wave: 8, 4 and 2 rows
                                 (8203, 1024), (4099, 1024), (2051, 2048), (700, 16384)])
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


# ---------------------------------------------------------------- batched (matrix-core) product
def _gemm(xbits, qw, sc, mn, b, n, k):
    y = hip.DeviceBuffer(b * n * 2)
    y.fill(0xFF)
    kernels.launch_qgemm_q4g32_bf16(_dev(xbits), qw, sc, mn, y, b, n, k)
    hip.synchronize()
    return y.to_numpy(np.uint16, (b, n))


def _batched_case(b, n, k, has_min, seed, wscale=0.02):
    rng = np.random.default_rng(seed)
    xbits = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    w = rng.standard_normal((n, k), np.float32) * np.float32(wscale)
    blocks = O.quantize_q4_blocks(w, n, k, has_min)
    return xbits, blocks


@pytest.mark.parametrize("has_min", [False, True])
@pytest.mark.parametrize("b,n,k", [
    (1, 1, 128), (2, 17, 256), (3, 16, 896),      # fewer 128-column chunks than waves
    (5, 33, 1024), (16, 130, 2176),               # 17 chunks: an odd share per wave
    (17, 47, 1152), (32, 257, 4096),              # two batch tiles
    (9, 4096 + 48, 1024),                         # two row tiles per workgroup + a ragged last
    (32, 12288, 4096), (16, 12288 + 16, 2048),    # three row tiles per workgroup
    (8, 1040, 12288),                             # 96 chunks: twelve per wave
])
def test_batched_product_matches_oracle(b, n, k, has_min):
    xbits, blocks = _batched_case(b, n, k, has_min, b * 104729 + n * 31 + k + has_min)
    qw, sc, mn = _repack_gpu(blocks, n, k, has_min)
    got = _gemm(xbits, qw, sc, mn, b, n, k)
    pq, ps, pm = O.q4_blocks_to_q4g32(blocks, n, k, has_min)
    want32 = O.qgemm_q4g32_f32(xbits, pq, ps, pm, b, n, k)
    # bf16 output of an fp32 accumulation: the tolerance of the decode path
    assert_parity(O.bf16_bits_to_f32(got), want32, max_abs=2e-3, max_rel=1e-2,
                  what=f"qgemm_q4g32 b={b} {n}x{k}")
    # and nearly always the very same bf16 value as the oracle's rounding of its own sum
    want = O.qgemm_q4g32_bf16(xbits, pq, ps, pm, b, n, k)
    assert (got == want).mean() > 0.97


def test_batched_rows_do_not_depend_on_the_batch():
    # row i of a batch of 32 equals the same x sent alone, bit for bit: the matrix-core
    # product never mixes batch rows and the summation order does not depend on b
    b, n, k = 32, 1000, 2048
    xbits, blocks = _batched_case(b, n, k, True, 77)
    qw, sc, mn = _repack_gpu(blocks, n, k, True)
    full = _gemm(xbits, qw, sc, mn, b, n, k)
    for i in (0, 15, 16, 31):
        one = _gemm(xbits[i:i + 1], qw, sc, mn, 1, n, k)
        assert np.array_equal(one[0], full[i])
    part = _gemm(xbits[:7], qw, sc, mn, 7, n, k)
    assert np.array_equal(part, full[:7])


def test_batched_product_agrees_with_the_gemv():
    # the same weights through the fp32 GEMV: x is bf16-exact, so only the output rounding
    # and the summation order differ
    b, n, k = 4, 512, 1024
    xbits, blocks = _batched_case(b, n, k, False, 78)
    qw, sc, mn = _repack_gpu(blocks, n, k, False)
    got = O.bf16_bits_to_f32(_gemm(xbits, qw, sc, mn, b, n, k))
    x = O.bf16_bits_to_f32(xbits)
    for i in range(b):
        y = _gemv(x[i], qw, sc, mn, n, k)
        assert_parity(got[i], y, max_abs=2e-3, max_rel=1e-2, what="gemm row vs gemv")


def test_batched_one_hot_reads_back_columns_of_every_group_position():
    # one-hot x in batch row r selects column c_r: pins the lane / dword transpose of the
    # weight tile (a wrong dword would return another column's value)
    n, k = 48, 512
    rng = np.random.default_rng(79)
    w = rng.standard_normal((n, k), np.float32)
    blocks = O.quantize_q4_blocks(w, n, k, True)
    qw, sc, mn = _repack_gpu(blocks, n, k, True)
    pq, ps, pm = O.q4_blocks_to_q4g32(blocks, n, k, True)
    deq = O.dequantize_q4g32(pq, ps, pm, n, k)
    cols = np.array([(37 * r + 5) % k for r in range(32)])
    assert len(set(cols % 32)) == 32                       # every position inside a group
    x = np.zeros((32, k), np.float32)
    x[np.arange(32), cols] = 1.0
    got = O.bf16_bits_to_f32(_gemm(O.f32_to_bf16_bits(x), qw, sc, mn, 32, n, k))
    want = O.bf16_bits_to_f32(O.f32_to_bf16_bits(deq[:, cols].T.copy()))
    assert np.array_equal(got, want)


def test_batched_shape_guards():
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_qgemm_q4g32_shape(4, 64, 96)          # K not a multiple of 128
    kernels.check_qgemm_q4g32_shape(33, 64, 128)            # any m: 32 rows per pass
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_qgemm_q4g32_shape(0, 64, 128)
    with pytest.raises(kernels.UnsupportedShape):
        kernels.check_qgemm_q4g32_shape(2, 65536, 65536)
