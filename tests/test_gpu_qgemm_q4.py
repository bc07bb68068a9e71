"""GPU parity: Q4G128 dequant-fused GEMV/GEMM vs the CPU oracle, through the C ABI.

Tolerance (bf16 outputs, fp32 accumulation): 2e-3 max-abs or 1e-2 relative.
"""
import numpy as np
import pytest

import oracle as O
from tests import workloads
from tests.gpu_harness import QgemmQ4Runner, assert_parity

pytestmark = pytest.mark.gpu

_cache = {}


def _config3():
    if "c3" not in _cache:
        c = workloads.config3()
        qw, s, z = O.quantize_q4g128(c["w"], c["n"], c["k"])
        _cache["c3"] = (c, qw, s, z)
    return _cache["c3"]


def _run(x_f32, qw, s, z, b, n, k, force_mfma=False):
    xb = O.f32_to_bf16_bits(x_f32[:b])
    r = QgemmQ4Runner(xb, qw, s, z, b, n, k)
    r.launch(force_mfma=force_mfma)
    got = O.bf16_bits_to_f32(r.result_bits())
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb, qw, s, z, b, n, k))
    return got, want


@pytest.mark.parametrize("b", [1, 2, 4, 8, 16])
def test_config3_matches_oracle(b):
    c, qw, s, z = _config3()
    got, want = _run(c["x"], qw, s, z, b, c["n"], c["k"])
    assert_parity(got, want, what=f"qgemm_q4 config 3 batch {b}")


@pytest.mark.parametrize("b", [1, 3, 4])
def test_config3_mfma_path_at_small_batch(b):
    c, qw, s, z = _config3()
    got, want = _run(c["x"], qw, s, z, b, c["n"], c["k"], force_mfma=True)
    assert_parity(got, want, what=f"qgemm_q4 config 3 batch {b} (mfma)")


@pytest.mark.parametrize("b,n,k", [(5, 16, 128), (7, 33, 256), (8, 17, 1152), (16, 1000, 2048),
                                   (9, 4096, 12288), (32, 4100, 4096), (17, 1024, 4096),
                                   (32, 12288, 4096), (32, 4096, 12288), (24, 70000, 256)])
def test_mfma_ragged_shapes(b, n, k):
    rng = np.random.default_rng(b * 1000003 + n * 101 + k)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    got, want = _run(x, qw, s, z, b, n, k)
    assert_parity(got, want, what=f"qgemm_q4 mfma {b}x{n}x{k}")


@pytest.mark.parametrize("b,n,k", [(1, 1, 128), (3, 5, 256), (2, 17, 1152), (4, 1000, 2048),
                                   (1, 4096, 12288), (4, 4100, 4096), (3, 1024, 4096)])
def test_ragged_shapes(b, n, k):
    rng = np.random.default_rng(b * 1000003 + n * 101 + k)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    got, want = _run(x, qw, s, z, b, n, k)
    assert_parity(got, want, what=f"qgemm_q4 {b}x{n}x{k}")


def test_one_hot_x_reads_back_the_dequantised_column():
    # orientation, nibble order and zero-point handling in one exact check
    rng = np.random.default_rng(8)
    n, k = 64, 256
    w = rng.standard_normal((n, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    wd = O.dequantize_q4g128(qw, s, z, n, k)
    for col in (0, 1, 5, 127, 128, 255):
        x = np.zeros((1, k), np.float32)
        x[0, col] = 1.0
        got, _ = _run(x, qw, s, z, 1, n, k)
        want = O.bf16_bits_to_f32(O.f32_to_bf16_bits(wd[:, col]))
        assert np.abs(got[0] - want).max() <= np.abs(want).max() * 2.0**-7, col


def test_batch_rows_are_independent():
    # a batch row's result does not depend on its neighbours or its position
    c, qw, s, z = _config3()
    n, k = c["n"], c["k"]
    got4, _ = _run(c["x"], qw, s, z, 4, n, k)                 # MFMA kernel
    got3, _ = _run(c["x"][[2, 0, 1]], qw, s, z, 3, n, k)      # MFMA kernel, row 2 first
    assert np.array_equal(got4[2], got3[0])
    # batch 2 of a matrix this large takes the same MFMA kernel: its rows are those of batch 4
    got2, _ = _run(c["x"], qw, s, z, 2, n, k)
    assert np.array_equal(got2, got4[:2])
    # the VALU GEMV (batch 1, and batch 2 of smaller matrices): same property
    got1, _ = _run(c["x"][1:2], qw, s, z, 1, n, k)
    ns = 2048                                                  # 2048 x 4096: batch 2 stays on the GEMV
    small2, _ = _run(c["x"], qw[:ns], s[:ns], z[:ns], 2, ns, k)
    small1, _ = _run(c["x"][1:2], qw[:ns], s[:ns], z[:ns], 1, ns, k)
    assert np.array_equal(small2[1], small1[0])
    assert np.array_equal(small1[0], got1[0][:ns])             # and of the matrix height
    # the two kernels agree to bf16 rounding
    assert_parity(got4[1], got1[0], what="mfma vs gemv")


# ------------------------------------------------------------------ split-K form (fp32 parts)
def _run_splitk(x_f32, qw, s, z, b, n, k, prepared=False):
    from logismos_amd import hip, kernels
    xb = O.f32_to_bf16_bits(x_f32[:b])
    j = kernels.qgemm_q4g128_splitk_parts(b, n, k, prepared)
    assert j >= 1
    d_parts = hip.DeviceBuffer(j * b * n * 4)
    d_parts.fill(0xFF)
    d_x = hip.DeviceBuffer.from_numpy(xb)
    if prepared:
        d_xp = hip.DeviceBuffer(kernels.q4_xprep_bytes(b, k))
        d_xp.fill(0xFF)  # padding rows stay NaN: they must not leak into stored results
        kernels.launch_q4_prepare_x_bf16(d_x, d_xp, b, k)
        d_x = d_xp
    kernels.launch_qgemm_q4g128_f32_splitk(
        d_x, hip.DeviceBuffer.from_numpy(np.ascontiguousarray(qw)),
        hip.DeviceBuffer.from_numpy(np.ascontiguousarray(s).view(np.uint16)),
        hip.DeviceBuffer.from_numpy(np.ascontiguousarray(z).view(np.uint16)), d_parts, b, n, k,
        prepared=prepared)
    hip.synchronize()
    parts = d_parts.to_numpy(np.float32, (j, b, n))
    assert np.isfinite(parts).all()
    return parts.sum(axis=0, dtype=np.float32), O.qgemm_q4g128_f32(xb, qw, s, z, b, n, k), j


@pytest.mark.parametrize("b", [1, 8, 16, 32])
def test_splitk_config3_matches_oracle(b):
    c, qw, s, z = _config3()
    x = np.concatenate([c["x"], c["x"][::-1]])  # 32 rows
    got, want, _ = _run_splitk(x, qw, s, z, b, c["n"], c["k"])
    # fp32 result of fp32 accumulation: only the summation order differs
    assert_parity(got, want, max_abs=2e-4, max_rel=1e-3, what=f"qgemm_q4 split-K batch {b}")


@pytest.mark.parametrize("b,n,k", [(32, 6144, 4096), (32, 4096, 4096), (32, 24576, 4096),
                                   (32, 4096, 12288), (5, 16, 128), (17, 33, 384),
                                   (32, 1000, 1152), (31, 4100, 2048), (9, 70000, 256)])
def test_splitk_ragged_shapes(b, n, k):
    rng = np.random.default_rng(b * 1000003 + n * 101 + k)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    got, want, j = _run_splitk(x, qw, s, z, b, n, k)
    assert_parity(got, want, max_abs=2e-4, max_rel=1e-3, what=f"split-K {b}x{n}x{k} (J={j})")


@pytest.mark.parametrize("b,n,k", [(5, 16, 128), (17, 33, 384), (16, 1000, 1152), (2, 12288, 4096),
                                   (32, 1000, 4096),
                                   # streaming kernel, one batch tile (same MFMA shape)
                                   (7, 45003, 1024), (16, 24576, 1024)])
def test_splitk_with_prepared_x_is_bit_identical(b, n, k):
    # shapes that stay on the split-K / streaming kernels (K not a multiple of 2048, fewer
    # than 3 batch rows or fewer than 1024 weight rows): the same arithmetic in the same order
    rng = np.random.default_rng(b * 1000003 + n * 101 + k + 1)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    plain, want, _ = _run_splitk(x, qw, s, z, b, n, k)
    prep, _, _ = _run_splitk(x, qw, s, z, b, n, k, prepared=True)
    assert np.array_equal(plain, prep)
    assert_parity(prep, want, max_abs=2e-4, max_rel=1e-3, what="split-K, prepared x")


@pytest.mark.parametrize("b,n,k", [(17, 45003, 1024), (32, 24576, 1024), (25, 16384, 3072)])
def test_streaming_kernel_with_two_batch_tiles(b, n, k):
    # batch 17..32 on large shapes whose K is a multiple of 1024 only: against the oracle and
    # the plain-x path, whole and ragged row tiles
    rng = np.random.default_rng(b * 1000003 + n * 101 + k + 2)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    plain, want, _ = _run_splitk(x, qw, s, z, b, n, k)
    prep, _, j = _run_splitk(x, qw, s, z, b, n, k, prepared=True)
    assert j == k // 1024
    assert_parity(prep, want, max_abs=2e-4, max_rel=1e-3, what="streaming kernel vs oracle")
    assert_parity(prep, plain, max_abs=5e-5, max_rel=1e-4, what="streaming vs split-K kernel")


@pytest.mark.parametrize("b,n,k,parts", [
    # the step's four projections at batch 32: 32-row tiles, slices of two groups up to
    # K = 4096 (two parts), of four beyond (three parts)
    (32, 6144, 4096, 2), (32, 4096, 4096, 2), (32, 24576, 4096, 2), (32, 4096, 12288, 3),
    # ragged: last tile short, batch rows short of the tile, one tile per workgroup
    (31, 4100, 2048, 1), (17, 1030, 8192, 2), (25, 12289, 4096, 2), (20, 1024, 6144, 3),
    # up to 16 batch rows: 16-row tiles
    (16, 24576, 4096, 2), (3, 12288, 4096, 2), (9, 2001, 6144, 3), (12, 5000, 12288, 3),
    (16, 70000, 2048, 1)])
def test_register_x_kernels_match_oracle_and_split_k(b, n, k, parts):
    # x in registers, weights through the LDS ring: against the oracle and the plain-x path.
    # The zero-point term is summed apart from the products here (one fp32 MFMA per tile), so
    # the two kernels agree to fp32 rounding, not bit for bit.
    rng = np.random.default_rng(b * 1000003 + n * 101 + k + 3)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    plain, want, _ = _run_splitk(x, qw, s, z, b, n, k)
    prep, _, j = _run_splitk(x, qw, s, z, b, n, k, prepared=True)
    assert j == parts
    assert_parity(prep, want, max_abs=2e-4, max_rel=1e-3, what="register-x kernel vs oracle")
    assert_parity(prep, plain, max_abs=5e-5, max_rel=1e-4, what="register-x vs split-K kernel")


def test_register_x_kernel_rows_do_not_depend_on_the_batch():
    # a batch row's result is the same whatever its neighbours are and wherever it sits,
    # within one kernel (32-row tiles) and across the two (16- and 32-row tiles)
    b, n, k = 32, 4096, 4096
    rng = np.random.default_rng(77)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((b, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    full, _, _ = _run_splitk(x, qw, s, z, 32, n, k, prepared=True)
    part, _, _ = _run_splitk(x[5:25], qw, s, z, 20, n, k, prepared=True)
    assert np.array_equal(full[5:25], part)
    small, _, _ = _run_splitk(x[8:20], qw, s, z, 12, n, k, prepared=True)
    assert_parity(small, full[8:20], max_abs=5e-5, max_rel=1e-4, what="16-row vs 32-row tiles")
