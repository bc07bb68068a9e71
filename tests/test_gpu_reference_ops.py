"""GPU parity of the launchers the reference already has (rms_norm, softmax, rope, matmul in
fp16), through the C ABI, against the CPU references the oracle restates.

The first test of each operator uses the shape of the reference's own GPU parity test
(crates/kernels/tests/op_parity.rs, matmul_parity.rs) and its metric and tolerance: max
relative error 5e-3 with the denominator floor 1e-3 (matmul_parity.rs:83-99).  The naive
matmul reproduces the CPU reference's summation order and is compared bit for bit.
"""
import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu

TOL = 5e-3


def _parity(gpu, cpu, tol=TOL):
    """`parity_check` (crates/kernels/tests/matmul_parity.rs:83-99)."""
    max_abs, max_rel = O.parity_metric(np.asarray(gpu, np.float32), np.asarray(cpu, np.float32))
    assert np.isfinite(np.asarray(gpu, np.float32)).all()
    assert max_rel <= tol, f"max_rel {max_rel:.3e} (max_abs {max_abs:.3e}) exceeds {tol}"


def _f16(rng, *shape):
    # `random_f16` of the reference's tests draws uniform values in [-1, 1)
    return (rng.random(shape, np.float32) * 2 - 1).astype(np.float16)


def _dev(a):
    from logismos_amd import hip
    return hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("m,n,eps", [(8, 1024, 1e-5), (1, 1, 1e-6), (3, 7, 1e-5), (5, 4096, 1e-6),
                                     (2, 10000, 1e-5)])
def test_rms_norm_parity(m, n, eps):
    """first case: crates/kernels/tests/op_parity.rs:72-110"""
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(42 + n)
    x, w = _f16(rng, m, n), _f16(rng, n)
    d_y = hip.DeviceBuffer(m * n * 2)
    d_y.fill(0xFF)
    kernels.launch_rms_norm_fp16(_dev(x), _dev(w), d_y, m, n, eps)
    hip.synchronize()
    _parity(d_y.to_numpy(np.float16, (m * n,)), O.rms_norm_fp16_ref(x, w, m, n, eps))


@pytest.mark.parametrize("m,n", [(4, 512), (1, 1), (3, 5), (2, 300), (6, 5000)])
def test_softmax_parity(m, n):
    """first case: crates/kernels/tests/op_parity.rs:113-145"""
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(7 + n)
    x = _f16(rng, m, n)
    d_y = hip.DeviceBuffer(m * n * 2)
    d_y.fill(0xFF)
    kernels.launch_softmax_fp16(_dev(x), d_y, m, n)
    hip.synchronize()
    got = d_y.to_numpy(np.float16, (m, n))
    _parity(got.ravel(), O.softmax_fp16_ref(x, m, n))
    assert np.allclose(got.astype(np.float32).sum(axis=1), 1.0, atol=2e-3 * max(1, n ** 0.5))


def test_softmax_rows_of_minus_infinity_become_uniform():
    """crates/kernels/src/softmax/cpu.rs:118-137 (all -inf -> 0.25 each), next to a mixed row"""
    from logismos_amd import hip, kernels
    x = np.array([[-np.inf] * 4, [0.0, -np.inf, 0.0, -np.inf]], np.float16)
    d_y = hip.DeviceBuffer(x.size * 2)
    kernels.launch_softmax_fp16(_dev(x), d_y, 2, 4)
    hip.synchronize()
    got = d_y.to_numpy(np.float16, (2, 4)).astype(np.float32)
    assert got[0].tolist() == [0.25] * 4
    assert got[1].tolist() == [0.5, 0.0, 0.5, 0.0]
    assert np.array_equal(got.astype(np.float16).view(np.uint16).ravel(),
                          O.softmax_fp16_ref(x, 2, 4).view(np.uint16))


@pytest.mark.parametrize("batch,seq,heads,d", [(2, 64, 8, 128), (1, 1, 1, 2), (3, 5, 2, 6),
                                               (1, 300, 4, 64)])
def test_rope_parity(batch, seq, heads, d):
    """first case: crates/kernels/tests/op_parity.rs:148-190 (theta 10000)"""
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(13 + seq)
    qk = _f16(rng, batch, seq, heads, d)
    table = O.build_cos_sin_table(seq, d, 10_000.0)
    d_qk = _dev(qk)
    kernels.launch_rope_fp16_in_place(d_qk, _dev(table), batch, seq, heads, d)
    hip.synchronize()
    _parity(d_qk.to_numpy(np.float16, (qk.size,)),
            O.rope_apply_fp16_ref(qk, table, batch, seq, heads, d))


def test_rope_position_zero_is_the_identity():
    """crates/kernels/src/rope/cpu.rs:133-158, on the GPU"""
    from logismos_amd import hip, kernels
    orig = np.array([1.0, 2.0, 3.0, 4.0], np.float16)
    d_qk = _dev(orig)
    kernels.launch_rope_fp16_in_place(d_qk, _dev(O.build_cos_sin_table(1, 4, 10_000.0)), 1, 1, 1, 4)
    hip.synchronize()
    assert np.array_equal(d_qk.to_numpy(np.uint16, (4,)), orig.view(np.uint16))


def _matmul(variant, m, n, k, seed):
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(seed)
    a, b = _f16(rng, m, k), _f16(rng, k, n)
    d_d = hip.DeviceBuffer(m * n * 2)
    d_d.fill(0xFF)
    kernels.launch_matmul_fp16(variant, _dev(a), _dev(b), d_d, m, n, k)
    hip.synchronize()
    return d_d.to_numpy(np.float16, (m * n,)), O.matmul_fp16_ref(a, b, m, n, k)


@pytest.mark.parametrize("m,n,k", [(32, 48, 64), (1, 1, 1), (5, 3, 7), (70, 130, 257)])
def test_matmul_naive_is_bit_identical_to_the_cpu_reference(m, n, k):
    """first case: crates/kernels/tests/matmul_parity.rs:101-113"""
    got, want = _matmul("naive", m, n, k, 1)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (256, 256, 256), (1, 1, 1), (5, 3, 7),
                                   (70, 130, 257), (33, 64, 40), (128, 65, 96), (200, 72, 1000)])
def test_matmul_matrix_core_parity(m, n, k):
    """first two cases: crates/kernels/tests/matmul_parity.rs:115-142 (the reference's WMMA
    variant wants multiples of 16; this one takes any shape)"""
    got, want = _matmul("wmma", m, n, k, 3)
    _parity(got, want)


def test_matmul_identity_returns_the_other_operand():
    """crates/kernels/src/matmul/cpu.rs:70-89, on both GPU variants"""
    n = 48
    rng = np.random.default_rng(5)
    from logismos_amd import hip, kernels
    b = _f16(rng, n, n)
    eye = np.eye(n, dtype=np.float16)
    for variant in ("naive", "wmma"):
        d_d = hip.DeviceBuffer(n * n * 2)
        kernels.launch_matmul_fp16(variant, _dev(eye), _dev(b), d_d, n, n, n)
        hip.synchronize()
        assert np.array_equal(d_d.to_numpy(np.uint16, (n, n)), b.view(np.uint16))


def test_shape_guards_reject_before_any_launch():
    """crates/kernels/src/matmul/mod.rs:213-247, crates/kernels/src/rope/mod.rs:215-269"""
    from logismos_amd import hip, kernels
    buf = hip.DeviceBuffer(64)
    big = 2 ** 31 - 1
    for m, n, k in [(0, 1, 1), (1, -1, 1), (1, 1, 0), (65536, 1, 65536), (1, 65536, 65536),
                    (65536, 65536, 1)]:
        for variant in ("naive", "wmma"):
            with pytest.raises(kernels.LaunchError) as e:
                kernels.launch_matmul_fp16(variant, buf, buf, buf, m, n, k)
            assert e.value.code == 1
    for shape in [(0, 1, 1, 2), (1, 1, 1, 0), (1, 1, 1, 3), (65536, 65536, 1, 2),
                  (big, big, 2, 2)]:
        with pytest.raises(kernels.LaunchError) as e:
            kernels.launch_rope_fp16_in_place(buf, buf, *shape)
        assert e.value.code == 1


@pytest.mark.parametrize("rows,n,mask_rows", [(12, 37, 3), (8, 128, 8), (6, 5, 1), (64, 1000, 2)])
@pytest.mark.parametrize("fp16", [False, True])
def test_mask_additive_matches_the_reference_function(rows, n, mask_rows, fp16):
    """`cpu_f32::mask_additive_in_place` (crates/kernels/src/cpu_f32/mod.rs:451-486): one mask
    row serves rows / mask_rows CONSECUTIVE score rows; bit for bit (the op only writes -inf)"""
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(rows * 1000 + n)
    scores = rng.standard_normal((rows, n)).astype(np.float32)
    mask = (rng.random((mask_rows, n)) < 0.6).astype(np.uint8)
    mask[0, :] = 0  # a mask row that hides every key
    want = scores.copy()
    O.mask_additive_in_place(want, mask, rows, n)
    dt = np.float16 if fp16 else np.float32
    d_s = _dev(scores.astype(dt))
    kernels.launch_mask_additive(d_s, _dev(mask), mask.size, rows, n, fp16=fp16)
    hip.synchronize()
    got = d_s.to_numpy(dt, (rows, n))
    want = want.astype(dt)  # (fp16: rounding the unmasked scores commutes with masking)
    assert np.array_equal(got.view(np.uint16 if fp16 else np.uint32),
                          want.view(np.uint16 if fp16 else np.uint32))
    repeat = rows // mask_rows
    assert np.isneginf(got[:repeat]).all()
    if mask_rows > 1:
        assert not np.isneginf(got[repeat:]).all()


def test_mask_additive_edge_cases_of_the_reference():
    """nothing to do without columns, rows or a mask (`:452-454, 459-461`); a row count the mask
    rows do not divide is refused where the reference panics (`:462-465`)"""
    from logismos_amd import hip, kernels
    scores = np.arange(12, dtype=np.float32).reshape(3, 4)
    d_s = _dev(scores)
    mask = np.zeros(8, np.uint8)
    for mask_len, rows, n in ((8, 3, 0), (8, 0, 4), (0, 3, 4), (3, 3, 4)):
        kernels.launch_mask_additive(d_s, _dev(mask), mask_len, rows, n)
    hip.synchronize()
    assert np.array_equal(d_s.to_numpy(np.float32, (3, 4)), scores)
    with pytest.raises(kernels.LaunchError):
        kernels.launch_mask_additive(d_s, _dev(mask), 8, 3, 4)   # 3 rows, 2 mask rows
    with pytest.raises(kernels.LaunchError):
        kernels.launch_mask_additive(d_s, _dev(mask), 7, 4, 4)   # not whole mask rows
    hip.synchronize()
    assert np.array_equal(d_s.to_numpy(np.float32, (3, 4)), scores)


def test_masked_scores_through_the_softmax_launcher():
    """the unfused attention of a padded batch: fp16 scores, key-padding mask, softmax; a query
    whose keys are all padding attends uniformly (crates/kernels/src/cpu_f32/mod.rs:395-416)"""
    from logismos_amd import hip, kernels
    rng = np.random.default_rng(99)
    heads, seq, n = 4, 3, 8
    scores = rng.standard_normal((2 * heads * seq, n)).astype(np.float16)
    mask = np.ones((2, n), np.uint8)
    mask[0, 5:] = 0     # batch row 0: keys 5.. are padding
    mask[1, :] = 0      # batch row 1: nothing but padding
    d_s = _dev(scores)
    kernels.launch_mask_additive(d_s, _dev(mask), mask.size, scores.shape[0], n, fp16=True)
    d_p = hip.DeviceBuffer(scores.size * 2)
    kernels.launch_softmax_fp16(d_s, d_p, scores.shape[0], n)
    hip.synchronize()
    p = d_p.to_numpy(np.float16, scores.shape).astype(np.float32)
    half = heads * seq
    assert (p[:half, 5:] == 0).all() and np.allclose(p[:half, :5].sum(axis=1), 1.0, atol=2e-3)
    assert (p[half:] == 0.125).all()
    masked = scores.astype(np.float32)
    O.mask_additive_in_place(masked, mask, scores.shape[0], n)
    assert np.array_equal(p.astype(np.float16).view(np.uint16),
                          O.softmax_fp16_ref(masked.astype(np.float16), scores.shape[0], n)
                          .view(np.uint16).reshape(p.shape))
