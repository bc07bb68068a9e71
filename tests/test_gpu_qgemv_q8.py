"""GPU parity: Q8G32 dequant-fused GEMV vs the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip
from tests import workloads
from tests.gpu_harness import QgemvQ8Runner, assert_parity

pytestmark = pytest.mark.gpu


def _run(x, w, n, k):
    qs, d = O.quantize_q8g32(w, n, k)
    r = QgemvQ8Runner(x, qs, d, n, k)
    r.launch()
    return r.result(), O.qgemv_q8g32_f32(x, qs, d, n, k), qs, d


def test_config1_up_proj_matches_oracle():
    c = workloads.config1()
    got, want, _, _ = _run(c["x"], c["w"], c["n"], c["k"])
    # fp32 in, fp32 accumulate, fp32 out: only the summation order differs
    assert_parity(got, want, max_abs=2e-5, max_rel=1e-4, what="qgemv_q8 config 1")


@pytest.mark.parametrize("n,k", [(1, 32), (3, 64), (5, 1024), (7, 1056), (130, 2048), (257, 8960),
                                 (4096, 4096),
                                 # several rows per wave with a ragged last wave: 8, 4 and 2 rows
                                 (8195, 512), (4099, 1024), (2051, 1536), (1500, 8192)])
def test_ragged_shapes(n, k):
    rng = np.random.default_rng(n * 7919 + k)
    x = rng.standard_normal(k, np.float32)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    got, want, _, _ = _run(x, w, n, k)
    assert_parity(got, want, max_abs=5e-5, max_rel=2e-4, what=f"qgemv_q8 {n}x{k}")


def test_orientation_and_scale_with_a_one_hot_x():
    rng = np.random.default_rng(5)
    n, k = 64, 256
    w = rng.standard_normal((n, k), np.float32)
    qs, d = O.quantize_q8g32(w, n, k)
    x = np.zeros(k, np.float32)
    x[37] = 1.0
    r = QgemvQ8Runner(x, qs, d, n, k)
    r.launch()
    want = O.dequantize_q8g32(qs, d, n, k)[:, 37]
    assert np.array_equal(r.result(), want)  # a single product per row: exact


def test_linearity_at_full_size():
    # size-independent property at config-1 size: y(a*x1 + x2) = a*y(x1) + y(x2)
    c = workloads.config1()
    rng = np.random.default_rng(9)
    n, k = c["n"], c["k"]
    qs, d = O.quantize_q8g32(c["w"], n, k)
    x2 = rng.standard_normal(k, np.float32)
    ys = []
    for x in (c["x"], x2, np.float32(0.5) * c["x"] + x2):
        r = QgemvQ8Runner(x, qs, d, n, k)
        r.launch()
        ys.append(r.result())
    assert np.abs(ys[2] - (0.5 * ys[0] + ys[1])).max() < 1e-5


def test_repack_from_ggml_q8_0_blocks_is_bit_exact():
    rng = np.random.default_rng(6)
    n, k = 33, 1536
    qs, d = O.quantize_q8g32(rng.standard_normal((n, k), np.float32), n, k)
    blocks = O.q8g32_to_q8_0_blocks(qs, d, n, k)
    from logismos_amd import kernels
    b = hip.DeviceBuffer.from_numpy(blocks)
    qs_d = hip.DeviceBuffer(n * k)
    d_d = hip.DeviceBuffer(n * (k // 32) * 2)
    kernels.launch_repack_q8_0(b, qs_d, d_d, n, k)
    hip.synchronize()
    assert np.array_equal(qs_d.to_numpy(np.int8, (n, k)), qs)
    assert np.array_equal(d_d.to_numpy(np.uint16, (n, k // 32)), d.view(np.uint16))
