"""GPU parity of what `cpu_f32::linear_t` is beyond a bare decode GEMV
(crates/kernels/src/cpu_f32/mod.rs:271-345): the optional bias (the q/k/v projections of
Qwen2 carry one, crates/transformers/src/attention.rs:49-57) and any number of activation
rows m (`seq` rows of a prefill chunk, crates/transformers/src/mlp.rs:104-111), through the
C ABI, against the CPU oracle.  bf16 / fp32 outputs with fp32 accumulation: 2e-3 absolute or
1e-2 relative (fp32 GEMV outputs: 2e-5 / 1e-4)."""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip, kernels
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu

up = hip.DeviceBuffer.from_numpy


def _q4(rng, n, k):
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    return O.quantize_q4g128(w, n, k)


def _gemm_q4(xb, qw, s, z, b, n, k, bias):
    d_y = hip.DeviceBuffer(b * n * 2)
    d_y.fill(0xFF)
    kernels.launch_qgemm_q4g128_bf16(up(xb), up(qw), up(s.view(np.uint16)), up(z.view(np.uint16)),
                                     d_y, b, n, k, bias=up(bias) if bias is not None else None)
    hip.synchronize()
    return O.bf16_bits_to_f32(d_y.to_numpy(np.uint16, (b, n)))


# every kernel behind the Q4G128 entry point: VALU GEMV (b = 1, 2), x-in-registers kernels
# for 16- and 32-row tiles (K = 4096 / 2048, N >= 1024), the MFMA kernel (other K)
@pytest.mark.parametrize("b,n,k", [(1, 2048, 1536), (2, 300, 1536), (2, 12288, 4096),
                                   (4, 1100, 4096), (16, 4096, 2048), (32, 6144, 4096),
                                   (5, 2048, 1536), (24, 777, 1152)])
def test_q4g128_bias_epilogue(b, n, k):
    rng = np.random.default_rng(1000 * b + n + k)
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    bias = (rng.standard_normal(n) * 2).astype(np.float32)
    got = _gemm_q4(xb, qw, s, z, b, n, k, bias)
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb, qw, s, z, b, n, k, bias))
    assert_parity(got, want, what=f"q4g128 + bias {b}x{n}x{k}")
    # the bias really is in there (outputs without it differ by about |bias|)
    plain = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb, qw, s, z, b, n, k))
    assert np.abs(got - plain).max() > 1.0


def test_q8g32_gemv_bias_qwen2_qkv_shape():
    # Qwen2-1.5B q/k/v projection with its bias: 1536 -> (12 + 2 * 2) * 128
    rng = np.random.default_rng(5)
    n, k = 2048, 1536
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    qs, d = O.quantize_q8g32(w, n, k)
    x = rng.standard_normal(k, np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    d_y = hip.DeviceBuffer(n * 4)
    for shape_n in (n, 37):  # the flat kernel and the short-matrix kernel
        kernels.launch_qgemv_q8g32_f32(up(x), up(qs[:shape_n]), up(d[:shape_n].view(np.uint16)), d_y,
                                       shape_n, k, bias=up(bias[:shape_n]))
        hip.synchronize()
        got = d_y.to_numpy(np.float32, (shape_n,))
        want = O.qgemv_q8g32_f32(x, qs[:shape_n], d[:shape_n], shape_n, k, bias[:shape_n])
        assert_parity(got, want, max_abs=2e-5, max_rel=1e-4, what="q8g32 gemv + bias")


def test_q4g32_gemv_and_gemm_bias():
    rng = np.random.default_rng(6)
    n, k, b = 1500, 1024, 7
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    q32, s32, m32 = O.q4_blocks_to_q4g32(O.quantize_q4_blocks(w, n, k, True), n, k, True)
    bias = rng.standard_normal(n).astype(np.float32)
    x = rng.standard_normal((b, k), np.float32)
    d_q, d_s, d_m = up(q32), up(s32.view(np.uint16)), up(m32.view(np.uint16))
    d_y = hip.DeviceBuffer(n * 4)
    kernels.launch_qgemv_q4g32_f32(up(x[0]), d_q, d_s, d_m, d_y, n, k, bias=up(bias))
    hip.synchronize()
    assert_parity(d_y.to_numpy(np.float32, (n,)), O.qgemv_q4g32_f32(x[0], q32, s32, m32, n, k, bias),
                  max_abs=2e-5, max_rel=1e-4, what="q4g32 gemv + bias")
    xb = O.f32_to_bf16_bits(x)
    d_yb = hip.DeviceBuffer(b * n * 2)
    kernels.launch_qgemm_q4g32_bf16(up(xb), d_q, d_s, d_m, d_yb, b, n, k, bias=up(bias))
    hip.synchronize()
    assert_parity(O.bf16_bits_to_f32(d_yb.to_numpy(np.uint16, (b, n))),
                  O.bf16_bits_to_f32(O.qgemm_q4g32_bf16(xb, q32, s32, m32, b, n, k, bias)),
                  what="q4g32 gemm + bias")


def test_q4g128_512_rows_through_the_mlp_up_projection():
    # one 512-token prefill chunk through gate/up-sized weights: m = 512, 12288 x 4096
    rng = np.random.default_rng(7)
    b, n, k = 512, 12288, 4096
    qw = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    s = (rng.random((n, k // 128), np.float32) * 0.004 + 0.004).astype(np.float16)
    z = (rng.random((n, k // 128), np.float32) * 2 + 6.5).astype(np.float16)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    got = _gemm_q4(xb, qw, s, z, b, n, k, None)
    # the oracle on a sample of rows that straddles the 32-row passes (each row of the product
    # depends on its own row of x only)
    rows = np.r_[0:34, 250:262, 480:512]
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb[rows], qw, s, z, len(rows), n, k))
    assert_parity(got[rows], want, what="q4g128 m = 512")
    assert np.isfinite(got).all()
    # every row was written by its own pass: a row of x repeated gives the same output row
    xb2 = xb.copy()
    xb2[300] = xb2[3]
    xb2[511] = xb2[3]
    got2 = _gemm_q4(xb2, qw, s, z, b, n, k, None)
    assert np.array_equal(got2[300], got2[3]) and np.array_equal(got2[511], got2[3])


def test_q4g128_packed_mixed_batch_rows_with_a_ragged_tail_and_bias():
    # config 4's packed token buffer (48 decode rows + 16 x 512 prefill rows = 8240 = 257 * 32
    # + 16) through an attention-output-sized projection, with a bias
    rng = np.random.default_rng(8)
    b, n, k = 8240, 4096, 4096
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    bias = rng.standard_normal(n).astype(np.float32)
    got = _gemm_q4(xb, qw, s, z, b, n, k, bias)
    rows = np.r_[0:3, 30:35, 4111:4114, 8222:8240]
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb[rows], qw, s, z, len(rows), n, k, bias))
    assert_parity(got[rows], want, what="q4g128 m = 8240 + bias")
    assert np.isfinite(got).all()


def test_q4g32_tall_x():
    rng = np.random.default_rng(9)
    b, n, k = 83, 1024, 512
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    q32, s32, m32 = O.q4_blocks_to_q4g32(O.quantize_q4_blocks(w, n, k, False), n, k, False)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    d_yb = hip.DeviceBuffer(b * n * 2)
    kernels.launch_qgemm_q4g32_bf16(up(xb), up(q32), up(s32.view(np.uint16)),
                                    up(m32.view(np.uint16)), d_yb, b, n, k)
    hip.synchronize()
    assert_parity(O.bf16_bits_to_f32(d_yb.to_numpy(np.uint16, (b, n))),
                  O.bf16_bits_to_f32(O.qgemm_q4g32_bf16(xb, q32, s32, m32, b, n, k)),
                  what="q4g32 gemm m = 83")


@pytest.mark.parametrize("b,n,k,with_bias", [(97, 128, 128, False), (130, 200, 256, True),
                                             (257, 1000, 1152, True), (300, 4100, 4096, False),
                                             (1000, 333, 2048, True)])
def test_q4g128_tiled_kernel_ragged_shapes(b, n, k, with_bias):
    # the 128 x 128-tile kernel that serves tall x: partial tiles in rows and in weight rows,
    # K of one group and of an odd number of groups, with and without a bias
    rng = np.random.default_rng(b + 7 * n + 13 * k)
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    bias = rng.standard_normal(n).astype(np.float32) if with_bias else None
    got = _gemm_q4(xb, qw, s, z, b, n, k, bias)
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb, qw, s, z, b, n, k, bias))
    assert_parity(got, want, what=f"q4g128 tiled {b}x{n}x{k}")


def test_q4g128_tiled_kernel_one_hot_rows_read_back_dequantised_columns():
    # orientation, nibble order, pair order of x and the zero-point term in one exact check:
    # row i of x is the unit vector of column c_i, so row i of y is column c_i of the
    # dequantised matrix (one product, one rounding)
    rng = np.random.default_rng(10)
    b, n, k = 256, 160, 384
    w = rng.standard_normal((n, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    wd = O.dequantize_q4g128(qw, s, z, n, k)
    cols = rng.integers(0, k, size=b)
    cols[:8] = [0, 1, 4, 7, 8, 63, 64, 127]
    x = np.zeros((b, k), np.float32)
    x[np.arange(b), cols] = 1.0
    got = _gemm_q4(O.f32_to_bf16_bits(x), qw, s, z, b, n, k, None)
    want = O.bf16_bits_to_f32(O.f32_to_bf16_bits(wd[:, cols].T.copy()))
    # (128 + q) - (128 + zero) in fp32, times scale: the same value the oracle rounds
    assert_parity(got, want, max_abs=1e-6, max_rel=4e-3, what="one-hot rows")


def _gemm_q4_ws(xb, qw, s, z, b, n, k, bias, f32_out=False, ws_fill=0xFF):
    """`logismos_launch_qgemm_q4g128_tall`: the same product through the entry point with a
    workspace (first pass over x, then the tiled kernel that reads x straight into LDS)."""
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(b, k))
    ws.fill(ws_fill)
    d_y = hip.DeviceBuffer(b * n * (4 if f32_out else 2))
    d_y.fill(0xFF)
    kernels.launch_qgemm_q4g128_tall(up(xb), up(qw), up(s.view(np.uint16)), up(z.view(np.uint16)),
                                     d_y, ws, b, n, k, bias=up(bias) if bias is not None else None,
                                     f32_out=f32_out)
    hip.synchronize()
    if f32_out:
        return d_y.to_numpy(np.float32, (b, n))
    return O.bf16_bits_to_f32(d_y.to_numpy(np.uint16, (b, n)))


@pytest.mark.parametrize("b,n,k,with_bias", [(1, 16, 256, True), (97, 128, 256, False),
                                             (130, 200, 512, True), (257, 1000, 1280, True),
                                             (300, 4100, 4096, False), (1000, 333, 2048, True),
                                             (142, 576, 512, True), (200, 300, 1536, True),
                                             (130, 520, 3072, False)])
def test_q4g128_workspace_kernel_ragged_shapes(b, n, k, with_bias):
    # partial tiles in rows (128) and in weight rows (256), K of two groups up to 32, with and
    # without a bias; the fp32 product (what the step executor keeps) tightly, the bf16 one at
    # the decode path's tolerance; what the workspace held before does not matter.  K decides
    # how many pairs of groups a lane loads scales / zeros / sums for at once (a multiple of
    # 1024: four, 1536 = 3 x 512: two, else one), each with one and with several such blocks;
    # every one of these launches is smaller than the device, so its tiles are split over K
    # (evenly or not: 24 groups in parts of 8, 12 in parts of 4) and summed by the reduce kernel
    rng = np.random.default_rng(b + 7 * n + 13 * k)
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    bias = rng.standard_normal(n).astype(np.float32) if with_bias else None
    got32 = _gemm_q4_ws(xb, qw, s, z, b, n, k, bias, f32_out=True)
    want32 = O.qgemm_q4g128_f32(xb, qw, s, z, b, n, k, bias)
    assert_parity(got32, want32, max_abs=2e-4, max_rel=1e-3, what=f"q4g128 workspace f32 {b}x{n}x{k}")
    got = _gemm_q4_ws(xb, qw, s, z, b, n, k, bias, ws_fill=0x00)
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb, qw, s, z, b, n, k, bias))
    assert_parity(got, want, what=f"q4g128 workspace bf16 {b}x{n}x{k}")
    # the bf16 product is the one rounding of the fp32 one
    assert np.array_equal(O.f32_to_bf16_bits(got32).reshape(b, n),
                          O.f32_to_bf16_bits(got).reshape(b, n))


@pytest.mark.parametrize("shift", [0, 8, 4])
def test_q4g128_workspace_kernel_takes_scales_and_zeros_at_any_4_byte_alignment(shift):
    # the kernel loads a lane's scales and zeros for four pairs of groups at once where they
    # are 16-byte aligned (and K allows), for two at 8 bytes, for one otherwise: the same
    # arrays at 16-, 8- and 4-byte aligned addresses, each against the oracle
    rng = np.random.default_rng(91)
    b, n, k = 200, 520, 2048
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    bias = rng.standard_normal(n).astype(np.float32)

    def shifted(a):
        raw = np.zeros(a.nbytes + 16, np.uint8)
        raw[shift:shift + a.nbytes] = a.view(np.uint8).reshape(-1)
        buf = up(raw)
        return buf, buf.offset(shift)
    s_buf, s_ptr = shifted(s.view(np.uint16))
    z_buf, z_ptr = shifted(z.view(np.uint16))
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(b, k))
    d_y = hip.DeviceBuffer(b * n * 4)
    d_y.fill(0xFF)
    kernels.launch_qgemm_q4g128_tall(up(xb), up(qw), s_ptr, z_ptr, d_y, ws, b, n, k,
                                     bias=up(bias), f32_out=True)
    hip.synchronize()
    got = d_y.to_numpy(np.float32, (b, n))
    want = O.qgemm_q4g128_f32(xb, qw, s, z, b, n, k, bias)
    assert_parity(got, want, max_abs=2e-4, max_rel=1e-3, what=f"scales at +{shift} bytes")
    del s_buf, z_buf


@pytest.mark.parametrize("rows,inter,n", [(200, 1024, 300), (130, 1536, 256), (97, 768, 520)])
def test_swiglu_written_as_the_workspace_kernels_operand(rows, inter, n):
    # `silu_mul_f32p_tall` + `qgemm_q4g128_tall_prepared` against `silu_mul_f32p` + the entry
    # point that makes its own first pass: the same workspace contents (x in pair order, rows
    # padded with zeros, group sums), hence the same product, bit for bit; and both against
    # the oracle.  inter a multiple of 1024 / 512 / 256: four, two, one pair of groups per load.
    from oracle import decode_step as OS
    rng = np.random.default_rng(rows + inter)
    parts = rng.standard_normal((2, rows, 2 * inter), np.float32)
    qw, s, z = _q4(rng, n, inter)
    d_parts, d_qw = up(parts), up(qw)
    d_s, d_z = up(s.view(np.uint16)), up(z.view(np.uint16))
    nbytes = kernels.qgemm_q4g128_tall_workspace_bytes(rows, inter)
    w = kernels.qgemm_q4g128_tall_pairs_per_load(inter, d_s, d_z)
    assert w == (4 if inter % 1024 == 0 else 2 if inter % 512 == 0 else 1)

    ws_a = hip.DeviceBuffer(nbytes)
    ws_a.fill(0xFF)
    d_ya = hip.DeviceBuffer(rows * n * 4)
    kernels.launch_silu_mul_f32p_tall(d_parts, 2, ws_a, rows, inter, w)
    kernels.launch_qgemm_q4g128_tall_prepared(d_qw, d_s, d_z, d_ya, ws_a, rows, n, inter,
                                              f32_out=True)
    ws_b = hip.DeviceBuffer(nbytes)
    ws_b.fill(0x00)
    d_act = hip.DeviceBuffer(rows * inter * 2)
    d_yb = hip.DeviceBuffer(rows * n * 4)
    kernels.launch_silu_mul_f32p(d_parts, 2, d_act, rows, inter)
    kernels.launch_qgemm_q4g128_tall(d_act, d_qw, d_s, d_z, d_yb, ws_b, rows, n, inter,
                                     f32_out=True)
    hip.synchronize()
    rows_pad = -(-rows // 128) * 128
    head = rows_pad * inter * 2                      # x in pair order
    sums_at = (head + 255) // 256 * 256
    sums = rows_pad * (inter // 128) * 4
    a, b = ws_a.to_numpy(np.uint8, (nbytes,)), ws_b.to_numpy(np.uint8, (nbytes,))
    assert np.array_equal(a[:head], b[:head])
    assert np.array_equal(a[sums_at:sums_at + sums], b[sums_at:sums_at + sums])
    assert not a[rows * inter * 2:head].any()        # the padding rows
    ya, yb = d_ya.to_numpy(np.float32, (rows, n)), d_yb.to_numpy(np.float32, (rows, n))
    assert np.array_equal(ya.view(np.uint32), yb.view(np.uint32))
    act = OS.silu_mul_bf16(parts[0] + parts[1], inter)
    assert np.array_equal(d_act.to_numpy(np.uint16, (rows, inter)), act)
    want = O.qgemm_q4g128_f32(act, qw, s, z, rows, n, inter, None)
    assert_parity(ya, want, max_abs=2e-4, max_rel=1e-3, what=f"swiglu -> down {rows}x{n}x{inter}")


@pytest.mark.parametrize("rows,inter,k", [(200, 300, 1024), (130, 1000, 512), (97, 128, 768),
                                          (520, 2560, 2048)])
def test_gate_up_projection_with_the_swiglu_in_the_kernel(rows, inter, k):
    # one kernel for the gate/up projection and silu(gate) * up against the two-step form
    # (fp32 products of all 2 * inter weight rows, then `silu_mul_f32p`): a workgroup tile
    # pairs 128 gate rows with the up rows of the same outputs, the sums are the same fp32
    # sums in the same order, so the bf16 activations are the same bits -- whole tiles and
    # tiles split over K (every launch here is smaller than the device; the last shape splits
    # unevenly), ragged in rows and in outputs; and against the oracle.
    from oracle import decode_step as OS
    rng = np.random.default_rng(rows + inter + k)
    qw, s, z = _q4(rng, 2 * inter, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((rows, k), np.float32))
    d_x, d_qw = up(xb), up(qw)
    d_s, d_z = up(s.view(np.uint16)), up(z.view(np.uint16))
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(rows, k))
    # two steps: products (which also leaves x prepared in the workspace), then the activation
    d_gu = hip.DeviceBuffer(rows * 2 * inter * 4)
    kernels.launch_qgemm_q4g128_tall(d_x, d_qw, d_s, d_z, d_gu, ws, rows, 2 * inter, k, f32_out=True)
    d_two = hip.DeviceBuffer(rows * inter * 2)
    kernels.launch_silu_mul_f32p(d_gu, 1, d_two, rows, inter)
    # one step over the same prepared workspace
    d_one = hip.DeviceBuffer(rows * inter * 2)
    d_one.fill(0xFF)
    kernels.launch_qgemm_q4g128_tall_swiglu_prepared(d_qw, d_s, d_z, d_one, ws, rows, inter, k)
    hip.synchronize()
    one = d_one.to_numpy(np.uint16, (rows, inter))
    two = d_two.to_numpy(np.uint16, (rows, inter))
    assert np.array_equal(one, two)
    gu = O.qgemm_q4g128_f32(xb, qw, s, z, rows, 2 * inter, k, None)
    want = OS.silu_mul_bf16(gu, inter)
    assert_parity(O.bf16_bits_to_f32(one), O.bf16_bits_to_f32(want), what="gate/up + swiglu")


@pytest.mark.parametrize("rows,inter,k", [(200, 1024, 512), (130, 512, 1024), (97, 256, 768),
                                          (520, 2560, 2048), (1100, 3840, 512)])
def test_gate_up_projection_writing_the_down_projections_operand(rows, inter, k):
    # the gate/up projection with the SwiGLU, its result written straight into the workspace of
    # the product that follows (K = inter), against the route through memory: fp32 gate/up
    # products, then `silu_mul_f32p_tall`.  The same bf16 values in the same places, zero
    # padding rows, the group sums added in the same order: the operand part of the two
    # workspaces is the same bytes -- for whole tiles (the last shape has more tiles than the
    # device has units) and for tiles split over K (the others), four, two and one pair of
    # groups per load of the following product.
    rng = np.random.default_rng(rows + inter + k + 1)
    qw, s, z = _q4(rng, 2 * inter, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((rows, k), np.float32))
    d_x, d_qw = up(xb), up(qw)
    d_s, d_z = up(s.view(np.uint16)), up(z.view(np.uint16))
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(rows, k))
    w_next = 4 if inter % 1024 == 0 else 2 if inter % 512 == 0 else 1
    nbytes = kernels.qgemm_q4g128_tall_workspace_bytes(rows, inter)
    d_gu = hip.DeviceBuffer(rows * 2 * inter * 4)
    kernels.launch_qgemm_q4g128_tall(d_x, d_qw, d_s, d_z, d_gu, ws, rows, 2 * inter, k, f32_out=True)
    ws_two = hip.DeviceBuffer(nbytes)
    ws_two.fill(0xFF)
    kernels.launch_silu_mul_f32p_tall(d_gu, 1, ws_two, rows, inter, w_next)
    ws_one = hip.DeviceBuffer(nbytes)
    ws_one.fill(0xEE)
    kernels.launch_qgemm_q4g128_tall_swiglu_operand(d_qw, d_s, d_z, ws_one, w_next, ws, rows,
                                                    inter, k)
    hip.synchronize()
    rows_pad = -(-rows // 128) * 128
    head = rows_pad * inter * 2
    sums_at = (head + 255) // 256 * 256
    sums = rows_pad * (inter // 128) * 4
    a, b = ws_one.to_numpy(np.uint8, (nbytes,)), ws_two.to_numpy(np.uint8, (nbytes,))
    assert np.array_equal(a[:head], b[:head])
    assert not a[rows * inter * 2:head].any()
    sa = a[sums_at:sums_at + sums].view(np.float32)
    sb = b[sums_at:sums_at + sums].view(np.float32)
    assert np.array_equal(sa.view(np.uint32), sb.view(np.uint32))
    # what lies behind the operand (the following product's partial tiles) is not touched
    assert np.all(a[sums_at + sums:] == 0xEE)


def test_gate_up_operand_refusals():
    rng = np.random.default_rng(3)
    rows, inter, k = 130, 384, 512  # inter is not a multiple of 256
    qw, s, z = _q4(rng, 2 * inter, k)
    d_qw, d_s, d_z = up(qw), up(s.view(np.uint16)), up(z.view(np.uint16))
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(rows, k))
    nxt = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(rows, 512))
    with pytest.raises(kernels.LaunchError):
        kernels.launch_qgemm_q4g128_tall_swiglu_operand(d_qw, d_s, d_z, nxt, 1, ws, rows, inter, k)
    qw, s, z = _q4(rng, 1024, k)
    d_qw, d_s, d_z = up(qw), up(s.view(np.uint16)), up(z.view(np.uint16))
    with pytest.raises(kernels.LaunchError):  # 512 is not a whole block of four pairs
        kernels.launch_qgemm_q4g128_tall_swiglu_operand(d_qw, d_s, d_z, nxt, 4, ws, rows, 512, k)
    with pytest.raises(kernels.LaunchError):  # one workspace for both
        kernels.launch_qgemm_q4g128_tall_swiglu_operand(d_qw, d_s, d_z, ws, 2, ws, rows, 512, k)
    hip.synchronize()


def test_gate_up_with_the_swiglu_on_more_tiles_than_the_device_has_units():
    # 9 x 30 = 270 tiles of 128 rows x 128 outputs: the first 256 whole, the other 14 split over
    # K with the activation applied where their parts are summed; bit for bit the two-step form
    # everywhere, and the oracle on the first and the last rows
    from oracle import decode_step as OS
    rows, inter, k = 1100, 3840, 512
    rng = np.random.default_rng(97)
    qw, s, z = _q4(rng, 2 * inter, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((rows, k), np.float32))
    d_x, d_qw = up(xb), up(qw)
    d_s, d_z = up(s.view(np.uint16)), up(z.view(np.uint16))
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(rows, k))
    d_gu = hip.DeviceBuffer(rows * 2 * inter * 4)
    kernels.launch_qgemm_q4g128_tall(d_x, d_qw, d_s, d_z, d_gu, ws, rows, 2 * inter, k, f32_out=True)
    d_two = hip.DeviceBuffer(rows * inter * 2)
    kernels.launch_silu_mul_f32p(d_gu, 1, d_two, rows, inter)
    d_one = hip.DeviceBuffer(rows * inter * 2)
    d_one.fill(0xFF)
    kernels.launch_qgemm_q4g128_tall_swiglu_prepared(d_qw, d_s, d_z, d_one, ws, rows, inter, k)
    hip.synchronize()
    one = d_one.to_numpy(np.uint16, (rows, inter))
    assert np.array_equal(one, d_two.to_numpy(np.uint16, (rows, inter)))
    for r0, r1 in ((0, 40), (rows - 40, rows)):
        gu = O.qgemm_q4g128_f32(xb[r0:r1], qw, s, z, r1 - r0, 2 * inter, k, None)
        assert_parity(O.bf16_bits_to_f32(one[r0:r1]), O.bf16_bits_to_f32(OS.silu_mul_bf16(gu, inter)),
                      what=f"gate/up + swiglu, rows {r0}..{r1}")


def test_q4g128_workspace_kernel_is_deterministic():
    # parts of a tile split over K are summed in part order: two launches, the same bits
    rng = np.random.default_rng(92)
    b, n, k = 300, 1000, 4096
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    first = _gemm_q4_ws(xb, qw, s, z, b, n, k, None, f32_out=True)
    again = _gemm_q4_ws(xb, qw, s, z, b, n, k, None, f32_out=True, ws_fill=0x00)
    assert np.array_equal(first.view(np.uint32), again.view(np.uint32))


def test_q4g128_workspace_kernel_one_hot_rows_read_back_dequantised_columns():
    # orientation, nibble order, the pair order the first pass writes, the LDS swizzles of x
    # and of the weights, and the zero-point product in one exact check: row i of x is the unit
    # vector of column c_i, so row i of y is column c_i of the dequantised matrix
    rng = np.random.default_rng(11)
    b, n, k = 384, 300, 768
    w = rng.standard_normal((n, k), np.float32)
    qw, s, z = O.quantize_q4g128(w, n, k)
    wd = O.dequantize_q4g128(qw, s, z, n, k)
    cols = rng.integers(0, k, size=b)
    cols[:10] = [0, 1, 4, 7, 8, 63, 64, 127, 128, 767]
    x = np.zeros((b, k), np.float32)
    x[np.arange(b), cols] = 1.0
    got = _gemm_q4_ws(O.f32_to_bf16_bits(x), qw, s, z, b, n, k, None, f32_out=True)
    # scale * (128 + q) and scale * (128 + zero) * 1 are rounded apart (values of ~50 here, one
    # fp32 ulp 4e-6) before they cancel to the dequantised weight of order 1
    assert_parity(got, wd[:, cols].T.copy(), max_abs=8e-6, max_rel=1e-5, what="one-hot rows")


def test_q4g128_workspace_kernel_config4_rows():
    # config 4's 8240 packed rows through an attention-output-sized projection with a bias
    rng = np.random.default_rng(12)
    b, n, k = 8240, 4096, 4096
    qw, s, z = _q4(rng, n, k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
    bias = rng.standard_normal(n).astype(np.float32)
    got = _gemm_q4_ws(xb, qw, s, z, b, n, k, bias)
    rows = np.r_[0:3, 126:131, 4111:4114, 8190:8194, 8222:8240]
    want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb[rows], qw, s, z, len(rows), n, k, bias))
    assert_parity(got[rows], want, what="q4g128 workspace m = 8240 + bias")
    assert np.isfinite(got).all()


def test_q4g128_workspace_entry_point_refuses_what_it_cannot_run():
    with pytest.raises(kernels.UnsupportedShape):
        kernels.launch_qgemm_q4g128_tall(None, None, None, None, None, None, 128, 128, 384)
    with pytest.raises(kernels.UnsupportedShape):
        kernels.launch_qgemm_q4g128_tall(None, None, None, None, None, None, 0, 128, 256)
    # the copy of x, its group sums, and room for 512 fp32 partial tiles of 128 x 256
    assert kernels.qgemm_q4g128_tall_workspace_bytes(130, 512) == (
        256 * 512 * 2 + 256 * 4 * 4 + 512 * 128 * 256 * 4)
