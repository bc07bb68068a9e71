"""GPU parity of the small decode-step operators vs the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from logismos_amd import hip, kernels
from tests.gpu_harness import assert_parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,n,with_y", [(1, 128, False), (5, 1536, True), (32, 4096, True),
                                           (3, 1000, True)])
def test_add_rms_norm(rows, n, with_y):
    rng = np.random.default_rng(rows * n)
    h = rng.standard_normal((rows, n), np.float32)
    y = O.f32_to_bf16_bits(rng.standard_normal((rows, n), np.float32)) if with_y else None
    w = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
    d_h = hip.DeviceBuffer.from_numpy(h)
    d_y = hip.DeviceBuffer.from_numpy(y) if with_y else None
    d_out = hip.DeviceBuffer(rows * n * 2)
    kernels.launch_add_rms_norm_bf16(d_h, d_y, hip.DeviceBuffer.from_numpy(w), d_out, rows, n, 1e-6)
    hip.synchronize()
    h_ref = h.copy()
    want = OS.add_rms_norm_bf16(h_ref, y, w, 1e-6)
    # the residual add is one fp32 add: bit-exact
    assert np.array_equal(d_h.to_numpy(np.float32, (rows, n)), h_ref)
    got = O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (rows, n)))
    assert_parity(got, O.bf16_bits_to_f32(want), max_abs=2e-3, max_rel=1e-2, what="add_rms_norm")


def test_rope_kv_write_matches_oracle_and_reference_table():
    rng = np.random.default_rng(21)
    t, hq, hkv, d, bs, nblk, max_pos = 7, 8, 2, 128, 16, 12, 4096
    qkv = O.f32_to_bf16_bits(rng.standard_normal((t, (hq + 2 * hkv) * d), np.float32))
    positions = np.array([0, 1, 17, 4095, 300, 4094, 2], np.int32)
    slots = rng.permutation(nblk * bs)[:t].astype(np.int64)
    slots[3] = -1
    cos, sin = O.build_rope_table_f32(max_pos, d, 1_000_000.0)
    k_pool = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    v_pool = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    d_kp, d_vp = hip.DeviceBuffer.from_numpy(k_pool), hip.DeviceBuffer.from_numpy(v_pool)
    d_q = hip.DeviceBuffer(t * hq * d * 2)
    kernels.launch_rope_kv_write_fp16(
        hip.DeviceBuffer.from_numpy(qkv), hip.DeviceBuffer.from_numpy(positions),
        hip.DeviceBuffer.from_numpy(cos), hip.DeviceBuffer.from_numpy(sin),
        hip.DeviceBuffer.from_numpy(slots), d_q, d_kp, d_vp, t, hq, hkv, d, max_pos)
    hip.synchronize()
    q_want = OS.rope_kv_write(qkv, positions, cos, sin, slots, k_pool, v_pool, hq, hkv, d)
    q_got = d_q.to_numpy(np.float16, (t, hq, d))
    # fp32 rotate of two products then one fp16 rounding: allow 1 ulp (fma contraction)
    assert_parity(q_got, q_want, max_abs=1e-3, max_rel=2e-3, what="rope q")
    assert_parity(d_kp.to_numpy(np.float16, k_pool.shape), k_pool, max_abs=1e-3, max_rel=2e-3,
                  what="rope k pool")
    # v is copied unrotated: bit-exact (bf16 -> fp16 is exact or the same rounding)
    assert np.array_equal(d_vp.to_numpy(np.float16, v_pool.shape).view(np.uint16),
                          v_pool.view(np.uint16))
    # position 0 is the identity rotation
    x0 = O.bf16_bits_to_f32(qkv[0]).reshape(hq + 2 * hkv, d)[:hq]
    assert np.array_equal(q_got[0], x0.astype(np.float16))


@pytest.mark.parametrize("d", [32, 64, 96, 256])
def test_rope_kv_write_at_other_head_dims(d):
    # the rotation pairs (i, i + d/2) of `rope_halves_in_place`
    # (crates/kernels/src/cpu_f32/mod.rs:599-619) at head widths other than 128, from bf16
    # rows and from fp32 split-K parts with a bias
    rng = np.random.default_rng(210 + d)
    t, hq, hkv, bs, nblk, max_pos = 9, 6, 2, 16, 12, 2048
    width = (hq + 2 * hkv) * d
    positions = np.array([0, 1, 17, 2047, 300, 2046, 2, 5, 1000], np.int32)
    slots = rng.permutation(nblk * bs)[:t].astype(np.int64)
    slots[3] = -1
    cos, sin = O.build_rope_table_f32(max_pos, d, 10_000.0)
    k0 = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    v0 = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    dev = hip.DeviceBuffer.from_numpy

    qkv = O.f32_to_bf16_bits(rng.standard_normal((t, width), np.float32))
    k_pool, v_pool = k0.copy(), v0.copy()
    d_kp, d_vp, d_q = dev(k_pool), dev(v_pool), hip.DeviceBuffer(t * hq * d * 2)
    kernels.launch_rope_kv_write_fp16(dev(qkv), dev(positions), dev(cos), dev(sin), dev(slots),
                                      d_q, d_kp, d_vp, t, hq, hkv, d, max_pos)
    hip.synchronize()
    q_want = OS.rope_kv_write(qkv, positions, cos, sin, slots, k_pool, v_pool, hq, hkv, d)
    q_got = d_q.to_numpy(np.float16, (t, hq, d))
    assert_parity(q_got, q_want, max_abs=1e-3, max_rel=2e-3, what=f"rope q d={d}")
    assert_parity(d_kp.to_numpy(np.float16, k_pool.shape), k_pool, max_abs=1e-3, max_rel=2e-3,
                  what=f"rope k pool d={d}")
    assert np.array_equal(d_vp.to_numpy(np.float16, v_pool.shape).view(np.uint16),
                          v_pool.view(np.uint16))
    x0 = O.bf16_bits_to_f32(qkv[0]).reshape(hq + 2 * hkv, d)[:hq]
    assert np.array_equal(q_got[0], x0.astype(np.float16))  # position 0: identity

    parts = rng.standard_normal((3, t, width), np.float32)
    bias = rng.standard_normal(width).astype(np.float32)
    k_pool, v_pool = k0.copy(), v0.copy()
    d_kp, d_vp, d_q = dev(k_pool), dev(v_pool), hip.DeviceBuffer(t * hq * d * 2)
    kernels.launch_rope_kv_write_f32p(dev(parts), 3, dev(positions), dev(cos), dev(sin),
                                      dev(slots), d_q, d_kp, d_vp, t, hq, hkv, d, max_pos,
                                      bias=dev(bias))
    hip.synchronize()
    q_want = OS.rope_kv_write(parts[0] + parts[1] + parts[2] + bias, positions, cos, sin, slots,
                              k_pool, v_pool, hq, hkv, d)
    assert_parity(d_q.to_numpy(np.float16, (t, hq, d)), q_want, max_abs=1e-3, max_rel=2e-3,
                  what=f"rope_f32p q d={d}")
    assert_parity(d_kp.to_numpy(np.float16, k_pool.shape), k_pool, max_abs=1e-3, max_rel=2e-3,
                  what=f"rope_f32p k d={d}")
    assert_parity(d_vp.to_numpy(np.float16, v_pool.shape), v_pool, max_abs=1e-3, max_rel=2e-3,
                  what=f"rope_f32p v d={d}")


def test_silu_mul_and_cast():
    rng = np.random.default_rng(22)
    rows, inter = 5, 1000
    gu = O.f32_to_bf16_bits(rng.standard_normal((rows, 2 * inter), np.float32) * 3)
    d_out = hip.DeviceBuffer(rows * inter * 2)
    kernels.launch_silu_mul_bf16(hip.DeviceBuffer.from_numpy(gu), d_out, rows, inter)
    hip.synchronize()
    got = O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (rows, inter)))
    assert_parity(got, O.bf16_bits_to_f32(OS.silu_mul_bf16(gu, inter)), what="silu_mul")
    a = rng.standard_normal(777, np.float32).astype(np.float16)
    d_b = hip.DeviceBuffer(777 * 2)
    kernels.launch_cast_f16_bf16(hip.DeviceBuffer.from_numpy(a), d_b, 777)
    hip.synchronize()
    assert np.array_equal(d_b.to_numpy(np.uint16, (777,)), OS.cast_f16_bf16(a))


def test_greedy_first_maximum_wins():
    """crates/decode/src/lib.rs:90-92 plus a vocabulary-sized row"""
    rng = np.random.default_rng(23)
    rows, n = 4, 151936
    logits = rng.standard_normal((rows, n), np.float32)
    logits[0, :3] = [0.0, 2.0, 2.0]
    logits[0, 3:] = -1.0
    logits[1, [5, 70000, 150000]] = 9.0       # three equal maxima: index 5
    logits[2, :] = -np.inf                     # all -inf: index 0
    d_out = hip.DeviceBuffer(rows * 4)
    kernels.launch_greedy_f32(hip.DeviceBuffer.from_numpy(logits), d_out, rows, n)
    hip.synchronize()
    got = d_out.to_numpy(np.uint32, (rows,))
    want = [O.greedy(logits[r]) for r in range(rows)]
    assert got.tolist() == want
    assert got[0] == 1 and got[1] == 5 and got[2] == 0


def test_f32_parts_variants_add_the_parts_in_order():
    rng = np.random.default_rng(24)
    rows, n, j = 6, 2048, 3
    # add_rms_norm over three fp32 parts
    h = rng.standard_normal((rows, n), np.float32)
    parts = rng.standard_normal((j, rows, n), np.float32)
    w = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
    d_h, d_out = hip.DeviceBuffer.from_numpy(h), hip.DeviceBuffer(rows * n * 2)
    kernels.launch_add_rms_norm_f32p(d_h, hip.DeviceBuffer.from_numpy(parts), j,
                                     hip.DeviceBuffer.from_numpy(w), d_out, rows, n, 1e-6)
    hip.synchronize()
    y = (parts[0] + parts[1]) + parts[2]            # same order: bit-exact residual
    h_ref = h + parts[0]
    h_ref += parts[1]
    h_ref += parts[2]
    assert np.array_equal(d_h.to_numpy(np.float32, (rows, n)), h_ref)
    want = O.f32_to_bf16_bits(O.rms_norm(h_ref, w, rows, n, 1e-6)).reshape(rows, n)
    assert_parity(O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (rows, n))),
                  O.bf16_bits_to_f32(want), what="add_rms_norm_f32p")
    # zero parts: plain RMSNorm of h
    d_h2 = hip.DeviceBuffer.from_numpy(h)
    kernels.launch_add_rms_norm_f32p(d_h2, None, 0, hip.DeviceBuffer.from_numpy(w), d_out, rows, n,
                                     1e-6)
    hip.synchronize()
    assert np.array_equal(d_h2.to_numpy(np.float32, (rows, n)), h)

    # silu_mul over two parts
    inter = 1000
    gp = rng.standard_normal((2, rows, 2 * inter), np.float32)
    d_o = hip.DeviceBuffer(rows * inter * 2)
    kernels.launch_silu_mul_f32p(hip.DeviceBuffer.from_numpy(gp), 2, d_o, rows, inter)
    hip.synchronize()
    want = OS.silu_mul_bf16(gp[0] + gp[1], inter)
    assert_parity(O.bf16_bits_to_f32(d_o.to_numpy(np.uint16, (rows, inter))),
                  O.bf16_bits_to_f32(want), what="silu_mul_f32p")

    # rope over two parts
    t, hq, hkv, d, bs, nblk, max_pos = 5, 4, 2, 128, 16, 8, 512
    qp = rng.standard_normal((2, t, (hq + 2 * hkv) * d), np.float32)
    positions = np.array([0, 3, 511, 17, 100], np.int32)
    slots = rng.permutation(nblk * bs)[:t].astype(np.int64)
    cos, sin = O.build_rope_table_f32(max_pos, d, 1_000_000.0)
    k_pool = np.zeros((nblk * bs, hkv * d), np.float16)
    v_pool = np.zeros((nblk * bs, hkv * d), np.float16)
    d_kp, d_vp = hip.DeviceBuffer.from_numpy(k_pool), hip.DeviceBuffer.from_numpy(v_pool)
    d_q = hip.DeviceBuffer(t * hq * d * 2)
    kernels.launch_rope_kv_write_f32p(
        hip.DeviceBuffer.from_numpy(qp), 2, hip.DeviceBuffer.from_numpy(positions),
        hip.DeviceBuffer.from_numpy(cos), hip.DeviceBuffer.from_numpy(sin),
        hip.DeviceBuffer.from_numpy(slots), d_q, d_kp, d_vp, t, hq, hkv, d, max_pos)
    hip.synchronize()
    q_want = OS.rope_kv_write(qp[0] + qp[1], positions, cos, sin, slots, k_pool, v_pool, hq, hkv, d)
    assert_parity(d_q.to_numpy(np.float16, (t, hq, d)), q_want, max_abs=1e-3, max_rel=2e-3,
                  what="rope_f32p q")
    assert_parity(d_kp.to_numpy(np.float16, k_pool.shape), k_pool, max_abs=1e-3, max_rel=2e-3,
                  what="rope_f32p k")
    assert np.array_equal(d_vp.to_numpy(np.float16, v_pool.shape).view(np.uint16),
                          v_pool.view(np.uint16))

    # the same into turbo3 pools: the encoder sees the fp16 rows the fp16 pools hold.  V is
    # not rotated (its fp16 rows are exact above), so its encoded bytes must be identical;
    # a rotated K row may differ from the oracle's in the last fp16 bit, and the byte-exact
    # comparison is made against the encoding of the rows the GPU wrote above.
    k3 = np.zeros((nblk * bs, hkv * 56), np.uint8)
    v3 = np.zeros((nblk * bs, hkv * 56), np.uint8)
    d_k3, d_v3 = hip.DeviceBuffer.from_numpy(k3), hip.DeviceBuffer.from_numpy(v3)
    d_q3 = hip.DeviceBuffer(t * hq * d * 2)
    kernels.launch_rope_kv_write_f32p(
        hip.DeviceBuffer.from_numpy(qp), 2, hip.DeviceBuffer.from_numpy(positions),
        hip.DeviceBuffer.from_numpy(cos), hip.DeviceBuffer.from_numpy(sin),
        hip.DeviceBuffer.from_numpy(slots), d_q3, d_k3, d_v3, t, hq, hkv, d, max_pos, turbo3=True)
    hip.synchronize()
    assert np.array_equal(d_q3.to_numpy(np.uint16, (t, hq, d)), d_q.to_numpy(np.uint16, (t, hq, d)))
    gpu_k16 = d_kp.to_numpy(np.float16, k_pool.shape)
    gpu_v16 = d_vp.to_numpy(np.float16, v_pool.shape)
    k3_want, v3_want = k3.copy(), v3.copy()
    O.kv_write_turbo3(gpu_k16[slots], gpu_v16[slots], k3_want, v3_want, slots, hkv)
    assert np.array_equal(d_k3.to_numpy(np.uint8, k3.shape), k3_want)
    assert np.array_equal(d_v3.to_numpy(np.uint8, v3.shape), v3_want)


def test_rope_kv_write_over_many_rows_equals_the_per_head_kernel_bit_for_bit():
    # from 64 tokens on 128-wide heads take the kernel with four rotation pairs per thread;
    # below, one workgroup per (token, head).  The same 200 tokens in one launch and in
    # launches of 50: same q rows, same pool rows, bit for bit -- with three parts, a bias, a
    # token without a slot (skipped) and a position at the end of the table -- and both against
    # the oracle.
    rng = np.random.default_rng(77)
    t, hq, hkv, d, bs, nblk, max_pos = 200, 8, 2, 128, 16, 20, 700
    width = (hq + 2 * hkv) * d
    parts = rng.standard_normal((3, t, width), np.float32)
    bias = rng.standard_normal(width).astype(np.float32)
    positions = rng.integers(0, max_pos, size=t).astype(np.int32)
    positions[:3] = [0, max_pos - 1, 17]
    slots = rng.permutation(nblk * bs)[:t].astype(np.int64)
    slots[5] = -1
    cos, sin = O.build_rope_table_f32(max_pos, d, 1_000_000.0)
    k0 = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    v0 = rng.standard_normal((nblk * bs, hkv * d), np.float32).astype(np.float16)
    dev = hip.DeviceBuffer.from_numpy

    def run(chunk):
        d_kp, d_vp, d_q = dev(k0), dev(v0), hip.DeviceBuffer(t * hq * d * 2)
        for r0 in range(0, t, chunk):
            n = min(chunk, t - r0)
            sub = np.ascontiguousarray(parts[:, r0:r0 + n])
            d_qs = hip.DeviceBuffer(n * hq * d * 2)
            kernels.launch_rope_kv_write_f32p(dev(sub), 3, dev(positions[r0:r0 + n]), dev(cos),
                                              dev(sin), dev(slots[r0:r0 + n]), d_qs, d_kp, d_vp, n,
                                              hq, hkv, d, max_pos, bias=dev(bias))
            hip.synchronize()
            d_q.copy_from_device(d_qs, n * hq * d * 2, dst_offset=r0 * hq * d * 2)
        hip.synchronize()
        return (d_q.to_numpy(np.uint16, (t, hq, d)), d_kp.to_numpy(np.uint16, k0.shape),
                d_vp.to_numpy(np.uint16, v0.shape))
    q_rows, k_rows, v_rows = run(t)       # one launch: the many-row kernel
    q_head, k_head, v_head = run(50)      # launches of 50 tokens: the per-head kernel
    assert np.array_equal(q_rows, q_head)
    assert np.array_equal(k_rows, k_head)
    assert np.array_equal(v_rows, v_head)
    k_want, v_want = k0.copy(), v0.copy()
    keep = slots >= 0
    q_want = OS.rope_kv_write((parts[0] + parts[1] + parts[2] + bias)[keep], positions[keep], cos,
                              sin, slots[keep], k_want, v_want, hq, hkv, d)
    assert_parity(q_rows.view(np.float16)[keep], q_want, max_abs=1e-3, max_rel=2e-3,
                  what="rope rows q")
    assert_parity(k_rows.view(np.float16), k_want, max_abs=1e-3, max_rel=2e-3, what="rope rows k")
    assert_parity(v_rows.view(np.float16), v_want, max_abs=1e-3, max_rel=2e-3, what="rope rows v")
    # the token without a slot left both pools alone (its q row is still written)
    untouched = np.setdiff1d(np.arange(nblk * bs), slots[keep])
    assert np.array_equal(k_rows[untouched], k0.view(np.uint16)[untouched])


def _unprepare(buf, b, k):
    """prepared layout -> (bf16 bits [b][k], group sums [b][k/128])"""
    bp = 16 if b <= 16 else 32
    chunks = k // 8
    xp = buf[: chunks * bp * 16].view(np.uint16).reshape(chunks, bp, 8)
    # pair order (x0,x4)(x1,x5)(x2,x6)(x3,x7) -> natural
    nat = np.empty_like(xp)
    nat[..., [0, 4, 1, 5, 2, 6, 3, 7]] = xp
    x = nat.transpose(1, 0, 2).reshape(bp, k)[:b]
    xg = buf[chunks * bp * 16:].view(np.float32).reshape(k // 128, bp).T[:b]
    return x, xg


def test_prepared_layout_producers_match_the_plain_ones():
    rng = np.random.default_rng(25)
    rows, n, j = 20, 4096, 5
    h = rng.standard_normal((rows, n), np.float32)
    parts = rng.standard_normal((j, rows, n), np.float32)
    w = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
    d_w, d_parts = hip.DeviceBuffer.from_numpy(w), hip.DeviceBuffer.from_numpy(parts)
    d_h1, d_h2 = hip.DeviceBuffer.from_numpy(h), hip.DeviceBuffer.from_numpy(h)
    d_plain = hip.DeviceBuffer(rows * n * 2)
    d_prep = hip.DeviceBuffer(kernels.q4_xprep_bytes(rows, n))
    kernels.launch_add_rms_norm_f32p(d_h1, d_parts, j, d_w, d_plain, rows, n, 1e-6)
    kernels.launch_add_rms_norm_f32p_xprep(d_h2, d_parts, j, d_w, d_prep, rows, n, 1e-6)
    hip.synchronize()
    assert np.array_equal(d_h1.to_numpy(np.float32, (rows, n)), d_h2.to_numpy(np.float32, (rows, n)))
    x, xg = _unprepare(d_prep.to_numpy(np.uint8, (d_prep.nbytes,)), rows, n)
    plain = d_plain.to_numpy(np.uint16, (rows, n))
    # the two kernels reduce the sum of squares in a different order: allow one bf16 ulp
    assert_parity(O.bf16_bits_to_f32(x), O.bf16_bits_to_f32(plain), max_abs=1e-6, max_rel=8e-3,
                  what="prepared add_rms_norm")
    assert np.abs(xg - O.bf16_bits_to_f32(x).reshape(rows, n // 128, 128).sum(axis=2)).max() < 1e-3

    inter = 1536
    gp = rng.standard_normal((3, rows, 2 * inter), np.float32)
    d_gp = hip.DeviceBuffer.from_numpy(gp)
    d_o = hip.DeviceBuffer(rows * inter * 2)
    d_op = hip.DeviceBuffer(kernels.q4_xprep_bytes(rows, inter))
    kernels.launch_silu_mul_f32p(d_gp, 3, d_o, rows, inter)
    kernels.launch_silu_mul_f32p_xprep(d_gp, 3, d_op, rows, inter)
    hip.synchronize()
    x, xg = _unprepare(d_op.to_numpy(np.uint8, (d_op.nbytes,)), rows, inter)
    assert np.array_equal(x, d_o.to_numpy(np.uint16, (rows, inter)))
    assert np.abs(xg - O.bf16_bits_to_f32(x).reshape(rows, inter // 128, 128).sum(axis=2)).max() < 1e-3
    # prepare kernel on the plain output gives the same bytes
    d_op2 = hip.DeviceBuffer(kernels.q4_xprep_bytes(rows, inter))
    kernels.launch_q4_prepare_x_bf16(d_o, d_op2, rows, inter)
    hip.synchronize()
    x2, xg2 = _unprepare(d_op2.to_numpy(np.uint8, (d_op2.nbytes,)), rows, inter)
    assert np.array_equal(x2, x) and np.array_equal(xg2, xg)


def _untall(buf, rows, k, pairs):
    """operand of the many-row GEMM -> (bf16 bits [rows_pad][k], group sums [rows_pad][k/128])"""
    rows_pad = -(-rows // 128) * 128
    xp = buf[: rows_pad * k * 2].view(np.uint16).reshape(rows_pad, k // 8, 8)
    nat = np.empty_like(xp)
    nat[..., [0, 4, 1, 5, 2, 6, 3, 7]] = xp
    at = (rows_pad * k * 2 + 255) // 256 * 256
    groups, bl = k // 128, 2 * pairs
    xs = buf[at: at + rows_pad * groups * 4].view(np.float32).reshape(
        rows_pad // 128, groups // bl, 2, 128, pairs)
    # [row tile][block][place in pair][row][pair] -> [row][group = block * bl + 2 * pair + place]
    sums = xs.transpose(0, 3, 1, 4, 2).reshape(rows_pad, groups)
    return nat.reshape(rows_pad, k), sums


@pytest.mark.parametrize("rows,n,pairs", [(32, 4096, 4), (150, 1536, 2), (130, 768, 1),
                                          (20, 2048, 1)])
def test_add_rms_norm_written_as_the_many_row_gemms_operand(rows, n, pairs):
    # the same kernel as the prepared-layout producer of the decode chunks, storing into the
    # tiled GEMM's workspace: x in pair order row by row, padding rows zero, group sums in the
    # kernel's block order (for every number of pairs per block the GEMM may ask for).  Up to
    # 32 rows the chunk producer runs beside it: same h, same bits, same sums.
    rng = np.random.default_rng(rows + n)
    j = 3
    h = rng.standard_normal((rows, n), np.float32)
    parts = rng.standard_normal((j, rows, n), np.float32)
    w = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
    dev = hip.DeviceBuffer.from_numpy
    d_w, d_parts, d_h = dev(w), dev(parts), dev(h)
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(rows, n))
    ws.fill(0xFF)
    kernels.launch_add_rms_norm_f32p_tall(d_h, d_parts, j, d_w, ws, rows, n, 1e-6, pairs)
    hip.synchronize()
    x, sums = _untall(ws.to_numpy(np.uint8, (ws.nbytes,)), rows, n, pairs)
    assert not x[rows:].any() and not sums[rows:].any()
    h_want = h.copy()
    want = OS.add_rms_norm_bf16(h_want, parts[0] + parts[1] + parts[2], w, 1e-6)
    assert_parity(d_h.to_numpy(np.float32, (rows, n)), h_want, max_abs=1e-5, max_rel=1e-5,
                  what="h")
    assert_parity(O.bf16_bits_to_f32(x[:rows]), O.bf16_bits_to_f32(want), max_abs=1e-6,
                  max_rel=8e-3, what="normed rows")
    assert np.abs(sums[:rows] -
                  O.bf16_bits_to_f32(x[:rows]).reshape(rows, n // 128, 128).sum(axis=2)).max() < 1e-3
    if rows <= 32:
        d_h2 = dev(h)
        d_prep = hip.DeviceBuffer(kernels.q4_xprep_bytes(rows, n))
        kernels.launch_add_rms_norm_f32p_xprep(d_h2, d_parts, j, d_w, d_prep, rows, n, 1e-6)
        hip.synchronize()
        x2, xg2 = _unprepare(d_prep.to_numpy(np.uint8, (d_prep.nbytes,)), rows, n)
        assert np.array_equal(x[:rows], x2) and np.array_equal(sums[:rows], xg2)
        assert np.array_equal(d_h.to_numpy(np.float32, (rows, n)),
                              d_h2.to_numpy(np.float32, (rows, n)))
