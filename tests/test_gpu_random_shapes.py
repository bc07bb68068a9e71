"""Seeded random shapes: the tiled Q4G128 GEMM with a workspace in every output mode, the
step executor at random geometries and the paged-attention launcher on random ragged batches,
against the CPU oracle through the C ABI.

The parametrised tests of the other files pick their shapes by hand (tile edges, split tiles,
alignment classes); these draw them, so that a combination nobody thought of is still seen:
rows around the 128-row tile and the 97-row switch of the executor, widths off every tile,
K from two groups to twenty-four, scales and zeros at 4-, 8- and 16-byte alignment, head
widths of 64, 96 and 128, grouped heads, a q/k/v bias, turbo3 pools, decode-only, few-row and
many-row batches.  Tolerances are those of the hand-picked tests.
"""
import copy
import ctypes as C

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from logismos_amd import hip, kernels
from tests import workloads
from tests.gpu_harness import DecodeStepRunner

pytestmark = pytest.mark.gpu

up = hip.DeviceBuffer.from_numpy


def _at_offset(a, mis):
    """Device copy of `a` starting `mis` bytes into its allocation (keeps the allocation)."""
    buf = hip.DeviceBuffer(a.nbytes + 16)
    hip.check(hip._runtime().hipMemcpy(buf.offset(mis), a.ctypes.data_as(C.c_void_p),
                                       C.c_size_t(a.nbytes), C.c_int(1)), "hipMemcpy(H2D)")
    return buf, buf.offset(mis)


def _out_of_tolerance(got, want, max_abs, max_rel):
    err = np.abs(got - want)
    rel = err / np.maximum(np.abs(want), 1e-3)
    return int(((err > max_abs) & (rel > max_rel)).sum())


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_workspace_gemm_random_shapes_and_modes(seed):
    rng = np.random.default_rng(seed)
    for case in range(24):
        k = int(rng.choice([256, 512, 768, 1024, 1536, 2048, 3072]))
        m = int(rng.choice([1, 5, 97, 128, 129, 255, 256, 257, 300, 383, 400]))
        mode = int(rng.integers(0, 4))  # bf16, fp32, SwiGLU, SwiGLU as the next operand
        if mode == 2:
            inter = int(rng.choice([128, 256, 384, 512, 640, 1024, 1280]))
        elif mode == 3:
            inter = int(rng.choice([256, 512, 768, 1024, 1280, 2048]))
        n = 2 * inter if mode >= 2 else int(rng.integers(1, 1500))
        w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
        qw, s, z = O.quantize_q4g128(w, n, k)
        xb = O.f32_to_bf16_bits(rng.standard_normal((m, k), np.float32))
        bias = rng.standard_normal(n).astype(np.float32) if mode < 2 and rng.integers(0, 2) else None
        mis = int(rng.choice([0, 0, 4, 8]))
        s_keep, sp = _at_offset(s, mis)
        z_keep, zp = _at_offset(z, mis)
        ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(m, k))
        ws.fill(0xFF)
        d_x, d_qw = up(xb), up(qw)
        what = f"seed {seed} case {case}: m={m} n={n} k={k} mode={mode} bias={bias is not None} mis={mis}"
        if mode < 2:
            d_y = hip.DeviceBuffer(m * n * (4 if mode == 1 else 2))
            d_y.fill(0xFF)
            kernels.launch_qgemm_q4g128_tall(d_x, d_qw, sp, zp, d_y, ws, m, n, k,
                                             bias=up(bias) if bias is not None else None,
                                             f32_out=mode == 1)
            hip.synchronize()
            want = O.qgemm_q4g128_f32(xb, qw, s, z, m, n, k, bias)
            if mode == 1:
                got, tol = d_y.to_numpy(np.float32, (m, n)), (2e-4, 1e-3)
            else:
                got, tol = O.bf16_bits_to_f32(d_y.to_numpy(np.uint16, (m, n))), (2e-3, 1e-2)
                want = O.bf16_bits_to_f32(O.f32_to_bf16_bits(want))
        else:
            # (the first pass over x, which the SwiGLU launches expect to have happened)
            kernels.launch_qgemm_q4g128_tall(d_x, d_qw, sp, zp, hip.DeviceBuffer(m * n * 4), ws, m,
                                             n, k, f32_out=True)
            gu = O.qgemm_q4g128_f32(xb, qw, s, z, m, n, k, None)
            want, tol = O.bf16_bits_to_f32(OS.silu_mul_bf16(gu, inter)), (2e-3, 1e-2)
            if mode == 2:
                d_a = hip.DeviceBuffer(m * inter * 2)
                d_a.fill(0xFF)
                kernels.launch_qgemm_q4g128_tall_swiglu_prepared(d_qw, sp, zp, d_a, ws, m, inter, k)
                hip.synchronize()
                got = O.bf16_bits_to_f32(d_a.to_numpy(np.uint16, (m, inter)))
            else:
                pairs = int(rng.choice([x for x in (1, 2, 4) if inter % (256 * x) == 0]))
                nxt = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(m, inter))
                nxt.fill(0xEE)
                kernels.launch_qgemm_q4g128_tall_swiglu_operand(d_qw, sp, zp, nxt, pairs, ws, m,
                                                                inter, k)
                hip.synchronize()
                m_pad = -(-m // 128) * 128
                chunks = nxt.to_numpy(np.uint16, (m_pad, inter // 8, 8))
                rows = np.empty_like(chunks)  # out of pair order: (x0,x4)(x1,x5)(x2,x6)(x3,x7)
                for j in range(8):
                    rows[:, :, j] = chunks[:, :, 2 * (j & 3) + (j >> 2)]
                rows = rows.reshape(m_pad, inter)
                assert not rows[m:].any(), what + ": padding rows"
                got = O.bf16_bits_to_f32(rows[:m])
        assert np.isfinite(got).all(), what
        assert _out_of_tolerance(got, want, *tol) == 0, what
        del s_keep, z_keep


@pytest.mark.parametrize("seed", [201, 202])
def test_step_executor_random_geometries(seed):
    rng0 = np.random.default_rng(seed)
    for case in range(20):
        d = int(rng0.choice([128, 128, 128, 64, 96]))
        hkv = int(rng0.choice([1, 2, 4]))
        hq = hkv * int(rng0.choice([1, 2, 4]))
        while (hq * d) % 128:  # the o projection's K in whole groups
            hq *= 2
        hidden = int(rng0.choice([256, 512, 768, 1024]))
        inter = int(rng0.choice([256, 384, 512, 640, 1024, 1280, 2048]))
        nseq = int(rng0.integers(1, 8))
        kind = int(rng0.integers(0, 3))  # decode rows only; a few rows per chunk; many rows
        if kind == 0:
            new = [1] * nseq
        elif kind == 1:
            new = [int(rng0.choice([1, 1, 3, 9, 20])) for _ in range(nseq)]
        else:
            new = [int(rng0.choice([1, 40, 70, 120, 200])) for _ in range(nseq)]
            if sum(new) < 97:
                new[0] = 130
        ctx = [n + int(rng0.integers(0, 600)) for n in new]
        t3 = bool(d == 128 and rng0.integers(0, 4) == 0)
        bias = bool(rng0.integers(0, 2))
        layers_n = int(rng0.integers(1, 3))
        what = (f"seed {seed} case {case}: d={d} hq={hq} hkv={hkv} hidden={hidden} inter={inter} "
                f"new={new} ctx={ctx} turbo3={t3} bias={bias} layers={layers_n}")
        rng = np.random.default_rng(seed * 1000 + case)
        cfg, layers, batch = workloads.decode_step_problem(
            rng, num_layers=layers_n, hidden=hidden, hq=hq, hkv=hkv, inter=inter, ctx=ctx, d=d,
            new_tokens=new, qkv_bias=bias, kv_turbo3=t3)
        r = DecodeStepRunner(cfg, layers, batch)
        r.launch()
        got = O.bf16_bits_to_f32(r.result_bits())
        lay = copy.deepcopy(layers)
        bat = dict(batch, h=batch["h"].copy())
        want = O.bf16_bits_to_f32(OS.decode_step(cfg, lay, bat))
        rel = float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-12))
        assert np.isfinite(got).all(), what
        # (the whole-step bounds of test_gpu_decode_step.py: 6e-3 over fp16 pools, wider over
        # turbo3 pools, whose encoder turns a last-bit difference of a row into another code)
        assert rel < (2.5e-2 if t3 else 6e-3), f"{what}: rel L2 {rel:.2e}"


@pytest.mark.parametrize("seed", [301, 302])
def test_paged_attention_random_ragged_batches(seed):
    # head widths 32..256, GQA groups 1..16, block sizes 16 / 32 / 64, decode rows, short and
    # long chunks, prior contexts on and around block edges, narrow block tables (static
    # split) and wide ones (balanced split), causal and not
    from tests.gpu_harness import PagedAttnRunner
    rng = np.random.default_rng(seed)
    for case in range(25):
        d = int(rng.choice([128, 128, 128, 32, 64, 96, 160, 256]))
        hkv = int(rng.choice([1, 2, 4, 8]))
        group = int(rng.integers(1, 9)) if d == 128 else int(rng.choice([1, 2, 3, 4, 7, 8, 16]))
        hq = hkv * group
        bs = int(rng.choice([16, 32, 64]))
        nseq = int(rng.integers(1, 20))
        kind = int(rng.integers(0, 3))
        if kind == 0:
            new = np.ones(nseq, np.int32)
        elif kind == 1:
            new = rng.choice([1, 1, 2, 5, 17, 40], size=nseq).astype(np.int32)
        else:
            new = rng.choice([1, 64, 100, 130], size=nseq).astype(np.int32)
        prior = rng.choice([0, 1, 15, 16, 17, 100, 500, 1500, 3000], size=nseq).astype(np.int32)
        wide = int(rng.choice([1, 1, 600]))
        causal = bool(rng.integers(0, 4) > 0)
        what = (f"seed {seed} case {case}: d={d} hq={hq} hkv={hkv} block={bs} new={new.tolist()} "
                f"prior={prior.tolist()} min_max_blocks={wide} causal={causal}")
        c = workloads.paged_case(rng, new, prior, hq, hkv, d, bs, min_max_blocks=wide)
        r = PagedAttnRunner(c, causal=causal)
        r.launch()
        got = r.result().astype(np.float32)
        want = O.paged_attn_varlen_fp16(c["q"], c["k_pool"], c["v_pool"], c["block_tables"],
                                        c["cu_seqlens"], c["context_lens"], hq, hkv, d, bs,
                                        c["scale"], causal).astype(np.float32)
        assert np.isfinite(got).all(), what
        assert _out_of_tolerance(got, want, 2e-3, 1e-2) == 0, what


@pytest.mark.parametrize("seed", [401, 402])
def test_small_batch_products_random_shapes(seed):
    # the Q8G32 GEMV and the Q4G128 product at any batch (the GEMV for 1-2 rows, the
    # matrix-core kernels in passes of 32 rows, a ragged last pass), N from 1 to thousands,
    # K from one group up and off the kernels' fast paths, with and without a bias
    rng = np.random.default_rng(seed)
    for case in range(40):
        n = int(rng.choice([1, 7, 16, 33, 100, 1000, 1024, 1536, 4096, 5000]))
        bias = rng.standard_normal(n).astype(np.float32) if rng.integers(0, 2) else None
        d_bias = up(bias) if bias is not None else None
        if rng.integers(0, 2):
            k = int(rng.choice([32, 64, 96, 512, 1536, 4096, 8192, 2080]))
            w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
            qs, d = O.quantize_q8g32(w, n, k)
            x = rng.standard_normal(k).astype(np.float32)
            what = f"seed {seed} case {case}: Q8G32 GEMV n={n} k={k} bias={bias is not None}"
            y = hip.DeviceBuffer(n * 4)
            y.fill(0xFF)
            kernels.launch_qgemv_q8g32_f32(up(x), up(qs), up(d.view(np.uint16)), y, n, k,
                                           bias=d_bias)
            hip.synchronize()
            got, tol = y.to_numpy(np.float32, (n,)), (2e-4, 1e-3)
            want = O.qgemv_q8g32_f32(x, qs, d, n, k, bias)
        else:
            k = int(rng.choice([128, 256, 384, 1024, 2048, 4096, 4224]))
            b = int(rng.choice([1, 2, 3, 4, 7, 8, 15, 16, 17, 31, 32, 33, 40, 64, 65, 70]))
            w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
            qw, s, z = O.quantize_q4g128(w, n, k)
            xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
            what = f"seed {seed} case {case}: Q4G128 b={b} n={n} k={k} bias={bias is not None}"
            y = hip.DeviceBuffer(b * n * 2)
            y.fill(0xFF)
            kernels.launch_qgemm_q4g128_bf16(up(xb), up(qw), up(s.view(np.uint16)),
                                             up(z.view(np.uint16)), y, b, n, k, bias=d_bias)
            hip.synchronize()
            got, tol = O.bf16_bits_to_f32(y.to_numpy(np.uint16, (b, n))), (2e-3, 1e-2)
            want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb, qw, s, z, b, n, k, bias))
        assert np.isfinite(got).all(), what
        assert _out_of_tolerance(got, want, *tol) == 0, what
