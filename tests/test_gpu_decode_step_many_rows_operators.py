"""The many-row form of the step (97 packed rows or more: a mixed chunked-prefill + decode
batch) operator by operator, through the C ABI.

As for the decode batch of the full-step workload, every GPU operator this form launches is
fed the CPU oracle's input for that operator (the `trace=` hook of oracle/decode_step.py) and
held to the decode path's tolerance, 2e-3 absolute or 1e-2 relative: the add + RMSNorm over all
rows with a bf16 result, the tiled Q4G128 GEMM over a workspace with its fp32 product (q/k/v
with a bias, o, gate/up, down), RoPE + K/V append from one fp32 part, the ragged attention
over decode rows and chunks, SiLU * up.  The whole step is then judged by its relative L2
error, which per-operator agreement of this kind bounds.
"""
import copy

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from logismos_amd import hip, kernels
from tests import workloads
from tests.gpu_harness import DecodeStepRunner, assert_parity

pytestmark = pytest.mark.gpu

HIDDEN, HQ, HKV, D, INTER = 1024, 8, 2, 128, 2048
CTX, NEW = [700, 140, 3, 33, 37], [1, 100, 3, 1, 37]
T = sum(NEW)

up = hip.DeviceBuffer.from_numpy


class _Case:
    pass


@pytest.fixture(scope="module")
def case():
    c = _Case()
    rng = np.random.default_rng(45)
    c.cfg, c.layers, c.batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=HIDDEN, hq=HQ, hkv=HKV, inter=INTER, ctx=CTX, new_tokens=NEW,
        qkv_bias=True)
    assert c.batch["h"].shape[0] == T == 142
    c.lay = copy.deepcopy(c.layers)
    c.bat = dict(c.batch, h=c.batch["h"].copy())
    c.trace = []
    c.out = OS.decode_step(c.cfg, c.lay, c.bat, trace=c.trace)
    c.t = c.trace[0]
    return c


def _gemm(x_bits, w, bias=None):
    qw, s, z = w
    n, k = qw.shape[0], qw.shape[1] * 2
    ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(T, k))
    ws.fill(0xFF)
    d_y = hip.DeviceBuffer(T * n * 4)
    d_y.fill(0xFF)
    kernels.launch_qgemm_q4g128_tall(
        up(np.ascontiguousarray(x_bits, np.uint16)), up(qw), up(s.view(np.uint16)),
        up(z.view(np.uint16)), d_y, ws, T, n, k, bias=up(bias) if bias is not None else None,
        f32_out=True)
    hip.synchronize()
    return d_y.to_numpy(np.float32, (T, n))


def test_norm1_over_all_rows(case):
    h = case.batch["h"]
    d_h, d_out = up(h), hip.DeviceBuffer(T * HIDDEN * 2)
    kernels.launch_add_rms_norm_f32p(d_h, None, 0, up(case.layers[0]["norm1"]), d_out, T, HIDDEN,
                                     case.cfg["eps"])
    hip.synchronize()
    assert np.array_equal(d_h.to_numpy(np.float32, h.shape), h)
    assert_parity(O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (T, HIDDEN))),
                  O.bf16_bits_to_f32(case.t["xn"]), what="norm1")


@pytest.mark.parametrize("name,src,dst", [("qkv", "xn", "qkv"), ("gate_up", "xn2", "gu"),
                                          ("down", "act", "down")])
def test_projection(case, name, src, dst):
    bias = case.layers[0]["qkv_bias"] if name == "qkv" else None
    assert_parity(_gemm(case.t[src], case.layers[0][name], bias), case.t[dst],
                  what=f"{name} projection, {T} rows")


def test_o_projection(case):
    x = O.f32_to_bf16_bits(case.t["attn"].reshape(T, HQ * D))
    assert_parity(_gemm(x, case.layers[0]["o"]), case.t["o"], what="o projection")


def test_rope_and_kv_append_from_one_part(case):
    b, L0 = case.batch, case.layers[0]
    max_pos = b["cos"].size // (D // 2)
    d_kp, d_vp = up(L0["k_pool"]), up(L0["v_pool"])
    d_q = hip.DeviceBuffer(T * HQ * D * 2)
    kernels.launch_rope_kv_write_f32p(
        up(case.t["qkv"]), 1, up(np.ascontiguousarray(b["positions"], np.int32)), up(b["cos"]),
        up(b["sin"]), up(np.ascontiguousarray(b["slots"], np.int64)), d_q, d_kp, d_vp, T, HQ, HKV,
        D, max_pos)
    hip.synchronize()
    assert_parity(d_q.to_numpy(np.float16, (T, HQ, D)), case.t["q"], max_abs=1e-3, max_rel=2e-3,
                  what="roped q")
    slots = np.asarray(b["slots"])
    kp = d_kp.to_numpy(np.float16, L0["k_pool"].shape)
    vp = d_vp.to_numpy(np.float16, L0["v_pool"].shape)
    assert_parity(kp[slots], case.lay[0]["k_pool"][slots], max_abs=1e-3, max_rel=2e-3,
                  what="appended K rows")
    assert np.array_equal(vp[slots].view(np.uint16), case.lay[0]["v_pool"][slots].view(np.uint16))
    rest = np.ones(kp.shape[0], bool)
    rest[slots] = False
    assert np.array_equal(kp[rest].view(np.uint16), L0["k_pool"][rest].view(np.uint16))
    assert np.array_equal(vp[rest].view(np.uint16), L0["v_pool"][rest].view(np.uint16))


def test_ragged_attention_over_decode_rows_and_chunks(case):
    b = case.batch
    nseq = len(CTX)
    max_blocks = b["block_tables"].shape[1]
    ns = kernels.paged_attn_num_splits(nseq, HKV, case.cfg["block_size"], max_blocks)
    d_ws = hip.DeviceBuffer(max(16, kernels.paged_attn_workspace_bytes(nseq, HQ, D, ns)))
    d_out = hip.DeviceBuffer(T * HQ * D * 2)
    kernels.launch_paged_attn_varlen_fp16(
        up(case.t["q"]), up(case.lay[0]["k_pool"]), up(case.lay[0]["v_pool"]),
        up(b["block_tables"]), up(np.ascontiguousarray(b["cu_seqlens"], np.int32)),
        up(np.ascontiguousarray(b["context_lens"], np.int32)), d_out, d_ws, nseq, T, max(NEW), HQ,
        HKV, D, case.cfg["block_size"], max_blocks, ns, 1.0 / np.sqrt(float(D)))
    hip.synchronize()
    assert_parity(d_out.to_numpy(np.float16, (T, HQ * D)), case.t["attn"].reshape(T, HQ * D),
                  what="ragged attention")


def test_residual_add_and_norm2(case):
    h0 = case.batch["h"]
    d_h, d_out = up(h0), hip.DeviceBuffer(T * HIDDEN * 2)
    kernels.launch_add_rms_norm_f32p(d_h, up(case.t["o"]), 1, up(case.layers[0]["norm2"]), d_out,
                                     T, HIDDEN, case.cfg["eps"])
    hip.synchronize()
    assert np.array_equal(d_h.to_numpy(np.float32, h0.shape), case.t["h"])  # one fp32 add
    assert_parity(O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (T, HIDDEN))),
                  O.bf16_bits_to_f32(case.t["xn2"]), what="norm2")


def test_silu_mul(case):
    d_out = hip.DeviceBuffer(T * INTER * 2)
    kernels.launch_silu_mul_f32p(up(case.t["gu"]), 1, d_out, T, INTER)
    hip.synchronize()
    assert_parity(O.bf16_bits_to_f32(d_out.to_numpy(np.uint16, (T, INTER))),
                  O.bf16_bits_to_f32(case.t["act"]), what="silu * up")


def test_whole_step_over_many_rows(case):
    r = DecodeStepRunner(case.cfg, case.layers, case.batch)
    r.launch()
    got = O.bf16_bits_to_f32(r.result_bits())
    want = O.bf16_bits_to_f32(case.out)
    rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    assert rel < 4e-3, rel
    assert np.all(np.abs(got - want) <= 1.2e-2 + 1.6e-2 * np.abs(want))
    h_gpu = r.h.to_numpy(np.float32, case.bat["h"].shape)
    assert float(np.linalg.norm(h_gpu - case.bat["h"]) / np.linalg.norm(case.bat["h"])) < 2e-3
