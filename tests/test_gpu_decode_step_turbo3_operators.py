"""The operators that differ when a step runs over TurboQuant 3-bit pools, each fed the CPU
oracle's input for it (the `trace=` hook of oracle/decode_step.py), through the C ABI.

The end-to-end comparison of such a step has to allow for the quantiser: a one-ulp difference
in a new K/V row between the two paths can move a 3-bit index to the neighbouring centroid.
Fed the same input, the operators themselves have no such freedom:

* RoPE + K/V encode from the oracle's fp32 projection: the roped queries to the decode path's
  tolerance; the encoded rows byte for byte against the reference encoder applied to the fp16
  rows the same kernel writes into fp16 pools (V is not rotated, so there it is also byte for
  byte against the oracle's own pool);
* attention over the oracle's turbo3 pools with the oracle's queries: 2e-3 absolute or 1e-2
  relative, like the attention over fp16 pools.
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
CTX = [1, 17, 300, 64, 999, 5]
T = len(CTX)

up = hip.DeviceBuffer.from_numpy


class _Case:
    pass


@pytest.fixture(scope="module")
def case():
    c = _Case()
    rng = np.random.default_rng(46)
    c.cfg, c.layers, c.batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=HIDDEN, hq=HQ, hkv=HKV, inter=INTER, ctx=CTX, kv_turbo3=True)
    c.lay = copy.deepcopy(c.layers)
    c.bat = dict(c.batch, h=c.batch["h"].copy())
    c.trace = []
    c.out = OS.decode_step(c.cfg, c.lay, c.bat, trace=c.trace)
    c.t = c.trace[0]
    return c


def test_rope_and_encode_from_the_oracles_projection(case):
    b, L0 = case.batch, case.layers[0]
    max_pos = b["cos"].size // (D // 2)
    slots = np.asarray(b["slots"])
    common = (up(np.ascontiguousarray(b["positions"], np.int32)), up(b["cos"]), up(b["sin"]),
              up(np.ascontiguousarray(slots, np.int64)))
    # the same kernel into fp16 pools: the rows the encoder sees
    rows = L0["k_pool"].shape[0]
    d_k16, d_v16 = hip.DeviceBuffer(rows * HKV * D * 2), hip.DeviceBuffer(rows * HKV * D * 2)
    d_k16.fill(0)
    d_v16.fill(0)
    d_q16 = hip.DeviceBuffer(T * HQ * D * 2)
    kernels.launch_rope_kv_write_f32p(up(case.t["qkv"]), 1, *common, d_q16, d_k16, d_v16, T, HQ,
                                      HKV, D, max_pos)
    d_k3, d_v3 = up(L0["k_pool"]), up(L0["v_pool"])
    d_q = hip.DeviceBuffer(T * HQ * D * 2)
    kernels.launch_rope_kv_write_f32p(up(case.t["qkv"]), 1, *common, d_q, d_k3, d_v3, T, HQ, HKV,
                                      D, max_pos, turbo3=True)
    hip.synchronize()
    q = d_q.to_numpy(np.float16, (T, HQ, D))
    assert np.array_equal(q.view(np.uint16), d_q16.to_numpy(np.uint16, (T, HQ, D)))
    assert_parity(q, case.t["q"], max_abs=1e-3, max_rel=2e-3, what="roped q")
    k16 = d_k16.to_numpy(np.float16, (rows, HKV * D))
    v16 = d_v16.to_numpy(np.float16, (rows, HKV * D))
    k3_want, v3_want = L0["k_pool"].copy(), L0["v_pool"].copy()
    O.kv_write_turbo3(k16[slots], v16[slots], k3_want, v3_want, slots, HKV)
    gk = d_k3.to_numpy(np.uint8, L0["k_pool"].shape)
    gv = d_v3.to_numpy(np.uint8, L0["v_pool"].shape)
    assert np.array_equal(gk, k3_want)  # appended rows and everything else
    assert np.array_equal(gv, v3_want)
    # V is cast, not rotated: identical to the oracle's pool as well
    assert np.array_equal(gv, case.lay[0]["v_pool"])
    # K: the rotation is fp32 on both sides; where the fp16 rows agree, so do the bytes
    same = sum(np.array_equal(gk[s], case.lay[0]["k_pool"][s]) for s in slots)
    assert same >= len(slots) // 2, same


def test_attention_over_the_oracles_turbo3_pools(case):
    b = case.batch
    nseq = len(CTX)
    max_blocks = b["block_tables"].shape[1]
    ns = kernels.paged_attn_num_splits(nseq, HKV, case.cfg["block_size"], max_blocks)
    d_ws = hip.DeviceBuffer(max(16, kernels.paged_attn_workspace_bytes(nseq, HQ, D, ns)))
    d_out = hip.DeviceBuffer(T * HQ * D * 2)
    kernels.launch_paged_attn_varlen_turbo3(
        up(case.t["q"]), up(case.lay[0]["k_pool"]), up(case.lay[0]["v_pool"]),
        up(b["block_tables"]), up(np.ascontiguousarray(b["cu_seqlens"], np.int32)),
        up(np.ascontiguousarray(b["context_lens"], np.int32)), d_out, d_ws, nseq, T, 1, HQ, HKV,
        case.cfg["block_size"], max_blocks, ns, 1.0 / np.sqrt(float(D)))
    hip.synchronize()
    assert_parity(d_out.to_numpy(np.float16, (T, HQ * D)), case.t["attn"].reshape(T, HQ * D),
                  what="attention over turbo3 pools")


def test_whole_step_over_turbo3_pools(case):
    r = DecodeStepRunner(case.cfg, case.layers, case.batch)
    r.launch()
    got = O.bf16_bits_to_f32(r.result_bits())
    want = O.bf16_bits_to_f32(case.out)
    rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    assert rel < 1e-2, rel
