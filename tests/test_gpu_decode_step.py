"""GPU parity of the full decode step vs the CPU oracle step, through the C ABI."""
import copy

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from tests import workloads
from tests.gpu_harness import DecodeStepRunner, assert_parity

pytestmark = pytest.mark.gpu


def _run_both(cfg, layers, batch, num_splits=None):
    r = DecodeStepRunner(cfg, layers, batch, num_splits=num_splits)
    r.launch()
    got = O.bf16_bits_to_f32(r.result_bits())
    lay = copy.deepcopy(layers)
    bat = dict(batch, h=batch["h"].copy())
    want = O.bf16_bits_to_f32(OS.decode_step(cfg, lay, bat))
    return r, got, want, lay, bat


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def test_small_geometry_three_layers():
    rng = np.random.default_rng(31)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=3, hidden=512, hq=4, hkv=2, inter=1024, ctx=[1, 17, 300, 64, 999])
    r, got, want, lay, bat = _run_both(cfg, layers, batch)
    # bf16 roundings of intermediate GEMM outputs can differ by one ulp between the two
    # paths and propagate through the layers: judge the step as a whole by its relative L2
    # error, and every element by the fp16/bf16 tolerance widened for three layers
    assert _rel_l2(got, want) < 5e-3
    assert np.all(np.abs(got - want) <= 2e-2 + 3e-2 * np.abs(want))
    # the KV append is part of the step: pools on the device match the oracle's
    import numpy as _np
    for (kp, vp), L in zip(r.pools, lay):
        gk = kp.to_numpy(_np.float16, L["k_pool"].shape).astype(_np.float32)
        assert_parity(gk, L["k_pool"].astype(_np.float32), max_abs=4e-3, max_rel=1e-2,
                      what="appended K rows")
    # the residual stream after the step
    h_gpu = r.h.to_numpy(np.float32, bat["h"].shape)
    assert _rel_l2(h_gpu, bat["h"]) < 5e-3


def test_single_layer_qwen3_8b_geometry_32_sequences():
    rng = np.random.default_rng(32)
    ctx = rng.integers(16, 600, size=32)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=4096, hq=32, hkv=8, inter=12288, ctx=ctx)
    _, got, want, _, _ = _run_both(cfg, layers, batch)
    assert _rel_l2(got, want) < 6e-3  # one-ulp bf16 differences of intermediates, compounded
    # element-wise: outputs are bf16 (ulp 2^-8 relative) of values up to ~4; allow two ulps
    assert np.all(np.abs(got - want) <= 1.5e-2 + 2e-2 * np.abs(want))


def test_step_is_deterministic_and_split_invariant():
    rng = np.random.default_rng(33)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=512, hq=4, hkv=2, inter=1024, ctx=[700, 33, 2000])
    _, a, want, _, _ = _run_both(cfg, layers, batch, num_splits=1)
    _, b, _, _, _ = _run_both(cfg, layers, batch, num_splits=1)
    _, c, _, _, _ = _run_both(cfg, layers, batch, num_splits=8)
    assert np.array_equal(a, b)
    assert _rel_l2(c, a) < 5e-3


def test_tokens_in_tokens_out():
    # embedding lookup in front, vocabulary projection + greedy behind: token ids to token ids
    rng = np.random.default_rng(34)
    vocab = 5003
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=1024, hq=8, hkv=2, inter=2048, ctx=[1, 17, 300, 64, 999, 5],
        vocab=vocab)
    batch["token_ids"][3] = vocab  # outside the vocabulary: a zero embedding row
    r, got, want, lay, bat = _run_both(cfg, layers, batch)
    assert _rel_l2(got, want) < 5e-3
    tokens, logits = r.result_tokens()
    assert np.isfinite(logits).all()
    assert _rel_l2(logits, bat["logits"]) < 6e-3
    # the selection rule exactly, on the logits the step stored
    assert np.array_equal(tokens, np.array([O.greedy(x) for x in logits], np.uint32))
    # and the oracle's token wherever its winner is clear of the logit error
    err = float(np.abs(logits - bat["logits"]).max())
    top2 = np.sort(bat["logits"], axis=1)[:, -2:]
    clear = (top2[:, 1] - top2[:, 0]) > 4 * err
    assert clear.any()
    assert np.array_equal(tokens[clear], bat["tokens"][clear])
    h_gpu = r.h.to_numpy(np.float32, bat["h"].shape)
    assert _rel_l2(h_gpu, bat["h"]) < 5e-3


def test_tokens_out_without_the_bf16_state_or_logits():
    rng = np.random.default_rng(35)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=1024, hq=8, hkv=2, inter=2048, ctx=[40, 7, 129], vocab=3000)
    full = DecodeStepRunner(cfg, layers, batch)
    full.launch()
    want, _ = full.result_tokens()
    lean = DecodeStepRunner(cfg, layers, batch)
    lean.batch.out_bf16 = None
    lean.batch.logits_f32 = None
    lean.launch()
    got, _ = lean.result_tokens()
    assert np.array_equal(got, want)


def test_step_over_turbo3_pools():
    # TurboQuant 3-bit KV: new rows encoded as they are written, attention decoding in its
    # gather; everything else as the fp16 step
    rng = np.random.default_rng(36)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=1024, hq=8, hkv=2, inter=2048, ctx=[1, 17, 300, 64, 999, 5],
        kv_turbo3=True)
    r, got, want, lay, bat = _run_both(cfg, layers, batch)
    # The encoder is a quantiser: a one-ulp difference in a new K/V row between the two paths
    # can move a 3-bit index to the neighbouring centroid, which a one-token context (row 0:
    # its output IS the decoded new V row) shows undamped.  Hence the wider bounds than for
    # the fp16 step; the first layer's appended rows are compared byte for byte below.
    assert _rel_l2(got, want) < 1e-2
    assert np.all(np.abs(got - want) <= 5e-2 + 3e-2 * np.abs(want))
    # the encoded rows the step appended: integer work, compared byte for byte wherever the
    # fp16 row that went into the encoder was the same on both sides (first layer: its input
    # does not depend on earlier GPU arithmetic beyond one GEMM; count the agreeing rows)
    kp, vp = r.pools[0]
    gk = kp.to_numpy(np.uint8, lay[0]["k_pool"].shape)
    gv = vp.to_numpy(np.uint8, lay[0]["v_pool"].shape)
    slots = np.asarray(batch["slots"])
    untouched = np.setdiff1d(np.arange(gk.shape[0]), slots)
    assert np.array_equal(gk[untouched], layers[0]["k_pool"][untouched])
    assert np.array_equal(gv[untouched], layers[0]["v_pool"][untouched])
    same = sum(np.array_equal(gk[s], lay[0]["k_pool"][s]) for s in slots)
    assert same >= len(slots) // 2, same
    # norms (fp16, first two bytes of every 14-byte block) agree to an fp16 ulp everywhere
    def norms(p):
        return p.reshape(p.shape[0], -1, 14)[:, :, :2].copy().view(np.float16).astype(np.float32)
    assert_parity(norms(gk[slots]), norms(lay[0]["k_pool"][slots]), max_abs=1e-3, max_rel=2e-3,
                  what="turbo3 K norms")
    assert_parity(norms(gv[slots]), norms(lay[0]["v_pool"][slots]), max_abs=1e-3, max_rel=2e-3,
                  what="turbo3 V norms")
