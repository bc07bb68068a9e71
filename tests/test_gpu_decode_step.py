"""GPU parity of the full decode step vs the CPU oracle step, through the C ABI."""
import copy

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from tests import workloads
from logismos_amd import hip, kernels
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


def _check_step(cfg, layers, batch, what, layers_n):
    r, got, want, lay, bat = _run_both(cfg, layers, batch)
    assert _rel_l2(got, want) < 5e-3, what
    assert np.all(np.abs(got - want) <= 2e-2 + 3e-2 * np.abs(want)), what
    h_gpu = r.h.to_numpy(np.float32, bat["h"].shape)
    assert _rel_l2(h_gpu, bat["h"]) < 5e-3, what
    slots = np.asarray(batch["slots"])
    for (kp, vp), L in zip(r.pools, lay):
        gk = kp.to_numpy(np.float16, L["k_pool"].shape)
        assert_parity(gk[slots], L["k_pool"][slots], max_abs=4e-3, max_rel=1e-2,
                      what=f"{what}: appended K rows")
        rest = np.ones(gk.shape[0], bool)
        rest[slots] = False
        assert np.array_equal(gk[rest].view(np.uint16), L["k_pool"][rest].view(np.uint16))
    return r


def test_mixed_batch_in_one_chunk_with_qkv_bias():
    # a decode row, a 7-token chunk with prior context, a whole 3-token prompt, a 5-token
    # chunk: 16 packed rows, causal inside each chunk; the q/k/v projections carry a bias
    rng = np.random.default_rng(37)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=512, hq=4, hkv=2, inter=1024, ctx=[90, 400, 3, 21],
        new_tokens=[1, 7, 3, 5], qkv_bias=True)
    _check_step(cfg, layers, batch, "mixed batch, one chunk", 2)


def test_mixed_batch_over_several_chunks_of_rows():
    # 1 + 40 + 3 + 1 + 37 = 82 packed rows: three passes of 32, 32 and 18 rows through the
    # projections, one attention launch over the ragged batch per layer
    rng = np.random.default_rng(38)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=512, hq=4, hkv=2, inter=1024, ctx=[700, 140, 3, 33, 37],
        new_tokens=[1, 40, 3, 1, 37], qkv_bias=True)
    assert batch["h"].shape[0] == 82
    _check_step(cfg, layers, batch, "mixed batch, three chunks", 2)


def test_mixed_batch_with_many_rows_on_the_tiled_gemm():
    # 1 + 100 + 3 + 1 + 37 = 142 packed rows: from 97 rows on every projection is one launch of
    # the tiled GEMM over all rows; two layers, q/k/v bias, a ragged last tile (142 = 128 + 14)
    rng = np.random.default_rng(42)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=512, hq=4, hkv=2, inter=1024, ctx=[700, 140, 3, 33, 37],
        new_tokens=[1, 100, 3, 1, 37], qkv_bias=True)
    assert batch["h"].shape[0] == 142
    _check_step(cfg, layers, batch, "mixed batch, tiled GEMM", 2)


def test_many_rows_at_head_dim_96_with_a_projection_width_off_the_tile():
    # the tiled-GEMM path (97 rows or more) at another head width: 4 query / 1 KV head of 96,
    # so the q/k/v projection is 576 columns wide -- four and a half 128-column tiles, the
    # last one half empty -- and the attention runs on the general kernel
    rng = np.random.default_rng(43)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=512, hq=4, hkv=1, inter=1024, ctx=[700, 140, 3, 33, 37],
        new_tokens=[1, 100, 3, 1, 37], d=96, qkv_bias=True)
    assert batch["h"].shape[0] == 142 and ((4 + 2) * 96) % 128 != 0
    _check_step(cfg, layers, batch, "142 rows, head_dim 96, width 576", 2)


def test_many_rows_over_turbo3_pools():
    # the same path over TurboQuant 3-bit pools: the chunk's new rows are rotated, rounded and
    # encoded by one launch over all 142 rows, the prefill kernel decodes inside its gather
    rng = np.random.default_rng(44)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=1024, hq=8, hkv=2, inter=2048, ctx=[700, 140, 3, 33, 37],
        new_tokens=[1, 100, 3, 1, 37], kv_turbo3=True)
    assert batch["h"].shape[0] == 142
    r, got, want, lay, bat = _run_both(cfg, layers, batch)
    assert _rel_l2(got, want) < 1e-2
    assert np.all(np.abs(got - want) <= 5e-2 + 3e-2 * np.abs(want))
    # rows of the pools the step did not write are untouched (integer work, bit-exact)
    slots = np.asarray(batch["slots"])
    for (kp, vp), L0 in zip(r.pools, layers):
        gk = kp.to_numpy(np.uint8, L0["k_pool"].shape)
        gv = vp.to_numpy(np.uint8, L0["v_pool"].shape)
        rest = np.setdiff1d(np.arange(gk.shape[0]), slots)
        assert np.array_equal(gk[rest], L0["k_pool"][rest])
        assert np.array_equal(gv[rest], L0["v_pool"][rest])


def test_more_than_32_decode_sequences():
    rng = np.random.default_rng(39)
    ctx = rng.integers(1, 300, size=45)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=512, hq=4, hkv=2, inter=1024, ctx=ctx)
    _check_step(cfg, layers, batch, "45 decode sequences", 2)


def test_full_layer_mixed_batch_at_qwen3_8b_geometry():
    # one layer at config 5's geometry over a mixed batch: 6 decode rows and two prefill chunks
    # (130 and 64 tokens, prior contexts 200 and 0) = 200 packed rows, 7 passes of rows
    rng = np.random.default_rng(40)
    ctx = [300, 17, 1024, 330, 2000, 64, 5, 77]
    new = [1, 1, 1, 130, 1, 64, 1, 1]
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=4096, hq=32, hkv=8, inter=12288, ctx=ctx, new_tokens=new)
    assert batch["h"].shape[0] == 200
    r, got, want, lay, bat = _run_both(cfg, layers, batch)
    assert _rel_l2(got, want) < 4e-3
    assert np.all(np.abs(got - want) <= 1.2e-2 + 1.6e-2 * np.abs(want))


def test_step_at_qwen2_05b_geometry_head_dim_64():
    # Qwen2-0.5B's layer geometry: hidden 896, 14 query / 2 KV heads of 64, MLP 4864, q/k/v
    # biases (crates/transformers/src/attention.rs:49-57); decode rows only, two layers
    rng = np.random.default_rng(64)
    ctx = rng.integers(1, 700, size=12)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=896, hq=14, hkv=2, inter=4864, ctx=ctx, d=64, qkv_bias=True,
        theta=1e4)
    _check_step(cfg, layers, batch, "head_dim 64, decode rows", 2)


@pytest.mark.parametrize("d,hq,hkv,hidden", [(64, 8, 2, 512), (96, 4, 4, 384), (256, 2, 1, 512)])
def test_mixed_batch_at_other_head_dims(d, hq, hkv, hidden):
    # decode rows and chunks in one chunk of rows, then over three chunks of rows
    rng = np.random.default_rng(640 + d)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=hidden, hq=hq, hkv=hkv, inter=1024, ctx=[90, 400, 3, 21],
        new_tokens=[1, 7, 3, 5], d=d, qkv_bias=True)
    _check_step(cfg, layers, batch, f"head_dim {d}, one chunk", 2)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=hidden, hq=hq, hkv=hkv, inter=1024, ctx=[300, 40, 70, 9, 33],
        new_tokens=[1, 40, 30, 1, 8], d=d)
    _check_step(cfg, layers, batch, f"head_dim {d}, three chunks", 1)


def test_step_rejects_what_it_cannot_run():
    import ctypes as C
    rng = np.random.default_rng(41)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=512, hq=4, hkv=2, inter=1024, ctx=[5, 9])
    r = DecodeStepRunner(cfg, layers, batch)
    lib = kernels.library()
    call = lambda: lib.logismos_launch_decode_step(C.byref(r.cfg), r.layers, C.byref(r.batch),
                                                   r.ws.ptr, None)
    assert call() == 0
    # RoPE tables shorter than what the block tables can hold
    keep = r.cfg.max_pos
    r.cfg.max_pos = r.cfg.block_size * r.cfg.max_blocks_per_seq - 1
    assert call() == 1
    r.cfg.max_pos = keep
    # fewer packed rows than sequences, or a chunk longer than the batch
    r.batch.total_tokens, r.batch.max_seqlen_q = 1, 1
    assert call() == 1
    r.batch.total_tokens, r.batch.max_seqlen_q = 2, 3
    assert call() == 1
    r.batch.total_tokens, r.batch.max_seqlen_q = 0, 0
    assert call() == 0
    hip.synchronize()
    # head widths and GQA groups the attention launchers would refuse are refused up front
    keep = (r.cfg.head_dim, r.cfg.num_q_heads, r.cfg.kv_turbo3)
    for head_dim, hq_, t3 in ((80, 4, 0), (288, 4, 0), (64, 8, 1), (128, 18, 0), (64, 34, 0),
                              (128, 5, 0)):
        r.cfg.head_dim, r.cfg.num_q_heads, r.cfg.kv_turbo3 = head_dim, hq_, t3
        assert call() == 1, (head_dim, hq_, t3)
    r.cfg.head_dim, r.cfg.num_q_heads, r.cfg.kv_turbo3 = keep
    assert call() == 0
    hip.synchronize()
