"""Tokens out of a step for the LAST packed row of every sequence (`tokens_for_last_rows`),
through the C ABI: the form a mixed chunked-prefill + decode batch of any size needs (a
sequence's next token is the choice at its last row; `decode::greedy`,
crates/decode/src/lib.rs:73-83, applied to that row's logits), where the per-row form is
limited to 32 packed rows.
"""
import copy

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from logismos_amd import kernels
from tests import workloads
from tests.gpu_harness import DecodeStepRunner

pytestmark = pytest.mark.gpu


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _oracle(cfg, layers, batch):
    lay = copy.deepcopy(layers)
    bat = dict(batch, h=batch["h"].copy())
    out = OS.decode_step(cfg, lay, bat)
    return O.bf16_bits_to_f32(out), bat["logits"], bat["tokens"]


def _last_rows(r, nseq, vocab):
    r.launch()
    tok, logits = r.result_tokens()          # (the runner sizes its buffers for every row)
    return tok[:nseq].copy(), logits.reshape(-1)[: nseq * vocab].reshape(nseq, vocab).copy()


def _check_against_oracle(tok, logits, want_logits, want_tok, last, what):
    assert _rel_l2(logits, want_logits[last]) < 6e-3, what
    # the selection rule exactly, on the logits the step stored ...
    assert np.array_equal(tok, np.array([O.greedy(x) for x in logits], np.uint32)), what
    # ... and the oracle's token wherever its winner is clear of the logit error
    err = float(np.abs(logits - want_logits[last]).max())
    top2 = np.sort(want_logits[last], axis=1)[:, -2:]
    clear = (top2[:, 1] - top2[:, 0]) > 4 * err
    assert clear.sum() >= len(tok) // 2, what
    assert np.array_equal(tok[clear], want_tok[last][clear]), what


def test_last_rows_of_a_small_mixed_batch_equal_the_per_row_choice():
    rng = np.random.default_rng(61)
    ctx, new = [40, 7, 129, 20], [1, 7, 1, 12]
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=2, hidden=1024, hq=8, hkv=2, inter=2048, ctx=ctx, new_tokens=new,
        vocab=3000)
    last = np.cumsum(new) - 1
    every = DecodeStepRunner(cfg, layers, batch)
    every.launch()
    tok_all, logits_all = every.result_tokens()
    r = DecodeStepRunner(cfg, layers, batch)
    r.batch.tokens_for_last_rows = 1
    tok, logits = _last_rows(r, len(ctx), 3000)
    assert np.array_equal(tok, tok_all[last])
    # same bf16 rows into the same projection: the logits agree to the last bits
    assert np.allclose(logits, logits_all[last], rtol=1e-5, atol=1e-5)
    # the rows behind the sequences' in the token buffer were left alone
    assert (r.tokens.to_numpy(np.uint32, (sum(new),))[len(ctx):] == 0xFFFFFFFF).all()
    assert np.array_equal(r.result_bits(), every.result_bits())


def test_many_rows_with_tokens_for_the_last_rows():
    # 142 packed rows: the projections on the tiled GEMM, tokens for five sequences
    rng = np.random.default_rng(62)
    ctx, new = [700, 140, 3, 33, 37], [1, 100, 3, 1, 37]
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=1024, hq=8, hkv=2, inter=2048, ctx=ctx, new_tokens=new,
        vocab=3000)
    want_out, want_logits, want_tok = _oracle(cfg, layers, batch)
    last = np.cumsum(new) - 1
    r = DecodeStepRunner(cfg, layers, batch)
    r.batch.tokens_for_last_rows = 1
    tok, logits = _last_rows(r, len(ctx), 3000)
    _check_against_oracle(tok, logits, want_logits, want_tok, last, "142 rows")
    got = O.bf16_bits_to_f32(r.result_bits())
    assert _rel_l2(got, want_out) < 5e-3
    # without a buffer for the normed rows of the whole batch: the same tokens
    lean = DecodeStepRunner(cfg, layers, batch)
    lean.batch.tokens_for_last_rows = 1
    lean.batch.out_bf16 = None
    tok2, logits2 = _last_rows(lean, len(ctx), 3000)
    assert np.array_equal(tok2, tok) and np.array_equal(logits2, logits)


def test_more_sequences_than_one_chunk_of_the_vocabulary_projection():
    # 40 sequences, 45 packed rows: the layers 32 rows at a time, the last rows 32 + 8
    rng = np.random.default_rng(63)
    nseq = 40
    ctx = [int(x) for x in rng.integers(1, 90, size=nseq)]
    new = [1] * nseq
    new[5], new[33] = 4, 3
    ctx[5], ctx[33] = max(ctx[5], 4), max(ctx[33], 3)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=1024, hq=4, hkv=2, inter=1024, ctx=ctx, new_tokens=new,
        vocab=2000)
    want_out, want_logits, want_tok = _oracle(cfg, layers, batch)
    last = np.cumsum(new) - 1
    r = DecodeStepRunner(cfg, layers, batch)
    r.batch.tokens_for_last_rows = 1
    r.batch.out_bf16 = None
    tok, logits = _last_rows(r, nseq, 2000)
    _check_against_oracle(tok, logits, want_logits, want_tok, last, "40 sequences")


def test_a_token_for_every_row_of_more_than_32_rows_stays_refused():
    rng = np.random.default_rng(64)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=1024, hq=4, hkv=2, inter=1024, ctx=[50, 9], new_tokens=[40, 1],
        vocab=2000)
    r = DecodeStepRunner(cfg, layers, batch)
    with pytest.raises(kernels.LaunchError):
        r.launch()
    r.batch.tokens_for_last_rows = 1
    r.launch()
    tok, _ = r.result_tokens()
    assert (tok[:2] < 2000).all()
