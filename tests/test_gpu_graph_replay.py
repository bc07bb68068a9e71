"""Captured HIP graphs of the launchers, replayed: every replay against the eager result.

The benchmark times replays of captured graphs and an executor that serves tokens would run
its step the same way, so what a replay computes is held to the eager launch here -- bit for
bit, the kernels being deterministic.  A graph is replayed several times with the program's
own eager work between the replays (inputs restored with copies, outputs poisoned with fills,
another launch on the same stream, synchronisations): a node that only works the first time
shows on the second.  The library records kernel nodes only -- no launcher clears memory with
a memset.
"""
import numpy as np
import pytest

from logismos_amd import hip, kernels
from tests import workloads
from tests.gpu_harness import DecodeStepRunner, PagedAttnRunner

pytestmark = pytest.mark.gpu

REPLAYS = 3


def _step_state(r, layers):
    """Everything a step leaves behind: the bf16 output, the residual stream, the pools."""
    out = r.result_bits().copy()
    h = r.h.to_numpy(np.float32, (r.b, r.cfg_d["hidden"]))
    pools = []
    for (kp, vp), L in zip(r.pools, layers):
        dt = np.uint8 if r.cfg_d.get("kv_turbo3") else np.uint16
        pools.append((kp.to_numpy(dt, (kp.nbytes // np.dtype(dt).itemsize,)),
                      vp.to_numpy(dt, (vp.nbytes // np.dtype(dt).itemsize,))))
    toks = r.result_tokens() if r.vocab else None
    return out, h, pools, toks


def _restore(r, layers, batch):
    # the program's own eager work between replays: the step adds into h and appends to the
    # pools, so both are put back; the outputs are poisoned
    r.h.copy_from_host(batch["h"].astype(np.float32))
    for (kp, vp), L in zip(r.pools, layers):
        kp.copy_from_host(np.ascontiguousarray(L["k_pool"]))
        vp.copy_from_host(np.ascontiguousarray(L["v_pool"]))
    r.out.fill(0xFF)
    r.ws.fill(0xFF)
    if r.vocab:
        r.tokens.fill(0xFF)
        r.logits.fill(0xFF)


def _same_state(a, b, what):
    assert np.array_equal(a[0], b[0]), f"{what}: output"
    assert np.array_equal(a[1], b[1]), f"{what}: residual stream"
    for i, (pa, pb) in enumerate(zip(a[2], b[2])):
        assert np.array_equal(pa[0], pb[0]) and np.array_equal(pa[1], pb[1]), f"{what}: pools {i}"
    if a[3] is not None:
        assert np.array_equal(a[3][0], b[3][0]) and np.array_equal(a[3][1], b[3][1]), \
            f"{what}: tokens / logits"


STEPS = {
    # decode rows, 32-row chunks: register-x GEMMs, static split-K attention
    "decode": dict(num_layers=3, hidden=512, hq=4, hkv=2, inter=1024,
                   ctx=[1, 17, 300, 64, 999]),
    # token ids in, token ids out (embedding lookup, vocabulary projection with its choice)
    "tokens": dict(num_layers=2, hidden=1024, hq=8, hkv=2, inter=2048,
                   ctx=[1, 17, 300, 64, 999, 5], vocab=5003),
    # 142 packed rows: the tiled GEMMs with their workspace and split tiles, the prefill kernel
    "many_rows": dict(num_layers=2, hidden=512, hq=4, hkv=2, inter=1024,
                      ctx=[700, 140, 3, 33, 37], new_tokens=[1, 100, 3, 1, 37], qkv_bias=True),
    # TurboQuant-3 pools
    "turbo3": dict(num_layers=2, hidden=1024, hq=8, hkv=2, inter=2048,
                   ctx=[1, 17, 300, 64, 999, 5], kv_turbo3=True),
}


@pytest.mark.parametrize("kind", sorted(STEPS))
def test_replays_of_a_captured_step_equal_the_eager_step(kind):
    rng = np.random.default_rng({"decode": 11, "tokens": 12, "many_rows": 13, "turbo3": 14}[kind])
    cfg, layers, batch = workloads.decode_step_problem(rng, **STEPS[kind])
    stream = hip.Stream()
    eager = DecodeStepRunner(cfg, layers, batch, stream=stream)
    eager.launch()
    want = _step_state(eager, layers)

    r = DecodeStepRunner(cfg, layers, batch, stream=stream)
    g = hip.Graph(stream)
    with g:
        r.launch()
    stream.synchronize()
    # nothing ran during the capture
    assert np.all(r.out.to_numpy(np.uint16, (r.b, cfg["hidden"])) == 0xFFFF)
    for i in range(REPLAYS):
        _restore(r, layers, batch)
        # another eager launch on the same stream between the replays
        eager.h.copy_from_host(batch["h"].astype(np.float32))
        eager.launch()
        hip.synchronize()
        g.launch()
        _same_state(_step_state(r, layers), want, f"{kind}, replay {i}")


def _attn_cases():
    rng = np.random.default_rng(21)
    return {
        # balanced decode kernel + merge
        "balanced": workloads.paged_case(rng, np.ones(24, np.int32),
                                         rng.integers(300, 4000, size=24), hq=32, hkv=8,
                                         min_max_blocks=600),
        # static split, decode and chunk rows in one batch (prefill kernel + merge)
        "mixed": workloads.paged_case(rng, [1, 40, 1, 7, 1], [900, 31, 257, 40, 0], hq=12, hkv=2),
    }


@pytest.mark.parametrize("kind", ["balanced", "mixed"])
@pytest.mark.parametrize("noalloc", [False, True])
def test_replays_of_a_captured_attention_launch_equal_the_eager_launch(kind, noalloc):
    case = _attn_cases()[kind]
    stream = hip.Stream()
    eager = PagedAttnRunner(case, stream=stream)
    eager.launch()
    want = eager.result().view(np.uint16).copy()

    r = PagedAttnRunner(case, stream=stream)
    if noalloc:
        # the look-ups of the entry point that allocates nothing happen before the capture
        kernels.paged_attn_noalloc_init()
    g = hip.Graph(stream)
    with g:
        if noalloc:
            kernels.launch_paged_attn_varlen_fp16_noalloc(
                r.q, r.k_pool, r.v_pool, r.bt, r.cu, r.ctx, r.out, r.num_seqs, r.total_tokens,
                r.max_seqlen_q, case["hq"], case["hkv"], case["d"], case["block_size"],
                case["max_blocks"], r.num_splits, case["scale"], True, stream)
        else:
            r.launch()
    stream.synchronize()
    for i in range(REPLAYS):
        r.out.fill(0xFF)
        r.ws.fill(0xFF)
        eager.out.fill(0xFF)
        eager.launch()  # (with noalloc: not on the static array, which the replay then reuses)
        hip.synchronize()
        g.launch()
        got = r.result().view(np.uint16)
        assert np.array_equal(got, want), f"{kind}, noalloc={noalloc}, replay {i}"
