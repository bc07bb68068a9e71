"""CPU pins of the decode-step oracle (oracle/decode_step.py): no GPU.

The step oracle composes restated reference functions; what it must follow is
  * the pre-norm residual order of `StellaLayer::forward`
    (crates/encoders/src/stella.rs:190-206): x += attn(norm1(x)); x += mlp(norm2(x)),
  * the SwiGLU order of `Mlp::forward` (crates/transformers/src/mlp.rs:82-125):
    down(silu(gate(x)) * up(x)),
  * RoPE (halves convention, by position) on q and k before the attention / the cache
    (crates/transformers/src/attention.rs:199-216), scores scaled by 1/sqrt(d) after the dot
    (:226-241), softmax over the visible keys, P.V, GQA head h reading kv head h / groups
    (:366-382), the o projection (:300-302).

Nothing below calls the oracle to produce an expectation.  `DenseStep` is a float64 dense
composition written from those reference lines with textbook numpy (dequantised weights,
contiguous K/V gathered by the slot formula, `softmax(q k^T / sqrt d) v`); with `rounding=True`
it stores intermediates in the types the step oracle documents (bf16 activations, fp16 q/K/V),
rounded by its own numpy code.  The special cases further down are exact statements a wrong
composition fails (a residual added after the norm, a RoPE position off by one, swapped
gate/up halves, a wrong slot, a wrong GQA map).
"""
import copy

import numpy as np
import pytest

import oracle as O
from oracle import decode_step as OS
from tests import workloads


# ------------------------------------------------------------------ independent numpy pieces
def bf16_round(x):
    """float64/float32 -> nearest-even bf16, returned as float64 values."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def bf16_bits(x):
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def f16_round(x):
    return np.asarray(x, np.float64).astype(np.float16).astype(np.float64)


def dequant_q4g128(t):
    """(qw, scale, zero) -> float64 [n, k]: low nibble first
    (crates/quant/src/lib.rs:272-285), w = (q - zero) * scale per 128-group."""
    qw, s, z = t
    n, k = qw.shape[0], qw.shape[1] * 2
    q = np.empty((n, k), np.float64)
    q[:, 0::2] = qw & 15
    q[:, 1::2] = qw >> 4
    s = np.repeat(np.asarray(s, np.float16).astype(np.float64), 128, axis=1)
    z = np.repeat(np.asarray(z, np.float16).astype(np.float64), 128, axis=1)
    return (q - z) * s


def rope_halves(x, pos, theta, d):
    """y[i] = x[i] c - x[i+d/2] s ; y[i+d/2] = x[i] s + x[i+d/2] c with angle pos * theta^(-2i/d)
    (crates/kernels/src/cpu_f32/mod.rs:502-547, 599-619); the table is f64 angles cast to f32."""
    half = d // 2
    inv = theta ** (-2.0 * np.arange(half) / d)
    ang = np.float64(pos) * inv
    c = np.cos(ang).astype(np.float32).astype(np.float64)
    s = np.sin(ang).astype(np.float32).astype(np.float64)
    a, b = x[..., :half], x[..., half:]
    return np.concatenate([a * c - b * s, a * s + b * c], axis=-1)


class DenseStep:
    """Float64 dense restatement of one step: row t of the packed batch is new token
    t - cu[s] of its sequence s, at position ctx[s] - new[s] + (t - cu[s]), and sees the keys
    up to its own position."""

    def __init__(self, cfg, layers, batch, theta, rounding):
        self.cfg, self.rounding, self.theta = cfg, rounding, theta
        self.r16 = f16_round if rounding else (lambda v: np.asarray(v, np.float64))
        self.rb = bf16_round if rounding else (lambda v: np.asarray(v, np.float64))
        self.layers = [dict(
            norm1=L["norm1"].astype(np.float64), norm2=L["norm2"].astype(np.float64),
            qkv=dequant_q4g128(L["qkv"]), o=dequant_q4g128(L["o"]),
            gate_up=dequant_q4g128(L["gate_up"]), down=dequant_q4g128(L["down"]),
            k_pool=L["k_pool"].astype(np.float64), v_pool=L["v_pool"].astype(np.float64),
            qkv_bias=None if L.get("qkv_bias") is None else L["qkv_bias"].astype(np.float64))
            for L in layers]
        self.h = batch["h"].astype(np.float64)
        self.bt = batch["block_tables"]
        self.ctx = np.asarray(batch["context_lens"], np.int64)
        self.cu = np.asarray(batch["cu_seqlens"], np.int64)
        self.final_norm = batch["final_norm"].astype(np.float64)
        self.trace = []

    def norm(self, x, w):
        return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + self.cfg["eps"]) * w

    def slot(self, s, p):
        bs = self.cfg["block_size"]
        return int(self.bt[s, p // bs]) * bs + p % bs

    def run(self):
        c = self.cfg
        hq, hkv, d, inter = c["hq"], c["hkv"], c["d"], c["inter"]
        groups = hq // hkv
        rows = self.h.shape[0]
        nseq = len(self.ctx)
        for L in self.layers:
            xn = self.rb(self.norm(self.h, L["norm1"]))
            qkv = xn @ L["qkv"].T
            if L.get("qkv_bias") is not None:
                qkv = qkv + L["qkv_bias"]
            attn = np.zeros((rows, hq, d))
            qs = np.zeros((rows, hq, d))
            for s in range(nseq):
                n_ctx = int(self.ctx[s])
                r0, r1 = int(self.cu[s]), int(self.cu[s + 1])
                n_new = r1 - r0  # the new tokens are the last n_new of the context
                # RoPE on q and k by position, then K / V into the cache
                # (attention.rs:199-216), for every new token of the sequence
                for i in range(n_new):
                    t, pos = r0 + i, n_ctx - n_new + i
                    qs[t] = self.r16(rope_halves(qkv[t, :hq * d].reshape(hq, d), pos, self.theta, d))
                    k = self.r16(rope_halves(qkv[t, hq * d:(hq + hkv) * d].reshape(hkv, d), pos,
                                             self.theta, d))
                    v = self.r16(qkv[t, (hq + hkv) * d:].reshape(hkv, d))
                    L["k_pool"][self.slot(s, pos)] = k.reshape(-1)
                    L["v_pool"][self.slot(s, pos)] = v.reshape(-1)
                for i in range(n_new):
                    t, pos = r0 + i, n_ctx - n_new + i
                    slots = [self.slot(s, p) for p in range(pos + 1)]  # causal: keys 0..pos
                    kc = L["k_pool"][slots].reshape(pos + 1, hkv, d)
                    vc = L["v_pool"][slots].reshape(pos + 1, hkv, d)
                    for hh in range(hq):
                        g = hh // groups
                        sc = (kc[:, g] @ qs[t, hh]) / np.sqrt(np.float64(d))
                        p = np.exp(sc - sc.max())
                        attn[t, hh] = (p / p.sum()) @ vc[:, g]
            o = self.rb(attn.reshape(rows, hq * d)) @ L["o"].T
            self.h = self.h + o
            xn2 = self.rb(self.norm(self.h, L["norm2"]))
            gu = xn2 @ L["gate_up"].T
            gate, up = gu[:, :inter], gu[:, inter:]
            act = self.rb(gate / (1.0 + np.exp(-gate)) * up)
            down = act @ L["down"].T
            self.h = self.h + down
            self.trace.append(dict(xn=xn, qkv=qkv, q=qs, attn=attn.reshape(rows, -1), o=o,
                                   xn2=xn2, gu=gu, act=act, down=down, h=self.h.copy()))
        return self.rb(self.norm(self.h, self.final_norm))


THETA = 1e6


def _problem(seed, ctx, num_layers=2, hidden=256, hq=4, hkv=2, inter=384, **kw):
    rng = np.random.default_rng(seed)
    return workloads.decode_step_problem(rng, num_layers=num_layers, hidden=hidden, hq=hq,
                                         hkv=hkv, inter=inter, ctx=ctx, theta=THETA, **kw)


def _oracle(cfg, layers, batch, trace=None):
    lay = copy.deepcopy(layers)
    bat = dict(batch, h=batch["h"].copy())
    out = O.bf16_bits_to_f32(OS.decode_step(cfg, lay, bat, trace=trace))
    return out, lay, bat


def _close(got, want, abs_tol, rel_tol, what):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bad = np.abs(got - want) > abs_tol + rel_tol * np.abs(want)
    assert not bad.any(), (what, int(bad.sum()), float(np.abs(got - want).max()))


def _bf16_nearly_equal(got_bits, want_vals, what, max_flip_frac=0.01):
    """bf16 results of two paths whose pre-rounding values differ by fp32-vs-f64 summation
    noise: equal except where a value sits on a rounding boundary, and then one ulp apart."""
    got = O.bf16_bits_to_f32(np.asarray(got_bits)).astype(np.float64).reshape(want_vals.shape)
    ulp = np.maximum(np.abs(want_vals), 2.0 ** -126) * 2.0 ** -7
    assert np.all(np.abs(got - want_vals) <= ulp), what
    assert (got != want_vals).mean() <= max_flip_frac, (what, float((got != want_vals).mean()))


# ------------------------------------------------------------------ (i) dense brute force
def test_step_matches_float64_dense_composition_stage_by_stage():
    """Every intermediate of every layer against the f64 composition that rounds where the
    step oracle says it rounds; the difference left is fp32-vs-f64 accumulation."""
    cfg, layers, batch = _problem(101, ctx=[1, 5, 37, 16, 64, 17])
    trace = []
    out, lay, bat = _oracle(cfg, layers, batch, trace=trace)
    ref = DenseStep(cfg, layers, batch, THETA, rounding=True)
    want = ref.run()
    assert len(trace) == len(ref.trace) == 2
    for li, (t, r) in enumerate(zip(trace, ref.trace)):
        _bf16_nearly_equal(t["xn"], r["xn"], f"layer {li} norm1")
        _close(t["qkv"], r["qkv"], 2e-4, 2e-4, f"layer {li} qkv")
        _close(t["q"].astype(np.float64), r["q"], 2e-3, 1e-3, f"layer {li} roped q")
        _close(t["attn"].reshape(r["attn"].shape), r["attn"], 1e-3, 1e-3, f"layer {li} attn")
        _close(t["o"], r["o"], 2e-4, 1e-3, f"layer {li} o projection")
        _bf16_nearly_equal(t["xn2"], r["xn2"], f"layer {li} norm2", max_flip_frac=0.03)
        _close(t["gu"], r["gu"], 5e-4, 1e-3, f"layer {li} gate_up")
        _close(O.bf16_bits_to_f32(t["act"]), r["act"], 2e-4, 1.6e-2, f"layer {li} silu*up")
        _close(t["down"], r["down"], 2e-4, 1e-3, f"layer {li} down projection")
        # the oracle folds `down` into h at the start of the next layer: its trace holds h + o
        _close(t["h"].astype(np.float64) + t["down"], r["h"], 5e-4, 1e-3,
               f"layer {li} residual stream")
    _close(out, want, 1e-3, 1.6e-2, "final normed state")
    rel = np.linalg.norm(out - want) / np.linalg.norm(want)
    assert rel < 1e-3, rel
    # the K / V rows the step appended, at the slot the block table gives
    for L, R in zip(lay, ref.layers):
        _close(L["k_pool"].astype(np.float64), R["k_pool"], 2e-3, 1e-3, "K pool after the step")
        _close(L["v_pool"].astype(np.float64), R["v_pool"], 2e-3, 1e-3, "V pool after the step")


def test_mixed_batch_with_qkv_bias_matches_float64_dense_composition():
    """A mixed chunked-prefill + decode batch (packed rows, causal inside a chunk) whose
    q/k/v projections carry a bias (attention.rs:49-57): the same stage-by-stage check."""
    ctx = [9, 40, 3, 21]
    new = [1, 7, 3, 5]  # decode row, a chunk with prior context, a whole short prompt, a chunk
    cfg, layers, batch = _problem(111, ctx=ctx, new_tokens=new, qkv_bias=True)
    assert batch["h"].shape[0] == 16 and list(batch["cu_seqlens"]) == [0, 1, 8, 11, 16]
    assert list(batch["positions"][1:8]) == list(range(33, 40))
    trace = []
    out, lay, bat = _oracle(cfg, layers, batch, trace=trace)
    ref = DenseStep(cfg, layers, batch, THETA, rounding=True)
    want = ref.run()
    for li, (t, r) in enumerate(zip(trace, ref.trace)):
        _close(t["qkv"], r["qkv"], 2e-4, 2e-4, f"layer {li} qkv + bias")
        _close(t["q"].astype(np.float64), r["q"], 4e-3, 1e-3, f"layer {li} roped q")
        _close(t["attn"].reshape(r["attn"].shape), r["attn"], 1e-3, 1e-3, f"layer {li} attn")
        _close(t["down"], r["down"], 2e-4, 1e-3, f"layer {li} down projection")
    assert np.linalg.norm(out - want) / np.linalg.norm(want) < 1e-3
    for L, R in zip(lay, ref.layers):
        _close(L["k_pool"].astype(np.float64), R["k_pool"], 4e-3, 1e-3, "K pool after the step")
    # the bias is in the projection (not dropped, not added twice): without it the result moves
    nb = [dict(L, qkv_bias=None) for L in layers]
    out_nb, _, _ = _oracle(cfg, nb, batch)
    assert np.abs(out_nb - out).max() > 1e-2
    # causal inside a chunk: the first token of the 7-token chunk does not see the later six;
    # changing the LAST token's hidden row leaves the earlier rows of the chunk untouched
    b2 = dict(batch, h=batch["h"].copy())
    b2["h"][7] += 1.0
    out2, _, _ = _oracle(cfg, layers, b2)
    assert np.array_equal(out2[1:7], out[1:7]) and not np.array_equal(out2[7], out[7])


def test_step_rounding_points_cost_what_bf16_and_fp16_cost():
    """Against the same composition with NO rounding anywhere: the oracle's documented
    rounding points (bf16 activations 2^-9, fp16 q/K/V 2^-11) may move the result by a few
    bf16 ulps of the activations, not more."""
    cfg, layers, batch = _problem(102, ctx=[3, 40, 9, 128])
    out, _, bat = _oracle(cfg, layers, batch)
    ref = DenseStep(cfg, layers, batch, THETA, rounding=False)
    want = ref.run()
    assert np.linalg.norm(out - want) / np.linalg.norm(want) < 6e-3
    assert np.linalg.norm(bat["h"] - ref.h) / np.linalg.norm(ref.h) < 6e-3
    _close(out, want, 2e-2, 2e-2, "final state vs unrounded f64")


# ------------------------------------------------------------------ (ii) exact special cases
def _zero_q4(n, k):
    """A Q4G128 matrix that dequantises to exactly 0: q = zero = 8."""
    return (np.full((n, k // 2), 0x88, np.uint8), np.full((n, k // 128), 0.01, np.float16),
            np.full((n, k // 128), 8.0, np.float16))


def test_zero_o_and_down_weights_leave_the_residual_stream_untouched():
    """stella.rs:193-203: both sub-blocks only ADD to x.  With zero o and down weights
    h is bit-identical after the step and the output is bf16(rms_norm(h) * final_norm)."""
    cfg, layers, batch = _problem(103, ctx=[7, 1, 33])
    for L in layers:
        L["o"] = _zero_q4(cfg["hidden"], cfg["hq"] * cfg["d"])
        L["down"] = _zero_q4(cfg["hidden"], cfg["inter"])
    out, _, bat = _oracle(cfg, layers, batch)
    assert np.array_equal(bat["h"], batch["h"])
    h = batch["h"].astype(np.float64)
    want = h / np.sqrt((h * h).mean(axis=1, keepdims=True) + cfg["eps"]) * batch["final_norm"]
    _bf16_nearly_equal(O.f32_to_bf16_bits(out), bf16_round(want), "final norm of untouched h")


def test_residual_is_added_before_the_second_norm():
    """A residual added after norm2 (or a norm applied to the sub-block output) gives a
    different xn2: xn2 must be bf16(rms_norm(h0 + o) * norm2)."""
    cfg, layers, batch = _problem(104, ctx=[12, 5], num_layers=1)
    trace = []
    _oracle(cfg, layers, batch, trace=trace)
    t = trace[0]
    h1 = batch["h"].astype(np.float64) + t["o"].astype(np.float64)
    want = h1 / np.sqrt((h1 * h1).mean(axis=1, keepdims=True) + cfg["eps"]) * layers[0]["norm2"]
    _bf16_nearly_equal(t["xn2"], bf16_round(want), "xn2 = norm2(h + o)")
    # the stream after the attention block is h0 + o, nothing else (`down` is folded in by
    # the next add_rms_norm: checked by the stage-by-stage test and the final state)
    assert np.array_equal(t["h"], batch["h"] + t["o"])
    wrong = bf16_round(batch["h"].astype(np.float64)
                       / np.sqrt((batch["h"].astype(np.float64) ** 2).mean(axis=1, keepdims=True)
                                 + cfg["eps"]) * layers[0]["norm2"])
    assert (O.bf16_bits_to_f32(t["xn2"]) != wrong).mean() > 0.5


def test_position_zero_is_a_rope_identity_and_later_positions_are_not():
    """cpu_f32/tests.rs:277-343: position 0 leaves the vector unchanged.  Sequence 0 has a
    one-token context (position 0), sequence 1 sits at position 4."""
    cfg, layers, batch = _problem(105, ctx=[1, 5], num_layers=1)
    trace = []
    _, lay, _ = _oracle(cfg, layers, batch, trace=trace)
    t = trace[0]
    hq, hkv, d = cfg["hq"], cfg["hkv"], cfg["d"]
    q_plain = t["qkv"][:, :hq * d].astype(np.float16).reshape(2, hq, d)
    assert np.array_equal(t["q"][0], q_plain[0])
    assert not np.array_equal(t["q"][1], q_plain[1])
    # the rotation at position 4 is the closed form, and its inverse gives the plain q back
    want = f16_round(rope_halves(t["qkv"][1, :hq * d].astype(np.float64).reshape(hq, d), 4,
                                 THETA, d))
    _close(t["q"][1].astype(np.float64), want, 1e-3, 1e-3, "rope at position 4")
    # an off-by-one position would be visible: positions 3 and 5 give different vectors
    for wrong_pos in (3, 5):
        other = f16_round(rope_halves(t["qkv"][1, :hq * d].astype(np.float64).reshape(hq, d),
                                      wrong_pos, THETA, d))
        assert np.abs(other - t["q"][1].astype(np.float64)).max() > 0.05
    # the cached K of sequence 0 (position 0) is the plain k rounded to fp16
    slot0 = int(batch["block_tables"][0, 0]) * cfg["block_size"]
    k_plain = t["qkv"][0, hq * d:(hq + hkv) * d].astype(np.float16)
    assert np.array_equal(lay[0]["k_pool"][slot0], k_plain)


def test_one_token_context_attends_to_its_own_value_row():
    """softmax over one key is exactly 1, so the attention output of a sequence whose context
    is the new token alone is its own (fp16) V row, each q head reading kv head h / groups
    (`repeat_kv`, attention.rs:366-382)."""
    cfg, layers, batch = _problem(106, ctx=[1, 1, 9], num_layers=1, hq=4, hkv=2)
    trace = []
    _oracle(cfg, layers, batch, trace=trace)
    t = trace[0]
    hq, hkv, d = cfg["hq"], cfg["hkv"], cfg["d"]
    groups = hq // hkv
    attn = np.asarray(t["attn"]).reshape(3, hq, d)
    for s in (0, 1):
        v = t["qkv"][s, (hq + hkv) * d:].astype(np.float16).astype(np.float32).reshape(hkv, d)
        for hh in range(hq):
            assert np.array_equal(attn[s, hh], v[hh // groups]), (s, hh)
        # the two kv heads differ, so a wrong GQA map (h % hkv) would fail the line above
        assert not np.array_equal(v[0], v[1])


def test_new_rows_land_in_the_slot_the_block_table_names_and_nowhere_else():
    cfg, layers, batch = _problem(107, ctx=[16, 17, 1, 33], num_layers=1)
    _, lay, _ = _oracle(cfg, layers, batch)
    bs = cfg["block_size"]
    want_slots = [int(batch["block_tables"][s, (c - 1) // bs]) * bs + (c - 1) % bs
                  for s, c in enumerate([16, 17, 1, 33])]
    assert list(batch["slots"]) == want_slots
    for name in ("k_pool", "v_pool"):
        changed = np.nonzero((lay[0][name] != layers[0][name]).any(axis=1))[0]
        assert sorted(changed.tolist()) == sorted(want_slots), name


def test_gate_is_the_first_half_and_goes_through_silu():
    """mlp.rs:104-121: silu applies to gate, up is the plain factor.  act must be
    bf16(silu(gu[:, :inter]) * gu[:, inter:]); swapping the halves of the fused weight changes
    the step, and the swapped step equals the dense composition of the swapped weight."""
    cfg, layers, batch = _problem(108, ctx=[4, 21], num_layers=1)
    inter = cfg["inter"]
    trace = []
    out, _, _ = _oracle(cfg, layers, batch, trace=trace)
    gu = trace[0]["gu"].astype(np.float64)
    want = bf16_round(gu[:, :inter] / (1 + np.exp(-gu[:, :inter])) * gu[:, inter:])
    _bf16_nearly_equal(trace[0]["act"], want, "act = silu(gate) * up")
    swapped_wrong = bf16_round(gu[:, inter:] / (1 + np.exp(-gu[:, inter:])) * gu[:, :inter])
    assert (O.bf16_bits_to_f32(trace[0]["act"]) != swapped_wrong).mean() > 0.9
    sw = copy.deepcopy(layers)
    sw[0]["gate_up"] = tuple(np.concatenate([a[inter:], a[:inter]]) for a in layers[0]["gate_up"])
    out_sw, _, _ = _oracle(cfg, sw, batch)
    assert np.abs(out_sw - out).max() > 1e-2
    ref = DenseStep(cfg, sw, batch, THETA, rounding=True).run()
    assert np.linalg.norm(out_sw - ref) / np.linalg.norm(ref) < 1e-3


def test_attention_sees_the_new_token_and_all_earlier_ones():
    """The new token's K/V row is written before attention runs (RoPE-then-cache order) and
    is visible: zeroing every OTHER cached value row leaves p_new * v_new, and the output is
    invariant to the unused rows of the pool."""
    cfg, layers, batch = _problem(109, ctx=[6], num_layers=1, hq=2, hkv=1)
    hq, hkv, d = cfg["hq"], cfg["hkv"], cfg["d"]
    lz = copy.deepcopy(layers)
    lz[0]["v_pool"][:] = 0
    trace = []
    _oracle(cfg, lz, batch, trace=trace)
    t = trace[0]
    v_new = t["qkv"][0, (hq + hkv) * d:].astype(np.float16).astype(np.float64)
    attn = np.asarray(t["attn"]).reshape(hq, d).astype(np.float64)
    # attn[h] = p_h * v_new with 0 < p_h < 1: parallel to v_new, same factor on every lane
    for hh in range(hq):
        ratio = attn[hh] / v_new
        assert 0 < ratio.mean() < 1
        assert np.ptp(ratio) < 1e-4
    # rows of the pool outside the sequence's blocks are never read
    noise = copy.deepcopy(layers)
    used = set()
    bs = cfg["block_size"]
    for p in range(6):
        used.add(int(batch["block_tables"][0, p // bs]) * bs + p % bs)
    free = [r for r in range(noise[0]["k_pool"].shape[0]) if r not in used]
    noise[0]["k_pool"][free] = np.float16(37.0)
    noise[0]["v_pool"][free] = np.float16(-11.0)
    a, _, _ = _oracle(cfg, layers, batch)
    b, _, _ = _oracle(cfg, noise, batch)
    assert np.array_equal(a, b)


# ------------------------------------------------------------------ the fused operators alone
def test_add_rms_norm_bf16_against_closed_form():
    rng = np.random.default_rng(110)
    h = rng.standard_normal((5, 384), np.float32)
    y = rng.standard_normal((5, 384), np.float32)
    w = (1 + 0.1 * rng.standard_normal(384)).astype(np.float32)
    h0 = h.copy()
    got = OS.add_rms_norm_bf16(h, y, w, 1e-6)
    assert np.array_equal(h, h0 + y)  # one fp32 add, in place
    hh = (h0 + y).astype(np.float64)
    want = hh / np.sqrt((hh * hh).mean(axis=1, keepdims=True) + 1e-6) * w
    _bf16_nearly_equal(got, bf16_round(want), "add + rms_norm")
    # y given as bf16 bits is widened exactly; y = None adds nothing
    h = h0.copy()
    yb = bf16_bits(y)
    OS.add_rms_norm_bf16(h, yb, w, 1e-6)
    assert np.array_equal(h, h0 + bf16_round(y).astype(np.float32))
    h = h0.copy()
    OS.add_rms_norm_bf16(h, None, w, 1e-6)
    assert np.array_equal(h, h0)


def test_rope_kv_write_against_closed_form():
    rng = np.random.default_rng(111)
    hq, hkv, d, t = 4, 2, 128, 3
    qkv = rng.standard_normal((t, (hq + 2 * hkv) * d), np.float32)
    pos = np.array([0, 7, 130], np.int32)
    cos, sin = O.build_rope_table_f32(131, d, 1e4)
    slots = np.array([5, 0, 9], np.int64)
    kp = np.zeros((12, hkv * d), np.float16)
    vp = np.zeros((12, hkv * d), np.float16)
    q16 = OS.rope_kv_write(qkv, pos, cos, sin, slots, kp, vp, hq, hkv, d)
    x = qkv.astype(np.float64).reshape(t, hq + 2 * hkv, d)
    for i in range(t):
        want_q = f16_round(rope_halves(x[i, :hq], pos[i], 1e4, d))
        want_k = f16_round(rope_halves(x[i, hq:hq + hkv], pos[i], 1e4, d))
        _close(q16[i].astype(np.float64), want_q, 2e-3, 1e-3, "q")
        _close(kp[slots[i]].astype(np.float64).reshape(hkv, d), want_k, 2e-3, 1e-3, "k")
        # v is not rotated: exactly the fp16 rounding of the projection output
        assert np.array_equal(vp[slots[i]], qkv[i, (hq + hkv) * d:].astype(np.float16))
    untouched = np.setdiff1d(np.arange(12), slots)
    assert not kp[untouched].any() and not vp[untouched].any()


def test_rope_kv_write_rejects_positions_outside_the_table():
    rng = np.random.default_rng(112)
    hq, hkv, d = 2, 1, 128
    qkv = rng.standard_normal((1, (hq + 2 * hkv) * d), np.float32)
    cos, sin = O.build_rope_table_f32(8, d, 1e4)
    kp = np.zeros((4, hkv * d), np.float16)
    vp = np.zeros((4, hkv * d), np.float16)
    for bad in (8, -1):
        with pytest.raises(ValueError):
            OS.rope_kv_write(qkv, np.array([bad], np.int32), cos, sin, np.array([0], np.int64),
                             kp, vp, hq, hkv, d)


def test_silu_mul_bf16_against_closed_form():
    rng = np.random.default_rng(113)
    gu = (rng.standard_normal((4, 512)) * 3).astype(np.float32)
    got = OS.silu_mul_bf16(gu, 256)
    g, u = gu[:, :256].astype(np.float64), gu[:, 256:].astype(np.float64)
    _close(O.bf16_bits_to_f32(got), bf16_round(g / (1 + np.exp(-g)) * u), 1e-6, 8e-3, "silu*up")
    # silu(0) = 0, silu(x) -> x for large x, -> 0 for very negative x (cpu_f32/tests.rs:465-470)
    edge = np.array([[0.0, 30.0, -30.0, 1.0, 2.0, 2.0, 2.0, 2.0]], np.float32)
    e = O.bf16_bits_to_f32(OS.silu_mul_bf16(edge, 4))[0]
    assert e[0] == 0 and e[1] == 60.0 and abs(e[2]) < 1e-10
    assert abs(e[3] - 2 * 0.7310585786) < 8e-3
