"""CPU oracle of one decode step (TEST INFRASTRUCTURE, like the rest of oracle/).

The reference has no decoder; the step below composes the restated reference
functions in the order of its encoder layer (`StellaLayer::forward`,
crates/encoders/src/stella.rs:190-206: pre-norm residual blocks) with the
attention and MLP arithmetic of crates/transformers/src/{attention,mlp}.rs,
replacing dense fp32 weights by Q4G128 ones and the contiguous K/V by the paged
cache.  Rounding points (what is stored in which type between operators) are
part of the definition and are the ones the GPU path uses:

  hidden state h ............ fp32
  normed activations ........ bf16   (input of every quantized GEMM)
  GEMM outputs .............. fp32   (consumed un-rounded by the next operator)
  q, and K/V in the cache ... fp16   (RoPE in fp32 on the fp32 GEMM output)
  attention output .......... bf16   (one rounding of the fp32 result; feeds the o projection)
  silu(gate) * up ........... bf16
"""
from __future__ import annotations

import numpy as np

import oracle as O


def add_rms_norm_bf16(h: np.ndarray, y, w, eps: float) -> np.ndarray:
    """h (fp32, [rows, n]) += y in place (y: bf16 bits, or fp32); returns bf16 bits of
    rms_norm(h) * w."""
    rows, n = h.shape
    if y is not None:
        y = np.asarray(y)
        h += (y if y.dtype == np.float32 else O.bf16_bits_to_f32(y)).reshape(rows, n)
    return O.f32_to_bf16_bits(O.rms_norm(h, w, rows, n, eps)).reshape(rows, n)


def rope_kv_write(qkv, positions, cos, sin, slots, k_pool, v_pool, hq, hkv, d=128, turbo3=False):
    """qkv (bf16 bits or fp32) [T, (hq+2hkv)*d] -> q fp16 [T,hq,d]; roped k and v written into
    the pools: as fp16 rows, or (turbo3: uint8 pools of 56-byte head rows) those fp16 rows
    encoded with `encode_turbo3_0_head`."""
    qkv = np.asarray(qkv)
    t = qkv.shape[0]
    half = d // 2
    x = (qkv if qkv.dtype == np.float32 else O.bf16_bits_to_f32(qkv)).reshape(t, hq + 2 * hkv, d)
    q = np.ascontiguousarray(x[:, :hq]).reshape(t * hq, d)
    k = np.ascontiguousarray(x[:, hq:hq + hkv]).reshape(t * hkv, d)
    v = np.ascontiguousarray(x[:, hq + hkv:]).reshape(t, hkv * d)
    max_pos = cos.size // half
    pos = np.asarray(positions, np.int64)
    if pos.size and (pos.min() < 0 or pos.max() >= max_pos):
        # `RopeTable::gather` (crates/transformers/src/rope.rs) fails on a position past the
        # table; so does the oracle
        raise ValueError(f"rope_kv_write: position outside the RoPE table of {max_pos} rows")
    cos2, sin2 = cos.reshape(max_pos, half), sin.reshape(max_pos, half)
    # `RopeTable::gather` (crates/transformers/src/rope.rs): one cos/sin row per (token, head)
    O.rope_halves_in_place(q, np.repeat(cos2[pos], hq, axis=0), np.repeat(sin2[pos], hq, axis=0),
                           t * hq, d)
    O.rope_halves_in_place(k, np.repeat(cos2[pos], hkv, axis=0), np.repeat(sin2[pos], hkv, axis=0),
                           t * hkv, d)
    q16 = O.f32_to_f16_bits(q).view(np.float16).reshape(t, hq, d)
    k16 = O.f32_to_f16_bits(k).view(np.float16).reshape(t, hkv * d)
    v16 = O.f32_to_f16_bits(v).view(np.float16).reshape(t, hkv * d)
    if turbo3:
        O.kv_write_turbo3(k16, v16, k_pool, v_pool, slots, hkv)
    else:
        O.kv_write_fp16(k16, v16, k_pool, v_pool, slots, hkv * d)
    return q16


def silu_mul_bf16(gate_up, inter):
    gate_up = np.asarray(gate_up)
    x = gate_up if gate_up.dtype == np.float32 else O.bf16_bits_to_f32(gate_up)
    rows = x.shape[0]
    g = np.ascontiguousarray(x[:, :inter])
    u = np.ascontiguousarray(x[:, inter:])
    return O.f32_to_bf16_bits(O.hadamard(O.silu(g), u)).reshape(rows, inter)


def cast_f16_bf16(a16):
    return O.f32_to_bf16_bits(O.f16_bits_to_f32(np.ascontiguousarray(a16).view(np.uint16)))


def _gemm(x_bits, w, b, bias=None):
    qw, s, z = w
    n, k = qw.shape[0], qw.shape[1] * 2
    return O.qgemm_q4g128_f32(np.ascontiguousarray(x_bits), qw, s, z, b, n, k, bias)


def decode_step(cfg, layers, batch, trace=None):
    """One step over `batch`: one row per new token, in packed order -- one token per sequence
    for a decode step, `cu_seqlens[s+1] - cu_seqlens[s]` tokens of sequence s for a mixed batch
    (chunked prefill + decode; causal inside a chunk).

    cfg:    dict(hidden, hq, hkv, d, inter, eps, block_size[, kv_turbo3: the pools are uint8
            turbo3 pools [rows][hkv*56]])
    layers: list of dict(norm1, qkv, o, norm2, gate_up, down, k_pool, v_pool[, qkv_bias]); each
            weight a (qw, scale, zero) triple; qkv_bias fp32 [(hq+2hkv)*d] is the bias of the
            q/k/v projections (crates/transformers/src/attention.rs:49-57), added as `linear_t`
            adds it; pools are updated in place
    batch:  dict(h [B, hidden] fp32 (updated in place), block_tables, cu_seqlens, context_lens,
            positions, slots, cos, sin, final_norm); optionally token_ids (uint32 [B]) with
            embed_table (bf16 bits [vocab, hidden]): h is first filled by `embed_lookup`; and
            lm_head (a Q4G128 triple [vocab, hidden]): the step ends with the vocabulary
            projection and `greedy`, leaving batch["logits"] (fp32) and batch["tokens"]
    Returns the final normed hidden state as bf16 bits.
    """
    b = batch["h"].shape[0]
    h = batch["h"]
    if batch.get("token_ids") is not None:
        vocab, hidden = batch["embed_table"].shape
        table = O.bf16_bits_to_f32(batch["embed_table"])
        h[:] = O.embed_lookup(table, hidden, vocab, batch["token_ids"]).reshape(b, hidden)
    y = None
    for li, L in enumerate(layers):
        xn = add_rms_norm_bf16(h, y, L["norm1"], cfg["eps"])
        qkv = _gemm(xn, L["qkv"], b, L.get("qkv_bias"))
        t3 = bool(cfg.get("kv_turbo3"))
        q16 = rope_kv_write(qkv, batch["positions"], batch["cos"], batch["sin"], batch["slots"],
                            L["k_pool"], L["v_pool"], cfg["hq"], cfg["hkv"], cfg["d"], turbo3=t3)
        if t3:
            attn = O.paged_attn_varlen_turbo3(q16, L["k_pool"], L["v_pool"],
                                              batch["block_tables"], batch["cu_seqlens"],
                                              batch["context_lens"], cfg["hq"], cfg["hkv"],
                                              cfg["block_size"],
                                              1.0 / np.sqrt(np.float32(cfg["d"])), True,
                                              f32_out=True)
        else:
            attn = O.paged_attn_varlen_fp16(q16, L["k_pool"], L["v_pool"], batch["block_tables"],
                                            batch["cu_seqlens"], batch["context_lens"], cfg["hq"],
                                            cfg["hkv"], cfg["d"], cfg["block_size"],
                                            1.0 / np.sqrt(np.float32(cfg["d"])), True,
                                            f32_out=True)
        o = _gemm(O.f32_to_bf16_bits(attn.reshape(b, -1)), L["o"], b)
        xn2 = add_rms_norm_bf16(h, o, L["norm2"], cfg["eps"])
        gu = _gemm(xn2, L["gate_up"], b)
        act = silu_mul_bf16(gu, cfg["inter"])
        y = _gemm(act, L["down"], b)
        if trace is not None:
            trace.append(dict(xn=xn, qkv=qkv, q=q16, attn=attn, o=o, xn2=xn2, gu=gu, act=act,
                              down=y, h=h.copy()))
    out = add_rms_norm_bf16(h, y, batch["final_norm"], cfg["eps"])
    if batch.get("lm_head") is not None:
        batch["logits"] = _gemm(out, batch["lm_head"], b)
        batch["tokens"] = np.array([O.greedy(r) for r in batch["logits"]], np.uint32)
    return out
