"""Seeded synthetic inputs shared by the parity tests, smoke() and bench.py.

Everything is generated on the host with numpy's PCG64 (same numpy on every
box of this image), then uploaded: the oracle and the GPU see identical bytes.
"""
from __future__ import annotations

import math

import numpy as np

SEED = 0x10615


def paged_case(rng, new_tokens, prior_ctx, hq, hkv, d=128, block_size=16, spare_frac=0.25,
               kv_std=1.0, pool_period_rows=None, min_max_blocks=1):
    """Ragged paged-attention inputs: pools shared by all sequences, physical
    block ids a random permutation, block-table tail entries poisoned.  With
    pool_period_rows the pools repeat that many random rows (full-size cases whose
    pools would take minutes to draw); min_max_blocks widens the block tables (the launch
    heuristics size their work by what the tables could hold)."""
    new = np.asarray(new_tokens, np.int32)
    prior = np.asarray(prior_ctx, np.int32)
    ctx = (new + prior).astype(np.int32)
    nblk = [(int(c) + block_size - 1) // block_size for c in ctx]
    total_blocks = sum(nblk) + max(1, int(sum(nblk) * spare_frac))
    perm = rng.permutation(total_blocks).astype(np.int32)
    max_blocks = max(max(nblk), min_max_blocks, 1)
    bt = np.full((len(new), max_blocks), 0x3FFFFFF, np.int32)
    o = 0
    for s, nb in enumerate(nblk):
        bt[s, :nb] = perm[o:o + nb]
        o += nb
    rows = total_blocks * block_size
    def pool():
        n = min(rows, pool_period_rows or rows)
        base = (rng.standard_normal((n, hkv * d), np.float32) * kv_std).astype(np.float16)
        return base if n == rows else np.resize(base, (rows, hkv * d))

    k_pool = pool()
    v_pool = pool()
    cu = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    q = rng.standard_normal((int(cu[-1]), hq, d), np.float32).astype(np.float16)
    return dict(q=q, k_pool=k_pool, v_pool=v_pool, block_tables=bt, cu_seqlens=cu,
                context_lens=ctx, new_tokens=new, prior_ctx=prior, hq=hq, hkv=hkv, d=d,
                block_size=block_size, max_blocks=max_blocks, scale=1.0 / math.sqrt(d))


def config2(seed=SEED + 1):
    """Ragged paged decode, Qwen2-1.5B geometry: 16 sequences, ctx ~ U{64..2048},
    12 query / 2 KV heads, head_dim 128, block 16, one query token each."""
    rng = np.random.default_rng(seed)
    ctx = rng.integers(64, 2049, size=16)
    return paged_case(rng, np.ones(16, np.int32), ctx - 1, hq=12, hkv=2)


def config1(seed=SEED):
    """Q8G32 GEMV, Qwen2-1.5B MLP up-proj: x 1x1536 ~N(0,1), W 8960x1536 ~N(0,0.02)."""
    rng = np.random.default_rng(seed)
    n, k = 8960, 1536
    x = rng.standard_normal(k, np.float32)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    return dict(x=x, w=w, n=n, k=k)


def paged_attn_algorithmic_bytes(case) -> int:
    """K and V rows read once per sequence, q and out, block-table entries read,
    cu_seqlens and context_lens."""
    ctx = case["context_lens"].astype(np.int64)
    row_bytes = case["hkv"] * case["d"] * 2
    kv = int(ctx.sum()) * 2 * row_bytes
    qo = 2 * case["q"].size * 2
    bt = 4 * int(((ctx + case["block_size"] - 1) // case["block_size"]).sum())
    return kv + qo + bt + 4 * (2 * len(ctx) + 1)


def qgemv_q8_algorithmic_bytes(n, k) -> int:
    return n * k + n * (k // 32) * 2 + 4 * k + 4 * n


def config5_attention(seed=SEED + 5, num_seqs=32, lo=256, hi=8192):
    """One layer's attention of the Qwen3-8B-geometry decode step: 32 live sequences,
    ctx ~ U{256..8192}, 32 query / 8 KV heads, head_dim 128, block 16."""
    rng = np.random.default_rng(seed)
    ctx = rng.integers(lo, hi + 1, size=num_seqs)
    return paged_case(rng, np.ones(num_seqs, np.int32), ctx - 1, hq=32, hkv=8, spare_frac=0.05)


def config4(seed=SEED + 4, num_decode=48, num_prefill=16, chunk=512, max_decode_ctx=32768,
            max_prior=8192, hq=32, hkv=8, pool_period_rows=8191):
    """Mixed chunked-prefill + decode ragged batch, Qwen3-8B attention geometry: 48 decode
    rows (contexts log-uniform 128..32768) interleaved with 16 prefill chunks of 512 tokens
    (prior context uniform 0..8192), one packed token buffer."""
    rng = np.random.default_rng(seed)
    dec_ctx = np.exp(rng.uniform(np.log(128.0), np.log(float(max_decode_ctx)), num_decode))
    dec_ctx = np.clip(np.rint(dec_ctx).astype(np.int64), 128, max_decode_ctx)
    pre_prior = rng.integers(0, max_prior + 1, size=num_prefill)
    kind = np.array([0] * num_decode + [1] * num_prefill)
    rng.shuffle(kind)
    new, prior = [], []
    di = pi = 0
    for kd in kind:
        if kd == 0:
            new.append(1)
            prior.append(int(dec_ctx[di]) - 1)
            di += 1
        else:
            new.append(chunk)
            prior.append(int(pre_prior[pi]))
            pi += 1
    return paged_case(rng, new, prior, hq=hq, hkv=hkv, spare_frac=0.02,
                      pool_period_rows=pool_period_rows)


def paged_attn_flops(case, causal=True) -> int:
    """QK^T and PV multiply-adds (x2) over the visible (query, key) pairs."""
    new = case["new_tokens"].astype(np.int64)
    ctx = case["context_lens"].astype(np.int64)
    if causal:
        pairs = new * (ctx - new) + new * (new + 1) // 2
    else:
        pairs = new * ctx
    return int(pairs.sum()) * case["hq"] * case["d"] * 4


def config3(seed=SEED + 3, n=12288, k=4096, max_batch=16):
    """Q4G128 GEMV/GEMM at Qwen-8B geometry: W 12288x4096 ~N(0,0.02), x bf16 ~N(0,1)."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
    x = rng.standard_normal((max_batch, k), np.float32)
    return dict(w=w, x=x, n=n, k=k)


def qgemm_q4_algorithmic_bytes(b, n, k) -> int:
    return n * k // 2 + n * (k // 128) * 4 + b * k * 2 + b * n * 2


def decode_step_problem(rng, num_layers, hidden, hq, hkv, inter, ctx, d=128, block_size=16,
                        max_pos=None, eps=1e-6, theta=1e6, random_nibbles=False, vocab=0,
                        kv_turbo3=False, new_tokens=None, qkv_bias=False,
                        pool_period_rows=None):
    """A decode-step problem: `ctx[s]` is the context of sequence s INCLUDING its new tokens
    (one per sequence, or `new_tokens[s]` for a mixed chunked-prefill + decode batch: the batch
    then has sum(new_tokens) packed rows).  qkv_bias: every layer's q/k/v projection carries a
    bias ~N(0,1).
    Weights ~N(0,0.02) quantised to Q4G128 by the oracle (or raw random nibbles/scales when
    random_nibbles, for timing-only runs), RMSNorm gains 1+N(0,0.02), RoPE theta 1e6.
    With vocab > 0 the batch also carries token ids, a bf16 embedding table and a Q4G128
    lm_head (tokens in, tokens out).  kv_turbo3: the pools are TurboQuant 3-bit pools
    (uint8 [rows][hkv*56]) holding the encoded random rows.  pool_period_rows: the pools
    repeat that many random rows (timing runs of full-size batches)."""
    import oracle as O
    ctx = np.asarray(ctx, np.int32)
    new = np.ones(len(ctx), np.int32) if new_tokens is None else np.asarray(new_tokens, np.int32)
    assert len(new) == len(ctx) and (new >= 1).all() and (new <= ctx).all()
    b = int(new.sum())  # packed rows
    max_pos = max_pos or int(ctx.max()) + 1

    def q4(n, k):
        if random_nibbles:
            qw = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
            s = (rng.random((n, k // 128), np.float32) * 0.004 + 0.004).astype(np.float16)
            z = (rng.random((n, k // 128), np.float32) * 2 + 6.5).astype(np.float16)
            return qw, s, z
        w = rng.standard_normal((n, k), np.float32) * np.float32(0.02)
        return O.quantize_q4g128(w, n, k)

    base = paged_case(rng, new, ctx - new, hq=hq, hkv=hkv, d=d, block_size=block_size,
                      spare_frac=0.05, pool_period_rows=pool_period_rows)

    def pool(rows):
        n = min(rows, pool_period_rows or rows)
        p = rng.standard_normal((n, hkv * d), np.float32).astype(np.float16)
        return p if n == rows else np.resize(p, (rows, hkv * d))
    layers = []
    for _ in range(num_layers):
        rows = base["k_pool"].shape[0]
        layers.append(dict(
            norm1=(1 + 0.02 * rng.standard_normal(hidden)).astype(np.float32),
            norm2=(1 + 0.02 * rng.standard_normal(hidden)).astype(np.float32),
            qkv=q4((hq + 2 * hkv) * d, hidden), o=q4(hidden, hq * d),
            gate_up=q4(2 * inter, hidden), down=q4(hidden, inter),
            k_pool=pool(rows), v_pool=pool(rows)))
        if qkv_bias:
            layers[-1]["qkv_bias"] = rng.standard_normal((hq + 2 * hkv) * d).astype(np.float32)
    # the RoPE tables cover every position the block tables can hold
    max_pos = max(max_pos, block_size * base["block_tables"].shape[1])
    cos, sin = O.build_rope_table_f32(max_pos, d, theta)
    cu, slots, ctx_lens, _ = O.pack_ragged(new, ctx - new, base["block_tables"], block_size)
    # position of packed row t: prior context of its sequence + its index inside the chunk
    positions = np.concatenate([np.arange(c - n, c) for c, n in zip(ctx, new)]).astype(np.int32)
    batch = dict(h=rng.standard_normal((b, hidden), np.float32),
                 block_tables=base["block_tables"], cu_seqlens=cu, context_lens=ctx_lens,
                 positions=positions, slots=slots, cos=cos, sin=sin,
                 final_norm=(1 + 0.02 * rng.standard_normal(hidden)).astype(np.float32))
    cfg = dict(hidden=hidden, hq=hq, hkv=hkv, d=d, inter=inter, eps=eps, block_size=block_size)
    if kv_turbo3:
        cfg["kv_turbo3"] = True
        for L in layers:
            rows = L["k_pool"].shape[0]
            kp = np.zeros((rows, hkv * 56), np.uint8)
            vp = np.zeros((rows, hkv * 56), np.uint8)
            O.kv_write_turbo3(L["k_pool"], L["v_pool"], kp, vp, np.arange(rows), hkv)
            L["k_pool"], L["v_pool"] = kp, vp
    if vocab:
        batch["token_ids"] = rng.integers(0, vocab, size=b, dtype=np.uint32)
        batch["embed_table"] = O.f32_to_bf16_bits(
            rng.standard_normal((vocab, hidden), np.float32)).reshape(vocab, hidden)
        batch["lm_head"] = q4(vocab, hidden)
    return cfg, layers, batch
