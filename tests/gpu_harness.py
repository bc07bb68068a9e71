"""Host glue used by the GPU tests, smoke() and bench.py: uploads a case,
calls the C-ABI launchers, downloads results."""
from __future__ import annotations

import ctypes as C

import numpy as np

from logismos_amd import hip, kernels


class PagedAttnRunner:
    def __init__(self, case, num_splits=None, causal=True, stream=None):
        self.case = case
        self.stream = stream
        self.causal = causal
        c = case
        self.num_seqs = len(c["context_lens"])
        self.total_tokens = int(c["cu_seqlens"][-1])
        self.max_seqlen_q = int(c["new_tokens"].max()) if self.num_seqs else 0
        self.num_splits = num_splits or kernels.paged_attn_num_splits(
            self.num_seqs, c["hkv"], c["block_size"], c["max_blocks"], c["d"])
        self.q = hip.DeviceBuffer.from_numpy(c["q"])
        self.k_pool = hip.DeviceBuffer.from_numpy(c["k_pool"])
        self.v_pool = hip.DeviceBuffer.from_numpy(c["v_pool"])
        self.bt = hip.DeviceBuffer.from_numpy(c["block_tables"])
        self.cu = hip.DeviceBuffer.from_numpy(c["cu_seqlens"])
        self.ctx = hip.DeviceBuffer.from_numpy(c["context_lens"])
        self.out = hip.DeviceBuffer(max(c["q"].nbytes, 16))
        self.out.fill(0xFF)  # NaN pattern: unwritten outputs are caught
        ws = kernels.paged_attn_workspace_bytes(self.num_seqs, c["hq"], c["d"], self.num_splits)
        self.ws = hip.DeviceBuffer(max(ws, 16))
        self.ws.fill(0xFF)

    def launch(self, phases=None, k_pool=None, v_pool=None):
        c = self.case
        kernels.launch_paged_attn_varlen_fp16(
            self.q, k_pool or self.k_pool, v_pool or self.v_pool, self.bt, self.cu, self.ctx,
            self.out, self.ws, self.num_seqs, self.total_tokens, self.max_seqlen_q, c["hq"],
            c["hkv"], c["d"], c["block_size"], c["max_blocks"], self.num_splits, c["scale"],
            self.causal, self.stream, phases)

    def result(self) -> np.ndarray:
        (self.stream.synchronize() if self.stream else hip.synchronize())
        return self.out.to_numpy(np.float16, self.case["q"].shape)


class QgemvQ8Runner:
    def __init__(self, x, qs, d, n, k, stream=None):
        self.n, self.k, self.stream = n, k, stream
        self.x = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(x, np.float32))
        self.qs = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(qs, np.int8))
        self.d = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(d).view(np.uint16))
        self.y = hip.DeviceBuffer(n * 4)
        self.y.fill(0xFF)

    def launch(self):
        kernels.launch_qgemv_q8g32_f32(self.x, self.qs, self.d, self.y, self.n, self.k, self.stream)

    def result(self) -> np.ndarray:
        (self.stream.synchronize() if self.stream else hip.synchronize())
        return self.y.to_numpy(np.float32, (self.n,))


class QgemmQ4Runner:
    def __init__(self, x_bf16_bits, qw, scale, zero, b, n, k, stream=None):
        self.b, self.n, self.k, self.stream = b, n, k, stream
        self.x = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(x_bf16_bits, np.uint16))
        self.qw = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(qw, np.uint8))
        self.scale = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(scale).view(np.uint16))
        self.zero = hip.DeviceBuffer.from_numpy(np.ascontiguousarray(zero).view(np.uint16))
        self.y = hip.DeviceBuffer(b * n * 2)
        self.y.fill(0xFF)

    def launch(self, qw=None, scale=None, zero=None, force_mfma=False):
        kernels.launch_qgemm_q4g128_bf16(self.x, qw or self.qw, scale or self.scale,
                                         zero or self.zero, self.y, self.b, self.n, self.k,
                                         self.stream, force_mfma)

    def result_bits(self) -> np.ndarray:
        (self.stream.synchronize() if self.stream else hip.synchronize())
        return self.y.to_numpy(np.uint16, (self.b, self.n))


def _val(p):
    return p.ptr.value if isinstance(p, hip.DeviceBuffer) else p


class DecodeStepRunner:
    """Uploads a decode-step problem (see oracle/decode_step.py for the dict layout) and runs
    logismos_launch_decode_step.  `layer_bufs` keeps the device buffers alive."""

    def __init__(self, cfg, layers, batch, num_splits=None, stream=None, share_layer_data=False):
        self.cfg_d, self.stream = cfg, stream
        b = batch["h"].shape[0]  # packed rows (= sequences for a decode step)
        self.b = b
        nseq = len(batch["context_lens"])
        self.num_seqs = nseq
        max_blocks = batch["block_tables"].shape[1]
        self.num_splits = num_splits or kernels.paged_attn_num_splits(
            nseq, cfg["hkv"], cfg["block_size"], max_blocks, cfg["d"])
        half = cfg["d"] // 2
        self.cfg = kernels.DecodeConfig(len(layers), cfg["hidden"], cfg["hq"], cfg["hkv"], cfg["d"],
                                        cfg["inter"], cfg["eps"], cfg["block_size"], max_blocks,
                                        batch["cos"].size // half,
                                        batch["lm_head"][0].shape[0] if "lm_head" in batch else 0,
                                        1 if cfg.get("kv_turbo3") else 0)
        up = hip.DeviceBuffer.from_numpy
        self.keep = []

        def w3(t):
            bufs = [up(np.ascontiguousarray(t[0])), up(np.ascontiguousarray(t[1]).view(np.uint16)),
                    up(np.ascontiguousarray(t[2]).view(np.uint16))]
            self.keep += bufs
            return kernels.Q4Weight(*[_val(x) for x in bufs])

        self.layers = (kernels.DecodeLayer * len(layers))()
        self.pools = []
        first = None
        for i, L in enumerate(layers):
            if share_layer_data and first is not None:
                # same weights, own pools (device-to-device copies): timing runs only
                src = first
                kp, vp = hip.DeviceBuffer(src[6].nbytes), hip.DeviceBuffer(src[7].nbytes)
                kp.copy_from_device(src[6], src[6].nbytes)
                vp.copy_from_device(src[7], src[7].nbytes)
                q4 = []
                for j in range(2, 6):
                    trio = []
                    for buf in src[j]:
                        nb = hip.DeviceBuffer(buf.nbytes)
                        nb.copy_from_device(buf, buf.nbytes)
                        trio.append(nb)
                    q4.append(trio)
                n1, n2 = src[0], src[1]
            else:
                n1, n2 = up(L["norm1"].astype(np.float32)), up(L["norm2"].astype(np.float32))
                q4 = []
                for name in ("qkv", "o", "gate_up", "down"):
                    t = L[name]
                    q4.append([up(np.ascontiguousarray(t[0])),
                               up(np.ascontiguousarray(t[1]).view(np.uint16)),
                               up(np.ascontiguousarray(t[2]).view(np.uint16))])
                kp, vp = up(L["k_pool"]), up(L["v_pool"])
                if first is None:
                    first = (n1, n2, q4[0], q4[1], q4[2], q4[3], kp, vp)
            self.keep += [n1, n2, kp, vp] + [x for t in q4 for x in t]
            self.pools.append((kp, vp))
            lay = self.layers[i]
            lay.norm1_w_f32, lay.norm2_w_f32 = _val(n1), _val(n2)
            for name, trio in zip(("qkv", "o", "gate_up", "down"), q4):
                setattr(lay, name, kernels.Q4Weight(*[_val(x) for x in trio]))
            lay.k_pool_f16, lay.v_pool_f16 = _val(kp), _val(vp)
            if L.get("qkv_bias") is not None:
                bb = up(np.ascontiguousarray(L["qkv_bias"], np.float32))
                self.keep.append(bb)
                lay.qkv_bias_f32 = _val(bb)

        self.h = up(batch["h"].astype(np.float32))
        self.out = hip.DeviceBuffer(b * cfg["hidden"] * 2)
        self.out.fill(0xFF)
        names = ("block_tables", "cu_seqlens", "context_lens", "positions")
        self.idx = {n: up(np.ascontiguousarray(batch[n], np.int32)) for n in names}
        self.slots = up(np.ascontiguousarray(batch["slots"], np.int64))
        self.cos, self.sin = up(batch["cos"]), up(batch["sin"])
        self.fnorm = up(batch["final_norm"].astype(np.float32))
        self.batch = kernels.DecodeBatch(
            _val(self.h), _val(self.out), _val(self.fnorm), _val(self.idx["block_tables"]),
            _val(self.idx["cu_seqlens"]), _val(self.idx["context_lens"]),
            _val(self.idx["positions"]), _val(self.slots), _val(self.cos), _val(self.sin), nseq,
            self.num_splits)
        if b != nseq:
            cu = np.asarray(batch["cu_seqlens"])
            self.batch.total_tokens = b
            self.batch.max_seqlen_q = int(np.diff(cu).max())
        self.vocab = self.cfg.vocab
        if self.vocab:
            # tokens in (embedding lookup) and tokens out (vocabulary projection + greedy)
            self.token_ids = up(np.ascontiguousarray(batch["token_ids"], np.uint32))
            self.embed = up(np.ascontiguousarray(batch["embed_table"], np.uint16))
            self.head = w3(batch["lm_head"])
            self.tokens = hip.DeviceBuffer(b * 4)
            self.tokens.fill(0xFF)
            self.logits = hip.DeviceBuffer(b * self.vocab * 4)
            self.logits.fill(0xFF)
            self.batch.token_ids = _val(self.token_ids)
            self.batch.embed_table_bf16 = _val(self.embed)
            self.batch.lm_head = C.pointer(self.head)
            self.batch.out_tokens_u32 = _val(self.tokens)
            self.batch.logits_f32 = _val(self.logits)
        ws = kernels.decode_step_workspace_bytes_tokens(self.cfg, nseq, b, self.num_splits)
        assert ws > 0
        self.ws = hip.DeviceBuffer(ws)
        self.ws.fill(0xFF)

    def launch(self):
        kernels.launch_decode_step(self.cfg, self.layers, self.batch, self.ws, self.stream)

    def result_bits(self) -> np.ndarray:
        (self.stream.synchronize() if self.stream else hip.synchronize())
        return self.out.to_numpy(np.uint16, (self.b, self.cfg_d["hidden"]))

    def result_tokens(self):
        """(tokens uint32 [B], logits fp32 [B, vocab]) of a step with an lm_head."""
        (self.stream.synchronize() if self.stream else hip.synchronize())
        return (self.tokens.to_numpy(np.uint32, (self.b,)),
                self.logits.to_numpy(np.float32, (self.b, self.vocab)))


def assert_parity(got, want, max_abs=2e-3, max_rel=1e-2, what=""):
    """Tolerance of the decode path for fp16/bf16 outputs with fp32 accumulation:
    every element within max_abs OR within max_rel of the oracle (relative error
    with the reference's denominator floor, crates/kernels/tests/matmul_parity.rs:83-99)."""
    got = np.asarray(got, np.float32)
    want = np.asarray(want, np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    rel = err / np.maximum(np.abs(want), 1e-3)
    bad = (err > max_abs) & (rel > max_rel)
    assert not bad.any(), (f"{what}: {int(bad.sum())} elements out of tolerance; "
                           f"max_abs={err.max():.3e} max_rel={rel.max():.3e}")
    return float(err.max()), float(rel.max())
