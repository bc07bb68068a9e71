"""ctypes binding of the CPU oracle (``oracle/liblogismos_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  The shipped package
(``logismos_amd``) never imports this module.

The functions mirror ``oracle/logismos_oracle.h`` one to one, taking and
returning numpy arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblogismos_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_sz = C.c_size_t
_vp = C.c_void_p


def _p(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return a.ctypes.data_as(_vp)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


# ---------------------------------------------------------------- conversions
_f32_to_f16 = _sig("oracle_f32_to_f16_n", None, _vp, _vp, _sz)
_f16_to_f32 = _sig("oracle_f16_to_f32_n", None, _vp, _vp, _sz)
_f32_to_bf16 = _sig("oracle_f32_to_bf16_n", None, _vp, _vp, _sz)
_bf16_to_f32 = _sig("oracle_bf16_to_f32_n", None, _vp, _vp, _sz)


def f32_to_f16_bits(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty(x.shape, np.uint16)
    _f32_to_f16(_p(x), _p(y), x.size)
    return y


def f16_bits_to_f32(h) -> np.ndarray:
    h = _u16(h)
    y = np.empty(h.shape, np.float32)
    _f16_to_f32(_p(h), _p(y), h.size)
    return y


def f32_to_bf16_bits(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty(x.shape, np.uint16)
    _f32_to_bf16(_p(x), _p(y), x.size)
    return y


def bf16_bits_to_f32(h) -> np.ndarray:
    h = _u16(h)
    y = np.empty(h.shape, np.float32)
    _bf16_to_f32(_p(h), _p(y), h.size)
    return y


# ---------------------------------------------------------------- cpu_f32
_embed_lookup = _sig("oracle_embed_lookup", None, _vp, _sz, _sz, _vp, _sz, _vp)
_rms_norm = _sig("oracle_rms_norm", None, _vp, _vp, _vp, _sz, _sz, C.c_float)
_linear = _sig("oracle_linear", None, _vp, _vp, _vp, _vp, _sz, _sz, _sz)
_linear_t = _sig("oracle_linear_t", None, _vp, _vp, _vp, _vp, _sz, _sz, _sz)
_silu = _sig("oracle_silu", None, _vp, _vp, _sz)
_hadamard = _sig("oracle_hadamard", None, _vp, _vp, _vp, _sz)
_softmax = _sig("oracle_softmax_last_dim", None, _vp, _vp, _sz, _sz)
_mask = _sig("oracle_mask_additive_in_place", C.c_int, _vp, _vp, _sz, _sz, _sz)
_rope = _sig("oracle_rope_halves_in_place", None, _vp, _vp, _vp, _sz, _sz)
_rope_table = _sig("oracle_build_rope_table_f32", None, _sz, _sz, C.c_double, _vp, _vp)


def embed_lookup(weight, hidden, vocab, ids):
    weight = _f32(weight)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    out = np.empty(ids.size * hidden, np.float32)
    _embed_lookup(_p(weight), hidden, vocab, _p(ids), ids.size, _p(out))
    return out


def rms_norm(x, weight, rows, n, eps):
    x, weight = _f32(x), _f32(weight)
    y = np.empty(rows * n, np.float32)
    _rms_norm(_p(x), _p(weight), _p(y), rows, n, eps)
    return y


def linear(a, b, bias, m, n, k):
    a, b = _f32(a), _f32(b)
    if a.size != m * k or b.size != k * n or (bias is not None and np.size(bias) != n):
        raise ValueError("linear: operand length does not match declared shape")
    bias = None if bias is None else _f32(bias)
    c = np.empty(m * n, np.float32)
    _linear(_p(a), _p(b), _p(bias), _p(c), m, n, k)
    return c


def linear_t(a, b, bias, m, n, k):
    a, b = _f32(a), _f32(b)
    if a.size != m * k or b.size != n * k or (bias is not None and np.size(bias) != n):
        raise ValueError("linear_t: operand length does not match declared shape")
    bias = None if bias is None else _f32(bias)
    c = np.empty(m * n, np.float32)
    _linear_t(_p(a), _p(b), _p(bias), _p(c), m, n, k)
    return c


def silu(x):
    x = _f32(x)
    y = np.empty_like(x)
    _silu(_p(x), _p(y), x.size)
    return y


def hadamard(a, b):
    a, b = _f32(a), _f32(b)
    if a.size != b.size:
        raise ValueError("hadamard: mismatched operand lengths")
    c = np.empty_like(a)
    _hadamard(_p(a), _p(b), _p(c), a.size)
    return c


def softmax_last_dim(x, rows, n):
    x = _f32(x)
    y = np.empty(rows * n, np.float32)
    _softmax(_p(x), _p(y), rows, n)
    return y


def mask_additive_in_place(scores: np.ndarray, mask, rows, n):
    assert scores.dtype == np.float32
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    rc = _mask(_p(scores), _p(mask), mask.size, rows, n)
    if rc != 0:
        raise ValueError("mask_additive_in_place: rows is not a multiple of mask_rows")


def rope_halves_in_place(x: np.ndarray, cos, sin, rows, head_dim):
    assert x.dtype == np.float32
    cos, sin = _f32(cos), _f32(sin)
    _rope(_p(x), _p(cos), _p(sin), rows, head_dim)


def build_rope_table_f32(seq, head_dim, theta):
    half = head_dim // 2
    cos = np.empty(seq * half, np.float32)
    sin = np.empty(seq * half, np.float32)
    _rope_table(seq, head_dim, float(theta), _p(cos), _p(sin))
    return cos, sin


# ---------------------------------------------------------------- fp16 refs
_matmul_fp16 = _sig("oracle_matmul_fp16_ref", None, _vp, _vp, _vp, _sz, _sz, _sz)
_softmax_fp16 = _sig("oracle_softmax_fp16_ref", None, _vp, _vp, _sz, _sz)
_rms_norm_fp16 = _sig("oracle_rms_norm_fp16_ref", None, _vp, _vp, _vp, _sz, _sz, C.c_float)


def matmul_fp16_ref(a, b, m, n, k):
    a, b = _u16(a), _u16(b)
    d = np.empty(m * n, np.uint16)
    _matmul_fp16(_p(a), _p(b), _p(d), m, n, k)
    return d.view(np.float16)


def softmax_fp16_ref(x, m, n):
    x = _u16(x)
    if x.size != m * n:
        raise ValueError("softmax_fp16_ref: x.len() != m*n")
    y = np.empty(m * n, np.uint16)
    _softmax_fp16(_p(x), _p(y), m, n)
    return y.view(np.float16)


def rms_norm_fp16_ref(x, w, m, n, eps):
    x, w = _u16(x), _u16(w)
    y = np.empty(m * n, np.uint16)
    _rms_norm_fp16(_p(x), _p(w), _p(y), m, n, eps)
    return y.view(np.float16)


_cos_sin_table = _sig("oracle_build_cos_sin_table", None, _sz, _sz, C.c_float, _vp)
_rope_fp16 = _sig("oracle_rope_apply_fp16_ref", None, _vp, _vp, _sz, _sz, _sz, _sz)


def build_cos_sin_table(seq, head_dim, theta_base):
    """`build_cos_sin_table` (crates/kernels/src/rope/cpu.rs:19-40): f32 [seq*head_dim]."""
    assert head_dim % 2 == 0
    t = np.empty(seq * head_dim, np.float32)
    _cos_sin_table(seq, head_dim, theta_base, _p(t))
    return t


def rope_apply_fp16_ref(qk, cos_sin, batch, seq, heads, head_dim):
    """`rope_apply_fp16_ref` (crates/kernels/src/rope/cpu.rs:56-127), returns the rotated copy;
    length mismatches are refused as there (:63-84)."""
    qk = _u16(qk).copy()
    cos_sin = _f32(cos_sin)
    if qk.size != batch * seq * heads * head_dim:
        raise ValueError(f"rope_apply_fp16_ref: qk.len()={qk.size} != batch*seq*heads*head_dim="
                         f"{batch * seq * heads * head_dim}")
    if cos_sin.size != seq * head_dim:
        raise ValueError(f"rope_apply_fp16_ref: cos_sin.len()={cos_sin.size} != seq*head_dim="
                         f"{seq * head_dim}")
    _rope_fp16(_p(qk), _p(cos_sin), batch, seq, heads, head_dim)
    return qk.view(np.float16)


# ---------------------------------------------------------------- attention pieces
_transpose = _sig("oracle_transpose_seq_heads", None, _vp, _vp, _sz, _sz, _sz)
_merge = _sig("oracle_merge_heads", None, _vp, _vp, _sz, _sz, _sz)
_repeat_kv = _sig("oracle_repeat_kv", None, _vp, _vp, _sz, _sz, _sz, _sz)
_sdpa = _sig("oracle_sdpa_f32", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz)
_greedy = _sig("oracle_greedy", C.c_uint32, _vp, _sz)


def transpose_seq_heads(x, seq, heads, d):
    x = _f32(x)
    out = np.empty(seq * heads * d, np.float32)
    _transpose(_p(x), _p(out), seq, heads, d)
    return out


def merge_heads(attn, heads, seq, d):
    attn = _f32(attn)
    out = np.empty(seq * heads * d, np.float32)
    _merge(_p(attn), _p(out), heads, seq, d)
    return out


def repeat_kv(kv, n_kv, groups, seq, d):
    kv = _f32(kv)
    out = np.empty(n_kv * groups * seq * d, np.float32)
    _repeat_kv(_p(kv), _p(out), n_kv, groups, seq, d)
    return out


def sdpa_f32(q_hsd, k_hsd, v_hsd, mask, n_h, n_kv, seq, d):
    q_hsd, k_hsd, v_hsd = _f32(q_hsd), _f32(k_hsd), _f32(v_hsd)
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    out = np.empty(n_h * seq * d, np.float32)
    _sdpa(_p(q_hsd), _p(k_hsd), _p(v_hsd), _p(mask), _p(out), n_h, n_kv, seq, d)
    return out


def greedy(logits) -> int:
    logits = _f32(logits)
    return int(_greedy(_p(logits), logits.size))


# ---------------------------------------------------------------- nibbles / quant
_pack_nib = _sig("oracle_pack_nibbles", C.c_int, _vp, _sz, _vp)
_unpack_nib = _sig("oracle_unpack_nibbles", None, _vp, _sz, _vp)
_quant_q8 = _sig("oracle_quantize_q8g32", None, _vp, _vp, _vp, _sz, _sz)
_dequant_q8 = _sig("oracle_dequantize_q8g32", None, _vp, _vp, _vp, _sz, _sz)
_to_blocks = _sig("oracle_q8g32_to_q8_0_blocks", None, _vp, _vp, _vp, _sz, _sz)
_from_blocks = _sig("oracle_q8_0_blocks_to_q8g32", None, _vp, _vp, _vp, _sz, _sz)
_qgemv_q8 = _sig("oracle_qgemv_q8g32_f32", None, _vp, _vp, _vp, _vp, _sz, _sz)
_quant_q4 = _sig("oracle_quantize_q4g128", None, _vp, _vp, _vp, _vp, _sz, _sz)
_dequant_q4 = _sig("oracle_dequantize_q4g128", None, _vp, _vp, _vp, _vp, _sz, _sz)
_qgemm_q4 = _sig("oracle_qgemm_q4g128_bf16", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz)


def pack_nibbles(idx):
    idx = np.ascontiguousarray(idx, dtype=np.uint8)
    assert idx.size % 2 == 0
    out = np.empty(idx.size // 2, np.uint8)
    if _pack_nib(_p(idx), idx.size, _p(out)) != 0:
        raise ValueError("pack_nibbles: index out of range")
    return out


def unpack_nibbles(packed, n):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(n, np.uint8)
    _unpack_nib(_p(packed), n, _p(out))
    return out


_quant_q4_0 = _sig("oracle_quantize_q4_0_blocks", None, _vp, _vp, _sz, _sz)
_quant_q4_1 = _sig("oracle_quantize_q4_1_blocks", None, _vp, _vp, _sz, _sz)
_dequant_q4_0 = _sig("oracle_dequantize_q4_0_blocks", None, _vp, _vp, _sz, _sz)
_dequant_q4_1 = _sig("oracle_dequantize_q4_1_blocks", None, _vp, _vp, _sz, _sz)
_q4_blocks_to_planar = _sig("oracle_q4_blocks_to_q4g32", None, _vp, C.c_int, _vp, _vp, _vp, _sz,
                            _sz)
_dequant_q4g32 = _sig("oracle_dequantize_q4g32", None, _vp, _vp, _vp, _vp, _sz, _sz)
_qgemv_q4g32 = _sig("oracle_qgemv_q4g32_f32", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz)


def quantize_q4_blocks(w, n, k, has_min):
    """ggml Q4_0 (has_min False, 18-byte blocks) or Q4_1 (True, 20-byte blocks) stream."""
    w = _f32(w)
    assert w.size == n * k and k % 32 == 0
    blocks = np.empty(n * (k // 32) * (20 if has_min else 18), np.uint8)
    (_quant_q4_1 if has_min else _quant_q4_0)(_p(w), _p(blocks), n, k)
    return blocks


def dequantize_q4_blocks(blocks, n, k, has_min):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    w = np.empty((n, k), np.float32)
    (_dequant_q4_1 if has_min else _dequant_q4_0)(_p(blocks), _p(w), n, k)
    return w


def q4_blocks_to_q4g32(blocks, n, k, has_min):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    qw = np.empty((n, k // 2), np.uint8)
    scale = np.empty((n, k // 32), np.uint16)
    minv = np.empty((n, k // 32), np.uint16)
    _q4_blocks_to_planar(_p(blocks), 1 if has_min else 0, _p(qw), _p(scale), _p(minv), n, k)
    return qw, scale.view(np.float16), minv.view(np.float16)


def dequantize_q4g32(qw, scale, minv, n, k):
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    scale, minv = _u16(scale), _u16(minv)
    w = np.empty((n, k), np.float32)
    _dequant_q4g32(_p(qw), _p(scale), _p(minv), _p(w), n, k)
    return w



def _add_bias(y, bias):
    """`linear_t`'s bias (crates/kernels/src/cpu_f32/mod.rs:336-343): one fp32 add per output,
    after the accumulation, broadcast over the rows."""
    if bias is None:
        return y
    bias = _f32(bias)
    assert bias.shape == (y.shape[-1],)
    return (y + bias).astype(np.float32)


def qgemv_q4g32_f32(x, qw, scale, minv, n, k, bias=None):
    x = _f32(x)
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    scale, minv = _u16(scale), _u16(minv)
    y = np.empty(n, np.float32)
    _qgemv_q4g32(_p(x), _p(qw), _p(scale), _p(minv), _p(y), n, k)
    return _add_bias(y, bias)


def qgemm_q4g32_f32(x_bf16_bits, qw, scale, minv, b, n, k, bias=None):
    """`linear_t` (crates/kernels/src/cpu_f32/mod.rs:271-345) at m = b over the dequantised Q4G32
    matrix: the GEMV above once per batch row, x given as bf16 bits; fp32 result."""
    x = bf16_bits_to_f32(np.asarray(x_bf16_bits).reshape(b, k))
    return np.stack([qgemv_q4g32_f32(x[i], qw, scale, minv, n, k, bias) for i in range(b)])


def qgemm_q4g32_bf16(x_bf16_bits, qw, scale, minv, b, n, k, bias=None):
    """The same, rounded once to bf16 (round to nearest even) like the Q4G128 GEMM's output."""
    return f32_to_bf16_bits(qgemm_q4g32_f32(x_bf16_bits, qw, scale, minv, b, n, k, bias))


def quantize_q8g32(w, n, k):
    w = _f32(w)
    assert w.size == n * k and k % 32 == 0
    qs = np.empty((n, k), np.int8)
    d = np.empty((n, k // 32), np.uint16)
    _quant_q8(_p(w), _p(qs), _p(d), n, k)
    return qs, d.view(np.float16)


def dequantize_q8g32(qs, d, n, k):
    qs = np.ascontiguousarray(qs, dtype=np.int8)
    d = _u16(d)
    w = np.empty((n, k), np.float32)
    _dequant_q8(_p(qs), _p(d), _p(w), n, k)
    return w


def q8g32_to_q8_0_blocks(qs, d, n, k):
    qs = np.ascontiguousarray(qs, dtype=np.int8)
    d = _u16(d)
    blocks = np.empty(n * (k // 32) * 34, np.uint8)
    _to_blocks(_p(qs), _p(d), _p(blocks), n, k)
    return blocks


def q8_0_blocks_to_q8g32(blocks, n, k):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    qs = np.empty((n, k), np.int8)
    d = np.empty((n, k // 32), np.uint16)
    _from_blocks(_p(blocks), _p(qs), _p(d), n, k)
    return qs, d.view(np.float16)


def qgemv_q8g32_f32(x, qs, d, n, k, bias=None):
    x = _f32(x)
    qs = np.ascontiguousarray(qs, dtype=np.int8)
    d = _u16(d)
    y = np.empty(n, np.float32)
    _qgemv_q8(_p(x), _p(qs), _p(d), _p(y), n, k)
    return _add_bias(y, bias)


def quantize_q4g128(w, n, k):
    w = _f32(w)
    assert w.size == n * k and k % 128 == 0
    qw = np.empty((n, k // 2), np.uint8)
    scale = np.empty((n, k // 128), np.uint16)
    zero = np.empty((n, k // 128), np.uint16)
    _quant_q4(_p(w), _p(qw), _p(scale), _p(zero), n, k)
    return qw, scale.view(np.float16), zero.view(np.float16)


def dequantize_q4g128(qw, scale, zero, n, k):
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    scale, zero = _u16(scale), _u16(zero)
    w = np.empty((n, k), np.float32)
    _dequant_q4(_p(qw), _p(scale), _p(zero), _p(w), n, k)
    return w


_qgemm_q4_f32 = _sig("oracle_qgemm_q4g128_f32", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz)


def qgemm_q4g128_f32(x_bf16_bits, qw, scale, zero, b, n, k, bias=None):
    x = _u16(x_bf16_bits)
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    scale, zero = _u16(scale), _u16(zero)
    y = np.empty((b, n), np.float32)
    _qgemm_q4_f32(_p(x), _p(qw), _p(scale), _p(zero), _p(y), b, n, k)
    return _add_bias(y, bias)


def qgemm_q4g128_bf16(x_bf16_bits, qw, scale, zero, b, n, k, bias=None):
    if bias is not None:  # the bias goes onto the fp32 sum, before the one rounding
        return f32_to_bf16_bits(qgemm_q4g128_f32(x_bf16_bits, qw, scale, zero, b, n, k, bias))
    x = _u16(x_bf16_bits)
    qw = np.ascontiguousarray(qw, dtype=np.uint8)
    scale, zero = _u16(scale), _u16(zero)
    y = np.empty((b, n), np.uint16)
    _qgemm_q4(_p(x), _p(qw), _p(scale), _p(zero), _p(y), b, n, k)
    return y


# ---------------------------------------------------------------- ragged packing / paged KV
_pack_ragged = _sig("oracle_pack_ragged", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz)
_kv_write = _sig("oracle_kv_write_fp16", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz)
_gather = _sig("oracle_paged_gather_fp16", None, _vp, _vp, _sz, _sz, _sz, _vp)
_paged_attn = _sig("oracle_paged_attn_varlen_fp16", None, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz,
                   _sz, _sz, _sz, _sz, _sz, C.c_float, C.c_int)


def pack_ragged(new_tokens, prior_ctx, block_tables, block_size):
    new_tokens = np.ascontiguousarray(new_tokens, dtype=np.int32)
    prior_ctx = np.ascontiguousarray(prior_ctx, dtype=np.int32)
    block_tables = np.ascontiguousarray(block_tables, dtype=np.int32)
    s = new_tokens.size
    max_blocks = block_tables.shape[1] if s else 0
    total = int(new_tokens.clip(min=0).sum())
    cu = np.empty(s + 1, np.int32)
    slots = np.empty(total, np.int64)
    ctx = np.empty(s, np.int32)
    rc = _pack_ragged(_p(new_tokens), _p(prior_ctx), _p(block_tables), _p(cu), _p(slots), _p(ctx),
                      s, block_size, max_blocks)
    if rc < 0:
        raise ValueError("pack_ragged: negative token count")
    return cu, slots, ctx, rc


def kv_write_fp16(k_new, v_new, k_pool, v_pool, slot_mapping, row_elems):
    k_new, v_new = _u16(k_new), _u16(v_new)
    slot_mapping = np.ascontiguousarray(slot_mapping, dtype=np.int64)
    kp, vp = _u16(k_pool), _u16(v_pool)
    _kv_write(_p(k_new), _p(v_new), _p(kp), _p(vp), _p(slot_mapping), slot_mapping.size, row_elems)


def paged_gather_fp16(pool, block_table_row, ctx, block_size, row_elems):
    pool = _u16(pool)
    bt = np.ascontiguousarray(block_table_row, dtype=np.int32)
    out = np.empty((ctx, row_elems), np.uint16)
    _gather(_p(pool), _p(bt), ctx, block_size, row_elems, _p(out))
    return out.view(np.float16)


_paged_attn_f32 = _sig("oracle_paged_attn_varlen_fp16_f32out", None, _vp, _vp, _vp, _vp, _vp, _vp,
                       _vp, _sz, _sz, _sz, _sz, _sz, _sz, C.c_float, C.c_int)


def paged_attn_varlen_fp16(q, k_pool, v_pool, block_tables, cu_seqlens_q, context_lens,
                           num_q_heads, num_kv_heads, head_dim, block_size, scale, causal=True,
                           f32_out=False):
    q, k_pool, v_pool = _u16(q), _u16(k_pool), _u16(v_pool)
    block_tables = np.ascontiguousarray(block_tables, dtype=np.int32)
    cu = np.ascontiguousarray(cu_seqlens_q, dtype=np.int32)
    ctx = np.ascontiguousarray(context_lens, dtype=np.int32)
    num_seqs = ctx.size
    out = np.zeros(q.shape, np.float32 if f32_out else np.uint16)
    (_paged_attn_f32 if f32_out else _paged_attn)(
        _p(q), _p(k_pool), _p(v_pool), _p(block_tables), _p(cu), _p(ctx), _p(out), num_seqs,
        num_q_heads, num_kv_heads, head_dim, block_size,
        block_tables.shape[1] if num_seqs else 0, scale, 1 if causal else 0)
    return out if f32_out else out.view(np.float16)


# ---------------------------------------------------------------- TurboQuant 3-bit KV
_t3_codebook = _sig("oracle_turbo3_codebook", None, _vp)
_fwht = _sig("oracle_fwht_128", None, _vp)
_t3_pack = _sig("oracle_pack_turbo3_indices", C.c_int, _vp, _vp)
_t3_unpack = _sig("oracle_unpack_turbo3_indices", None, _vp, _vp)
_t3_encode = _sig("oracle_encode_turbo3_0_head", None, _vp, _vp)
_t3_decode = _sig("oracle_decode_turbo3_0_head", None, _vp, _vp)
_t3_kv_write = _sig("oracle_kv_write_turbo3", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz)
_t3_gather = _sig("oracle_paged_gather_turbo3", None, _vp, _vp, _sz, _sz, _sz, _vp)
_t3_attn = _sig("oracle_paged_attn_varlen_turbo3", None, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz,
                _sz, _sz, _sz, _sz, C.c_float, C.c_int)
_t3_attn_f32 = _sig("oracle_paged_attn_varlen_turbo3_f32out", None, _vp, _vp, _vp, _vp, _vp, _vp,
                    _vp, _sz, _sz, _sz, _sz, _sz, C.c_float, C.c_int)
TURBO3_BYTES_PER_HEAD = 56


def turbo3_codebook():
    out = np.empty(8, np.float32)
    _t3_codebook(_p(out))
    return out


def fwht_128(data):
    d = _f32(data).copy()
    assert d.size == 128
    _fwht(_p(d))
    return d


def pack_turbo3_indices(idx):
    idx = np.ascontiguousarray(idx, dtype=np.uint8)
    assert idx.size == 32
    out = np.empty(12, np.uint8)
    pos = _t3_pack(_p(idx), _p(out))
    if pos >= 0:
        raise ValueError(f"turbo3 index out of range at position {pos}: {int(idx[pos])} > 7")
    return out


def unpack_turbo3_indices(packed):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size == 12
    out = np.empty(32, np.uint8)
    _t3_unpack(_p(packed), _p(out))
    return out


def encode_turbo3_0_head(values):
    v = _f32(values)
    if v.size != 128:
        raise ValueError(f"invalid head dim: got {v.size}, expected 128")
    out = np.empty(56, np.uint8)
    _t3_encode(_p(v), _p(out))
    return out


def decode_turbo3_0_head(blocks):
    b = np.ascontiguousarray(blocks, dtype=np.uint8)
    if b.size != 56:
        raise ValueError(f"invalid block count: got {b.size} bytes, expected 56")
    out = np.empty(128, np.float32)
    _t3_decode(_p(b), _p(out))
    return out


def kv_write_turbo3(k_new, v_new, k_pool, v_pool, slot_mapping, num_kv_heads):
    """In place: k_pool / v_pool uint8 [rows][num_kv_heads*56]."""
    k_new, v_new = _u16(k_new), _u16(v_new)
    slots = np.ascontiguousarray(slot_mapping, dtype=np.int64)
    assert k_pool.dtype == np.uint8 and k_pool.flags.c_contiguous
    assert v_pool.dtype == np.uint8 and v_pool.flags.c_contiguous
    _t3_kv_write(_p(k_new), _p(v_new), _p(k_pool), _p(v_pool), _p(slots), slots.size, num_kv_heads)


def paged_gather_turbo3(pool, block_table_row, ctx, block_size, num_kv_heads):
    pool = np.ascontiguousarray(pool, dtype=np.uint8)
    bt = np.ascontiguousarray(block_table_row, dtype=np.int32)
    out = np.empty((ctx, num_kv_heads * 128), np.float32)
    _t3_gather(_p(pool), _p(bt), ctx, block_size, num_kv_heads, _p(out))
    return out


def paged_attn_varlen_turbo3(q, k_pool, v_pool, block_tables, cu_seqlens_q, context_lens,
                             num_q_heads, num_kv_heads, block_size, scale, causal=True,
                             f32_out=False):
    q = _u16(q)
    k_pool = np.ascontiguousarray(k_pool, dtype=np.uint8)
    v_pool = np.ascontiguousarray(v_pool, dtype=np.uint8)
    block_tables = np.ascontiguousarray(block_tables, dtype=np.int32)
    cu = np.ascontiguousarray(cu_seqlens_q, dtype=np.int32)
    ctx = np.ascontiguousarray(context_lens, dtype=np.int32)
    num_seqs = ctx.size
    out = np.zeros(q.shape, np.float32 if f32_out else np.uint16)
    (_t3_attn_f32 if f32_out else _t3_attn)(
        _p(q), _p(k_pool), _p(v_pool), _p(block_tables), _p(cu), _p(ctx), _p(out), num_seqs,
        num_q_heads, num_kv_heads, block_size, block_tables.shape[1] if num_seqs else 0, scale,
        1 if causal else 0)
    return out if f32_out else out.view(np.float16)


# ---------------------------------------------------------------- metric / threads
_metric = _sig("oracle_parity_metric_f32", None, _vp, _vp, _sz, C.POINTER(C.c_float),
               C.POINTER(C.c_float))
num_threads = _sig("oracle_num_threads", C.c_int)
set_num_threads = _sig("oracle_set_num_threads", None, C.c_int)


def parity_metric(got, want):
    """(max_abs, max_rel) with the reference's denominator floor of 1e-3."""
    got, want = _f32(got).ravel(), _f32(want).ravel()
    assert got.size == want.size
    ma, mr = C.c_float(), C.c_float()
    _metric(_p(got), _p(want), got.size, C.byref(ma), C.byref(mr))
    return ma.value, mr.value
