"""Python mirror of the reference's ``kernels::launch_*`` wrappers for the
decode path (crates/kernels/src/matmul/mod.rs:140-186 is the template):
host-side shape guard -> FFI call with raw device pointers, i32 dims and the
raw stream -> non-zero status becomes ``LaunchError`` carrying the classified
kind.  The library is loaded from ``logismos_amd/lib``; there is no fallback.
"""
from __future__ import annotations

import ctypes as C
import os

from . import hip

_HERE = os.path.dirname(os.path.abspath(__file__))
# LOGISMOS_KERNELS_LIB points at an alternative build of the same ABI.
LIB_PATH = os.environ.get("LOGISMOS_KERNELS_LIB") or os.path.join(_HERE, "lib",
                                                                 "liblogismos_kernels.so")

_lib = None


class NoGpuBuild(RuntimeError):
    """`Error::NoGpuBuild` (crates/kernels/src/error.rs:55-63): the kernel archive is absent."""


class UnsupportedShape(ValueError):
    """`Error::UnsupportedShape` (crates/kernels/src/error.rs:44-53)."""

    def __init__(self, kernel: str, msg: str):
        self.kernel, self.msg = kernel, msg
        super().__init__(f"kernel {kernel}: unsupported shape: {msg}")


class LaunchError(RuntimeError):
    """`Error::Launch` (crates/kernels/src/error.rs:27-42)."""

    def __init__(self, kernel: str, code: int):
        self.kernel, self.code, self.kind = kernel, int(code), hip.error_kind(code)
        super().__init__(f"kernel {kernel}: launch failed: {self.kind} (code {self.code})")


_vp, _i, _f, _sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t

_SIGNATURES = {
    "logismos_decode_abi_version": (C.c_int, []),
    "logismos_decode_offload_arch": (C.c_char_p, []),
    "logismos_check_qgemv_q8g32_shape": (C.c_uint32, [_i, _i, C.c_char_p, _sz]),
    "logismos_check_paged_attn_shape": (C.c_uint32, [_i] * 9 + [C.c_char_p, _sz]),
    "logismos_launch_qgemv_q8g32_f32": (C.c_uint32, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "logismos_launch_qgemv_q8g32_f32_bias": (C.c_uint32, [_vp] * 5 + [_i, _i, _vp]),
    "logismos_launch_qgemm_q4g128_bf16_bias": (C.c_uint32, [_vp] * 6 + [_i, _i, _i, _vp]),
    "logismos_launch_qgemv_q4g32_f32_bias": (C.c_uint32, [_vp] * 6 + [_i, _i, _vp]),
    "logismos_launch_qgemm_q4g32_bf16_bias": (C.c_uint32, [_vp] * 6 + [_i, _i, _i, _vp]),
    "logismos_check_qgemm_q4g128_shape": (C.c_uint32, [_i, _i, _i, C.c_char_p, _sz]),
    "logismos_launch_qgemm_q4g128_bf16": (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_launch_qgemm_q4g128_bf16_mfma": (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_check_qgemm_q4g128_tall_shape": (C.c_uint32, [_i, _i, _i, C.c_char_p, _sz]),
    "logismos_qgemm_q4g128_tall_workspace_bytes": (_sz, [_i, _i]),
    "logismos_launch_qgemm_q4g128_tall": (C.c_uint32, [_vp] * 6 + [_i, _vp, _i, _i, _i, _vp]),
    "logismos_qgemm_q4g128_tall_pairs_per_load": (C.c_int, [_i, _vp, _vp]),
    "logismos_launch_qgemm_q4g128_tall_prepared":
        (C.c_uint32, [_vp] * 5 + [_i, _vp, _i, _i, _i, _vp]),
    "logismos_launch_silu_mul_f32p_tall": (C.c_uint32, [_vp, _i, _vp, _i, _i, _i, _vp]),
    "logismos_launch_qgemm_q4g128_tall_swiglu_prepared":
        (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_launch_qgemm_q4g128_tall_swiglu_operand":
        (C.c_uint32, [_vp] * 4 + [_i, _vp, _i, _i, _i, _vp]),
    "logismos_launch_add_rms_norm_f32p_tall":
        (C.c_uint32, [_vp, _vp, _i, _vp, _vp, _i, _i, _f, _i, _vp]),
    "logismos_launch_repack_q8_0": (C.c_uint32, [_vp, _vp, _vp, _i, _i, _vp]),
    "logismos_check_qgemv_q4g32_shape": (C.c_uint32, [_i, _i, C.c_char_p, _sz]),
    "logismos_launch_qgemv_q4g32_f32": (C.c_uint32, [_vp] * 5 + [_i, _i, _vp]),
    "logismos_check_qgemm_q4g32_shape": (C.c_uint32, [_i, _i, _i, C.c_char_p, _sz]),
    "logismos_launch_qgemm_q4g32_bf16": (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_launch_repack_q4_0": (C.c_uint32, [_vp] * 4 + [_i, _i, _vp]),
    "logismos_launch_repack_q4_1": (C.c_uint32, [_vp] * 4 + [_i, _i, _vp]),
    "logismos_paged_attn_num_splits": (C.c_int, [_i, _i, _i, _i]),
    "logismos_paged_attn_num_splits_hd": (C.c_int, [_i, _i, _i, _i, _i]),
    "logismos_paged_attn_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "logismos_launch_paged_attn_varlen_fp16":
        (C.c_uint32, [_vp] * 8 + [_i] * 9 + [_f, _i, _vp]),
    "logismos_launch_paged_attn_varlen_fp16_phases":
        (C.c_uint32, [_vp] * 8 + [_i] * 9 + [_f, _i, _i, _vp]),
    "logismos_paged_attn_static_workspace_bytes": (_sz, []),
    "logismos_paged_attn_noalloc_init": (C.c_uint32, []),
    "logismos_launch_paged_attn_varlen_fp16_noalloc":
        (C.c_uint32, [_vp] * 7 + [_i] * 9 + [_f, _i, _vp]),
    "logismos_launch_paged_attn_decode_fp16_xprep":
        (C.c_uint32, [_vp] * 8 + [_i] * 7 + [_f, _vp]),
    "logismos_check_pack_ragged_shape": (C.c_uint32, [_i, _i, _i, C.c_char_p, _sz]),
    "logismos_launch_pack_ragged": (C.c_uint32, [_vp] * 6 + [_i, _i, _i, _vp]),
    "logismos_launch_kv_write_fp16": (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_launch_add_rms_norm_bf16": (C.c_uint32, [_vp] * 4 + [_i, _i, _f, _vp]),
    "logismos_launch_rope_kv_write_fp16": (C.c_uint32, [_vp] * 8 + [_i] * 5 + [_vp]),
    "logismos_launch_silu_mul_bf16": (C.c_uint32, [_vp, _vp, _i, _i, _vp]),
    "logismos_launch_cast_f16_bf16": (C.c_uint32, [_vp, _vp, _sz, _vp]),
    "logismos_launch_greedy_f32": (C.c_uint32, [_vp, _vp, _i, _i, _vp]),
    "logismos_launch_rms_norm_fp16": (C.c_uint32, [_vp, _vp, _vp, _i, _i, _f, _vp]),
    "logismos_launch_softmax_fp16": (C.c_uint32, [_vp, _vp, _i, _i, _vp]),
    "logismos_launch_mask_additive_f32": (C.c_uint32, [_vp, _vp, _sz, _sz, _sz, _vp]),
    "logismos_launch_mask_additive_fp16": (C.c_uint32, [_vp, _vp, _sz, _sz, _sz, _vp]),
    "logismos_launch_rope_fp16": (C.c_uint32, [_vp, _vp, _i, _i, _i, _i, _vp]),
    "logismos_launch_matmul_naive_fp16": (C.c_uint32, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "logismos_launch_matmul_wmma_fp16": (C.c_uint32, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "logismos_check_qgemm_q4g128_greedy_shape": (C.c_uint32, [_i, _i, _i, C.c_char_p, _sz]),
    "logismos_qgemm_q4g128_greedy_workspace_bytes": (_sz, [_i, _i, _i]),
    "logismos_launch_qgemm_q4g128_greedy_xprep": (C.c_uint32, [_vp] * 7 + [_i, _i, _i, _vp]),
    "logismos_launch_embed_lookup_f32": (C.c_uint32, [_vp, _vp, _vp, _i, _i, C.c_longlong, _vp]),
    "logismos_launch_embed_lookup_bf16": (C.c_uint32, [_vp, _vp, _vp, _i, _i, C.c_longlong, _vp]),
    "logismos_decode_step_workspace_bytes": (_sz, [_vp, _i, _i]),
    "logismos_decode_step_workspace_bytes_tokens": (_sz, [_vp, _i, _i, _i]),
    "logismos_launch_rope_kv_write_f32p_bias":
        (C.c_uint32, [_vp, _i] + [_vp] * 8 + [_i] * 5 + [_vp]),
    "logismos_launch_rope_kv_write_f32p_turbo3_bias":
        (C.c_uint32, [_vp, _i] + [_vp] * 8 + [_i] * 5 + [_vp]),
    "logismos_launch_decode_step": (C.c_uint32, [_vp, _vp, _vp, _vp, _vp]),
    "logismos_qgemm_q4g128_splitk_parts": (C.c_int, [_i, _i, _i]),
    "logismos_qgemm_q4g128_splitk_xprep_parts": (C.c_int, [_i, _i, _i]),
    "logismos_launch_qgemm_q4g128_f32_splitk": (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_launch_add_rms_norm_f32p": (C.c_uint32, [_vp, _vp, _i, _vp, _vp, _i, _i, _f, _vp]),
    "logismos_launch_rope_kv_write_f32p": (C.c_uint32, [_vp, _i] + [_vp] * 7 + [_i] * 5 + [_vp]),
    "logismos_launch_rope_kv_write_f32p_turbo3":
        (C.c_uint32, [_vp, _i] + [_vp] * 7 + [_i] * 5 + [_vp]),
    "logismos_launch_silu_mul_f32p": (C.c_uint32, [_vp, _i, _vp, _i, _i, _vp]),
    "logismos_q4_xprep_bytes": (_sz, [_i, _i]),
    "logismos_launch_q4_prepare_x_bf16": (C.c_uint32, [_vp, _vp, _i, _i, _vp]),
    "logismos_launch_qgemm_q4g128_f32_splitk_xprep": (C.c_uint32, [_vp] * 5 + [_i, _i, _i, _vp]),
    "logismos_launch_add_rms_norm_f32p_xprep":
        (C.c_uint32, [_vp, _vp, _i, _vp, _vp, _i, _i, _f, _vp]),
    "logismos_launch_silu_mul_f32p_xprep": (C.c_uint32, [_vp, _i, _vp, _i, _i, _vp]),
    "logismos_launch_kv_append_fp16": (C.c_uint32, [_vp] * 5 + [_i] * 5 + [_vp]),
    "logismos_launch_kv_gather_fp16": (C.c_uint32, [_vp] * 5 + [_i] * 5 + [_vp]),
    "logismos_paged_kv_cache_create": (C.c_int, [_vp, C.POINTER(_vp)]),
    "logismos_paged_kv_cache_destroy": (None, [_vp]),
    "logismos_paged_kv_cache_open_seq": (C.c_int, [_vp, C.POINTER(C.c_int)]),
    "logismos_paged_kv_cache_close_seq": (C.c_int, [_vp, _i]),
    "logismos_paged_kv_cache_reserve": (C.c_int, [_vp, _i, C.c_int64, _vp]),
    "logismos_paged_kv_cache_advance": (C.c_int, [_vp, _i, _i, _i]),
    "logismos_paged_kv_cache_put": (C.c_int, [_vp, _i, _i, _vp, _vp, _i, _vp]),
    "logismos_paged_kv_cache_get": (C.c_int, [_vp, _i, _i, C.c_int64, _vp, _vp, _vp]),
    "logismos_paged_kv_cache_len_of": (C.c_int64, [_vp, _i, _i]),
    "logismos_paged_kv_cache_num_layers": (C.c_int, [_vp]),
    "logismos_paged_kv_cache_reset": (None, [_vp]),
    "logismos_paged_kv_cache_free_blocks": (C.c_int, [_vp]),
    "logismos_paged_kv_cache_k_pool": (_vp, [_vp, _i]),
    "logismos_paged_kv_cache_v_pool": (_vp, [_vp, _i]),
    "logismos_paged_kv_cache_block_tables": (_vp, [_vp]),
    "logismos_paged_kv_cache_block_tables_host": (_vp, [_vp]),
    "logismos_launch_paged_attn_varlen_turbo3":
        (C.c_uint32, [_vp] * 8 + [_i] * 8 + [_f, _vp]),
    "logismos_launch_kv_write_turbo3": (C.c_uint32, [_vp] * 5 + [_i, _i, _vp]),
    "logismos_launch_kv_gather_turbo3_f32": (C.c_uint32, [_vp] * 5 + [_i] * 4 + [_vp]),
    "logismos_launch_probe_copy": (C.c_uint32, [_vp, _vp, _sz, _vp]),
    "logismos_launch_probe_read": (C.c_uint32, [_vp, _vp, _sz, _vp]),
    "logismos_launch_probe_read_ex": (C.c_uint32, [_vp, _vp, _sz, _i, _vp]),
    "logismos_launch_probe_mfma": (C.c_uint32, [_vp, _i, _i, _vp]),
    "logismos_probe_mfma_flops": (C.c_double, [_i]),
}

ATTN_PHASE_DECODE, ATTN_PHASE_PREFILL, ATTN_PHASE_MERGE, ATTN_PHASE_ALL = 1, 2, 4, 7


class PagedKvLayout(C.Structure):
    _fields_ = [("num_layers", _i), ("num_kv_heads", _i), ("head_dim", _i), ("block_size", _i),
                ("num_blocks", _i), ("max_seqs", _i), ("max_blocks_per_seq", _i)]


class Q4Weight(C.Structure):
    _fields_ = [("qw", _vp), ("scale", _vp), ("zero", _vp)]


class DecodeConfig(C.Structure):
    _fields_ = [("num_layers", _i), ("hidden", _i), ("num_q_heads", _i), ("num_kv_heads", _i),
                ("head_dim", _i), ("intermediate", _i), ("rms_eps", _f), ("block_size", _i),
                ("max_blocks_per_seq", _i), ("max_pos", _i), ("vocab", _i),
                ("kv_turbo3", _i)]


class DecodeLayer(C.Structure):
    _fields_ = [("norm1_w_f32", _vp), ("norm2_w_f32", _vp), ("qkv", Q4Weight), ("o", Q4Weight),
                ("gate_up", Q4Weight), ("down", Q4Weight), ("k_pool_f16", _vp),
                ("v_pool_f16", _vp), ("qkv_bias_f32", _vp)]


class DecodeBatch(C.Structure):
    _fields_ = [("hidden_f32", _vp), ("out_bf16", _vp), ("final_norm_w_f32", _vp),
                ("block_tables", _vp), ("cu_seqlens", _vp), ("context_lens", _vp),
                ("positions", _vp), ("slot_mapping", _vp), ("rope_cos_f32", _vp),
                ("rope_sin_f32", _vp), ("num_seqs", _i), ("num_splits", _i),
                ("token_ids", _vp), ("embed_table_bf16", _vp), ("lm_head", C.POINTER(Q4Weight)),
                ("out_tokens_u32", _vp), ("logits_f32", _vp), ("total_tokens", _i),
                ("max_seqlen_q", _i), ("tokens_for_last_rows", _i)]


def library() -> C.CDLL:
    """Loads the C-ABI library; raises NoGpuBuild when it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NoGpuBuild(f"{LIB_PATH} is missing: run `python -m logismos_amd.build` "
                             "(needs hipcc); there is no CPU fallback")
        hip._runtime()
        lib = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib


def exported_symbols() -> list[str]:
    return sorted(_SIGNATURES)


def _raw(stream) -> C.c_void_p | None:
    return stream.raw if stream is not None else None


def _ptr(x) -> C.c_void_p:
    return x.ptr if isinstance(x, (hip.DeviceBuffer, hip.DevicePtrView)) else x


def _guard(kernel: str, check_fn, *dims) -> None:
    msg = C.create_string_buffer(256)
    if check_fn(*dims, msg, len(msg)) != 0:
        raise UnsupportedShape(kernel, msg.value.decode())


def _status(kernel: str, code: int) -> None:
    if code != 0:
        raise LaunchError(kernel, code)


def check_qgemv_q4g32_shape(n: int, k: int) -> None:
    _guard("qgemv_q4g32_f32", library().logismos_check_qgemv_q4g32_shape, n, k)


def launch_qgemv_q4g32_f32(x, qw, scale, minv, y, n: int, k: int, stream=None,
                           bias=None) -> None:
    """`bias`: fp32 [n] on the device or None, as `linear_t`'s `bias: Option<&[f32]>`."""
    check_qgemv_q4g32_shape(n, k)
    _status("qgemv_q4g32_f32", library().logismos_launch_qgemv_q4g32_f32_bias(
        _ptr(x), _ptr(qw), _ptr(scale), _ptr(minv), _ptr(bias) if bias is not None else None,
        _ptr(y), n, k, _raw(stream)))


def check_qgemm_q4g32_shape(b: int, n: int, k: int) -> None:
    _guard("qgemm_q4g32_bf16", library().logismos_check_qgemm_q4g32_shape, b, n, k)


def launch_qgemm_q4g32_bf16(x, qw, scale, minv, y, b: int, n: int, k: int, stream=None,
                            bias=None) -> None:
    """Batched product over planar Q4G32 weights; x and y bf16; optional fp32 bias [n]."""
    check_qgemm_q4g32_shape(b, n, k)
    _status("qgemm_q4g32_bf16", library().logismos_launch_qgemm_q4g32_bf16_bias(
        _ptr(x), _ptr(qw), _ptr(scale), _ptr(minv), _ptr(bias) if bias is not None else None,
        _ptr(y), b, n, k, _raw(stream)))


def launch_repack_q4_blocks(blocks, qw, scale, minv, n: int, k: int, has_min: bool,
                            stream=None) -> None:
    """ggml Q4_1 (has_min) or Q4_0 block stream -> planar Q4G32."""
    check_qgemv_q4g32_shape(n, k)
    fn = (library().logismos_launch_repack_q4_1 if has_min
          else library().logismos_launch_repack_q4_0)
    _status("repack_q4_1" if has_min else "repack_q4_0",
            fn(_ptr(blocks), _ptr(qw), _ptr(scale), _ptr(minv), n, k, _raw(stream)))


def check_qgemv_q8g32_shape(n: int, k: int) -> None:
    _guard("qgemv_q8g32_f32", library().logismos_check_qgemv_q8g32_shape, n, k)


def launch_qgemv_q8g32_f32(x, qs, d, y, n: int, k: int, stream=None, bias=None) -> None:
    """`bias`: fp32 [n] on the device or None, as `linear_t`'s `bias: Option<&[f32]>`."""
    check_qgemv_q8g32_shape(n, k)
    if bias is None:
        code = library().logismos_launch_qgemv_q8g32_f32(
            _ptr(x), _ptr(qs), _ptr(d), _ptr(y), n, k, _raw(stream))
    else:
        code = library().logismos_launch_qgemv_q8g32_f32_bias(
            _ptr(x), _ptr(qs), _ptr(d), _ptr(bias), _ptr(y), n, k, _raw(stream))
    _status("qgemv_q8g32_f32", code)


def check_qgemm_q4g128_shape(b: int, n: int, k: int) -> None:
    _guard("qgemm_q4g128_bf16", library().logismos_check_qgemm_q4g128_shape, b, n, k)


def launch_qgemm_q4g128_bf16(x, qw, scale, zero, y, b: int, n: int, k: int, stream=None,
                             force_mfma: bool = False, bias=None) -> None:
    check_qgemm_q4g128_shape(b, n, k)
    if bias is not None:
        if force_mfma:
            raise ValueError("the forced matrix-core entry point takes no bias")
        _status("qgemm_q4g128_bf16", library().logismos_launch_qgemm_q4g128_bf16_bias(
            _ptr(x), _ptr(qw), _ptr(scale), _ptr(zero), _ptr(bias), _ptr(y), b, n, k,
            _raw(stream)))
        return
    fn = (library().logismos_launch_qgemm_q4g128_bf16_mfma if force_mfma
          else library().logismos_launch_qgemm_q4g128_bf16)
    _status("qgemm_q4g128_bf16", fn(_ptr(x), _ptr(qw), _ptr(scale), _ptr(zero), _ptr(y), b, n, k,
                                    _raw(stream)))


def qgemm_q4g128_tall_workspace_bytes(m: int, k: int) -> int:
    return library().logismos_qgemm_q4g128_tall_workspace_bytes(m, k)


def launch_qgemm_q4g128_tall(x, qw, scale, zero, y, workspace, m: int, n: int, k: int,
                             stream=None, bias=None, f32_out: bool = False) -> None:
    """`linear_t` over many rows through the tiled kernel with a workspace."""
    _guard("qgemm_q4g128_tall", library().logismos_check_qgemm_q4g128_tall_shape, m, n, k)
    _status("qgemm_q4g128_tall", library().logismos_launch_qgemm_q4g128_tall(
        _ptr(x), _ptr(qw), _ptr(scale), _ptr(zero), _ptr(bias) if bias is not None else None,
        _ptr(y), 1 if f32_out else 0, _ptr(workspace), m, n, k, _raw(stream)))


def qgemm_q4g128_tall_pairs_per_load(k: int, scale, zero) -> int:
    return library().logismos_qgemm_q4g128_tall_pairs_per_load(k, _ptr(scale), _ptr(zero))


def launch_qgemm_q4g128_tall_prepared(qw, scale, zero, y, workspace, m: int, n: int, k: int,
                                      stream=None, bias=None, f32_out: bool = False) -> None:
    """The tiled kernel alone over a workspace whose producer wrote x in the kernel's order."""
    _guard("qgemm_q4g128_tall", library().logismos_check_qgemm_q4g128_tall_shape, m, n, k)
    _status("qgemm_q4g128_tall_prepared", library().logismos_launch_qgemm_q4g128_tall_prepared(
        _ptr(qw), _ptr(scale), _ptr(zero), _ptr(bias) if bias is not None else None, _ptr(y),
        1 if f32_out else 0, _ptr(workspace), m, n, k, _raw(stream)))


def launch_qgemm_q4g128_tall_swiglu_prepared(qw, scale, zero, act, workspace, m: int, inter: int,
                                             k: int, stream=None) -> None:
    """gate/up projection + SwiGLU in one kernel over a prepared workspace: act bf16 [m][inter]."""
    _guard("qgemm_q4g128_tall", library().logismos_check_qgemm_q4g128_tall_shape, m, 2 * inter, k)
    _status("qgemm_q4g128_tall_swiglu_prepared",
            library().logismos_launch_qgemm_q4g128_tall_swiglu_prepared(
                _ptr(qw), _ptr(scale), _ptr(zero), _ptr(act), _ptr(workspace), m, inter, k,
                _raw(stream)))


def launch_qgemm_q4g128_tall_swiglu_operand(qw, scale, zero, next_workspace,
                                            next_pairs_per_load: int, workspace, m: int,
                                            inter: int, k: int, stream=None) -> None:
    """gate/up projection + SwiGLU, written as the operand of the following product."""
    _guard("qgemm_q4g128_tall", library().logismos_check_qgemm_q4g128_tall_shape, m, 2 * inter, k)
    _status("qgemm_q4g128_tall_swiglu_operand",
            library().logismos_launch_qgemm_q4g128_tall_swiglu_operand(
                _ptr(qw), _ptr(scale), _ptr(zero), _ptr(next_workspace), next_pairs_per_load,
                _ptr(workspace), m, inter, k, _raw(stream)))


def launch_silu_mul_f32p_tall(parts, num_parts: int, workspace, rows: int, inter: int,
                              pairs_per_load: int, stream=None) -> None:
    _status("silu_mul_f32p_tall", library().logismos_launch_silu_mul_f32p_tall(
        _ptr(parts), num_parts, _ptr(workspace), rows, inter, pairs_per_load, _raw(stream)))


def launch_add_rms_norm_f32p_tall(h, parts, num_parts: int, w, workspace, rows: int, n: int,
                                  eps: float, pairs_per_load: int, stream=None) -> None:
    _status("add_rms_norm_f32p_tall", library().logismos_launch_add_rms_norm_f32p_tall(
        _ptr(h), _ptr(parts) if parts is not None else None, num_parts, _ptr(w), _ptr(workspace),
        rows, n, float(eps), pairs_per_load, _raw(stream)))


def launch_repack_q8_0(blocks, qs, d, n: int, k: int, stream=None) -> None:
    check_qgemv_q8g32_shape(n, k)
    _status("repack_q8_0", library().logismos_launch_repack_q8_0(
        _ptr(blocks), _ptr(qs), _ptr(d), n, k, _raw(stream)))


def paged_attn_num_splits(num_seqs, num_kv_heads, block_size, max_blocks_per_seq,
                          head_dim: int = 128) -> int:
    return library().logismos_paged_attn_num_splits_hd(num_seqs, num_kv_heads, head_dim,
                                                       block_size, max_blocks_per_seq)


def paged_attn_workspace_bytes(num_seqs, num_q_heads, head_dim, num_splits) -> int:
    return library().logismos_paged_attn_workspace_bytes(num_seqs, num_q_heads, head_dim,
                                                         num_splits)


def check_paged_attn_shape(num_seqs, total_tokens, max_seqlen_q, num_q_heads, num_kv_heads,
                           head_dim, block_size, max_blocks_per_seq, num_splits) -> None:
    _guard("paged_attn_varlen_fp16", library().logismos_check_paged_attn_shape, num_seqs,
           total_tokens, max_seqlen_q, num_q_heads, num_kv_heads, head_dim, block_size,
           max_blocks_per_seq, num_splits)


def launch_paged_attn_varlen_fp16(q, k_pool, v_pool, block_tables, cu_seqlens_q, context_lens, out,
                                  workspace, num_seqs, total_tokens, max_seqlen_q, num_q_heads,
                                  num_kv_heads, head_dim, block_size, max_blocks_per_seq,
                                  num_splits, scale, causal=True, stream=None,
                                  phases=None) -> None:
    check_paged_attn_shape(num_seqs, total_tokens, max_seqlen_q, num_q_heads, num_kv_heads,
                           head_dim, block_size, max_blocks_per_seq, num_splits)
    args = (_ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables), _ptr(cu_seqlens_q),
            _ptr(context_lens), _ptr(out), _ptr(workspace) if workspace is not None else None,
            num_seqs, total_tokens, max_seqlen_q, num_q_heads, num_kv_heads, head_dim, block_size,
            max_blocks_per_seq, num_splits, float(scale), 1 if causal else 0)
    if phases is None:
        code = library().logismos_launch_paged_attn_varlen_fp16(*args, _raw(stream))
    else:
        code = library().logismos_launch_paged_attn_varlen_fp16_phases(*args, int(phases),
                                                                       _raw(stream))
    _status("paged_attn_varlen_fp16", code)


def paged_attn_noalloc_init() -> None:
    """Set-up of the entry point that allocates nothing, for the current device."""
    _status("paged_attn_noalloc_init", library().logismos_paged_attn_noalloc_init())


def launch_paged_attn_varlen_fp16_noalloc(q, k_pool, v_pool, block_tables, cu_seqlens_q,
                                          context_lens, out, num_seqs, total_tokens, max_seqlen_q,
                                          num_q_heads, num_kv_heads, head_dim, block_size,
                                          max_blocks_per_seq, num_splits, scale, causal=True,
                                          stream=None) -> None:
    """The paged-attention launch over the library's static workspace: allocates nothing."""
    check_paged_attn_shape(num_seqs, total_tokens, max_seqlen_q, num_q_heads, num_kv_heads,
                           head_dim, block_size, max_blocks_per_seq, num_splits)
    need = paged_attn_workspace_bytes(num_seqs, num_q_heads, head_dim, num_splits)
    cap = library().logismos_paged_attn_static_workspace_bytes()
    if need > cap:
        raise UnsupportedShape("paged_attn_varlen_fp16_noalloc",
                               f"split-K partials need {need} bytes, the static workspace "
                               f"holds {cap}")
    _status("paged_attn_varlen_fp16_noalloc",
            library().logismos_launch_paged_attn_varlen_fp16_noalloc(
                _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables), _ptr(cu_seqlens_q),
                _ptr(context_lens), _ptr(out), num_seqs, total_tokens, max_seqlen_q, num_q_heads,
                num_kv_heads, head_dim, block_size, max_blocks_per_seq, num_splits, float(scale),
                1 if causal else 0, _raw(stream)))


def launch_paged_attn_decode_fp16_xprep(q, k_pool, v_pool, block_tables, cu_seqlens_q,
                                        context_lens, out_prepared, workspace, num_seqs,
                                        num_q_heads, num_kv_heads, head_dim, block_size,
                                        max_blocks_per_seq, num_splits, scale,
                                        stream=None) -> None:
    """Decode rows only, result in the prepared layout of the o projection."""
    check_paged_attn_shape(num_seqs, num_seqs, 1, num_q_heads, num_kv_heads, head_dim, block_size,
                           max_blocks_per_seq, num_splits)
    _status("paged_attn_decode_fp16_xprep", library().logismos_launch_paged_attn_decode_fp16_xprep(
        _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables), _ptr(cu_seqlens_q),
        _ptr(context_lens), _ptr(out_prepared),
        _ptr(workspace) if workspace is not None else None, num_seqs, num_q_heads, num_kv_heads,
        head_dim, block_size, max_blocks_per_seq, num_splits, float(scale), _raw(stream)))


def launch_probe_copy(src, dst, nbytes: int, stream=None) -> None:
    _status("probe_copy", library().logismos_launch_probe_copy(_ptr(src), _ptr(dst), nbytes,
                                                               _raw(stream)))


PROBE_NON_TEMPORAL, PROBE_STRIDED = 1, 2


def launch_probe_read(src, sink, nbytes: int, stream=None, flags: int = 0) -> None:
    _status("probe_read", library().logismos_launch_probe_read_ex(_ptr(src), _ptr(sink), nbytes,
                                                                  flags, _raw(stream)))


PROBE_MFMA_CHANGING, PROBE_MFMA_BF16 = 1, 2


def launch_probe_mfma(sink, iters: int, flags: int = 0, stream=None) -> None:
    """Nothing but MFMAs on every CU (fp16 or bf16; constant or changing operands)."""
    _status("probe_mfma", library().logismos_launch_probe_mfma(_ptr(sink), iters, flags,
                                                               _raw(stream)))


def probe_mfma_flops(iters: int) -> float:
    return float(library().logismos_probe_mfma_flops(iters))


def launch_pack_ragged(new_tokens, prior_ctx, block_tables, cu_seqlens, slot_mapping, context_lens,
                       num_seqs: int, block_size: int, max_blocks: int, stream=None) -> None:
    _guard("pack_ragged", library().logismos_check_pack_ragged_shape, num_seqs, block_size,
           max_blocks)
    _status("pack_ragged", library().logismos_launch_pack_ragged(
        _ptr(new_tokens), _ptr(prior_ctx), _ptr(block_tables), _ptr(cu_seqlens),
        _ptr(slot_mapping), _ptr(context_lens), num_seqs, block_size, max_blocks, _raw(stream)))


def launch_paged_attn_varlen_turbo3(q, k_pool, v_pool, block_tables, cu_seqlens_q, context_lens,
                                    out, workspace, num_seqs, total_tokens, max_seqlen_q,
                                    num_q_heads, num_kv_heads, block_size, max_blocks_per_seq,
                                    num_splits, scale, stream=None) -> None:
    check_paged_attn_shape(num_seqs, total_tokens, max_seqlen_q, num_q_heads, num_kv_heads, 128,
                           block_size, max_blocks_per_seq, num_splits)
    _status("paged_attn_varlen_turbo3", library().logismos_launch_paged_attn_varlen_turbo3(
        _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables), _ptr(cu_seqlens_q),
        _ptr(context_lens), _ptr(out), _ptr(workspace) if workspace is not None else None,
        num_seqs, total_tokens, max_seqlen_q, num_q_heads, num_kv_heads, block_size,
        max_blocks_per_seq, num_splits, float(scale), _raw(stream)))


def launch_kv_write_turbo3(k_new, v_new, k_pool, v_pool, slot_mapping, total_tokens: int,
                           num_kv_heads: int, stream=None) -> None:
    _status("kv_write_turbo3", library().logismos_launch_kv_write_turbo3(
        _ptr(k_new), _ptr(v_new), _ptr(k_pool), _ptr(v_pool), _ptr(slot_mapping), total_tokens,
        num_kv_heads, _raw(stream)))


def launch_kv_gather_turbo3_f32(k_pool, v_pool, block_table_row, k_out, v_out, start_pos: int,
                                n_tokens: int, num_kv_heads: int, block_size: int,
                                stream=None) -> None:
    _status("kv_gather_turbo3_f32", library().logismos_launch_kv_gather_turbo3_f32(
        _ptr(k_pool), _ptr(v_pool), _ptr(block_table_row), _ptr(k_out), _ptr(v_out), start_pos,
        n_tokens, num_kv_heads, block_size, _raw(stream)))


def launch_kv_write_fp16(k_new, v_new, k_pool, v_pool, slot_mapping, total_tokens: int,
                         num_kv_heads: int, head_dim: int, stream=None) -> None:
    _status("kv_write_fp16", library().logismos_launch_kv_write_fp16(
        _ptr(k_new), _ptr(v_new), _ptr(k_pool), _ptr(v_pool), _ptr(slot_mapping), total_tokens,
        num_kv_heads, head_dim, _raw(stream)))


def launch_add_rms_norm_bf16(h, y, w, out, rows: int, n: int, eps: float, stream=None) -> None:
    _status("add_rms_norm_bf16", library().logismos_launch_add_rms_norm_bf16(
        _ptr(h), _ptr(y) if y is not None else None, _ptr(w), _ptr(out), rows, n, float(eps),
        _raw(stream)))


def launch_rope_kv_write_fp16(qkv, positions, cos, sin, slot_mapping, q_out, k_pool, v_pool,
                              total_tokens: int, hq: int, hkv: int, head_dim: int, max_pos: int,
                              stream=None) -> None:
    _status("rope_kv_write_fp16", library().logismos_launch_rope_kv_write_fp16(
        _ptr(qkv), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping), _ptr(q_out),
        _ptr(k_pool), _ptr(v_pool), total_tokens, hq, hkv, head_dim, max_pos, _raw(stream)))


def launch_silu_mul_bf16(gate_up, out, rows: int, inter: int, stream=None) -> None:
    _status("silu_mul_bf16", library().logismos_launch_silu_mul_bf16(
        _ptr(gate_up), _ptr(out), rows, inter, _raw(stream)))


def launch_cast_f16_bf16(src, dst, count: int, stream=None) -> None:
    _status("cast_f16_bf16", library().logismos_launch_cast_f16_bf16(
        _ptr(src), _ptr(dst), count, _raw(stream)))


def launch_greedy_f32(logits, out, rows: int, n: int, stream=None) -> None:
    _status("greedy_f32", library().logismos_launch_greedy_f32(
        _ptr(logits), _ptr(out), rows, n, _raw(stream)))


# ---- the reference's existing launchers (same names as its Rust wrappers,
# crates/kernels/src/{rms_norm,softmax,rope,matmul}/mod.rs)
def launch_rms_norm_fp16(x, w, y, m: int, n: int, eps: float, stream=None) -> None:
    _status("rms_norm_fp16", library().logismos_launch_rms_norm_fp16(
        _ptr(x), _ptr(w), _ptr(y), m, n, eps, _raw(stream)))


def launch_mask_additive(scores, mask, mask_len: int, rows: int, n: int, fp16: bool = False,
                         stream=None) -> None:
    """`cpu_f32::mask_additive_in_place` on device scores (fp32, or fp16 with fp16=True)."""
    fn = (library().logismos_launch_mask_additive_fp16 if fp16
          else library().logismos_launch_mask_additive_f32)
    _status("mask_additive", fn(_ptr(scores) if scores is not None else None,
                                _ptr(mask) if mask is not None else None, mask_len, rows, n,
                                _raw(stream)))


def launch_softmax_fp16(x, y, m: int, n: int, stream=None) -> None:
    _status("softmax_fp16", library().logismos_launch_softmax_fp16(
        _ptr(x), _ptr(y), m, n, _raw(stream)))


def launch_rope_fp16_in_place(qk, cos_sin, batch: int, seq: int, heads: int, head_dim: int,
                              stream=None) -> None:
    _status("rope_fp16", library().logismos_launch_rope_fp16(
        _ptr(qk), _ptr(cos_sin), batch, seq, heads, head_dim, _raw(stream)))


def launch_matmul_fp16(variant: str, a, b, d, m: int, n: int, k: int, stream=None) -> None:
    """variant: "naive" or "wmma" (`Variant`, crates/kernels/src/matmul/mod.rs:58-69)."""
    fn = {"naive": library().logismos_launch_matmul_naive_fp16,
          "wmma": library().logismos_launch_matmul_wmma_fp16}[variant]
    _status(f"matmul_{variant}_fp16", fn(_ptr(a), _ptr(b), _ptr(d), m, n, k, _raw(stream)))


def check_qgemm_q4g128_greedy_shape(b: int, n: int, k: int) -> None:
    _guard("qgemm_q4g128_greedy", library().logismos_check_qgemm_q4g128_greedy_shape, b, n, k)


def qgemm_q4g128_greedy_workspace_bytes(b: int, n: int, k: int) -> int:
    return library().logismos_qgemm_q4g128_greedy_workspace_bytes(b, n, k)


def launch_qgemm_q4g128_greedy_xprep(x_prepared, qw, scale, zero, out_tokens, logits, workspace,
                                     b: int, n: int, k: int, stream=None) -> None:
    """Vocabulary projection + greedy token per batch row; `logits` may be None."""
    check_qgemm_q4g128_greedy_shape(b, n, k)
    _status("qgemm_q4g128_greedy", library().logismos_launch_qgemm_q4g128_greedy_xprep(
        _ptr(x_prepared), _ptr(qw), _ptr(scale), _ptr(zero), _ptr(out_tokens),
        _ptr(logits) if logits is not None else None, _ptr(workspace), b, n, k, _raw(stream)))


def launch_embed_lookup(table, ids, out, rows: int, hidden: int, vocab: int, bf16: bool,
                        stream=None) -> None:
    fn = (library().logismos_launch_embed_lookup_bf16 if bf16
          else library().logismos_launch_embed_lookup_f32)
    _status("embed_lookup", fn(_ptr(table), _ptr(ids), _ptr(out), rows, hidden, vocab,
                               _raw(stream)))


def decode_step_workspace_bytes_tokens(cfg: DecodeConfig, num_seqs: int, total_tokens: int,
                                       num_splits: int) -> int:
    return library().logismos_decode_step_workspace_bytes_tokens(C.byref(cfg), num_seqs,
                                                                 total_tokens, num_splits)


def decode_step_workspace_bytes(cfg: DecodeConfig, num_seqs: int, num_splits: int) -> int:
    return library().logismos_decode_step_workspace_bytes(C.byref(cfg), num_seqs, num_splits)


def launch_decode_step(cfg: DecodeConfig, layers, batch: DecodeBatch, workspace, stream=None) -> None:
    """`layers` is a ctypes array of DecodeLayer (host memory)."""
    _status("decode_step", library().logismos_launch_decode_step(
        C.byref(cfg), C.cast(layers, _vp), C.byref(batch), _ptr(workspace), _raw(stream)))


def qgemm_q4g128_splitk_parts(b: int, n: int, k: int, prepared: bool = False) -> int:
    if prepared:
        return library().logismos_qgemm_q4g128_splitk_xprep_parts(b, n, k)
    return library().logismos_qgemm_q4g128_splitk_parts(b, n, k)


def launch_qgemm_q4g128_f32_splitk(x, qw, scale, zero, parts, b: int, n: int, k: int,
                                   stream=None, prepared: bool = False) -> None:
    check_qgemm_q4g128_shape(b, n, k)
    fn = (library().logismos_launch_qgemm_q4g128_f32_splitk_xprep if prepared
          else library().logismos_launch_qgemm_q4g128_f32_splitk)
    _status("qgemm_q4g128_f32_splitk", fn(_ptr(x), _ptr(qw), _ptr(scale), _ptr(zero), _ptr(parts),
                                          b, n, k, _raw(stream)))


def q4_xprep_bytes(b: int, k: int) -> int:
    return library().logismos_q4_xprep_bytes(b, k)


def launch_q4_prepare_x_bf16(x, xprep, b: int, k: int, stream=None) -> None:
    _status("q4_prepare_x_bf16", library().logismos_launch_q4_prepare_x_bf16(
        _ptr(x), _ptr(xprep), b, k, _raw(stream)))


def launch_add_rms_norm_f32p(h, parts, num_parts: int, w, out, rows: int, n: int, eps: float,
                             stream=None) -> None:
    _status("add_rms_norm_f32p", library().logismos_launch_add_rms_norm_f32p(
        _ptr(h), _ptr(parts) if parts is not None else None, num_parts, _ptr(w), _ptr(out), rows,
        n, float(eps), _raw(stream)))


def launch_rope_kv_write_f32p(parts, num_parts: int, positions, cos, sin, slot_mapping, q_out,
                              k_pool, v_pool, total_tokens: int, hq: int, hkv: int, head_dim: int,
                              max_pos: int, stream=None, turbo3: bool = False, bias=None) -> None:
    fn = (library().logismos_launch_rope_kv_write_f32p_turbo3_bias if turbo3
          else library().logismos_launch_rope_kv_write_f32p_bias)
    _status("rope_kv_write_f32p", fn(
        _ptr(parts), num_parts, _ptr(bias) if bias is not None else None, _ptr(positions),
        _ptr(cos), _ptr(sin), _ptr(slot_mapping), _ptr(q_out), _ptr(k_pool), _ptr(v_pool),
        total_tokens, hq, hkv, head_dim, max_pos, _raw(stream)))


def launch_silu_mul_f32p(parts, num_parts: int, out, rows: int, inter: int, stream=None) -> None:
    _status("silu_mul_f32p", library().logismos_launch_silu_mul_f32p(
        _ptr(parts), num_parts, _ptr(out), rows, inter, _raw(stream)))


def launch_add_rms_norm_f32p_xprep(h, parts, num_parts: int, w, xprep, rows: int, n: int,
                                   eps: float, stream=None) -> None:
    _status("add_rms_norm_f32p_xprep", library().logismos_launch_add_rms_norm_f32p_xprep(
        _ptr(h), _ptr(parts) if parts is not None else None, num_parts, _ptr(w), _ptr(xprep), rows,
        n, float(eps), _raw(stream)))


def launch_silu_mul_f32p_xprep(parts, num_parts: int, xprep, rows: int, inter: int,
                               stream=None) -> None:
    _status("silu_mul_f32p_xprep", library().logismos_launch_silu_mul_f32p_xprep(
        _ptr(parts), num_parts, _ptr(xprep), rows, inter, _raw(stream)))
