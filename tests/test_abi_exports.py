"""The C-ABI library loads without a GPU and exports every symbol that
include/logismos_decode.h declares (no compute calls here)."""
import ctypes
import os
import re

import pytest

from logismos_amd import hip, kernels

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "logismos_decode.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(logismos_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_all_exported():
    lib = ctypes.CDLL(kernels.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 8
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_binding_covers_exactly_the_header():
    assert kernels.exported_symbols() == _declared_symbols()


def test_identity():
    lib = kernels.library()
    assert lib.logismos_decode_abi_version() == 5
    assert lib.logismos_decode_offload_arch() == b"gfx950"


def test_error_kind_mapping_matches_reference_table():
    """crates/hipcore/src/error.rs:161-181"""
    table = {0: None, 1: "InvalidValue", 2: "OutOfMemory", 3: "NotInitialized", 4: "Deinitialized",
             35: "InsufficientDriver", 53: "PriorLaunchFailure", 500: "NotFound", 600: "NotReady",
             700: "IllegalAddress", 701: "LaunchOutOfResources", 702: "LaunchTimeout",
             719: "LaunchFailure"}
    for code, kind in table.items():
        if kind:
            assert hip.error_kind(code) == kind
    assert hip.error_kind(12345) == "Unknown(12345)"
    err = kernels.LaunchError("matmul_naive_fp16", 719)
    assert "LaunchFailure" in str(err) and "719" in str(err)


@pytest.mark.parametrize("n,k,frag", [
    (0, 32, "N must be positive"), (8, 0, "K must be positive"), (8, -32, "K must be positive"),
    (8, 48, "multiple of the group size 32"), (1 << 20, 1 << 12, "exceeds i32::MAX"),
])
def test_qgemv_q8_shape_guard(n, k, frag):
    """Counterpart of check_matmul_shape's tests (crates/kernels/src/matmul/mod.rs:213-247)."""
    with pytest.raises(kernels.UnsupportedShape) as e:
        kernels.check_qgemv_q8g32_shape(n, k)
    assert frag in str(e.value)


def test_qgemv_q8_shape_guard_accepts_config1():
    kernels.check_qgemv_q8g32_shape(8960, 1536)


@pytest.mark.parametrize("args,frag", [
    (dict(num_seqs=0), "num_seqs must be positive"),
    (dict(head_dim=80), "head_dim must be a multiple of 32 up to 256"),
    (dict(head_dim=288), "head_dim must be a multiple of 32 up to 256"),
    (dict(head_dim=64, num_q_heads=34, num_kv_heads=2), "group size 17 exceeds 16"),
    (dict(head_dim=64, num_seqs=2, total_tokens=65530, max_seqlen_q=40000), "<= 65520"),
    (dict(block_size=24), "multiple of 16"),
    (dict(num_q_heads=12, num_kv_heads=5), "not a multiple of num_kv_heads"),
    (dict(num_q_heads=32, num_kv_heads=2), "group size 16 exceeds 8"),
    (dict(max_seqlen_q=99), "exceeds total_tokens"),
    (dict(num_splits=0), "num_splits must be positive"),
    (dict(block_size=1 << 16, max_blocks_per_seq=1 << 16), "exceeds i32::MAX"),
    (dict(num_seqs=70000, total_tokens=70000), "<= 65535"),
])
def test_paged_attn_shape_guard(args, frag):
    base = dict(num_seqs=16, total_tokens=16, max_seqlen_q=1, num_q_heads=12, num_kv_heads=2,
                head_dim=128, block_size=16, max_blocks_per_seq=128, num_splits=4)
    base.update(args)
    with pytest.raises(kernels.UnsupportedShape) as e:
        kernels.check_paged_attn_shape(**base)
    assert frag in str(e.value)


def test_launchers_reject_bad_shapes_with_invalid_value_and_do_not_touch_the_device():
    lib = kernels.library()
    assert lib.logismos_launch_qgemv_q8g32_f32(None, None, None, None, 8, 48, None) == 1
    assert lib.logismos_launch_paged_attn_varlen_fp16(
        None, None, None, None, None, None, None, None, 16, 16, 1, 12, 2, 80, 16, 8, 1, 0.1, 1,
        None) == 1


def test_num_splits_and_workspace_are_pure_functions():
    assert kernels.paged_attn_num_splits(16, 2, 16, 128) == kernels.paged_attn_num_splits(16, 2, 16, 128)
    ns = kernels.paged_attn_num_splits(32, 8, 16, 512)
    assert ns >= 1
    assert kernels.paged_attn_workspace_bytes(32, 32, 128, ns) == 32 * ns * 32 * 130 * 4
    assert kernels.paged_attn_workspace_bytes(32, 32, 128, 1) == 0


@pytest.mark.parametrize("b,n,k,frag", [
    (0, 8, 128, "batch must be positive"), (1, 0, 128, "N must be positive"),
    (1, 8, 64, "multiple of the group size 128"), (1, 1 << 20, 1 << 12, "exceeds i32::MAX"),
    # scales and zeros of all of K next to the partial sums exceed 160 KiB on the MFMA path
    (32, 12288, 45056, "bytes of LDS"),
    # a 33rd row is a second pass of one row on the GEMV path, whose x staging K = 77824 exceeds:
    # refused as a whole, not after the first 32 rows were written
    (33, 16, 77824, "do not fit the LDS staging"),
])
def test_qgemm_q4_shape_guard(b, n, k, frag):
    with pytest.raises(kernels.UnsupportedShape) as e:
        kernels.check_qgemm_q4g128_shape(b, n, k)
    assert frag in str(e.value)
    kernels.check_qgemm_q4g128_shape(1, 12288, 4096)
    kernels.check_qgemm_q4g128_shape(8240, 4096, 4096)  # any m, as linear_t; 32 rows per pass
    kernels.check_qgemm_q4g128_shape(32, 16, 77824)     # one full pass on the matrix cores
    kernels.check_qgemm_q4g128_shape(37, 16, 77824)     # ... and a last pass of five rows
    # the split-K forms hold the whole batch in one launch: at most 32 rows
    assert kernels.qgemm_q4g128_splitk_parts(33, 4096, 4096) == 0
    assert kernels.qgemm_q4g128_splitk_parts(33, 4096, 4096, prepared=True) == 0


@pytest.mark.parametrize("b,n,k,frag", [
    (0, 8, 128, "batch must be positive"),
    (1, 0, 128, "N must be positive"), (1, 8, 96, "multiple of 128"),
    (1, 1 << 20, 1 << 12, "exceeds i32::MAX"),
])
def test_qgemm_q4g32_shape_guard(b, n, k, frag):
    with pytest.raises(kernels.UnsupportedShape) as e:
        kernels.check_qgemm_q4g32_shape(b, n, k)
    assert frag in str(e.value)
    kernels.check_qgemm_q4g32_shape(16, 12288, 4096)
    kernels.check_qgemm_q4g32_shape(8240, 4096, 4096)  # any m, as linear_t; 32 rows per pass


def test_q4g32_launchers_reject_bad_arguments_without_touching_the_device():
    lib = kernels.library()
    # null pointers, then a K that is not a multiple of the group size
    assert lib.logismos_launch_qgemm_q4g32_bf16(None, None, None, None, None, 4, 64, 128, None) == 1
    assert lib.logismos_launch_qgemm_q4g32_bf16(None, None, None, None, None, 4, 64, 96, None) == 1
    assert lib.logismos_launch_qgemv_q4g32_f32(None, None, None, None, None, 64, 48, None) == 1
