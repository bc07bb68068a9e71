"""Host-side checks of the paged KV cache that need no GPU: layouts are validated before
any HIP call, and null handles are tolerated by the accessors."""
import ctypes as C
import os
import subprocess

import pytest

from logismos_amd import kernels


def _create(**kw):
    lay = dict(num_layers=2, num_kv_heads=2, head_dim=8, block_size=16, num_blocks=4, max_seqs=2,
               max_blocks_per_seq=2)
    lay.update(kw)
    layout = kernels.PagedKvLayout(*[lay[k] for k, _ in kernels.PagedKvLayout._fields_])
    h = C.c_void_p()
    rc = kernels.library().logismos_paged_kv_cache_create(C.byref(layout), C.byref(h))
    return rc, h


@pytest.mark.parametrize("bad", [dict(num_layers=0), dict(num_kv_heads=-1), dict(head_dim=0),
                                 dict(block_size=0), dict(block_size=24), dict(num_blocks=0),
                                 dict(max_seqs=0), dict(max_blocks_per_seq=0),
                                 dict(num_kv_heads=1, head_dim=4),              # row % 8 != 0
                                 dict(block_size=1 << 20, max_blocks_per_seq=1 << 12)])
def test_invalid_layouts_are_rejected_before_touching_the_device(bad):
    rc, h = _create(**bad)
    assert rc == 4 and not h.value     # ShapeMismatch, no object


def test_null_handles_are_harmless():
    lib = kernels.library()
    assert lib.logismos_paged_kv_cache_num_layers(None) == 0
    assert lib.logismos_paged_kv_cache_len_of(None, 0, 0) == -1
    assert lib.logismos_paged_kv_cache_free_blocks(None) == 0
    assert lib.logismos_paged_kv_cache_block_tables(None) is None
    assert lib.logismos_paged_kv_cache_close_seq(None, 0) == 5
    lib.logismos_paged_kv_cache_reset(None)
    lib.logismos_paged_kv_cache_destroy(None)


def test_append_and_gather_reject_bad_arguments_on_the_host():
    lib = kernels.library()
    assert lib.logismos_launch_kv_append_fp16(None, None, None, None, None, -1, 1, 2, 8, 16,
                                              None) == 1
    assert lib.logismos_launch_kv_append_fp16(None, None, None, None, None, 0, 1, 1, 4, 16,
                                              None) == 1   # row % 8 != 0
    assert lib.logismos_launch_kv_gather_fp16(None, None, None, None, None, 0, 0, 2, 8, 16,
                                              None) == 0   # nothing to do
    assert lib.logismos_launch_kv_gather_fp16(None, None, None, None, None, 0, 3, 2, 8, 16,
                                              None) == 1   # null pointers


def test_block_table_updates_are_staged_until_their_copy_has_run(tmp_path):
    """The deferral rule of the cache's block-table mirror (lg::StagingRing): a queued copy
    delivers what the table row held when it was queued, whatever the host writes to the row
    afterwards, and a staging slot is reused only behind its fence.  Exercised with a
    simulated stream (tests/cpp/staging_ring_test.cpp, plain g++, no device)."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = tmp_path / "staging_ring_test"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror",
                    "-I", os.path.join(root, "logismos_amd", "csrc"),
                    os.path.join(root, "tests", "cpp", "staging_ring_test.cpp"), "-o", str(exe)],
                   check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "staging ring ok" in r.stdout
