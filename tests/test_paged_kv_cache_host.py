"""Host-side checks of the paged KV cache that need no GPU: layouts are validated before
any HIP call, and null handles are tolerated by the accessors."""
import ctypes as C

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
