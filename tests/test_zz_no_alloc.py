"""The entry point that allocates nothing: `logismos_launch_paged_attn_varlen_fp16_noalloc`
keeps its split-K partials in the library's static device array.  Through the C ABI, against
the existing launcher with a caller workspace: same kernels, same split, so the outputs are
bit-identical; two calls in a row, the second on a smaller input, and every call also against
the CPU oracle."""
import numpy as np
import pytest

import oracle as O
from logismos_amd import hip, kernels
from tests import workloads
from tests.gpu_harness import PagedAttnRunner, assert_parity

pytestmark = pytest.mark.gpu


def _both(case, num_splits=None):
    r = PagedAttnRunner(case, num_splits=num_splits)
    r.launch()
    want_gpu = r.result().copy()
    d_out = hip.DeviceBuffer(max(case["q"].nbytes, 16))
    d_out.fill(0xFF)
    kernels.launch_paged_attn_varlen_fp16_noalloc(
        r.q, r.k_pool, r.v_pool, r.bt, r.cu, r.ctx, d_out, r.num_seqs, r.total_tokens,
        r.max_seqlen_q, case["hq"], case["hkv"], case["d"], case["block_size"],
        case["max_blocks"], r.num_splits, case["scale"], True)
    hip.synchronize()
    got = d_out.to_numpy(np.float16, case["q"].shape)
    assert np.array_equal(got.view(np.uint16), want_gpu.view(np.uint16))
    want = O.paged_attn_varlen_fp16(case["q"], case["k_pool"], case["v_pool"],
                                    case["block_tables"], case["cu_seqlens"],
                                    case["context_lens"], case["hq"], case["hkv"], case["d"],
                                    case["block_size"], case["scale"], True)
    assert_parity(got, want, what="no-alloc paged attention")
    return r.num_splits


def test_two_calls_in_a_row_the_second_smaller():
    rng = np.random.default_rng(71)
    # balanced decode kernel (wide block tables), partials of many workers in the static array
    big = workloads.paged_case(rng, np.ones(24, np.int32), rng.integers(300, 4000, size=24),
                               hq=32, hkv=8, min_max_blocks=600)
    ns = _both(big)
    assert ns > 2
    # then a smaller problem on the same array (static split-K kernel, fewer partials): what
    # the first call left behind must not matter
    small = workloads.paged_case(rng, [1, 1, 1, 7, 1], [900, 31, 257, 40, 0], hq=12, hkv=2)
    _both(small, num_splits=5)
    # and the first once more
    _both(big)


def test_refuses_partials_beyond_the_static_array_and_allocates_nothing():
    cap = kernels.library().logismos_paged_attn_static_workspace_bytes()
    assert cap == 16 << 20
    rng = np.random.default_rng(72)
    case = workloads.paged_case(rng, [1, 1], [100, 50], hq=32, hkv=8)
    r = PagedAttnRunner(case, num_splits=2)
    d_out = hip.DeviceBuffer(case["q"].nbytes)
    # 2 sequences x 4096 splits x 32 heads x 130 floats = 136 MB of partials: refused
    need = kernels.paged_attn_workspace_bytes(2, 32, 128, 4096)
    assert need > cap
    code = kernels.library().logismos_launch_paged_attn_varlen_fp16_noalloc(
        r.q.ptr, r.k_pool.ptr, r.v_pool.ptr, r.bt.ptr, r.cu.ptr, r.ctx.ptr, d_out.ptr, 2, 2, 1,
        32, 8, 128, 16, case["max_blocks"], 4096, float(case["scale"]), 1, None)
    assert code == 1  # hipErrorInvalidValue
    # device memory in use does not move across calls of the entry point: after the set-up
    # call (symbol look-up, which may load the code object and place the array; CU count),
    # whatever ran in this process before
    kernels.paged_attn_noalloc_init()
    hip.synchronize()
    free0, _ = hip.mem_info()
    for _ in range(3):
        kernels.launch_paged_attn_varlen_fp16_noalloc(
            r.q, r.k_pool, r.v_pool, r.bt, r.cu, r.ctx, d_out, 2, 2, 1, 32, 8, 128, 16,
            case["max_blocks"], 2, case["scale"], True)
    hip.synchronize()
    free1, _ = hip.mem_info()
    assert free1 == free0
