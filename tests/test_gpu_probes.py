"""The measurement probes run and refuse what they cannot take (through the C ABI).

Their rates are what bench.py reports as the box's ceilings; nothing is asserted about the
rates here beyond the two forms of the matrix-core probe finishing in comparable time.
"""
import numpy as np
import pytest

from logismos_amd import hip, kernels

pytestmark = pytest.mark.gpu


def test_read_probe_all_forms_leave_the_sink_alone():
    src = hip.DeviceBuffer(1 << 20)
    src.fill(0x5A)
    sink = hip.DeviceBuffer(16)
    sink.fill(0)
    for flags in (0, kernels.PROBE_NON_TEMPORAL, kernels.PROBE_STRIDED,
                  kernels.PROBE_NON_TEMPORAL | kernels.PROBE_STRIDED):
        kernels.launch_probe_read(src, sink, 1 << 20, flags=flags)
    hip.synchronize()
    assert not sink.to_numpy(np.uint32, (4,)).any()
    with pytest.raises(kernels.LaunchError):
        kernels.launch_probe_read(src, sink, (1 << 20) + 8)  # not a multiple of 16 bytes


def test_matrix_core_probe_runs_in_all_four_forms():
    sink = hip.DeviceBuffer(16)
    sink.fill(0)
    assert kernels.probe_mfma_flops(10) == 256 * 8 * 10 * 4 * 32768.0
    times = {}
    for flags in (0, kernels.PROBE_MFMA_CHANGING, kernels.PROBE_MFMA_BF16,
                  kernels.PROBE_MFMA_CHANGING | kernels.PROBE_MFMA_BF16):
        kernels.launch_probe_mfma(sink, 50, flags)  # warm-up
        hip.synchronize()
        e0, e1 = hip.Event(), hip.Event()
        stream = hip.Stream()
        e0.record(stream)
        kernels.launch_probe_mfma(sink, 2000, flags, stream)
        e1.record(stream)
        e1.synchronize()
        times[flags] = e0.elapsed_ms(e1)
    hip.synchronize()
    assert not sink.to_numpy(np.uint32, (4,)).any()
    # 2000 x 4 MFMAs of 32 clocks per wave, two waves per SIMD: 0.2 ms at 2.4 GHz; the form
    # with changing operands may be held back by the part, but not by an order of magnitude
    for flags, ms in times.items():
        assert 0.1 < ms < 5.0, (flags, ms)
    for bad in (dict(iters=0, flags=0), dict(iters=10, flags=4)):
        with pytest.raises(kernels.LaunchError):
            kernels.launch_probe_mfma(sink, bad["iters"], bad["flags"])
