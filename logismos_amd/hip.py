"""ctypes view of the HIP runtime: the plumbing `hipcore` provides in the
reference (crates/hipcore/src/{device,stream,memory,error}.rs) -- device
selection, streams, events, owned device buffers, status-to-error mapping.
No PyTorch involved.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_lib = None


def _runtime() -> C.CDLL:
    global _lib
    if _lib is None:
        last = None
        for name in ("libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6",
                     os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib", "libamdhip64.so")):
            try:
                _lib = C.CDLL(name, mode=C.RTLD_GLOBAL)
                break
            except OSError as e:  # pragma: no cover
                last = e
        if _lib is None:
            raise RuntimeError(f"HIP runtime not found: {last}")
        _lib.hipGetErrorString.restype = C.c_char_p
        _lib.hipGetErrorString.argtypes = [C.c_int]
    return _lib


# crates/hipcore/src/error.rs:125-201 -- the codes the reference classifies.
ERROR_KINDS = {
    1: "InvalidValue", 2: "OutOfMemory", 3: "NotInitialized", 4: "Deinitialized",
    35: "InsufficientDriver", 53: "PriorLaunchFailure", 500: "NotFound", 600: "NotReady",
    700: "IllegalAddress", 701: "LaunchOutOfResources", 702: "LaunchTimeout", 719: "LaunchFailure",
}


def error_kind(code: int) -> str:
    """`ErrorKind::from_raw` (crates/hipcore/src/error.rs:125-150)."""
    return ERROR_KINDS.get(int(code), f"Unknown({int(code)})")


class HipError(RuntimeError):
    def __init__(self, code: int, op: str):
        self.code = int(code)
        self.kind = error_kind(code)
        self.op = op
        super().__init__(f"{op}: {self.kind} (code {self.code})")


def check(code: int, op: str) -> None:
    if code != 0:
        raise HipError(code, op)


def device_count() -> int:
    n = C.c_int(0)
    try:
        rc = _runtime().hipGetDeviceCount(C.byref(n))
    except RuntimeError:
        return 0
    return n.value if rc == 0 else 0


def set_device(ordinal: int) -> None:
    check(_runtime().hipSetDevice(C.c_int(ordinal)), "hipSetDevice")


def synchronize() -> None:
    check(_runtime().hipDeviceSynchronize(), "hipDeviceSynchronize")


def device_attribute(attr: int, ordinal: int = 0) -> int:
    v = C.c_int(0)
    check(_runtime().hipDeviceGetAttribute(C.byref(v), C.c_int(attr), C.c_int(ordinal)),
          "hipDeviceGetAttribute")
    return v.value


def mem_info() -> tuple[int, int]:
    free, total = C.c_size_t(0), C.c_size_t(0)
    check(_runtime().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value, total.value


class Stream:
    """An owned HIP stream at the default priority."""

    def __init__(self):
        self._h = C.c_void_p()
        check(_runtime().hipStreamCreate(C.byref(self._h)), "hipStreamCreate")

    @property
    def raw(self) -> C.c_void_p:
        return self._h

    def synchronize(self) -> None:
        check(_runtime().hipStreamSynchronize(self._h), "hipStreamSynchronize")

    def wait_event(self, event: "Event") -> None:
        """Work enqueued on this stream from now on starts after `event` (as recorded so far)."""
        check(_runtime().hipStreamWaitEvent(self._h, event._h, C.c_uint(0)), "hipStreamWaitEvent")

    def __del__(self):
        try:
            if self._h:
                _runtime().hipStreamDestroy(self._h)
        except Exception:
            pass


class Event:
    def __init__(self):
        self._h = C.c_void_p()
        check(_runtime().hipEventCreate(C.byref(self._h)), "hipEventCreate")

    def record(self, stream: Stream | None = None) -> None:
        check(_runtime().hipEventRecord(self._h, stream.raw if stream else None), "hipEventRecord")

    def synchronize(self) -> None:
        check(_runtime().hipEventSynchronize(self._h), "hipEventSynchronize")

    def elapsed_ms(self, end: "Event") -> float:
        ms = C.c_float(0)
        check(_runtime().hipEventElapsedTime(C.byref(ms), self._h, end._h), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            if self._h:
                _runtime().hipEventDestroy(self._h)
        except Exception:
            pass


class DevicePtrView:
    """Borrowed device memory (owned by someone else, e.g. a cache's pool): read-back only."""

    def __init__(self, ptr: C.c_void_p, nbytes: int):
        self._p = C.c_void_p(ptr.value if isinstance(ptr, C.c_void_p) else int(ptr))
        self.nbytes = int(nbytes)

    @property
    def ptr(self) -> C.c_void_p:
        return self._p

    def to_numpy(self, dtype, shape=None) -> np.ndarray:
        out = np.empty(self.nbytes // np.dtype(dtype).itemsize if shape is None else shape, dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(_runtime().hipMemcpy(out.ctypes.data_as(C.c_void_p), self._p,
                                       C.c_size_t(out.nbytes), C.c_int(2)), "hipMemcpy(D2H)")
        return out


class DeviceBuffer:
    """Owned device allocation (`hipcore::DeviceBuffer`, crates/hipcore/src/memory.rs)."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self._p = C.c_void_p()
        check(_runtime().hipMalloc(C.byref(self._p), C.c_size_t(max(self.nbytes, 1))), "hipMalloc")

    @property
    def ptr(self) -> C.c_void_p:
        return self._p

    def offset(self, nbytes: int) -> C.c_void_p:
        return C.c_void_p(self._p.value + int(nbytes))

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        buf.copy_from_host(a)
        return buf

    def copy_from_host(self, a: np.ndarray, dst_offset: int = 0) -> None:
        a = np.ascontiguousarray(a)
        assert dst_offset + a.nbytes <= self.nbytes
        if a.nbytes == 0:
            return
        check(_runtime().hipMemcpy(self.offset(dst_offset), a.ctypes.data_as(C.c_void_p),
                                   C.c_size_t(a.nbytes), C.c_int(1)), "hipMemcpy(H2D)")

    def to_numpy(self, dtype, shape, src_offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype)
        assert src_offset + out.nbytes <= self.nbytes
        if out.nbytes:
            check(_runtime().hipMemcpy(out.ctypes.data_as(C.c_void_p), self.offset(src_offset),
                                       C.c_size_t(out.nbytes), C.c_int(2)), "hipMemcpy(D2H)")
        return out

    def copy_from_device(self, src: "DeviceBuffer", nbytes: int, dst_offset: int = 0,
                         src_offset: int = 0) -> None:
        assert dst_offset + nbytes <= self.nbytes and src_offset + nbytes <= src.nbytes
        check(_runtime().hipMemcpy(self.offset(dst_offset), src.offset(src_offset),
                                   C.c_size_t(nbytes), C.c_int(3)), "hipMemcpy(D2D)")

    def copy_from_device_async(self, src: "DeviceBuffer", nbytes: int, stream: "Stream",
                               dst_offset: int = 0, src_offset: int = 0) -> None:
        assert dst_offset + nbytes <= self.nbytes and src_offset + nbytes <= src.nbytes
        check(_runtime().hipMemcpyAsync(self.offset(dst_offset), src.offset(src_offset),
                                        C.c_size_t(nbytes), C.c_int(3), stream.raw),
              "hipMemcpyAsync(D2D)")

    def fill(self, byte: int) -> None:
        check(_runtime().hipMemset(self._p, C.c_int(byte), C.c_size_t(self.nbytes)), "hipMemset")

    def free(self) -> None:
        if self._p:
            _runtime().hipFree(self._p)
            self._p = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Graph:
    """A captured, instantiated HIP graph: the launches enqueued on `stream`
    inside the `with` block replay with one `launch()`.  Kernel launches only;
    nothing captured here records a memset node."""

    def __init__(self, stream: Stream):
        self.stream = stream
        self._graph = C.c_void_p()
        self._exec = C.c_void_p()

    def __enter__(self):
        check(_runtime().hipStreamBeginCapture(self.stream.raw, C.c_int(2)), "hipStreamBeginCapture")
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = _runtime().hipStreamEndCapture(self.stream.raw, C.byref(self._graph))
        if exc_type is not None:
            return False
        check(rc, "hipStreamEndCapture")
        check(_runtime().hipGraphInstantiate(C.byref(self._exec), self._graph, None, None,
                                             C.c_size_t(0)), "hipGraphInstantiate")
        return False

    def launch(self) -> None:
        check(_runtime().hipGraphLaunch(self._exec, self.stream.raw), "hipGraphLaunch")

    def __del__(self):
        try:
            if self._exec:
                _runtime().hipGraphExecDestroy(self._exec)
            if self._graph:
                _runtime().hipGraphDestroy(self._graph)
        except Exception:
            pass
