"""Device, stream, event and memory handles over the C ABI."""

from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import check


def device_count() -> int:
    n = C.c_int()
    check(_lib.load().pf_device_count(C.byref(n)))
    return n.value


def set_device(device: int) -> None:
    check(_lib.load().pf_set_device(device))


def device_synchronize() -> None:
    check(_lib.load().pf_device_synchronize())


def device_numa_node(device: int) -> int:
    n = C.c_int()
    check(_lib.load().pf_device_numa_node(device, C.byref(n)))
    return n.value


def device_name(device: int) -> str:
    buf = C.create_string_buffer(256)
    check(_lib.load().pf_device_name(device, buf, 256))
    return buf.value.decode()


class Stream:
    """A non-blocking HIP stream at the default priority, or a wrapper around
    an existing one (``Stream.wrap(torch_stream.cuda_stream)``)."""

    def __init__(self, _handle=None):
        self._lib = _lib.load()
        if _handle is None:
            h = C.c_void_p()
            check(self._lib.pf_stream_create(C.byref(h)))
            _handle = h
        self.handle = _handle

    @classmethod
    def wrap(cls, native_stream: int) -> "Stream":
        h = C.c_void_p()
        check(_lib.load().pf_stream_wrap(C.c_void_p(native_stream), C.byref(h)))
        return cls(h)

    @property
    def native(self) -> int:
        return self._lib.pf_stream_native(self.handle) or 0

    def synchronize(self) -> None:
        check(self._lib.pf_stream_synchronize(self.handle))

    def runs_concurrently_with(self, other: "Stream") -> bool:
        """Whether kernels of this stream and of ``other`` execute at the same
        time (they do not when the runtime put both on one hardware queue)."""
        out = C.c_int()
        check(self._lib.pf_streams_run_concurrently(self.handle, other.handle, C.byref(out)))
        return bool(out.value)

    def wait_event(self, event: "Event") -> None:
        check(self._lib.pf_stream_wait_event(self.handle, event.handle))

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_stream_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Event:
    def __init__(self, timing: bool = False):
        self._lib = _lib.load()
        h = C.c_void_p()
        check(self._lib.pf_event_create(1 if timing else 0, C.byref(h)))
        self.handle = h

    def record(self, stream: Stream) -> None:
        check(self._lib.pf_event_record(self.handle, stream.handle))

    def synchronize(self) -> None:
        check(self._lib.pf_event_synchronize(self.handle))

    def query(self) -> bool:
        done = C.c_int()
        check(self._lib.pf_event_query(self.handle, C.byref(done)))
        return bool(done.value)

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        check(self._lib.pf_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_event_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class PinnedMemory:
    """Pinned, device-mapped host memory (the reference's ``PinnedMemory``,
    pegaflow-core/src/pinned_mem.rs:113-289)."""

    def __init__(self, size: int, strategy: int = _lib.PF_HOST_HIP_ALLOC, numa_node: int = -1):
        self._lib = _lib.load()
        self._mem = _lib.PfHostMem()
        check(self._lib.pf_host_alloc(size, strategy, numa_node, C.byref(self._mem)))

    @property
    def host_ptr(self) -> int:
        return self._mem.host or 0

    @property
    def device_ptr(self) -> int:
        return self._mem.device

    @property
    def size(self) -> int:
        return self._mem.size

    def as_numpy(self) -> np.ndarray:
        """uint8 view of the whole region (no copy)."""
        buf = (C.c_uint8 * self.size).from_address(self.host_ptr)
        return np.frombuffer(buf, dtype=np.uint8)

    def close(self) -> None:
        if self._mem.host:
            check(self._lib.pf_host_free(C.byref(self._mem)))

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class DeviceBuffer:
    """Raw device allocation with blocking copies, for tests and benches
    (the reference's test-only ``GpuBuffer``,
    pegaflow-core/tests/common/gpu_buffer.rs:13-69)."""

    def __init__(self, size: int):
        self._lib = _lib.load()
        p = C.c_uint64()
        check(self._lib.pf_dev_malloc(size, C.byref(p)))
        self.ptr = p.value
        self.size = size

    def fill(self, value: int) -> None:
        check(self._lib.pf_dev_memset(self.ptr, value, self.size))

    def copy_from_host(self, data: np.ndarray, offset: int = 0) -> None:
        data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        assert offset + data.nbytes <= self.size
        check(self._lib.pf_dev_copy_from_host(self.ptr + offset, data.ctypes.data, data.nbytes))

    def copy_to_host(self, offset: int = 0, size: int | None = None) -> np.ndarray:
        size = self.size - offset if size is None else size
        out = np.empty(size, dtype=np.uint8)
        check(self._lib.pf_dev_copy_to_host(out.ctypes.data, self.ptr + offset, size))
        return out

    def close(self) -> None:
        if self.ptr:
            self._lib.pf_dev_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def memcpy_h2d_async(dst_dev: int, src_host: int, size: int, stream: Stream) -> None:
    check(_lib.load().pf_memcpy_h2d_async(dst_dev, src_host, size, stream.handle))


def memcpy_d2h_async(dst_host: int, src_dev: int, size: int, stream: Stream) -> None:
    check(_lib.load().pf_memcpy_d2h_async(dst_host, src_dev, size, stream.handle))
