"""Device buffers, streams and events over the C ABI's runtime helpers (no torch involved)."""
import ctypes as C

import numpy as np

from ._lib import lib, check


class Stream:
    def __init__(self):
        h = C.c_void_p()
        check(lib().flexllm_rt_stream_create(C.byref(h)))
        self.handle = h

    def sync(self):
        check(lib().flexllm_rt_stream_sync(self.handle))

    def __del__(self):
        try:
            lib().flexllm_rt_stream_destroy(self.handle)
        except Exception:
            pass


class Event:
    def __init__(self):
        h = C.c_void_p()
        check(lib().flexllm_rt_event_create(C.byref(h)))
        self.handle = h

    def record(self, stream=None):
        check(lib().flexllm_rt_event_record(self.handle, _s(stream)))

    def sync(self):
        check(lib().flexllm_rt_event_sync(self.handle))

    def elapsed_ms(self, later):
        ms = C.c_float()
        check(lib().flexllm_rt_event_elapsed_ms(self.handle, later.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            lib().flexllm_rt_event_destroy(self.handle)
        except Exception:
            pass


def _s(stream):
    return stream.handle if stream is not None else None


def device_sync():
    check(lib().flexllm_rt_device_sync())


def device_name():
    buf = C.create_string_buffer(256)
    check(lib().flexllm_rt_device_name(buf, 256))
    return buf.value.decode()


class DeviceArray:
    """A dense device allocation with a numpy-style shape/dtype."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(d) for d in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib().flexllm_rt_malloc(C.byref(p), C.c_size_t(max(self.nbytes, 1))))     # size_t: an untyped int would be cut to 32 bits
        self.ptr = p.value
        self._owner = True

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def copy_from(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        assert host.nbytes == self.nbytes, (host.shape, self.shape)
        check(lib().flexllm_rt_memcpy_h2d(C.c_void_p(self.ptr), host.ctypes.data_as(C.c_void_p), C.c_size_t(self.nbytes), None))
        return self

    def numpy(self):
        device_sync()
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            check(lib().flexllm_rt_memcpy_d2h(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr), C.c_size_t(self.nbytes), None))
        return out

    def zero_(self, stream=None):
        check(lib().flexllm_rt_memset(C.c_void_p(self.ptr), 0, C.c_size_t(self.nbytes), _s(stream)))
        return self

    def view(self, offset_bytes, shape, dtype=None):
        v = DeviceArray.__new__(DeviceArray)
        v.shape = tuple(shape)
        v.dtype = np.dtype(dtype or self.dtype)
        v.nbytes = int(np.prod(v.shape, dtype=np.int64)) * v.dtype.itemsize
        assert offset_bytes + v.nbytes <= self.nbytes
        v.ptr = self.ptr + offset_bytes
        v._owner = False
        v._base = self
        return v

    def __del__(self):
        if getattr(self, "_owner", False) and self.ptr:
            try:
                lib().flexllm_rt_free(C.c_void_p(self.ptr))
            except Exception:
                pass
            self.ptr = 0


def empty(shape, dtype):
    return DeviceArray(shape, dtype)


def zeros(shape, dtype):
    return DeviceArray(shape, dtype).zero_()


def to_device(host, dtype=None):
    host = np.ascontiguousarray(host, dtype=dtype)
    return DeviceArray(host.shape, host.dtype).copy_from(host)
