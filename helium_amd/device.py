"""Device-side plumbing over the C ABI: context init, streams, events, device buffers.

Mirrors what helium/src/cuda/context.rs and tensor_storage.rs give the reference's backend. Host data is
exchanged as numpy arrays; 16-bit float tensors travel as uint16 bit patterns.
"""
import ctypes as C

import numpy as np

from . import _ffi
from ._ffi import check, lib

_initialised = False

NP_STORAGE = {_ffi.F16: np.uint16, _ffi.BF16: np.uint16, _ffi.F32: np.float32, _ffi.U32: np.uint32,
              _ffi.BOOL: np.uint32}


def init(device=0):
    """he_init once per process; raises HeliumError when no GPU is visible."""
    global _initialised
    if not _initialised:
        check(lib.he_init(device))
        _initialised = True


def device_count():
    n = C.c_int(0)
    status = lib.he_device_count(C.byref(n))
    return n.value if status == 0 else 0


def device_attr(attr, device=0):
    v = C.c_int64(0)
    check(lib.he_device_attr(device, attr, C.byref(v)))
    return v.value


def device_arch(device=0):
    buf = C.create_string_buffer(256)
    check(lib.he_device_arch(device, buf, 256))
    return buf.value.decode()


def synchronize():
    check(lib.he_device_synchronize())


class Stream:
    def __init__(self):
        init()
        self.handle = C.c_void_p()
        check(lib.he_stream_create(C.byref(self.handle)))
        self._callbacks = []

    def synchronize(self):
        check(lib.he_stream_synchronize(self.handle))
        self._callbacks.clear()

    def host_callback(self, fn):
        cb = _ffi.HOST_FN(lambda _user: fn())
        self._callbacks.append(cb)  # keep the trampoline alive until the stream is synchronised
        check(lib.he_stream_host_callback(self.handle, cb, None))

    def close(self):
        if self.handle:
            check(lib.he_stream_destroy(self.handle))
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _h(stream):
    return stream.handle if stream is not None else None


class Event:
    def __init__(self):
        init()
        self.handle = C.c_void_p()
        check(lib.he_event_create(C.byref(self.handle)))

    def record(self, stream=None):
        check(lib.he_event_record(self.handle, _h(stream)))

    def wait(self, stream=None):
        check(lib.he_event_wait(self.handle, _h(stream)))

    def synchronize(self):
        check(lib.he_event_synchronize(self.handle))

    def elapsed_ms(self, stop):
        ms = C.c_float(0)
        check(lib.he_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                lib.he_event_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass


class DeviceBuffer:
    """A raw device allocation (he_malloc) with synchronous numpy upload/download helpers."""

    def __init__(self, nbytes):
        init()
        self.nbytes = int(nbytes)
        self.ptr = C.c_void_p()
        check(lib.he_malloc(C.byref(self.ptr), self.nbytes))

    @classmethod
    def from_numpy(cls, array, stream=None):
        array = np.ascontiguousarray(array)
        buf = cls(array.nbytes)
        buf.upload(array, stream)
        return buf

    def upload(self, array, stream=None):
        array = np.ascontiguousarray(array)
        assert array.nbytes <= self.nbytes, (array.nbytes, self.nbytes)
        if array.nbytes:
            check(lib.he_memcpy_h2d_async(self.ptr, array.ctypes.data_as(C.c_void_p), array.nbytes, _h(stream)))
            check(lib.he_stream_synchronize(_h(stream)))

    def to_numpy(self, dtype, shape=None, stream=None):
        dtype = np.dtype(dtype)
        count = self.nbytes // dtype.itemsize if shape is None else int(np.prod(shape, dtype=np.int64))
        out = np.empty(count, dtype=dtype)
        if out.nbytes:
            check(lib.he_memcpy_d2h_async(out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes, _h(stream)))
            check(lib.he_stream_synchronize(_h(stream)))
        return out if shape is None else out.reshape(shape)

    def read(self, byte_offset, dtype, count, stream=None):
        """`count` elements of `dtype` starting `byte_offset` bytes into the buffer (a sampled download)."""
        dtype = np.dtype(dtype)
        out = np.empty(int(count), dtype=dtype)
        assert 0 <= byte_offset and byte_offset + out.nbytes <= self.nbytes, (byte_offset, out.nbytes, self.nbytes)
        if out.nbytes:
            src = C.c_void_p(self.ptr.value + int(byte_offset))
            check(lib.he_memcpy_d2h_async(out.ctypes.data_as(C.c_void_p), src, out.nbytes, _h(stream)))
            check(lib.he_stream_synchronize(_h(stream)))
        return out

    def fill_u32(self, value, stream=None):
        check(lib.he_memset_d32_async(self.ptr, value, self.nbytes // 4, _h(stream)))

    def fill_u8(self, value, stream=None):
        check(lib.he_memset_d8_async(self.ptr, value, self.nbytes, _h(stream)))

    def free(self):
        if self.ptr:
            check(lib.he_free(self.ptr))
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def rtc_compile(source, name="kernel", options=()):
    """he_rtc_compile → bytes of the gfx950 code object. Needs no GPU."""
    opts = _ffi.arr(C.c_char_p, [o.encode() for o in options])
    code, size = C.c_void_p(), C.c_size_t(0)
    check(lib.he_rtc_compile(source.encode(), name.encode(), opts, len(options), C.byref(code), C.byref(size)))
    blob = C.string_at(code, size.value)
    lib.he_rtc_free(code)
    return blob


def rtc_stats():
    s = (C.c_uint64 * 3)()
    check(lib.he_rtc_stats(s))
    return {"compiles": s[0], "memory_hits": s[1], "disk_hits": s[2]}


class Module:
    """he_module_load + he_module_get_function + he_launch, for hand-launching a compiled code object."""

    def __init__(self, code):
        init()
        self._code = code
        self.handle = C.c_void_p()
        check(lib.he_module_load(C.byref(self.handle), code, len(code)))

    def function(self, name):
        f = C.c_void_p()
        check(lib.he_module_get_function(self.handle, name.encode(), C.byref(f)))
        return f

    def launch(self, function, grid, block, args, lds_bytes=0, stream=None):
        g = _ffi.arr(C.c_uint32, grid)
        b = _ffi.arr(C.c_uint32, block)
        holders = list(args)  # ctypes values
        argv = (C.c_void_p * len(holders))(*[C.cast(C.pointer(a), C.c_void_p) for a in holders])
        check(lib.he_launch(function, g, b, lds_bytes, _h(stream), argv))

    def __del__(self):
        try:
            if self.handle:
                lib.he_module_unload(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass
