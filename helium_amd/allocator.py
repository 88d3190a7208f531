"""The device memory pool over the C ABI: the block allocator (helium/src/cuda/allocator/block.rs), which is pure host
logic, and the device pool built on it (allocator/device.rs)."""
import ctypes as C

from . import _ffi
from ._ffi import check, lib


class Block(C.Structure):
    _fields_ = [("page", C.c_uint32), ("start", C.c_uint64), ("size", C.c_uint64), ("streams", C.c_uint64 * 8),
                ("num_streams", C.c_int32)]

    def end(self):
        return self.start + self.size

    def in_use(self):
        return sorted(self.streams[: self.num_streams])


_ffi._sig("he_block_allocator_create", C.POINTER(C.c_void_p))
_ffi._sig("he_block_allocator_destroy", C.c_void_p)
_ffi._sig("he_block_allocator_add_page", C.c_void_p, C.c_uint64, C.POINTER(C.c_uint32))
_ffi._sig("he_block_allocator_allocate", C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.POINTER(Block), C.POINTER(C.c_int))
_ffi._sig("he_block_allocator_deallocate", C.c_void_p, C.POINTER(Block))
_ffi._sig("he_block_allocator_begin_stream", C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64))
_ffi._sig("he_block_allocator_end_stream", C.c_void_p, C.c_uint64)
_ffi._sig("he_block_allocator_stats", C.c_void_p, C.POINTER(C.c_uint64))
_ffi._sig("he_pool_begin_scope", C.c_uint64, C.POINTER(C.c_uint64))
_ffi._sig("he_pool_end_scope", C.c_uint64)
_ffi._sig("he_pool_allocate", C.c_size_t, C.c_uint64, C.POINTER(C.c_void_p), C.POINTER(Block))
_ffi._sig("he_pool_release", C.c_void_p, C.POINTER(Block), C.c_uint64)


class BlockAllocator:
    def __init__(self):
        self.handle = C.c_void_p()
        check(lib.he_block_allocator_create(C.byref(self.handle)))

    def __del__(self):
        try:
            if self.handle:
                lib.he_block_allocator_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass

    def add_page(self, size):
        page = C.c_uint32()
        check(lib.he_block_allocator_add_page(self.handle, size, C.byref(page)))
        return page.value

    def allocate(self, size, align, stream=0):
        """The block, or None when nothing fits."""
        b, found = Block(), C.c_int()
        check(lib.he_block_allocator_allocate(self.handle, size, align, stream, C.byref(b), C.byref(found)))
        return b if found.value else None

    def deallocate(self, block):
        check(lib.he_block_allocator_deallocate(self.handle, C.byref(block)))

    def begin_stream(self, parent=0):
        s = C.c_uint64()
        check(lib.he_block_allocator_begin_stream(self.handle, parent, C.byref(s)))
        return s.value

    def end_stream(self, stream):
        check(lib.he_block_allocator_end_stream(self.handle, stream))

    def stats(self):
        """Also verifies the allocator's internal indices."""
        s = (C.c_uint64 * 4)()
        check(lib.he_block_allocator_stats(self.handle, s))
        return dict(zip(["free_blocks", "free_bytes", "largest_free_block", "streams"], [int(v) for v in s]))


def pool_begin_scope(thread=0):
    s = C.c_uint64()
    check(lib.he_pool_begin_scope(thread, C.byref(s)))
    return s.value


def pool_end_scope(scope):
    check(lib.he_pool_end_scope(scope))


def pool_allocate(nbytes, scope=0):
    """(device address, Block)"""
    ptr, b = C.c_void_p(), Block()
    check(lib.he_pool_allocate(nbytes, scope, C.byref(ptr), C.byref(b)))
    return ptr.value, b


def pool_release(ptr, block, scope=0):
    check(lib.he_pool_release(C.c_void_p(ptr), C.byref(block), scope))
