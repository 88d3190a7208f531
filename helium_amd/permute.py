"""PermuteDims — host-side mirror of helium/src/cuda/instr/permute_dims.rs over the C ABI."""
import ctypes as C

from . import _ffi
from ._ffi import check, lib
from .device import _h


def _dtype_code(dtype):
    return _ffi.DTYPES[dtype] if isinstance(dtype, str) else int(dtype)


class PermuteDims:
    """A compiled permute kernel for one (shape, permutation, dtype).

    `perm` follows numpy.transpose (out.shape[i] == shape[perm[i]]); `swaps` is a sequence of SwapDims
    (axis_a, axis_b) applied in order, the form enumerate_swaps produces (permute_dims.rs:112-142).
    Construction generates and compiles the kernel and needs no GPU; `execute` launches it.
    """

    def __init__(self, shape, dtype, perm=None, swaps=None):
        assert (perm is None) != (swaps is None), "give exactly one of perm / swaps"
        self.shape = tuple(int(d) for d in shape)
        self.dtype = _dtype_code(dtype)
        rank = len(self.shape)
        self.handle = C.c_void_p()
        shp = _ffi.arr(C.c_int64, self.shape)
        if perm is not None:
            self.perm = tuple(int(p) for p in perm)
            check(lib.he_permute_create(C.byref(self.handle), shp, _ffi.arr(C.c_int32, self.perm), rank, self.dtype))
        else:
            flat = [int(x) for s in swaps for x in s]
            p = list(range(rank))
            for a, b in swaps:
                p[a], p[b] = p[b], p[a]
            self.perm = tuple(p)
            check(lib.he_permute_create_from_swaps(C.byref(self.handle), shp, rank, _ffi.arr(C.c_int32, flat),
                                                   len(flat) // 2, self.dtype))
        self.out_shape = tuple(self.shape[p] for p in self.perm)

    @property
    def source(self):
        return lib.he_permute_source(self.handle).decode()

    @property
    def description(self):
        return lib.he_permute_describe(self.handle).decode()

    def execute(self, src, dst, stream=None):
        """src/dst: DeviceBuffer (or raw device addresses)."""
        sp = src.ptr if hasattr(src, "ptr") else C.c_void_p(src)
        dp = dst.ptr if hasattr(dst, "ptr") else C.c_void_p(dst)
        check(lib.he_permute_execute(self.handle, sp, dp, _h(stream)))

    def close(self):
        if self.handle:
            lib.he_permute_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def reference_output_strides(shape, swaps):
    """compute_output_strides as written in permute_dims.rs:159-171 (see the header for its quirk)."""
    rank = len(shape)
    flat = [int(x) for s in swaps for x in s]
    out = (C.c_int64 * rank)()
    check(lib.he_permute_reference_output_strides(_ffi.arr(C.c_int64, shape), rank, _ffi.arr(C.c_int32, flat),
                                                  len(flat) // 2, out))
    return list(out)
