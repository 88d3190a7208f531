"""Compiled tile kernels over the C ABI: the pointwise/reduction instruction (helium/src/cuda/instr/pointwise.rs)
and anchor-less fusion-IR kernels (helium-playground/src/templates/auxiliary.cu)."""
import ctypes as C

from . import _ffi
from ._ffi import check, lib
from .device import _h

_ffi._sig("he_pointwise_supports", C.c_void_p, C.POINTER(C.c_uint32), C.c_int, C.POINTER(C.c_int))
_ffi._sig("he_pointwise_create", C.POINTER(C.c_void_p), C.c_void_p, C.POINTER(C.c_uint32), C.c_int)
_ffi._sig("he_aux_kernel_create", C.POINTER(C.c_void_p), C.c_void_p)
_ffi._sig("he_fused_kernel_create", C.POINTER(C.c_void_p), C.c_void_p)
_ffi._sig("he_tile_kernel_num_args", C.c_void_p, C.POINTER(C.c_int))
_ffi._sig("he_tile_kernel_arg_info", C.c_void_p, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_int32),
          C.POINTER(C.c_int32), C.POINTER(C.c_int64))
_ffi._sig("he_tile_kernel_execute", C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_void_p)
_ffi._sig("he_tile_kernel_execute_noalloc", C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_void_p)
_ffi._sig("he_tile_kernel_source", C.c_void_p, restype=C.c_char_p)
_ffi._sig("he_tile_kernel_describe", C.c_void_p, restype=C.c_char_p)
_ffi._sig("he_tile_kernel_destroy", C.c_void_p)


def pointwise_supports(graph, nodes):
    ok = C.c_int()
    check(lib.he_pointwise_supports(graph.handle, _ffi.arr(C.c_uint32, nodes), len(nodes), C.byref(ok)))
    return bool(ok.value)


class TileKernel:
    """args: list of dicts {node, is_output, dtype, numel} in kernel-argument order."""

    def __init__(self, handle):
        self.handle = handle
        n = C.c_int()
        check(lib.he_tile_kernel_num_args(handle, C.byref(n)))
        self.args = []
        for i in range(n.value):
            node, is_out, dtype, numel = C.c_uint64(), C.c_int32(), C.c_int32(), C.c_int64()
            check(lib.he_tile_kernel_arg_info(handle, i, C.byref(node), C.byref(is_out), C.byref(dtype), C.byref(numel)))
            self.args.append({"node": node.value, "is_output": bool(is_out.value),
                              "dtype": _ffi.DTYPE_NAMES[dtype.value], "numel": numel.value})

    @classmethod
    def pointwise(cls, graph, nodes):
        """PointwiseGraph::new for the subgraph made of `nodes` of a helium-ir graph."""
        h = C.c_void_p()
        check(lib.he_pointwise_create(C.byref(h), graph.handle, _ffi.arr(C.c_uint32, nodes), len(nodes)))
        return cls(h)

    @classmethod
    def auxiliary(cls, fgraph):
        """KernelGenerator for an anchor-less fusion-IR graph."""
        h = C.c_void_p()
        check(lib.he_aux_kernel_create(C.byref(h), fgraph.handle))
        return cls(h)

    @classmethod
    def fused(cls, fgraph):
        """KernelGenerator for any fusion-IR graph: the fused GEMM when it holds a Matmul anchor (its mainloop ops
        run while operand tiles are staged, its epilogue ops on the accumulators), else the auxiliary kernel."""
        h = C.c_void_p()
        check(lib.he_fused_kernel_create(C.byref(h), fgraph.handle))
        return cls(h)

    @property
    def source(self):
        return lib.he_tile_kernel_source(self.handle).decode()

    @property
    def description(self):
        return lib.he_tile_kernel_describe(self.handle).decode()

    def execute(self, buffers, stream=None):
        """buffers: DeviceBuffers (or raw addresses) in kernel-argument order."""
        ptrs = [(b.ptr if hasattr(b, "ptr") else C.c_void_p(b)) for b in buffers]
        argv = (C.c_void_p * len(ptrs))(*ptrs)
        check(lib.he_tile_kernel_execute(self.handle, argv, len(ptrs), _h(stream)))

    def execute_noalloc(self, buffers, stream=None):
        """The same launches with the kernels' scratch in the library's own device array: no allocation happens."""
        ptrs = [(b.ptr if hasattr(b, "ptr") else C.c_void_p(b)) for b in buffers]
        argv = (C.c_void_p * len(ptrs))(*ptrs)
        check(lib.he_tile_kernel_execute_noalloc(self.handle, argv, len(ptrs), _h(stream)))

    def __del__(self):
        try:
            if self.handle:
                lib.he_tile_kernel_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass
