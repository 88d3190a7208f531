"""The HIP backend over the C ABI: tensors, plan generation and execute_graph — the host-side mirror of
helium/src/backend.rs (traits Backend / Executor), helium/src/backend/plan_generation.rs and helium/src/cuda.rs."""
import ctypes as C

import numpy as np

from . import _ffi
from ._ffi import check, lib
from .device import NP_STORAGE, init

_ffi._sig("he_matmul_kernel_create", C.POINTER(C.c_void_p), C.c_void_p, C.POINTER(C.c_uint32), C.c_int)
_ffi._sig("he_tensor_create_with_data", C.POINTER(C.c_void_p), C.c_void_p, C.c_int, C.c_size_t)
_ffi._sig("he_tensor_download", C.c_void_p, C.c_void_p)
_ffi._sig("he_tensor_info", C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
          C.POINTER(C.c_void_p))
_ffi._sig("he_tensor_free", C.c_void_p)
_ffi._sig("he_plan_generate", C.c_void_p, C.POINTER(C.c_void_p))
_ffi._sig("he_plan_num_steps", C.c_void_p, C.POINTER(C.c_int))
_ffi._sig("he_plan_describe", C.c_void_p, restype=C.c_char_p)
_ffi._sig("he_plan_graph", C.c_void_p, C.POINTER(C.c_void_p))
_ffi._sig("he_plan_describe_planned", C.c_void_p, restype=C.c_char_p)
_ffi._sig("he_plan_destroy", C.c_void_p)
_ffi._sig("he_plan_precompile", C.c_void_p)
_ffi._sig("he_plan_instruction_kernel", C.c_void_p, C.c_int, C.POINTER(C.c_void_p))
_ffi._sig("he_execute_graph", C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_uint32),
          C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_int))
_ffi._sig("he_backend_stats", C.POINTER(C.c_uint64))
_ffi._sig("he_backend_set_option", C.c_int, C.c_int64)
OPT_FUSE_MATMUL_EPILOGUE = 0
OPT_FOLD_SWAP_INTO_REDUCE = 1
OPT_REMATERIALIZE = 2
OPT_CANCEL_TRANSPOSES = 3
OPT_HOIST_BROADCASTS = 4
OPT_STREAM_FAN_OUT = 5  # 0 one stream, 1 where it pays (default), 2 every step with several instructions


def set_option(option, value):
    check(lib.he_backend_set_option(option, int(value)))


class Tensor:
    """TensorStorage: a reference to device storage of `len` elements of `dtype` (Bool: bits)."""

    def __init__(self, handle):
        self.handle = handle
        self._info = None  # (dtype, len, nbytes, ptr), asked for on first use: a result that is only passed on costs no call

    def _get(self, i):
        if self._info is None:
            dt, ln, nb, ptr = C.c_int32(), C.c_uint64(), C.c_uint64(), C.c_void_p()
            check(lib.he_tensor_info(self.handle, C.byref(dt), C.byref(ln), C.byref(nb), C.byref(ptr)))
            self._info = (_ffi.DTYPE_NAMES[dt.value], ln.value, nb.value, ptr)
        return self._info[i]

    dtype = property(lambda self: self._get(0))
    len = property(lambda self: self._get(1))
    nbytes = property(lambda self: self._get(2))
    ptr = property(lambda self: self._get(3))

    @classmethod
    def from_numpy(cls, storage, dtype, length=None):
        """Backend::create_tensor_with_data. `storage`: array in storage form (uint16 bit patterns for bf16/f16,
        packed uint32 words for bool)."""
        init()
        storage = np.ascontiguousarray(storage)
        length = storage.size if length is None else length
        h = C.c_void_p()
        check(lib.he_tensor_create_with_data(C.byref(h), storage.ctypes.data_as(C.c_void_p), _ffi.DTYPES[dtype], length))
        t = cls(h)
        assert t.nbytes == storage.nbytes, (t.nbytes, storage.nbytes)
        return t

    def to_numpy(self):
        """Backend::download_tensor (blocking): the storage-form array."""
        np_dtype = NP_STORAGE[_ffi.DTYPES[self.dtype]]
        out = np.empty(self.nbytes // np.dtype(np_dtype).itemsize, dtype=np_dtype)
        check(lib.he_tensor_download(self.handle, out.ctypes.data_as(C.c_void_p)))
        return out

    def free(self):
        if self.handle:
            lib.he_tensor_free(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Plan:
    """generate_plan for a graph: `steps` is a list of (instructions, released nodes); an instruction is
    (kind, [node ids])."""

    def __init__(self, graph):
        self.handle = C.c_void_p()
        check(lib.he_plan_generate(graph.handle, C.byref(self.handle)))
        self.text = lib.he_plan_describe(self.handle).decode()
        self.steps = self._parse(self.text)

    def planned_steps(self):
        """`steps` with the node ids of `graph()` instead of the planned graph's."""
        return self._parse(lib.he_plan_describe_planned(self.handle).decode())

    @staticmethod
    def _parse(text):
        steps = []
        for line in text.strip().split("\n"):
            body, rel = line.split("|")
            instrs = []
            for tok in body.split(":", 1)[1].split():
                kind, nodes = tok.split("{")
                instrs.append((kind, [int(x) for x in nodes.rstrip("}").split(",") if x]))
            released = [int(x) for x in rel.replace("release", "").split()]
            steps.append((instrs, released))
        return steps

    def graph(self):
        """The graph the instructions are made of (he_plan_graph): the planned graph as the backend's rewrites left
        it, as an ir.OpGraph whose node dicts carry "origin"."""
        from . import ir

        handle = C.c_void_p()
        check(lib.he_plan_graph(self.handle, C.byref(handle)))
        return ir.OpGraph.from_handle(handle)

    def kernel(self, index):
        """The compiled kernel of the index-th instruction (he_plan_instruction_kernel), as a kernels.TileKernel whose
        argument nodes are nodes of `graph()`."""
        from .kernels import TileKernel

        h = C.c_void_p()
        check(lib.he_plan_instruction_kernel(self.handle, index, C.byref(h)))
        return TileKernel(h)

    def precompile(self):
        """Compiles the kernels of all instructions (in parallel) into the kernel caches; needs no device."""
        check(lib.he_plan_precompile(self.handle))

    def __del__(self):
        try:
            if self.handle:
                lib.he_plan_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass


def execute_graph(graph, inputs):
    """BackendExt::execute_graph. `inputs`: {input node id: Tensor}. Returns {output node id: Tensor}."""
    init()
    n = len(inputs)
    # array types are cached per size: building a ctypes array type costs more than filling an array
    in_nodes_t, in_handles_t = _array_types(max(n, 1))
    nodes = in_nodes_t(*inputs.keys())
    handles = in_handles_t(*[t.handle for t in inputs.values()])
    cap = max(1, graph.num_outputs)
    out_nodes_t, out_handles_t = _array_types(cap)
    out_nodes = out_nodes_t()
    out_handles = out_handles_t()
    count = C.c_int()
    check(lib.he_execute_graph(graph.handle, nodes, handles, n, out_nodes, out_handles, cap, C.byref(count)))
    return {out_nodes[i]: Tensor(C.c_void_p(out_handles[i])) for i in range(count.value)}


_ARRAY_TYPES = {}


def _array_types(n):
    t = _ARRAY_TYPES.get(n)
    if t is None:
        t = _ARRAY_TYPES[n] = (C.c_uint32 * n, C.c_void_p * n)
    return t


def stats():
    s = (C.c_uint64 * 9)()
    check(lib.he_backend_stats(s))
    keys = ["steps", "instrs", "streams_used", "event_waits", "plan_cache_hits", "plan_cache_misses", "pool_bytes",
            "pool_driver_allocs", "pool_reuses"]
    return dict(zip(keys, [int(x) for x in s]))


def matmul_kernel(graph, nodes):
    """MatmulGenerator::new(subgraph).generate(..): the fused-GEMM kernel of a Matmul-anchored helium-ir subgraph."""
    from .kernels import TileKernel

    h = C.c_void_p()
    check(lib.he_matmul_kernel_create(C.byref(h), graph.handle, _ffi.arr(C.c_uint32, nodes), len(nodes)))
    return TileKernel(h)
