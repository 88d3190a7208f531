"""Fusion-IR graph builder over the C ABI — host-side mirror of helium-playground/src/opgraph.rs.

Shapes are [batch, rows, cols]. Like `ir.OpGraph`, every node is also recorded as plain data in `self.nodes`.
"""
import ctypes as C

from . import _ffi
from ._ffi import check, lib

KINDS = ["producer", "constant", "matmul", "unary", "reduction", "binary", "broadcast", "transpose", "consumer"]
UNARY = ["neg", "relu", "gelu", "tanh", "exp", "ln", "sqrt", "add_constant", "mul_constant", "pow_constant"]
BINARY = ["add", "sub", "mul", "div", "pow", "drelu"]
DEPTH = ["rows", "columns", "item", "batch"]
AUTO = 0xFFFFFFFFFFFFFFFF


class FOpDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("shape", C.c_uint32 * 3), ("value", C.c_float), ("a", C.c_uint64),
                ("b", C.c_uint64), ("sub_op", C.c_int32), ("constant", C.c_float), ("depth", C.c_int32),
                ("axis", C.c_uint32), ("amount", C.c_uint32), ("dtype", C.c_int32)]


_ffi._sig("he_fgraph_create", C.POINTER(C.c_void_p))
_ffi._sig("he_fgraph_destroy", C.c_void_p)
_ffi._sig("he_fgraph_insert", C.c_void_p, C.POINTER(FOpDesc), C.POINTER(C.c_uint64))
_ffi._sig("he_fgraph_shape", C.c_void_p, C.c_uint64, C.POINTER(C.c_uint32))


class OpGraph:
    def __init__(self):
        self.handle = C.c_void_p()
        check(lib.he_fgraph_create(C.byref(self.handle)))
        self.nodes = []

    def __del__(self):
        try:
            if self.handle:
                lib.he_fgraph_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass

    def _insert(self, kind, record, node_id=None, **f):
        d = FOpDesc()
        d.kind = KINDS.index(kind)
        d.dtype = _ffi.BF16
        for k, v in f.items():
            if k == "shape":
                for i in range(3):
                    d.shape[i] = v[i]
            else:
                setattr(d, k, v)
        node = C.c_uint64(AUTO if node_id is None else node_id)
        check(lib.he_fgraph_insert(self.handle, C.byref(d), C.byref(node)))
        self.nodes.append({"id": node.value, "op": kind, "shape": self.shape(node.value), **record})
        return node.value

    def shape(self, node):
        s = (C.c_uint32 * 3)()
        check(lib.he_fgraph_shape(self.handle, node, s))
        return list(s)

    def producer(self, shape, dtype="bf16", node_id=None):
        return self._insert("producer", {"dtype": dtype}, node_id, shape=shape, dtype=_ffi.DTYPES[dtype])

    def constant(self, shape, value, node_id=None):
        return self._insert("constant", {"value": float(value)}, node_id, shape=shape, value=float(value))

    def matmul(self, a, b, node_id=None):
        return self._insert("matmul", {"a": a, "b": b}, node_id, a=a, b=b)

    def unary(self, x, op, constant=0.0, node_id=None):
        return self._insert("unary", {"x": x, "fn": op, "constant": float(constant)}, node_id, a=x,
                            sub_op=UNARY.index(op), constant=float(constant))

    def binary(self, lhs, rhs, op, node_id=None):
        return self._insert("binary", {"lhs": lhs, "rhs": rhs, "fn": op}, node_id, a=lhs, b=rhs, sub_op=BINARY.index(op))

    def reduction(self, x, depth, node_id=None):
        return self._insert("reduction", {"x": x, "depth": depth}, node_id, a=x, depth=DEPTH.index(depth))

    def broadcast(self, x, axis, amount, node_id=None):
        return self._insert("broadcast", {"x": x, "axis": axis, "amount": amount}, node_id, a=x, axis=axis, amount=amount)

    def transpose(self, x, node_id=None):
        return self._insert("transpose", {"x": x}, node_id, a=x)

    def consumer(self, x, dtype="bf16", node_id=None):
        return self._insert("consumer", {"x": x, "dtype": dtype}, node_id, a=x, dtype=_ffi.DTYPES[dtype])
