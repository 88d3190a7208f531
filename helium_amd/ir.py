"""helium-ir OpGraph builder over the C ABI — the host-side mirror of helium-ir/src/opgraph.rs and op.rs.

Every node is created in the library (which performs the shape / dtype inference) and also recorded as plain
data in `self.nodes`, so that a test can hand the very same graph description to the CPU oracle.
"""
import ctypes as C
import struct

import numpy as np

from . import _ffi
from ._ffi import check, lib

KINDS = ["matmul", "unary", "binary", "change_dtype", "reduce", "broadcast", "reshape", "swap_dims", "compare",
         "select", "conv", "conv_bwd_data", "conv_bwd_filter", "constant"]
UNARY = ["recip", "neg", "exp", "sin", "cos", "tan", "sigmoid", "tanh", "relu", "sqrt", "log"]
BINARY = ["add", "mul", "pow", "min", "max", "and", "or", "xor"]
REDUCE = ["sum", "mean", "max", "min"]
COMPARE = ["eq", "ne", "lt", "le", "gt", "ge"]
PADDING = ["same", "valid", "full"]
PRECISION = ["f32_f32", "tf32_f32", "bf16_f32", "f16_f32", "f16_f16", "f8_f32", "f8_f16"]


class OpDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("inputs", C.c_uint32 * 3), ("num_inputs", C.c_int32), ("sub_op", C.c_int32),
                ("precision", C.c_int32), ("target_type", C.c_int32), ("depth", C.c_uint32),
                ("new_dim_count", C.c_int64), ("broadcast_axes", C.POINTER(C.c_int64)),
                ("num_broadcast_axes", C.c_int32), ("shape", C.POINTER(C.c_int64)), ("shape_rank", C.c_int32),
                ("axis_a", C.c_int64), ("axis_b", C.c_int64), ("const_bits", C.c_uint32), ("const_dtype", C.c_int32),
                ("conv_in_channels", C.c_int64), ("conv_out_channels", C.c_int64), ("conv_kernel", C.c_int64 * 2),
                ("conv_stride", C.c_int64 * 2), ("conv_dilation", C.c_int64 * 2), ("conv_padding_mode", C.c_int32),
                ("conv_input_size", C.c_int64 * 2)]


_ffi._sig("he_graph_create", C.POINTER(C.c_void_p))
_ffi._sig("he_graph_destroy", C.c_void_p)
_ffi._sig("he_graph_new_input", C.c_void_p, C.POINTER(C.c_int64), C.c_int, C.c_int, C.POINTER(C.c_uint32))
_ffi._sig("he_graph_new_op", C.c_void_p, C.POINTER(OpDesc), C.POINTER(C.c_uint32))
_ffi._sig("he_graph_new_output", C.c_void_p, C.c_uint32, C.POINTER(C.c_uint32))
_ffi._sig("he_graph_optimize", C.c_void_p)
_ffi._sig("he_graph_num_nodes", C.c_void_p, C.POINTER(C.c_uint32))
_ffi._sig("he_graph_node_info", C.c_void_p, C.c_uint32, C.POINTER(C.c_int32), C.POINTER(C.c_int32),
          C.POINTER(C.c_int32), C.POINTER(C.c_int64))
_ffi._sig("he_graph_node_op", C.c_void_p, C.c_uint32, C.POINTER(OpDesc), C.POINTER(C.c_int64), C.POINTER(C.c_int64),
          C.POINTER(C.c_uint32))
_ffi._sig("he_graph_capacity", C.c_void_p, C.POINTER(C.c_uint32))


def scalar_bits(value, dtype):
    """Bit pattern of a Constant's Scalar in its own dtype (helium-ir/src/data_type.rs:391-438)."""
    if dtype == "f32":
        return struct.unpack("<I", struct.pack("<f", float(value)))[0]
    if dtype == "bf16":
        u = struct.unpack("<I", struct.pack("<f", float(value)))[0]
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF
    if dtype == "f16":
        return int(np.array(value, dtype=np.float16).view(np.uint16))
    if dtype == "u32":
        return int(value) & 0xFFFFFFFF
    if dtype == "bool":
        return 1 if value else 0
    raise ValueError(dtype)


def scalar_from_bits(bits, dtype):
    """Inverse of scalar_bits."""
    if dtype == "f32":
        return struct.unpack("<f", struct.pack("<I", bits))[0]
    if dtype == "bf16":
        return struct.unpack("<f", struct.pack("<I", (bits & 0xFFFF) << 16))[0]
    if dtype == "f16":
        return float(np.array(bits & 0xFFFF, dtype=np.uint16).view(np.float16))
    if dtype == "u32":
        return int(bits)
    if dtype == "bool":
        return bool(bits)
    raise ValueError(dtype)


class OpGraph:
    def __init__(self):
        self.handle = C.c_void_p()
        check(lib.he_graph_create(C.byref(self.handle)))
        self.nodes = []  # plain-data record of the graph: dicts with id / kind / op fields
        self.num_outputs = 0

    def __del__(self):
        try:
            if self.handle:
                lib.he_graph_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass

    @classmethod
    def from_handle(cls, handle):
        """Takes over a graph handle the library made (he_plan_graph) and reads its nodes back; every node dict also
        carries "origin", the node of the planned graph it stands for."""
        self = cls.__new__(cls)
        self.handle, self.nodes, self.num_outputs = handle, [], 0
        cap = C.c_uint32()
        check(lib.he_graph_capacity(handle, C.byref(cap)))
        d, axes, shape, origin = OpDesc(), (C.c_int64 * 32)(), (C.c_int64 * 16)(), C.c_uint32()
        kind, dtype, rank, dims = C.c_int32(), C.c_int32(), C.c_int32(), (C.c_int64 * 16)()
        for i in range(cap.value):
            if lib.he_graph_node_info(handle, i, C.byref(kind), C.byref(dtype), C.byref(rank), dims) != 0 or kind.value == 3:
                continue  # pruned
            check(lib.he_graph_node_op(handle, i, C.byref(d), axes, shape, C.byref(origin)))
            desc = {"shape": list(dims[: rank.value]), "dtype": _ffi.DTYPE_NAMES[dtype.value]}
            if kind.value == 0:
                n = {"id": i, "node": "input", **desc}
            elif kind.value == 2:
                n = {"id": i, "node": "output", "from": d.inputs[0]}
                self.num_outputs += 1
            else:
                op = KINDS[d.kind]
                n = {"id": i, "node": "op", "op": op, "inputs": list(d.inputs[: d.num_inputs]), **desc}
                if op == "matmul":
                    n["precision"] = PRECISION[d.precision]
                elif op in ("unary", "binary", "reduce", "compare"):
                    n["fn"] = {"unary": UNARY, "binary": BINARY, "reduce": REDUCE, "compare": COMPARE}[op][d.sub_op]
                    if op == "reduce":
                        n["depth"] = d.depth
                elif op == "change_dtype":
                    n["target"] = _ffi.DTYPE_NAMES[d.target_type]
                elif op == "broadcast":
                    n["new_dim_count"] = d.new_dim_count
                    n["axes"] = [[axes[2 * k], axes[2 * k + 1]] for k in range(d.num_broadcast_axes)]
                elif op == "reshape":
                    n["new_shape"] = list(shape[: d.shape_rank])
                elif op == "swap_dims":
                    n["axis_a"], n["axis_b"] = d.axis_a, d.axis_b
                elif op == "constant":
                    n["const_dtype"] = _ffi.DTYPE_NAMES[d.const_dtype]
                    n["value"] = scalar_from_bits(d.const_bits, n["const_dtype"])
                elif op in ("conv", "conv_bwd_data", "conv_bwd_filter"):
                    n["params"] = {"in_channels": d.conv_in_channels, "out_channels": d.conv_out_channels,
                                   "kernel_size": list(d.conv_kernel), "stride": list(d.conv_stride),
                                   "dilation": list(d.conv_dilation), "padding_mode": PADDING[d.conv_padding_mode]}
                    if op == "conv_bwd_data":
                        n["input_size"] = list(d.conv_input_size)
            n["origin"] = origin.value
            self.nodes.append(n)
        return self

    # -- node creation -----------------------------------------------------------------------------------
    def new_input(self, shape, dtype):
        node = C.c_uint32()
        check(lib.he_graph_new_input(self.handle, _ffi.arr(C.c_int64, shape), len(shape), _ffi.DTYPES[dtype],
                                     C.byref(node)))
        self.nodes.append({"id": node.value, "node": "input", "shape": list(shape), "dtype": dtype})
        return node.value

    def new_output(self, from_node):
        node = C.c_uint32()
        check(lib.he_graph_new_output(self.handle, from_node, C.byref(node)))
        self.nodes.append({"id": node.value, "node": "output", "from": from_node})
        self.num_outputs += 1
        return node.value

    def _op(self, kind, inputs, record, **f):
        d = OpDesc()
        d.kind = KINDS.index(kind)
        for i, x in enumerate(inputs):
            d.inputs[i] = x
        d.num_inputs = len(inputs)
        keep = []
        for k, v in f.items():
            if k in ("broadcast_axes", "shape"):
                a = _ffi.arr(C.c_int64, v)
                keep.append(a)
                setattr(d, k, C.cast(a, C.POINTER(C.c_int64)))
            else:
                setattr(d, k, v)
        node = C.c_uint32()
        check(lib.he_graph_new_op(self.handle, C.byref(d), C.byref(node)))
        shape, dtype = self.descriptor(node.value)
        self.nodes.append({"id": node.value, "node": "op", "op": kind, "inputs": list(inputs), "shape": shape,
                           "dtype": dtype, **record})
        return node.value

    def matmul(self, a, b, precision="bf16_f32"):
        return self._op("matmul", [a, b], {"precision": precision}, precision=PRECISION.index(precision))

    def unary(self, x, op):
        return self._op("unary", [x], {"fn": op}, sub_op=UNARY.index(op))

    def binary(self, lhs, rhs, op):
        return self._op("binary", [lhs, rhs], {"fn": op}, sub_op=BINARY.index(op))

    def change_data_type(self, x, target):
        return self._op("change_dtype", [x], {"target": target}, target_type=_ffi.DTYPES[target])

    def reduce(self, x, op, depth):
        return self._op("reduce", [x], {"fn": op, "depth": depth}, sub_op=REDUCE.index(op), depth=depth)

    def broadcast(self, x, new_dim_count, axes):
        """axes: list of (axis, new_size) — BroadcastAxis (op.rs:397-407)."""
        flat = [int(v) for a in axes for v in a]
        return self._op("broadcast", [x], {"new_dim_count": new_dim_count, "axes": [list(a) for a in axes]},
                        new_dim_count=new_dim_count, broadcast_axes=flat, num_broadcast_axes=len(axes))

    def reshape(self, x, new_shape):
        return self._op("reshape", [x], {"new_shape": list(new_shape)}, shape=list(new_shape), shape_rank=len(new_shape))

    def swap_dims(self, x, axis_a, axis_b):
        return self._op("swap_dims", [x], {"axis_a": axis_a, "axis_b": axis_b}, axis_a=axis_a, axis_b=axis_b)

    def compare(self, lhs, rhs, op):
        return self._op("compare", [lhs, rhs], {"fn": op}, sub_op=COMPARE.index(op))

    def select(self, lhs, rhs, selector):
        """lhs where the selector is false, rhs where it is true (op.rs:439-445)."""
        return self._op("select", [lhs, rhs, selector], {})

    def _conv_fields(self, params, input_size=(0, 0)):
        """params: dict with in_channels, out_channels, kernel_size, stride, dilation, padding_mode (Conv2dParams)."""
        two = C.c_int64 * 2
        return dict(conv_in_channels=params["in_channels"], conv_out_channels=params["out_channels"],
                    conv_kernel=two(*params["kernel_size"]), conv_stride=two(*params.get("stride", (1, 1))),
                    conv_dilation=two(*params.get("dilation", (1, 1))),
                    conv_padding_mode=PADDING.index(params.get("padding_mode", "same")), conv_input_size=two(*input_size))

    def conv(self, image, filter_, params):
        """Op::Conv: NHWC image, [out_channels, kh, kw, in_channels] filter (op.rs:447-452)."""
        return self._op("conv", [image, filter_], {"params": dict(params)}, **self._conv_fields(params))

    def conv_backward_data(self, flow, filter_, params, input_size):
        return self._op("conv_bwd_data", [flow, filter_], {"params": dict(params), "input_size": list(input_size)},
                        **self._conv_fields(params, input_size))

    def conv_backward_filter(self, flow, image, params):
        return self._op("conv_bwd_filter", [flow, image], {"params": dict(params)}, **self._conv_fields(params))

    def constant(self, value, dtype, shape):
        return self._op("constant", [], {"value": value, "const_dtype": dtype}, shape=list(shape),
                        shape_rank=len(shape), const_bits=scalar_bits(value, dtype), const_dtype=_ffi.DTYPES[dtype])

    # -- queries -----------------------------------------------------------------------------------------
    def descriptor(self, node):
        kind, dtype, rank = C.c_int32(), C.c_int32(), C.c_int32()
        shape = (C.c_int64 * 16)()
        check(lib.he_graph_node_info(self.handle, node, C.byref(kind), C.byref(dtype), C.byref(rank), shape))
        return list(shape[: rank.value]), _ffi.DTYPE_NAMES[dtype.value]

    def num_nodes(self):
        n = C.c_uint32()
        check(lib.he_graph_num_nodes(self.handle, C.byref(n)))
        return n.value

    def optimize(self):
        check(lib.he_graph_optimize(self.handle))
