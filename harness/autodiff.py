"""Graph recorder with reverse-mode differentiation: the host-side mirror of the reference's lazy `RawTensor`
(helium/src/raw_tensor.rs), the `Tensor` methods with their gradient rules (helium/src/tensor.rs) and the tape that
replays them (helium/src/tensor/tape.rs). It only records helium-ir ops; running the recorded graph is the backend's job.

It exists so that tests and the benchmark can hand `execute_graph` the graphs the reference's front end would hand it
(forward, backward and optimizer step of a training iteration) - it is harness code, not part of the backend.

One `Graph` stands for one OpGraphBuilder: every tensor recorded on it is a node of the same helium-ir graph. A concrete
tensor becomes a graph input; a 1-element concrete tensor is shared per value, as the reference's scalar cache makes it
(raw_tensor.rs:63-75).
"""
import itertools

import numpy as np

from helium_amd import ir

FLOATS = ("f32", "bf16", "f16")


def _to_storage(values, dtype):
    values = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == "f32":
        return values
    if dtype == "bf16":
        u = values.view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    if dtype == "f16":
        return values.astype(np.float16).view(np.uint16)
    raise ValueError(dtype)


class Graph:
    def __init__(self):
        self.g = ir.OpGraph()
        self.feeds = {}  # input node -> storage array
        self._scalars = {}  # (value bits, dtype) -> Raw

    # -- concrete tensors ---------------------------------------------------------------------------------
    def raw_from_storage(self, storage, shape, dtype):
        node = self.g.new_input(list(shape), dtype)
        self.feeds[node] = np.ascontiguousarray(storage).reshape(-1)
        return Raw(self, node)

    def raw_from_slice(self, values, shape, dtype="f32"):
        """RawTensor::from_slice (raw_tensor.rs:61-76)."""
        values = np.asarray(values, dtype=np.float32)
        if values.size == 1:
            key = (values.reshape(-1).view(np.uint32)[0].item(), dtype, tuple(shape))
            if key not in self._scalars:
                self._scalars[key] = self.raw_from_storage(_to_storage(values, dtype), shape, dtype)
            return self._scalars[key]
        return self.raw_from_storage(_to_storage(values, dtype), shape, dtype)

    def raw_constant(self, value, shape, dtype="f32"):
        """RawTensor::from_constant: an Op::Constant (raw_tensor.rs:107-123)."""
        return Raw(self, self.g.constant(value, dtype, list(shape)))

    def tensor(self, values, shape=None, dtype="f32"):
        values = np.asarray(values, dtype=np.float32)
        return Tensor(self.raw_from_slice(values, list(values.shape) if shape is None else shape, dtype))

    def constant(self, value, shape, dtype="f32"):
        return Tensor(self.raw_constant(value, shape, dtype))

    def param(self, values, shape=None, dtype="f32"):
        return Param(self.tensor(values, shape, dtype))


class Raw:
    """A node of the graph with the reference's op lowerings as methods (raw_tensor.rs)."""

    def __init__(self, graph, node):
        self.G = graph
        self.node = node
        self._desc = None

    def _d(self):
        if self._desc is None:
            self._desc = self.G.g.descriptor(self.node)
        return self._desc

    shape = property(lambda self: list(self._d()[0]))
    dtype = property(lambda self: self._d()[1])

    def _new(self, node):
        return Raw(self.G, node)

    def _scalar(self, value):
        return self.G.raw_from_slice([value], [1]).broadcast_to(self.shape)

    def unary(self, fn):
        return self._new(self.G.g.unary(self.node, fn))

    def binary(self, other, fn):
        assert self.shape == other.shape, (fn, self.shape, other.shape)
        return self._new(self.G.g.binary(self.node, other.node, fn))

    def __neg__(self):
        return self.unary("neg")

    def __add__(self, other):
        return self.binary(other if isinstance(other, Raw) else self._scalar(other), "add")

    def __sub__(self, other):  # self + -rhs (raw_tensor.rs:647-661)
        return self + (-other)

    def __mul__(self, other):
        return self.binary(other if isinstance(other, Raw) else self._scalar(other), "mul")

    def __truediv__(self, other):  # self * rhs.recip() (raw_tensor.rs:679-695); an f32 is inverted on the host
        if isinstance(other, Raw):
            return self * other.recip()
        return self * float(np.float32(1.0) / np.float32(other))

    def recip(self):
        return self.unary("recip")

    def exp(self):
        return self.unary("exp")

    def log(self):
        return self.unary("log")

    def sin(self):
        return self.unary("sin")

    def cos(self):
        return self.unary("cos")

    def tan(self):
        return self.unary("tan")

    def sqrt(self):
        return self.unary("sqrt")

    def sigmoid(self):
        return self.unary("sigmoid")

    def tanh(self):
        return self.unary("tanh")

    def relu(self):
        return self.unary("relu")

    def min(self, other):
        return self.binary(other, "min")

    def max(self, other):
        return self.binary(other, "max")

    def pow(self, other):
        return self.broadcast_to(other.shape).binary(other, "pow")

    def pow_scalar(self, power):
        return self.pow(self._scalar(power))

    def into_data_type(self, dtype):
        return self if dtype == self.dtype else self._new(self.G.g.change_data_type(self.node, dtype))

    def matmul(self, rhs, precision):
        """raw_tensor.rs:179-231: the product comes in the accumulator type and is cast back to the lhs type."""
        assert self.dtype == rhs.dtype
        out = self._new(self.G.g.matmul(self.node, rhs.node, precision))
        return out.into_data_type(self.dtype)

    def conv2d(self, filt, params):
        return self._new(self.G.g.conv(self.node, filt.node, params))

    def conv2d_backward_data(self, filt, params, input_size):
        return self._new(self.G.g.conv_backward_data(self.node, filt.node, params, input_size))

    def conv2d_backward_filter(self, image, params):
        return self._new(self.G.g.conv_backward_filter(self.node, image.node, params))

    def swap_dims(self, a, b):
        return self if a == b else self._new(self.G.g.swap_dims(self.node, a, b))

    def transpose(self):
        n = len(self.shape)
        return self.swap_dims(n - 1, n - 2)

    def broadcast_to(self, new_shape):
        """raw_tensor.rs:370-424"""
        new_shape = list(new_shape)
        old = self.shape
        if new_shape == old:
            return self
        d, d2 = len(old), len(new_shape)
        axes = []
        for rev, (o, n) in enumerate(zip(reversed(old), reversed(new_shape))):
            if o != 1:
                assert o == n, f"cannot broadcast axis of size {o} to {n}"
            if o == 1 and n != 1:
                axes.append((d2 - rev - 1, n))
        for i in range(d2 - d):
            axes.append((i, new_shape[i]))
        return self._new(self.G.g.broadcast(self.node, d2, axes))

    def reshape(self, new_shape):
        new_shape = list(new_shape)
        return self if new_shape == self.shape else self._new(self.G.g.reshape(self.node, new_shape))

    def _reduce(self, fn, depth):
        """raw_tensor.rs:817-858: a Reduce yields f32 and is cast back to the input type."""
        if depth == 0:
            return self
        return self._new(self.G.g.reduce(self.node, fn, depth)).into_data_type(self.dtype)

    def reduce_sum(self, depth):
        return self._reduce("sum", depth)

    def reduce_mean(self, depth):
        return self._reduce("mean", depth)

    def reduce_min(self, depth):
        return self._reduce("min", depth)

    def reduce_max(self, depth):
        return self._reduce("max", depth)

    def compare(self, rhs, fn):
        return self._new(self.G.g.compare(self.node, rhs.node, fn))

    def select(self, true_case, false_case):
        """RawTensor::select on a Bool tensor: Op::Select { lhs: false case, rhs: true case } (raw_tensor.rs:548-579)."""
        return self._new(self.G.g.select(false_case.node, true_case.node, self.node))


# ---- tape (tensor/tape.rs) ------------------------------------------------------------------------------------
_positions = itertools.count()


class _Node:
    children = ()

    def __init__(self):
        self.position = next(_positions)


class _Constant(_Node):
    def __init__(self, activation):
        super().__init__()
        self._activation = activation

    def activation(self, state):
        return self._activation

    def backprop(self, state, grads, flow):
        pass


class _ParamNode(_Node):
    def __init__(self, pid, value):
        super().__init__()
        self.pid, self.value = pid, value

    def activation(self, state):
        return self.value

    def backprop(self, state, grads, flow):
        assert self.pid not in grads
        grads[self.pid] = flow


class _Unary(_Node):
    def __init__(self, prev, op, flow):
        super().__init__()
        self.children = (prev,)
        self.op, self.flow = op, flow

    def activation(self, state):
        return self.op(state.get_activation(self.children[0]))

    def backprop(self, state, grads, flow):
        x = state.get_activation(self.children[0])
        state.propagate(self.children[0], grads, self.flow(x, flow))


class _Binary(_Node):
    def __init__(self, prev1, prev2, op, flow1, flow2):
        super().__init__()
        self.children = (prev1, prev2)
        self.op, self.flow1, self.flow2 = op, flow1, flow2

    def activation(self, state):
        return self.op(state.get_activation(self.children[0]), state.get_activation(self.children[1]))

    def backprop(self, state, grads, flow):
        a = state.get_activation(self.children[0])
        b = state.get_activation(self.children[1])
        f1 = self.flow1(a, b, flow)
        f2 = self.flow2(a, b, flow)
        state.propagate(self.children[0], grads, f1)
        state.propagate(self.children[1], grads, f2)


class _Checkpoint(_Node):
    def __init__(self, prev, activation):
        super().__init__()
        self.children = (prev,)
        self._activation = activation

    def activation(self, state):
        return self._activation

    def backprop(self, state, grads, flow):
        state.propagate(self.children[0], grads, flow)


class _State:
    """tape.rs:93-158: activations are recomputed from the last checkpoint (memoised per backward pass); a node's flow
    is passed on when every one of its uses has delivered its share."""

    def __init__(self, root):
        self.remaining, self.acc, self.memo = {}, {}, {}
        stack, seen = [root], set()
        while stack:
            n = stack.pop()
            if n.position in seen:
                continue
            seen.add(n.position)
            for c in n.children:
                self.remaining[c.position] = self.remaining.get(c.position, 0) + 1
                stack.append(c)

    def get_activation(self, node):
        if node.position not in self.memo:
            self.memo[node.position] = node.activation(self)
        return self.memo[node.position]

    def propagate(self, child, grads, flow):
        self.remaining[child.position] -= 1
        self.acc[child.position] = flow if child.position not in self.acc else self.acc[child.position] + flow
        if self.remaining[child.position] == 0:
            child.backprop(self, grads, self.acc.pop(child.position))


_param_ids = itertools.count(1)


class Param:
    """tensor/param.rs"""

    def __init__(self, value):
        self.id = next(_param_ids)
        self.set_value(value)

    def set_value(self, value):
        self.value = Tensor(value.raw, _ParamNode(self.id, value.raw))


def _t(x):
    return x.value if isinstance(x, Param) else x


def apply_permutation_via_swaps(n, perm):
    """tensor.rs:840-857"""
    swaps = []
    perm = [perm(i) for i in range(n)]
    for i in range(n):
        if perm[i] == i:
            continue
        for j in range(i + 1, n):
            if perm[j] == i:
                swaps.append((i, j))
                perm[i], perm[j] = perm[j], perm[i]
                break
    return swaps


class Tensor:
    """Tensor<D, Float> (tensor.rs): a Raw plus an optional tape."""

    def __init__(self, raw, tape=None):
        self.raw = raw
        self.tape = tape

    shape = property(lambda self: self.raw.shape)
    dtype = property(lambda self: self.raw.dtype)
    G = property(lambda self: self.raw.G)

    # -- autodiff plumbing (tensor.rs:748-810) -------------------------------------------------------------
    def _op(self, compute, gradient):
        tape = _Unary(self.tape, compute, gradient) if self.tape is not None else None
        return Tensor(compute(self.raw), tape)

    def _op_binary(self, rhs, compute, grad_left, grad_right):
        rhs = _t(rhs)
        tape = None
        if self.tape is not None or rhs.tape is not None:
            lt = self.tape if self.tape is not None else _Constant(self.raw)
            rt = rhs.tape if rhs.tape is not None else _Constant(rhs.raw)
            tape = _Binary(lt, rt, compute, grad_left, grad_right)
        return Tensor(compute(self.raw, rhs.raw), tape)

    def checkpoint(self):
        return Tensor(self.raw, _Checkpoint(self.tape, self.raw) if self.tape is not None else None)

    def detach(self):
        return Tensor(self.raw)

    def backward(self):
        """tensor.rs:236-247: the flow that enters the tape is the constant 1.0 of shape [1]. Returns {param id: Raw}."""
        assert self.tape is not None, "backward() on a tensor without gradient tracking"
        grads = {}
        self.tape.backprop(_State(self.tape), grads, self.G.raw_constant(1.0, [1], "f32"))
        return grads

    def _scalar(self, value):
        return Tensor(self.G.raw_from_slice([value], [1])).broadcast_to(self.shape)

    # -- shape ops (tensor.rs:75-152) ----------------------------------------------------------------------
    def reshape(self, new_shape):
        old = self.shape
        return self._op(lambda x: x.reshape(new_shape), lambda _, flow: flow.reshape(old))

    def broadcast_to(self, new_shape):
        new_shape = list(new_shape)
        old = self.shape
        if old == new_shape:
            return self
        d, d2 = len(old), len(new_shape)
        axes = [(d2 - d) + i for i in range(d) if new_shape[(d2 - d) + i] != 1 and old[i] == 1]
        axes += list(range(d2 - d))
        mapping = {axis: k for k, axis in enumerate(axes)}
        offset = len(axes)
        for axis in range(d2):
            if axis not in axes:
                mapping[axis] = offset
                offset += 1
        mapping = {a: d2 - v - 1 for a, v in mapping.items()}
        inverse = {b: a for a, b in mapping.items()}

        def gradient(_, flow):
            for a, b in apply_permutation_via_swaps(d2, lambda x: mapping[x]):
                flow = flow.swap_dims(a, b)
            temp = old + [1] * (d2 - d)
            flow = flow.reduce_sum(len(axes)).reshape(temp)
            for a, b in apply_permutation_via_swaps(d2, lambda x: inverse[x]):
                flow = flow.swap_dims(a, b)
            return flow.reshape(old)

        return self._op(lambda x: x.broadcast_to(new_shape), gradient)

    def swap_dims(self, a, b):
        return self._op(lambda x: x.swap_dims(a, b), lambda _, flow: flow.swap_dims(a, b))

    def transpose(self):
        n = len(self.shape)
        return self.swap_dims(n - 1, n - 2)

    def to_data_type(self, dtype):
        old = self.dtype
        return self._op(lambda x: x.into_data_type(dtype), lambda _, flow: flow.into_data_type(old))

    # -- float math (tensor.rs:314-470) --------------------------------------------------------------------
    def recip(self):
        return self._op(lambda x: x.recip(), lambda x, flow: -(x.pow_scalar(-2.0)) * flow)

    def exp(self):
        return self._op(lambda x: x.exp(), lambda x, flow: x.exp() * flow)

    def log(self):
        return self._op(lambda x: x.log(), lambda x, flow: flow / x)

    def sigmoid(self):
        def gradient(x, flow):
            e = (-x).exp()
            return e / (e + 1.0).pow_scalar(2.0) * flow
        return self._op(lambda x: x.sigmoid(), gradient)

    def pow(self, power):
        def left(a, b, flow):
            return (b * a.pow(b - 1.0) * flow).into_data_type(flow.dtype)

        def right(a, b, flow):
            return (a.pow(b) * a.log() * flow).into_data_type(flow.dtype)
        return self._op_binary(power, lambda a, b: a.pow(b), left, right)

    def pow_scalar(self, power):
        return self.pow(self._scalar(power))

    def sqrt(self):
        return self._op(lambda x: x.sqrt(), lambda x, flow: flow / (x.sqrt() * 2.0))

    def sin(self):
        return self._op(lambda x: x.sin(), lambda x, flow: flow * x.cos())

    def cos(self):
        return self._op(lambda x: x.cos(), lambda x, flow: flow * -x.sin())

    def tan(self):
        return self._op(lambda x: x.tan(), lambda x, flow: flow / (x.cos().pow_scalar(2.0)))

    def relu(self):
        """tensor.rs:372-387: the mask is (x < 0) ? 0 : 1 through Compare + Select, cast to the flow's type."""
        def gradient(x, flow):
            zero = x.G.raw_constant(0.0, x.shape, "f32")
            one = x.G.raw_constant(1.0, x.shape, "f32")
            return x.compare(zero, "lt").select(zero, one).into_data_type(flow.dtype) * flow
        return self._op(lambda x: x.relu(), gradient)

    def _extremum(self, other, fn, cmp):
        def gradient(data, other_):
            ones = data.G.raw_constant(1.0, data.shape, "f32")
            zeros = data.G.raw_constant(0.0, data.shape, "f32")
            halves = data.G.raw_constant(0.5, data.shape, "f32")
            return data.compare(other_, cmp).select(ones, data.compare(other_, "eq").select(halves, zeros))
        return self._op_binary(other, lambda a, b: a.binary(b, fn), lambda a, b, flow: gradient(a, b) * flow,
                               lambda a, b, flow: gradient(b, a) * flow)

    def max(self, other):
        return self._extremum(other, "max", "gt")

    def min(self, other):
        return self._extremum(other, "min", "lt")

    def matmul(self, rhs, precision):
        """tensor.rs:447-455"""
        return self._op_binary(rhs, lambda a, b: a.matmul(b, precision),
                               lambda _a, b, flow: b.matmul(flow.transpose(), precision).transpose(),
                               lambda a, _b, flow: a.transpose().matmul(flow, precision)).checkpoint()

    def conv2d(self, filt, params):
        """tensor.rs:462-487"""
        input_size = self.shape[1:3]
        return self._op_binary(filt, lambda image, f: image.conv2d(f, params),
                               lambda _, f, flow: flow.conv2d_backward_data(f, params, input_size),
                               lambda image, _, flow: flow.conv2d_backward_filter(image, params)).checkpoint()

    def _reduced_shape(self, depth):
        shape = self.shape
        return shape[: len(shape) - depth] + [1] if depth else shape

    def reduce_sum(self, depth):
        shape, dtype = self.shape, self.dtype
        result_shape = self._reduced_shape(depth)

        def gradient(_, flow):
            padded = result_shape + [1] * (len(shape) - len(result_shape))
            return flow.reshape(padded).broadcast_to(shape).into_data_type(dtype)
        return self._op(lambda x: x.reduce_sum(depth), gradient)

    def reduce_mean(self, depth):
        shape, dtype = self.shape, self.dtype
        stride = int(np.prod(shape[len(shape) - depth:], dtype=np.int64))
        result_shape = self._reduced_shape(depth)

        def gradient(_, flow):
            padded = result_shape + [1] * (len(shape) - len(result_shape))
            scale = float(np.float32(1.0) / np.float32(stride))
            return (flow.reshape(padded).broadcast_to(shape) * scale).into_data_type(dtype)
        return self._op(lambda x: x.reduce_mean(depth), gradient)

    def _reduce_extremum(self, depth, which, count_dtype):
        """tensor.rs:522-592: the flow is shared evenly among the elements that equal the extremum; the count of
        matches is taken in f32 for min and in f16 for max."""
        shape, dtype = self.shape, self.dtype

        def gradient(x, flow):
            temp = flow.shape + [1] * (len(shape) - len(flow.shape))
            ext = getattr(x, "reduce_" + which)(depth).reshape(temp).broadcast_to(shape)
            mask = ext.compare(x, "eq")
            count = mask.into_data_type(count_dtype).reduce_sum(depth).reshape(temp).broadcast_to(shape)
            share = mask.select(count.recip(), x.G.raw_constant(0.0, shape, "f32"))
            return (share * flow.reshape(temp).broadcast_to(shape)).into_data_type(dtype)
        return self._op(lambda x: getattr(x, "reduce_" + which)(depth), gradient)

    def reduce_min(self, depth):
        return self._reduce_extremum(depth, "min", "f32")

    def reduce_max(self, depth):
        return self._reduce_extremum(depth, "max", "f16")

    def log_softmax(self):
        """tensor.rs:595-605 (rank 2)."""
        mx = self.reduce_max(1).broadcast_to(self.shape)
        return self - mx - (self - mx).exp().reduce_sum(1).log().broadcast_to(self.shape)

    # -- operators (tensor.rs:607-745) ---------------------------------------------------------------------
    def __neg__(self):
        return self._op(lambda x: -x, lambda _, flow: -flow)

    def __add__(self, rhs):
        if isinstance(rhs, (int, float)):
            rhs = self._scalar(rhs)
        return self._op_binary(rhs, lambda a, b: a + b, lambda _a, _b, flow: flow, lambda _a, _b, flow: flow)

    def __sub__(self, rhs):
        if isinstance(rhs, (int, float)):
            rhs = self._scalar(rhs)
        return self + (-_t(rhs))

    def __mul__(self, rhs):
        if isinstance(rhs, (int, float)):
            rhs = self._scalar(rhs)
        dtype = self.dtype
        return self._op_binary(rhs, lambda a, b: a * b, lambda _, b, flow: (b * flow).into_data_type(dtype),
                               lambda a, _, flow: (a * flow).into_data_type(dtype))

    def __truediv__(self, rhs):
        if isinstance(rhs, (int, float)):
            rhs = self._scalar(rhs)
        return self * _t(rhs).recip()


def cross_entropy_loss(logits, targets):
    """helium/src/loss.rs:5-8"""
    batch = logits.shape[0]
    return -(logits.log_softmax() * targets).reduce_sum(2) / float(batch)


def _clamped_log(x):
    return x.log().max(x.G.constant(-100.0, x.shape))


def binary_cross_entropy_loss(predictions, targets):
    """helium/src/loss.rs:10-20"""
    return -(targets * _clamped_log(predictions) + (-targets + 1.0) * _clamped_log(-predictions + 1.0)).reduce_mean(2)
