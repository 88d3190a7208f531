"""How the reference's lazy-tensor front end writes its tensor methods into helium-ir ops (helium/src/raw_tensor.rs,
helium/src/modules/batch_norm.rs, helium/src/optimizer/sgd.rs): scalar operands become 1-element inputs that are
broadcast, subtraction is add-of-negation, division is multiply-by-reciprocal. Used to build graphs of the shape the
reference would hand to `execute_graph`."""
import numpy as np


def scalar_tensor(g, value, like_shape):
    """`x op f32`: a 1-element f32 input broadcast to x's shape (raw_tensor.rs:638-645, broadcast_to :389-414).
    Returns (broadcast node, scalar input node, scalar storage)."""
    s = g.new_input([1], "f32")
    rank = len(like_shape)
    axes = []
    if like_shape[-1] != 1:
        axes.append((rank - 1, like_shape[-1]))
    for i in range(rank - 1):
        axes.append((i, like_shape[i]))
    b = g.broadcast(s, rank, axes)
    return b, s, np.array([value], dtype=np.float32)


def broadcast_to(g, x, x_shape, new_shape):
    """RawTensor::broadcast_to (raw_tensor.rs:370-424)."""
    d, d2 = len(x_shape), len(new_shape)
    axes = []
    for rev, (old, new) in enumerate(zip(reversed(x_shape), reversed(new_shape))):
        index = d2 - rev - 1
        if old != 1:
            assert old == new
        if old == 1 and new != 1:
            axes.append((index, new))
    for i in range(d2 - d):
        axes.append((i, new_shape[i]))
    return g.broadcast(x, d2, axes)


def sub(g, a, b):
    return g.binary(a, g.unary(b, "neg"), "add")  # a - b = a + (-b), raw_tensor.rs:647-653


def div(g, a, b):
    return g.binary(a, g.unary(b, "recip"), "mul")  # a / b = a * recip(b), raw_tensor.rs:679-686


class Recorder:
    """Collects the scalar inputs a graph needs next to its tensor inputs."""

    def __init__(self, g):
        self.g = g
        self.scalars = {}  # input node -> 1-element f32 array

    def shape(self, x):
        return self.g.descriptor(x)[0]

    def scalar_like(self, value, x):
        b, s, data = scalar_tensor(self.g, value, self.shape(x))
        self.scalars[s] = data
        return b

    def mul_scalar(self, x, value):
        return self.g.binary(x, self.scalar_like(value, x), "mul")

    def add_scalar(self, x, value):
        return self.g.binary(x, self.scalar_like(value, x), "add")

    def pow_scalar(self, x, value):
        return self.g.binary(x, self.scalar_like(value, x), "pow")


def batch_norm_train(rec, x, running_mean, running_variance, scale, bias, relu=True):
    """BatchNorm2d::forward in Train mode on an NHWC tensor (helium/src/modules/batch_norm.rs:32-72), followed by
    the Relu the resnet blocks apply (resnet-train/src/model.rs). Returns (y, new running mean, new running
    variance)."""
    g = rec.g
    shape, dtype = g.descriptor(x)
    c = shape[3]
    xt = g.swap_dims(x, 0, 3)  # statistics over N, H, W: swap N and C, fold the three trailing dims
    mean = g.reshape(g.reduce(xt, "mean", 3), [c])
    mean_square = g.reshape(g.reduce(rec.pow_scalar(xt, 2.0), "mean", 3), [c])
    variance = sub(g, mean_square, rec.pow_scalar(mean, 2.0))
    new_mean = g.change_data_type(g.binary(rec.mul_scalar(running_mean, 0.9), rec.mul_scalar(mean, 0.1), "add"), "f32")
    new_var = g.change_data_type(g.binary(rec.mul_scalar(running_variance, 0.9), rec.mul_scalar(variance, 0.1), "add"), "f32")
    mean_b = broadcast_to(g, mean, [c], shape)
    var_b = broadcast_to(g, variance, [c], shape)
    xh = div(g, sub(g, x, mean_b), g.unary(rec.add_scalar(var_b, 1e-3), "sqrt"))
    y = g.binary(g.binary(xh, broadcast_to(g, scale, [c], shape), "mul"), broadcast_to(g, bias, [c], shape), "add")
    y = g.change_data_type(y, dtype)
    if relu:
        y = g.unary(y, "relu")
    return y, new_mean, new_var


def sgd_momentum_step(rec, weights, gradient, average, momentum=0.9, learning_rate=0.1):
    """Sgd::step with momentum for one parameter that already has a gradient average
    (helium/src/optimizer/sgd.rs:42-66). Returns (new weights, new average as f32)."""
    g = rec.g
    updated = g.binary(rec.mul_scalar(gradient, 1.0 - momentum), rec.mul_scalar(average, momentum), "add")
    new_weights = sub(g, weights, rec.mul_scalar(updated, learning_rate))
    return new_weights, g.change_data_type(updated, "f32")


def conv2d(g, x, kernel, bias, params):
    """Conv2d::forward (helium/src/modules/conv.rs:62-68): the convolution, plus the bias broadcast over the pixels."""
    y = g.conv(x, kernel, params)
    if bias is not None:
        shape, _ = g.descriptor(y)
        y = g.binary(y, broadcast_to(g, bias, [shape[3]], shape), "add")
    return y


def basic_block_forward(rec, x, bn1, kernel1, bias1, bn2, kernel2, bias2):
    """BasicBlock::forward in Train mode (resnet-train/src/model.rs:155-165): bn1 -> relu -> conv1 -> bn2 -> relu ->
    conv2 -> + shortcut, 3x3 convolutions that keep the channel count. `bn1` / `bn2`: (running mean, running variance,
    scale, bias). Returns (output, [new running mean 1, new running variance 1, new running mean 2, ...])."""
    g = rec.g
    shape, _ = g.descriptor(x)
    c = shape[3]
    params = {"in_channels": c, "out_channels": c, "kernel_size": [3, 3]}
    h, m1, v1 = batch_norm_train(rec, x, *bn1, relu=True)
    h = conv2d(g, h, kernel1, bias1, params)
    h, m2, v2 = batch_norm_train(rec, h, *bn2, relu=True)
    h = conv2d(g, h, kernel2, bias2, params)
    return g.binary(h, x, "add"), [m1, v1, m2, v2]
