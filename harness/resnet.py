"""The training step of the reference's resnet-train example, recorded as one helium-ir graph.

Harness code, like autodiff.py: it restates the model (resnet-train/src/model.rs), the modules it is made of
(helium/src/modules/conv.rs, batch_norm.rs), the loss (helium/src/loss.rs), the optimizer (helium/src/optimizer/sgd.rs)
and the body of the training loop (resnet-train/src/train.rs:383-396: forward in Train mode, cross-entropy, backward,
Sgd::step with momentum) on top of the graph recorder, so that `execute_graph` gets the graph the reference's front end
would hand it. Parameters, running statistics and gradient averages are graph inputs; their updated values are graph
outputs, which the next step feeds back in.
"""
import numpy as np

from . import autodiff as ad

NUM_CLASSES = 1000


class Conv2d:
    """modules/conv.rs: kernel [K,R,S,C] and bias [K] are f32 parameters (Conv2dSettings::default), the kernel is cast to
    the activation's type where it is used."""

    def __init__(self, G, rng, in_channels, out_channels, kernel_size, stride=1):
        self.params = {"in_channels": in_channels, "out_channels": out_channels, "kernel_size": [kernel_size, kernel_size],
                       "stride": [stride, stride]}
        shape = [out_channels, kernel_size, kernel_size, in_channels]
        stdev = 1.0 / np.sqrt(kernel_size * kernel_size * out_channels)  # Initializer::KaimingNormal (initializer.rs:48-53)
        self.kernel = G.param((rng.standard_normal(shape) * stdev).astype(np.float32))
        self.bias = G.param(np.zeros([out_channels], dtype=np.float32))

    def forward(self, x):
        y = x.conv2d(self.kernel.value.to_data_type(x.dtype), self.params)
        return y + self.bias.value.broadcast_to(y.shape)

    def parameters(self):
        return [self.kernel, self.bias]


class BatchNorm2d:
    """modules/batch_norm.rs:32-72, Train mode: statistics over N, H, W of the NHWC activation."""

    def __init__(self, G, channels):
        self.channels = channels
        self.running_mean = G.tensor(np.zeros([channels], dtype=np.float32))
        self.running_variance = G.tensor(np.ones([channels], dtype=np.float32))
        self.scale = G.param(np.ones([channels], dtype=np.float32))
        self.bias = G.param(np.zeros([channels], dtype=np.float32))
        self.first_statistics = (self.running_mean.raw.node, self.running_variance.raw.node)

    def forward(self, x):
        dtype = x.dtype
        xt = x.swap_dims(0, 3)
        mean = xt.reduce_mean(3).reshape([self.channels])
        mean_square = xt.pow_scalar(2.0).reduce_mean(3).reshape([self.channels])
        variance = mean_square - mean.pow_scalar(2.0)
        self.running_mean = (self.running_mean * 0.9 + mean * 0.1).detach().to_data_type("f32")
        self.running_variance = (self.running_variance * 0.9 + variance * 0.1).detach().to_data_type("f32")
        x = (x - mean.broadcast_to(x.shape)) / (variance.broadcast_to(x.shape) + 1e-3).sqrt()
        return (x * self.scale.value.broadcast_to(x.shape) + self.bias.value.broadcast_to(x.shape)).to_data_type(dtype)

    def parameters(self):
        return [self.scale, self.bias]


class BasicBlock:
    """model.rs:115-166"""

    def __init__(self, G, rng, channels):
        self.bn1, self.conv1 = BatchNorm2d(G, channels), Conv2d(G, rng, channels, channels, 3)
        self.bn2, self.conv2 = BatchNorm2d(G, channels), Conv2d(G, rng, channels, channels, 3)

    def forward(self, x):
        shortcut = x
        x = self.conv1.forward(self.bn1.forward(x).relu())
        x = self.conv2.forward(self.bn2.forward(x).relu())
        return x + shortcut

    def modules(self):
        return [self.bn1, self.conv1, self.bn2, self.conv2]


class DownsampleBlock:
    """model.rs:168-249: extents halve, channels double. As the reference writes it, bn1 runs twice: once before the
    shortcut convolution and once more, on that result, before conv1."""

    def __init__(self, G, rng, in_channels):
        out_channels = in_channels * 2
        self.bn1, self.conv1 = BatchNorm2d(G, in_channels), Conv2d(G, rng, in_channels, out_channels, 3, stride=2)
        self.bn2, self.conv2 = BatchNorm2d(G, out_channels), Conv2d(G, rng, out_channels, out_channels, 3)
        self.shortcut_conv = Conv2d(G, rng, in_channels, out_channels, 1, stride=2)

    def forward(self, x):
        x = self.bn1.forward(x).relu()
        shortcut = self.shortcut_conv.forward(x)
        x = self.conv1.forward(self.bn1.forward(x).relu())
        x = self.conv2.forward(self.bn2.forward(x).relu())
        return x + shortcut

    def modules(self):
        return [self.bn1, self.conv1, self.bn2, self.conv2, self.shortcut_conv]


class Model:
    """model.rs:11-85: 7x7 stride-2 head, four segments (a downsample block and one basic block each), batch norm, relu,
    1x1 convolution to the classes, global average pooling. `width` is the head's channel count (32 in the reference)."""

    def __init__(self, G, rng, width=32, num_classes=NUM_CLASSES):
        self.num_classes = num_classes
        self.head = Conv2d(G, rng, 3, width, 7, stride=2)
        self.blocks = []
        for k in range(4):
            self.blocks += [DownsampleBlock(G, rng, width << k), BasicBlock(G, rng, width << (k + 1))]
        self.tail_bn = BatchNorm2d(G, width << 4)
        self.tail = Conv2d(G, rng, width << 4, num_classes, 1)

    def forward(self, x):
        x = self.head.forward(x)
        for block in self.blocks:
            x = block.forward(x)
        x = self.tail.forward(self.tail_bn.forward(x).relu())
        batch = x.shape[0]
        return x.swap_dims(2, 3).swap_dims(1, 2).reduce_mean(2).reshape([batch, self.num_classes])

    def modules(self):
        out = [self.head]
        for block in self.blocks:
            out += block.modules()
        return out + [self.tail_bn, self.tail]

    def parameters(self):
        return [p for m in self.modules() for p in m.parameters()]

    def batch_norms(self):
        return [m for m in self.modules() if isinstance(m, BatchNorm2d)]


def record_training_step(batch, image_size, width=32, num_classes=NUM_CLASSES, seed=66, learning_rate=0.1, momentum=0.9,
                         dtype="bf16"):
    """One iteration of train.rs:383-396 as a graph. Returns a dict:
    graph: the autodiff.Graph (its `.g` is the helium-ir graph, `.feeds` the storage of every input),
    image / labels: input nodes of the batch, loss / probs: output nodes,
    carried: [(input node, output node)] for every parameter, gradient average and running statistic: the output of one
    step is that input of the next.
    `dtype` is the storage type of the images and labels, hence of every activation and flow (bf16 in the reference,
    train.rs:68-87)."""
    G = ad.Graph()
    rng = np.random.default_rng(seed)
    model = Model(G, rng, width, num_classes)
    image = G.tensor(rng.standard_normal([batch, image_size, image_size, 3]).astype(np.float32), dtype=dtype)
    one_hot = np.zeros([batch, num_classes], dtype=np.float32)
    one_hot[np.arange(batch), rng.integers(0, num_classes, batch)] = 1.0
    labels = G.tensor(one_hot, dtype=dtype)

    logits = model.forward(image).to_data_type("f32")
    probs = logits.log_softmax().exp()
    loss = ad.cross_entropy_loss(logits, labels)
    grads = loss.backward()

    # Sgd::step with momentum and an average that already exists for every parameter (sgd.rs:42-66)
    carried = []
    for p in model.parameters():
        weights = p.value.detach()
        gradient = ad.Tensor(grads[p.id])
        average = G.tensor(np.zeros(weights.shape, dtype=np.float32))
        updated = gradient * (1.0 - momentum) + average * momentum
        new_average = updated.to_data_type("f32")
        new_weights = weights - updated * learning_rate
        carried.append((weights.raw.node, G.g.new_output(new_weights.raw.node)))
        carried.append((average.raw.node, G.g.new_output(new_average.raw.node)))
    for bn in model.batch_norms():
        carried.append((bn.first_statistics[0], G.g.new_output(bn.running_mean.raw.node)))
        carried.append((bn.first_statistics[1], G.g.new_output(bn.running_variance.raw.node)))
    return {"graph": G, "image": image.raw.node, "labels": labels.raw.node, "loss": G.g.new_output(loss.raw.node),
            "probs": G.g.new_output(probs.raw.node), "carried": carried, "model": model}
