"""Graph builders and seeded synthetic inputs for the benchmark configurations (BASELINE.json configs 1-5).

Used by bench.py, the kernel prebuild step and the parity tests, so that all three run the very same graphs.
Inputs come from numpy's PCG64 with a fixed seed per configuration.
"""
import numpy as np

from . import fusion


def bf16_rne(x):
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


PERMUTES = {
    # name: (shape, numpy.transpose axes) — bf16 N(0,1)
    "C2a": ((64, 56, 56, 256), (0, 3, 1, 2)),   # NHWC -> NCHW
    "C2b": ((4096, 4096), (1, 0)),              # 2-d transpose
    "C2c": ((32, 128, 28, 28), (0, 2, 3, 1)),   # arbitrary 4-d permute
}


def permute_input(name, seed=None):
    shape, _ = PERMUTES[name]
    seed = {"C2a": 21, "C2b": 22, "C2c": 23}[name] if seed is None else seed
    rng = np.random.default_rng(seed)
    return bf16_rne(rng.standard_normal(size=shape, dtype=np.float32))


def c3_chain(rows=4096, cols=4096, bias_axis=2, seed=31, make_inputs=True):
    """Config 3: Add, broadcast-add of a bias, Relu, Tanh, Neg, AddConstant(1.0), Mul, Sub, PowConstant(2.0),
    MulConstant(1/4096), then Sum over batch and over columns; f32, U(-1,1).
    bias_axis=2: bias [1,rows,1] as BASELINE.json words it; bias_axis=1: bias [1,1,cols] as the reference's README
    listing broadcasts its biases (README.md:42,46)."""
    g = fusion.OpGraph()
    full = [1, rows, cols]
    a, b, c, d = (g.producer(full, "f32") for _ in range(4))
    bshape = [1, rows, 1] if bias_axis == 2 else [1, 1, cols]
    bias = g.producer(bshape, "f32")
    x = g.binary(a, b, "add")
    x = g.binary(x, g.broadcast(bias, bias_axis, full[bias_axis]), "add")
    x = g.unary(x, "relu")
    x = g.unary(x, "tanh")
    x = g.unary(x, "neg")
    x = g.unary(x, "add_constant", 1.0)
    x = g.binary(x, c, "mul")
    x = g.binary(x, d, "sub")
    x = g.unary(x, "pow_constant", 2.0)
    r = g.unary(x, "mul_constant", 1.0 / 4096.0)
    out_batch = g.consumer(g.reduction(r, "batch"), "f32")
    out_cols = g.consumer(g.reduction(r, "columns"), "f32")
    inputs = {}
    if make_inputs:
        rng = np.random.default_rng(seed)
        inputs = {n: rng.uniform(-1, 1, size=full).astype(np.float32) for n in (a, b, c, d)}
        inputs[bias] = rng.uniform(-1, 1, size=bshape).astype(np.float32)
    return g, inputs, {"batch": out_batch, "columns": out_cols, "r": r}
