"""Fused-GEMM cases shared by the CPU-emulation and GPU parity tests (fusion IR built through the C ABI)."""
import numpy as np

import helium_amd as ha
from helium_amd import configs


def bf16_normal(rng, shape, scale=1.0):
    return configs.bf16_rne((rng.standard_normal(shape) * scale).astype(np.float32))


def plain(m, n, k, batch=1, seed=0, dtype="bf16", out_dtype="f32", scale=0.5):
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(seed)
    a = g.producer([batch, m, k], dtype); b = g.producer([batch, k, n], dtype)
    out = g.consumer(g.matmul(a, b), out_dtype)
    if dtype == "bf16":
        inputs = {a: bf16_normal(rng, (batch, m, k), scale), b: bf16_normal(rng, (batch, k, n), scale)}
    elif dtype == "f16":
        inputs = {a: (rng.standard_normal((batch, m, k)) * scale).astype(np.float16).view(np.uint16),
                  b: (rng.standard_normal((batch, k, n)) * scale).astype(np.float16).view(np.uint16)}
    else:
        inputs = {a: (rng.standard_normal((batch, m, k)) * scale).astype(np.float32),
                  b: (rng.standard_normal((batch, k, n)) * scale).astype(np.float32)}
    return g, inputs, [out]


def transposed_b(m, n, k, batch=1, seed=4, dtype="bf16", out_dtype="f32", scale=0.5, scaled=False):
    """C = A * Bt^T with Bt stored [batch, n, k] (k contiguous): the mainloop's Transpose op on the B operand.
    `scaled`: Bt is also multiplied by a [batch, n, 1] column before the transposition (a fused mainloop)."""
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(seed)
    a = g.producer([batch, m, k], dtype); bt = g.producer([batch, n, k], dtype)
    if dtype == "bf16":
        inputs = {a: bf16_normal(rng, (batch, m, k), scale), bt: bf16_normal(rng, (batch, n, k), scale)}
    else:
        inputs = {a: (rng.standard_normal((batch, m, k)) * scale).astype(np.float32),
                  bt: (rng.standard_normal((batch, n, k)) * scale).astype(np.float32)}
    b = bt
    if scaled:
        col = g.producer([batch, n, 1], "f32")
        inputs[col] = rng.uniform(0.5, 1.5, (batch, n, 1)).astype(np.float32)
        b = g.binary(bt, g.broadcast(col, 2, k), "mul")
    out = g.consumer(g.matmul(a, g.transpose(b)), out_dtype)
    return g, inputs, [out]


def transposed_a(m, n, k, batch=1, seed=5, dtype="bf16", out_dtype="f32", scale=0.5, both=False):
    """C = At^T * B with At stored [batch, k, m] (m contiguous); `both`: B is stored transposed as well."""
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(seed)
    bshape = (batch, n, k) if both else (batch, k, n)
    at = g.producer([batch, k, m], dtype); b = g.producer(list(bshape), dtype)
    if dtype == "bf16":
        inputs = {at: bf16_normal(rng, (batch, k, m), scale), b: bf16_normal(rng, bshape, scale)}
    else:
        inputs = {at: (rng.standard_normal((batch, k, m)) * scale).astype(np.float32),
                  b: (rng.standard_normal(bshape) * scale).astype(np.float32)}
    out = g.consumer(g.matmul(g.transpose(at), g.transpose(b) if both else b), out_dtype)
    return g, inputs, [out]


def linear_layer(m, k, n):
    """Config 1 at a small size: f32 Y = relu(X W + b) and its column sums."""
    from helium_amd import configs

    g, names = configs.c1_graph(m, k, n)
    return g, configs.c1_inputs(names, m, k, n), [names["y"], names["colsum"]]


def bias_relu_colsum(m, n, k, batch=1, seed=1, bias_axis=1, mainloop=False, a_dtype="bf16"):
    """Config 5a's shape of fusion: optional mainloop relu(A0) * T on the A operand, bias + Relu epilogue, the
    full-size result and its column sums as outputs."""
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(seed)
    a0 = g.producer([batch, m, k], a_dtype)
    inputs = {a0: bf16_normal(rng, (batch, m, k)) if a_dtype == "bf16" else rng.standard_normal((batch, m, k)).astype(np.float32)}
    a = a0
    if mainloop:
        t = g.producer([batch, m, k], "bf16")
        inputs[t] = bf16_normal(rng, (batch, m, k))
        a = g.binary(g.unary(a0, "relu"), t, "mul")
    b = g.producer([batch, k, n], "bf16")
    inputs[b] = bf16_normal(rng, (batch, k, n), 0.25)
    bshape = [batch, 1, n] if bias_axis == 1 else [batch, m, 1]
    bias = g.producer(bshape, "f32")
    inputs[bias] = rng.standard_normal(bshape).astype(np.float32)
    mm = g.matmul(a, b)
    y = g.unary(g.binary(mm, g.broadcast(bias, bias_axis, m if bias_axis == 1 else n), "add"), "relu")
    outs = [g.consumer(y, "bf16"), g.consumer(g.reduction(y, "columns"), "f32")]
    return g, inputs, outs


def all_reductions(m, n, k, batch=2, seed=2):
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(seed)
    a = g.producer([batch, m, k], "bf16"); b = g.producer([batch, k, n], "bf16"); aux = g.producer([batch, m, n], "bf16")
    inputs = {a: bf16_normal(rng, (batch, m, k), 0.5), b: bf16_normal(rng, (batch, k, n), 0.5), aux: bf16_normal(rng, (batch, m, n))}
    v = g.binary(g.unary(g.matmul(a, b), "tanh"), aux, "mul")
    outs = [g.consumer(g.reduction(v, d), "f32") for d in ("rows", "columns", "item", "batch")]
    outs.append(g.consumer(v, "f32"))
    return g, inputs, outs


MATMUL_DTYPES = ("f32", "bf16", "f16")
# helium-kernel-generator/tests/matmul.rs:171-181: the precisions of matmul_no_fusion (the four F8 mode pairs share one
# entry here: the modes change nothing on hardware whose F8 products run as bf16)
MATMUL_PRECISIONS = ("f32_f32", "tf32_f32", "bf16_f32", "f16_f32", "f16_f16", "f8_f32", "f8_f16")


def ir_matmul(m, n, k, dtype_a, dtype_b, precision, out_dtype, seed=7):
    """matmul_no_fusion of helium-kernel-generator/tests/matmul.rs:24-70: Input a, Input b, Matmul(precision),
    ChangeDataType(output type), Output, handed to the MatmulGenerator boundary as the subgraph {matmul, cast}.
    Operands are uniform in [0, 1) like the reference's `rand::random::<f32>()`. Returns (graph, kernel, inputs by
    node, the cast's node id)."""
    from helium_amd import backend, ir
    from oracle import numerics as nm

    g = ir.OpGraph()
    a, b = g.new_input([m, k], dtype_a), g.new_input([k, n], dtype_b)
    mm = g.matmul(a, b, precision)
    out = g.change_data_type(mm, out_dtype)
    g.new_output(out)
    rng = np.random.default_rng(seed)
    host = {a: nm.to_storage(rng.random((m, k), dtype=np.float32), dtype_a), b: nm.to_storage(rng.random((k, n), dtype=np.float32), dtype_b)}
    return g, backend.matmul_kernel(g, [mm, out]), host, out
