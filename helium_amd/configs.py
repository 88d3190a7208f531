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


# The reference's own permute benchmark (helium/examples/permute_dim_benchmark.rs:13-41): f32 [2048,128,128,32],
# swap_dims(0, 3): 4.3 GB in, 4.3 GB out - a size no cache flatters.
PERM_REF_SHAPE, PERM_REF_PERM = (2048, 128, 128, 32), (3, 1, 2, 0)


def perm_ref_expected(out_index):
    """With input element i holding the 32-bit value i, the value at linear index `out_index` (uint64 array) of
    swap_dims(0, 3) of a [2048,128,128,32] tensor: output coordinates (i3, i1, i2, i0) read input (i0, i1, i2, i3)."""
    n0, n1, n2, n3 = PERM_REF_SHAPE
    j = np.asarray(out_index, dtype=np.uint64)
    i0 = j % n0
    i2 = (j // n0) % n2
    i1 = (j // (n0 * n2)) % n1
    i3 = j // (n0 * n2 * n1)
    return (((i0 * n1 + i1) * n2 + i2) * n3 + i3).astype(np.uint32)


def permute_input(name, seed=None):
    shape, _ = PERMUTES[name]
    seed = {"C2a": 21, "C2b": 22, "C2c": 23}[name] if seed is None else seed
    rng = np.random.default_rng(seed)
    return bf16_rne(rng.standard_normal(size=shape, dtype=np.float32))


def c1_graph(rows=256, inner=512, cols=512):
    """Config 1 as one Core fusion: Y = relu(X W + b) and the sum of Y over columns (fold of the row axis), all f32."""
    g = fusion.OpGraph()
    x, w = g.producer([1, rows, inner], "f32"), g.producer([1, inner, cols], "f32")
    b = g.producer([1, 1, cols], "f32")
    y = g.unary(g.binary(g.matmul(x, w), g.broadcast(b, 1, rows), "add"), "relu")
    return g, {"x": x, "w": w, "b": b, "y": g.consumer(y, "f32"),
               "colsum": g.consumer(g.reduction(y, "columns"), "f32")}


def c1_ir_graph(rows=256, inner=512, cols=512):
    """Config 1 as the lazy-tensor front end records it (helium-ir): Matmul, broadcast-add, Relu, and the column
    sum as swap_dims + Reduce(depth 1); execute_graph plans it as a GEMM and two pointwise kernels."""
    from . import ir

    g = ir.OpGraph()
    x, w, b = g.new_input([rows, inner], "f32"), g.new_input([inner, cols], "f32"), g.new_input([cols], "f32")
    y = g.unary(g.binary(g.matmul(x, w, "f32_f32"), g.broadcast(b, 2, [(0, rows)]), "add"), "relu")
    colsum = g.reduce(g.swap_dims(y, 0, 1), "sum", 1)
    return g, {"x": x, "w": w, "b": b, "y": g.new_output(y), "colsum": g.new_output(colsum)}


def c1_inputs(names, rows=256, inner=512, cols=512, seed=11, batched=True):
    rng = np.random.default_rng(seed)
    lead = (1,) if batched else ()
    return {names["x"]: rng.uniform(-1, 1, lead + (rows, inner)).astype(np.float32),
            names["w"]: rng.uniform(-1, 1, lead + (inner, cols)).astype(np.float32),
            names["b"]: rng.uniform(-1, 1, (lead + (1, cols)) if batched else (cols,)).astype(np.float32)}


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


def c4_graph(size=4096, mainloop=False, full_size_outputs=False, bias_rows=False):
    """Config 4: the reference README's fusion (README.md:33-79), node ids as printed there.

    Core = Matmul{a: n1, b: n2} is node 12; n13, n24, n26 are the other GEMM results of the LSTM-cell-like graph
    and arrive as bf16 tensors, n9 is the previous state, n11 the target, n6 / n8 the f32 biases [1,1,size]
    broadcast along axis 1. 39 epilogue ops follow the anchor; the leaves are the three reductions n39 (Batch),
    n58 and n87 (Columns). With mainloop=True the anchor's A operand is n25 = Relu(n22) * n9 (README.md:36-38).
    With full_size_outputs=True n57 and n86 (the gradients the backward GEMMs would read) are also stored, as bf16.
    With bias_rows=True the biases are [1,size,1] columns broadcast along axis 2, as the headline configuration words
    them, and their gradients n58 / n87 are sums over each row.
    """
    g = fusion.OpGraph()
    full = [1, size, size]
    P = lambda i, shape=full, dt="bf16": g.producer(shape, dt, node_id=i)  # noqa: E731
    n1 = P(22) if mainloop else P(1)
    n2 = P(2)
    bias_shape, bias_axis, bias_sum = ([1, size, 1], 2, "rows") if bias_rows else ([1, 1, size], 1, "columns")
    n6, n8 = P(6, bias_shape, "f32"), P(8, bias_shape, "f32")
    n9, n11, n13, n24, n26 = P(9), P(11), P(13), P(24), P(26)
    a_operand = n1
    if mainloop:
        g.unary(22, "relu", node_id=23)
        a_operand = g.binary(23, n9, "mul", node_id=25)
    g.matmul(a_operand, n2, node_id=12)
    U = lambda i, x, fn, c=0.0: g.unary(x, fn, c, node_id=i)  # noqa: E731
    B = lambda i, lhs, rhs, fn: g.binary(lhs, rhs, fn, node_id=i)  # noqa: E731
    inv = np.float32(0.00024414063)
    B(14, 12, n13, "add"); g.broadcast(n6, bias_axis, size, node_id=15); B(16, 14, 15, "add"); U(17, 16, "relu")
    B(27, n24, n26, "add"); g.broadcast(n8, bias_axis, size, node_id=28); B(29, 27, 28, "add"); U(30, 29, "tanh")
    U(31, 17, "neg"); U(32, 31, "add_constant", 1.0); B(33, 32, n9, "mul"); B(34, 17, 30, "mul"); B(35, 33, 34, "add")
    B(36, 35, n11, "sub"); U(37, 36, "pow_constant", 2.0); U(38, 37, "mul_constant", inv)
    g.reduction(38, "batch", node_id=39)
    g.constant([1, 1, 1], 1.0, node_id=41)
    g.broadcast(41, 1, size, node_id=42); g.broadcast(42, 2, size, node_id=43); g.broadcast(43, 0, 1, node_id=44)
    U(45, 44, "mul_constant", inv)
    g.constant(full, 2.0, node_id=46); g.constant(full, 1.0, node_id=47)
    B(48, 36, 47, "pow"); B(49, 48, 46, "mul"); B(50, 49, 45, "mul")
    B(52, 50, 30, "mul"); B(53, 17, 50, "mul"); U(54, 30, "pow_constant", 2.0); U(55, 54, "neg")
    U(56, 55, "add_constant", 1.0); B(57, 53, 56, "mul")
    g.reduction(57, bias_sum, node_id=58)
    B(81, 50, n9, "mul"); U(84, 81, "neg"); B(85, 52, 84, "add"); B(86, 85, 16, "drelu")
    g.reduction(86, bias_sum, node_id=87)
    outs = {"loss": 39, "db8": 58, "db6": 87}
    if full_size_outputs:
        outs["dpre_c"] = g.consumer(57, "bf16", node_id=90)
        outs["dpre_z"] = g.consumer(86, "bf16", node_id=91)
    return g, outs


def c4_inputs(g, size=4096, seed=41):
    """A, B ~ N(0, 0.02) (bf16); the other GEMM results ~ N(0, 0.02 * 0.02 * sqrt(size)) like a product of two
    such matrices; previous state and target ~ N(0,1); biases ~ N(0,1) f32."""
    rng = np.random.default_rng(seed)
    inputs = {}
    for n in g.nodes:
        if n["op"] != "producer":
            continue
        shape = n["shape"]
        if n["dtype"] == "f32":
            inputs[n["id"]] = rng.standard_normal(shape).astype(np.float32)
        elif n["id"] in (1, 2, 22):
            inputs[n["id"]] = bf16_rne((rng.standard_normal(shape) * 0.02).astype(np.float32))
        elif n["id"] in (13, 24, 26):
            inputs[n["id"]] = bf16_rne((rng.standard_normal(shape) * (0.02 * 0.02 * np.sqrt(size))).astype(np.float32))
        else:
            inputs[n["id"]] = bf16_rne(rng.standard_normal(shape).astype(np.float32))
    return inputs


def c5a_graph(size=4096):
    """Config 5a: Y = relu(A' B + bias) with A' = Relu(A0) * T applied to the A tiles before the MFMA; bf16
    operands, f32 bias [1,1,size], bf16 output."""
    g = fusion.OpGraph()
    full = [1, size, size]
    a0, t, b = g.producer(full, "bf16"), g.producer(full, "bf16"), g.producer(full, "bf16")
    bias = g.producer([1, 1, size], "f32")
    a = g.binary(g.unary(a0, "relu"), t, "mul")
    y = g.unary(g.binary(g.matmul(a, b), g.broadcast(bias, 1, size), "add"), "relu")
    out = g.consumer(y, "bf16")
    return g, {"a0": a0, "t": t, "b": b, "bias": bias, "y": out}


def c5a_inputs(names, size=4096, seed=51):
    rng = np.random.default_rng(seed)
    full = (1, size, size)
    return {names["a0"]: bf16_rne(rng.standard_normal(full).astype(np.float32)),
            names["t"]: bf16_rne(rng.standard_normal(full).astype(np.float32)),
            names["b"]: bf16_rne((rng.standard_normal(full) * 0.02).astype(np.float32)),
            names["bias"]: rng.standard_normal((1, 1, size)).astype(np.float32)}
