"""Oracle for the fusion IR (helium-playground/src/opgraph.rs). Test infrastructure only.

Semantics follow the reference's own PyTorch rendering of the IR (helium-playground/src/torch_synthesizer.rs:30-84:
x ** c for PowConstant, where(rhs > 0, lhs, 0) for Drelu, keepdim sums over dim 2 / 1 / (1,2) / (0,1,2) for
Rows / Columns / Item / Batch, transpose(1, 2), matmul, implicit broadcast) and the shape rules of
opgraph.rs:386-426. All arithmetic is f32 (the build's stated precision); the reference's prototype kernels compute
in bf16 intrinsics (kernel_generator.rs:363-414), so bit-level agreement with them is "parity unpinned" — what is
pinned (tests/test_oracle_cpu.py): each unary / binary op against Python's `math` (`math.erf` for Gelu, Drelu as
torch_synthesizer.rs:76-78 writes it), the four reduction depths and the shape rules against loops, and the README
graph (README.md:33-79, with and without its mainloop ops) against its closed forms written directly in float64.

The graph is plain data: the list of dicts recorded by helium_amd.fusion.OpGraph.nodes.
"""
import numpy as np

from . import numerics as nm


def shape_of(node, shapes):
    """opgraph.rs:386-426"""
    op = node["op"]
    if op in ("producer", "constant"):
        return list(node["shape"])
    if op == "matmul":
        return [shapes[node["a"]][0], shapes[node["a"]][1], shapes[node["b"]][2]]
    if op in ("unary", "consumer"):
        return list(shapes[node["x"]])
    if op == "binary":
        return list(shapes[node["lhs"]])
    if op == "reduction":
        s = list(shapes[node["x"]])
        if node["depth"] == "rows":
            s[2] = 1
        elif node["depth"] == "columns":
            s[1] = 1
        elif node["depth"] == "item":
            s[1] = s[2] = 1
        else:
            s = [1, 1, 1]
        return s
    if op == "broadcast":
        s = list(shapes[node["x"]])
        s[node["axis"]] = node["amount"]
        return s
    if op == "transpose":
        s = list(shapes[node["x"]])
        return [s[0], s[2], s[1]]
    raise ValueError(op)


def unary(fn, x, c):
    one = np.float32(1.0)
    c = np.float32(c)
    with np.errstate(all="ignore"):
        if fn == "neg":
            return -x
        if fn == "relu":
            return np.fmax(x, np.float32(0))
        if fn == "gelu":
            from scipy.special import erf
            return (0.5 * x.astype(np.float64) * (1.0 + erf(x.astype(np.float64) / np.sqrt(2.0)))).astype(np.float32)
        if fn == "tanh":
            return np.tanh(x.astype(np.float64)).astype(np.float32)
        if fn == "exp":
            return np.exp(x.astype(np.float64)).astype(np.float32)
        if fn == "ln":
            return np.log(x.astype(np.float64)).astype(np.float32)
        if fn == "sqrt":
            return np.sqrt(x)
        if fn == "add_constant":
            return x + c
        if fn == "mul_constant":
            return x * c
        if fn == "pow_constant":
            if c == np.float32(2.0):
                return x * x
            return np.power(x.astype(np.float64), np.float64(c)).astype(np.float32)
    raise ValueError(fn)


def binary(fn, a, b):
    with np.errstate(all="ignore"):
        if fn == "add":
            return a + b
        if fn == "sub":
            return a - b
        if fn == "mul":
            return a * b
        if fn == "div":
            return a / b
        if fn == "pow":
            return np.power(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)
        if fn == "drelu":
            return np.where(b > 0, a, np.float32(0)).astype(np.float32)
    raise ValueError(fn)


def reduction(depth, x):
    axis = {"rows": 2, "columns": 1, "item": (1, 2), "batch": (0, 1, 2)}[depth]
    return x.astype(np.float64).sum(axis=axis, keepdims=True).astype(np.float32)


def matmul(a, b):
    """bf16/f16/f32 operands (already widened to f32), products accumulated without loss (float64)."""
    return np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)


def evaluate(nodes, inputs, round_mainloop_to=None, materialize=None):
    """inputs: {producer id: storage array}. Returns ({id: f32 array}, {id: shape}).
    materialize: {node id: storage dtype} of values that cross a kernel boundary when the graph runs as several
    kernels; they are rounded to that dtype where they are produced.
    round_mainloop_to: storage dtype the Matmul operands are rounded to after mainloop ops (the fused GEMM casts
    the mainloop chain's result back to the load type before the MMA, helium-kernel-generator/src/generators/
    matmul/sm80.rs:418-437); None leaves them in f32."""
    shapes, val = {}, {}
    for n in nodes:
        i, op = n["id"], n["op"]
        shapes[i] = shape_of(n, shapes)
        if op == "producer":
            val[i] = nm.from_storage(inputs[i], n["dtype"], n["shape"])
        elif op == "constant":
            val[i] = np.full(n["shape"], n["value"], dtype=np.float32)
        elif op == "matmul":
            a, b = val[n["a"]], val[n["b"]]
            if round_mainloop_to:
                a = nm.from_storage(nm.to_storage(a, round_mainloop_to), round_mainloop_to, a.shape)
                b = nm.from_storage(nm.to_storage(b, round_mainloop_to), round_mainloop_to, b.shape)
            val[i] = matmul(a, b)
        elif op == "unary":
            val[i] = unary(n["fn"], val[n["x"]], n["constant"])
        elif op == "binary":
            val[i] = binary(n["fn"], val[n["lhs"]], val[n["rhs"]])
        elif op == "reduction":
            val[i] = reduction(n["depth"], val[n["x"]])
        elif op == "broadcast":
            val[i] = np.ascontiguousarray(np.broadcast_to(val[n["x"]], shapes[i]))
        elif op == "transpose":
            val[i] = np.ascontiguousarray(np.swapaxes(val[n["x"]], 1, 2))
        elif op == "consumer":
            val[i] = val[n["x"]]
        else:
            raise ValueError(op)
        assert list(val[i].shape) == list(shapes[i]), (n, val[i].shape, shapes[i])
        if materialize and i in materialize:
            val[i] = nm.from_storage(nm.to_storage(val[i], materialize[i]), materialize[i], val[i].shape)
    return val, shapes


def outputs(nodes, inputs, **kw):
    """Storage-domain value of every leaf, keyed by leaf id. Reductions are stored as f32, other consumers in the
    consumer's dtype."""
    val, _ = evaluate(nodes, inputs, **kw)
    by_id = {n["id"]: n for n in nodes}
    used = set()
    for n in nodes:
        for k in ("a", "b", "x", "lhs", "rhs"):
            if k in n:
                used.add(n[k])
    out = {}
    for n in nodes:
        if n["id"] in used:
            continue
        src = by_id[n["x"]] if n["op"] == "consumer" else n
        dtype = "f32" if src["op"] == "reduction" else (n["dtype"] if n["op"] == "consumer" else "bf16")
        out[n["id"]] = nm.to_storage(val[n["id"]], dtype)
    return out
