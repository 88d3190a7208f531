"""Oracle for helium-ir graphs: shape/dtype inference and op-by-op evaluation. Test infrastructure only.

Follows helium-ir/src/opgraph/op.rs (inference), helium/src/cuda/instr/pointwise/jit.rs (arithmetic: every float
op is computed in f32 whatever the storage type; same-class casts are transparent inside a kernel; stores round
to the storage type) and helium/src/raw_tensor.rs (front-end lowerings, in `lower_*` helpers used by the tests).

Pinned by tests/test_oracle_cpu.py: `conv` against the reference's conv_simple vector and a seven-loop brute force
over the three padding modes, strides and dilations (with the output-size rule of conv.rs:51-73 checked against a
hand-made table); `conv_backward_data` / `conv_backward_filter` against scatter loops and the adjoint identities;
Compare / Select / casts / Reduce / Broadcast / SwapDims / Constant through the gradient graphs of
helium/tests/autodiff.rs and helium/tests/loss.rs with the values those tests assert (tests/golden/autodiff.json); the
matmul cases of tensor_ops.rs:172-318 (tests/golden/tensor_ops.json); unary and binary functions against Python's
`math`. tests/test_pointwise_cpu.py adds the pointwise known answers of tensor_ops.rs (add/mul/div/recip/scalar ops,
the op chain = 0.4, reductions incl. 200k elements, broadcast, reshape, relu, constant, max/min). Transcendentals
(`expf`, `tanhf`, `powf`, ...) are evaluated in float64 and rounded once to float32; the reference uses CUDA libdevice
for them, whose last-bit behaviour is "parity unpinned" beyond the exact-answer cases.

The graph is plain data: a list of dicts as recorded by helium_amd.ir.OpGraph.nodes
  {"id", "node": "input", "shape", "dtype"} | {"id", "node": "output", "from"} |
  {"id", "node": "op", "op": kind, "inputs": [...], ...op fields}.
"""
import numpy as np

from . import numerics as nm

FLOATS = ("f32", "bf16", "f16")


def accumulator_type(precision):
    """helium-ir/src/opgraph/op/precision.rs:87-96"""
    return "f16" if precision in ("f16_f16", "f8_f16") else "f32"


def infer(node, desc):
    """Output (shape, dtype) of an op node given `desc[id] = (shape, dtype)` (op.rs:52-179)."""
    op, ins = node["op"], node["inputs"]
    s0, t0 = desc[ins[0]] if ins else (None, None)
    if op == "change_dtype":
        return list(s0), node["target"]
    if op == "matmul":
        return list(s0[:-1]) + [desc[ins[1]][0][-1]], accumulator_type(node["precision"])
    if op in ("unary", "binary", "select"):
        return list(s0), t0
    if op == "reduce":
        return list(s0[: len(s0) - node["depth"]]) + [1], "f32"
    if op == "reshape":
        return list(node["new_shape"]), t0
    if op == "broadcast":
        shape = [1] * max(0, node["new_dim_count"] - len(s0)) + list(s0)
        for axis, size in node["axes"]:
            shape[axis] = size
        return shape, t0
    if op == "swap_dims":
        shape = list(s0)
        a, b = node["axis_a"], node["axis_b"]
        shape[a], shape[b] = shape[b], shape[a]
        return shape, t0
    if op == "compare":
        return list(s0), "bool"
    if op == "constant":
        return list(node["shape"]), node["const_dtype"]
    if op == "conv":  # op.rs:123-142
        image, filt = desc[ins[0]][0], desc[ins[1]][0]
        out = conv_output_size(node["params"], image[1:3], filt[1:3])
        return [image[0], out[0], out[1], node["params"]["out_channels"]], t0
    if op == "conv_bwd_data":  # op.rs:143-158
        return [s0[0], node["input_size"][0], node["input_size"][1], node["params"]["in_channels"]], t0
    if op == "conv_bwd_filter":  # op.rs:159-173
        p = node["params"]
        return [p["out_channels"], p["kernel_size"][0], p["kernel_size"][1], p["in_channels"]], t0
    raise ValueError(op)


def conv_output_size(params, input_size, kernel_size):
    """Conv2dParams::compute_output_size (helium-ir/src/opgraph/op/conv.rs:51-73): Full adds kernel/2, Valid
    subtracts kernel/2 (saturating), then the stride divides."""
    mode = params.get("padding_mode", "same")
    stride = params.get("stride", (1, 1))
    out = []
    for d in range(2):
        v = input_size[d]
        if mode == "full":
            v += kernel_size[d] // 2
        elif mode == "valid":
            v = max(0, v - kernel_size[d] // 2)
        out.append(v // stride[d])
    return out


def conv_padding(params):
    """PaddingMode::compute_padding_amount (conv.rs:85-91)."""
    k = params["kernel_size"]
    mode = params.get("padding_mode", "same")
    return [k[0] // 2, k[1] // 2] if mode == "same" else [0, 0] if mode == "valid" else [k[0] - 1, k[1] - 1]


def conv(image, filt, params, dtype):
    """Cross-correlation of an NHWC image with a [out_channels, kh, kw, in_channels] filter, zero padding of
    `conv_padding` on both sides, stride and dilation as given (the descriptor helium/src/cuda/instr/
    cudnn_graph.rs:384-396 builds: CUDNN_CROSS_CORRELATION, pre = post padding, f32 compute). Output element
    (n, p, q, o) = sum over (r, s, c) of image[n, p*sh + r*dh - ph, q*sw + s*dw - pw, c] * filter[o, r, s, c], taps
    outside the image contributing zero; evaluated in float64 on the stored operand values."""
    n, h, w, c = image.shape
    o, kr, ks, _ = filt.shape
    sh, sw = params.get("stride", (1, 1))
    dh, dw = params.get("dilation", (1, 1))
    ph, pw = conv_padding(params)
    oh, ow = conv_output_size(params, (h, w), (kr, ks))
    x = image.astype(np.float64)
    f = filt.astype(np.float64)
    out = np.zeros((n, oh, ow, o), dtype=np.float64)
    for r in range(kr):
        for s in range(ks):
            # rows / columns of the output whose tap (r, s) falls inside the image
            ih = np.arange(oh) * sh + r * dh - ph
            iw = np.arange(ow) * sw + s * dw - pw
            vh, vw = (ih >= 0) & (ih < h), (iw >= 0) & (iw < w)
            if not vh.any() or not vw.any():
                continue
            patch = x[:, ih[vh]][:, :, iw[vw]]  # [n, oh', ow', c]
            out[np.ix_(np.arange(n), np.nonzero(vh)[0], np.nonzero(vw)[0], np.arange(o))] += np.einsum("nhwc,oc->nhwo", patch, f[:, r, s, :])
    return out.astype(np.float32)


def _f64(fn, x):
    with np.errstate(all="ignore"):
        return fn(x.astype(np.float64)).astype(np.float32)


def unary(fn, x):
    """jit.rs:718-732, in f32."""
    one = np.float32(1.0)
    with np.errstate(all="ignore"):
        if fn == "recip":
            return one / x
        if fn == "neg":
            return -x
        if fn == "exp":
            return _f64(np.exp, x)
        if fn == "sin":
            return _f64(np.sin, x)
        if fn == "cos":
            return _f64(np.cos, x)
        if fn == "tan":
            return _f64(np.tan, x)
        if fn == "sigmoid":
            return one / (one + _f64(np.exp, -x))
        if fn == "tanh":
            return _f64(np.tanh, x)
        if fn == "relu":
            return np.fmax(x, np.float32(0.0))
        if fn == "sqrt":
            return np.sqrt(x)
        if fn == "log":
            return _f64(np.log, x)
    raise ValueError(fn)


def binary(fn, a, b):
    """jit.rs:734-747"""
    with np.errstate(all="ignore"):
        if a.dtype == np.bool_:
            return {"and": a & b, "or": a | b, "xor": a ^ b}[fn]
        if fn == "add":
            return a + b
        if fn == "mul":
            return a * b
        if fn == "pow":
            return np.power(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)
        if fn == "min":
            return np.fmin(a, b)
        if fn == "max":
            return np.fmax(a, b)
        if fn in ("and", "or", "xor"):
            return {"and": a & b, "or": a | b, "xor": a ^ b}[fn]
    raise ValueError(fn)


def compare(fn, a, b):
    return {"eq": a == b, "ne": a != b, "lt": a < b, "le": a <= b, "gt": a > b, "ge": a >= b}[fn]


def cast_class(x, src, dst):
    """jit.rs:663-672. Same-class casts do nothing to the math-domain value."""
    sf, df = src in FLOATS, dst in FLOATS
    if sf and df or src == dst:
        return x
    if sf and dst == "bool":
        return x != np.float32(0.0)
    if src == "bool" and df:
        return np.where(x, np.float32(1.0), np.float32(0.0)).astype(np.float32)
    if sf and dst == "u32":
        with np.errstate(all="ignore"):
            return np.clip(np.trunc(x.astype(np.float64)), 0, 0xFFFFFFFF).astype(np.uint32)
    if src == "u32" and df:
        return x.astype(np.float32)
    if src == "bool" and dst == "u32":
        return x.astype(np.uint32)
    if src == "u32" and dst == "bool":
        return x != 0
    raise ValueError((src, dst))


def reduce(fn, x, depth):
    """jit.rs:588-644 + op.rs:78-89: fold the last `depth` dims into one of extent 1; result is f32.
    Summation runs in float64 (the reference's order is unspecified: block tree + atomics)."""
    shape = list(x.shape)
    keep = shape[: len(shape) - depth]
    flat = x.reshape(keep + [-1])
    group = flat.shape[-1]
    if fn == "sum":
        r = flat.astype(np.float64).sum(axis=-1)
    elif fn == "mean":
        # every term is scaled by the double 1/group first, in double, then narrowed to float (jit.rs:599-604)
        r = (flat.astype(np.float64) * (1.0 / group)).astype(np.float32).astype(np.float64).sum(axis=-1)
    elif fn == "max":
        r = flat.max(axis=-1)
    elif fn == "min":
        r = flat.min(axis=-1)
    else:
        raise ValueError(fn)
    return r.astype(np.float32).reshape(keep + [1])


def matmul(a, b, precision, a_dtype, b_dtype):
    """Batched row-major A[..,M,K] x B[..,K,N] with operands rounded to the multiplicand type and f32
    accumulation, evaluated in float64 (helium-ir op.rs:61-73; precision.rs:3-35: actual precision may exceed the
    one asked for, never fall below)."""
    def to_mul(x):
        if precision in ("bf16_f32",):
            return nm.bf16_bits_to_f32(nm.f32_to_bf16_bits(x)).reshape(x.shape)
        if precision in ("f16_f32", "f16_f16"):
            return x.astype(np.float16).astype(np.float32)
        return x
    r = np.matmul(to_mul(a).astype(np.float64), to_mul(b).astype(np.float64)).astype(np.float32)
    if accumulator_type(precision) == "f16":
        r = r.astype(np.float16).astype(np.float32)
    return r


def evaluate(nodes, inputs, materialize=False):
    """Evaluates the graph. `inputs`: {input id: storage array}. Returns {node id: math-domain array} for every
    node plus the descriptors. With materialize=True every intermediate is rounded to its storage dtype (what
    happens when each op runs as its own kernel); with False none is (one fused kernel); with a set of node ids
    exactly those are (the tensors that cross kernel boundaries of a plan)."""
    desc, val = {}, {}
    for n in nodes:
        i = n["id"]
        if n["node"] == "input":
            desc[i] = (list(n["shape"]), n["dtype"])
            val[i] = nm.from_storage(inputs[i], n["dtype"], n["shape"])
        elif n["node"] == "output":
            desc[i] = desc[n["from"]]
            val[i] = val[n["from"]]
        else:
            desc[i] = infer(n, desc)
            val[i] = _eval_op(n, desc, val)
            shape, dtype = desc[i]
            assert list(val[i].shape) == list(shape), (n, val[i].shape, shape)
            if materialize is True or (materialize is not False and i in materialize):
                val[i] = nm.from_storage(nm.to_storage(val[i], dtype), dtype, shape)
    return val, desc


def _eval_op(n, desc, val):
    op, ins = n["op"], n["inputs"]
    if op == "unary":
        return unary(n["fn"], val[ins[0]])
    if op == "binary":
        return binary(n["fn"], val[ins[0]], val[ins[1]])
    if op == "change_dtype":
        return cast_class(val[ins[0]], desc[ins[0]][1], n["target"])
    if op == "reduce":
        return reduce(n["fn"], val[ins[0]], n["depth"])
    if op == "broadcast":
        shape, _ = infer(n, desc)
        x = val[ins[0]]
        x = x.reshape([1] * (len(shape) - x.ndim) + list(x.shape))
        # a listed axis always reads coordinate 0 of the input (jit.rs:877-879)
        index = tuple(slice(0, 1) if any(a == ax for ax, _ in n["axes"]) else slice(None) for a in range(len(shape)))
        return np.ascontiguousarray(np.broadcast_to(x[index], shape))
    if op == "reshape":
        return val[ins[0]].reshape(n["new_shape"])
    if op == "swap_dims":
        return np.ascontiguousarray(np.swapaxes(val[ins[0]], n["axis_a"], n["axis_b"]))
    if op == "compare":
        return compare(n["fn"], val[ins[0]], val[ins[1]])
    if op == "select":
        return np.where(val[ins[2]], val[ins[1]], val[ins[0]])  # rhs where the selector is true
    if op == "constant":
        dt = n["const_dtype"]
        math = nm.from_storage(nm.to_storage(np.array([n["value"]]), dt), dt, [1]) if dt != "bool" else np.array([bool(n["value"])])
        return np.ascontiguousarray(np.broadcast_to(math.reshape([1] * len(n["shape"])), n["shape"]))
    if op == "matmul":
        return matmul(val[ins[0]], val[ins[1]], n["precision"], desc[ins[0]][1], desc[ins[1]][1])
    if op == "conv":
        return conv(val[ins[0]], val[ins[1]], n["params"], desc[ins[0]][1])
    if op == "conv_bwd_data":
        return conv_backward_data(val[ins[0]], val[ins[1]], n["params"], n["input_size"])
    if op == "conv_bwd_filter":
        return conv_backward_filter(val[ins[0]], val[ins[1]], n["params"])
    raise ValueError(op)


def conv_backward_data(flow, filt, params, input_size):
    """Gradient of `conv` with respect to its image (what cuDNN's CONVOLUTION_BACKWARD_DATA computes for the
    descriptor of cudnn_graph.rs:205-216,384-396): the adjoint of the forward map, so every product
    flow[n,p,q,o] * filter[o,r,s,c] lands on the image pixel (p*sh + r*dh - ph, q*sw + s*dw - pw) the forward op
    read for it, if that pixel exists. Evaluated in float64."""
    n, oh, ow, o = flow.shape
    _, kr, ks, c = filt.shape
    h, w = input_size
    sh, sw = params.get("stride", (1, 1))
    dh, dw = params.get("dilation", (1, 1))
    ph, pw = conv_padding(params)
    dy = flow.astype(np.float64)
    f = filt.astype(np.float64)
    out = np.zeros((n, h, w, c), dtype=np.float64)
    for r in range(kr):
        for s in range(ks):
            ih = np.arange(oh) * sh + r * dh - ph
            iw = np.arange(ow) * sw + s * dw - pw
            vh, vw = (ih >= 0) & (ih < h), (iw >= 0) & (iw < w)
            if not vh.any() or not vw.any():
                continue
            contrib = np.einsum("nhwo,oc->nhwc", dy[:, vh][:, :, vw], f[:, r, s, :])
            out[np.ix_(np.arange(n), ih[vh], iw[vw], np.arange(c))] += contrib
    return out.astype(np.float32)


def conv_backward_filter(flow, image, params):
    """Gradient of `conv` with respect to its filter (cuDNN's CONVOLUTION_BACKWARD_FILTER for the descriptor of
    cudnn_graph.rs:217-228,384-396): filter tap (o, r, s, c) collects flow[n,p,q,o] * image[n, p*sh + r*dh - ph,
    q*sw + s*dw - pw, c] over every output pixel whose tap lies inside the image. Evaluated in float64."""
    n, oh, ow, o = flow.shape
    _, h, w, c = image.shape
    kr, ks = params["kernel_size"]
    sh, sw = params.get("stride", (1, 1))
    dh, dw = params.get("dilation", (1, 1))
    ph, pw = conv_padding(params)
    dy = flow.astype(np.float64)
    x = image.astype(np.float64)
    out = np.zeros((o, kr, ks, c), dtype=np.float64)
    for r in range(kr):
        for s in range(ks):
            ih = np.arange(oh) * sh + r * dh - ph
            iw = np.arange(ow) * sw + s * dw - pw
            vh, vw = (ih >= 0) & (ih < h), (iw >= 0) & (iw < w)
            if not vh.any() or not vw.any():
                continue
            out[:, r, s, :] = np.einsum("nhwo,nhwc->oc", dy[:, vh][:, :, vw], x[:, ih[vh]][:, :, iw[vw]])
    return out.astype(np.float32)


def kernel_outputs(nodes, inputs, leaf_ids):
    """Storage-domain outputs of ONE fused kernel whose leaves are `leaf_ids`."""
    val, desc = evaluate(nodes, inputs, materialize=False)
    return {i: nm.to_storage(val[i], desc[i][1]) for i in leaf_ids}


def plan_outputs(nodes, inputs, plan_steps):
    """Storage-domain value of every Output node when the graph runs as the kernels of `plan_steps`
    ([(instrs, released)], instrs = [(kind, [node ids])]): a value is rounded to its storage dtype exactly where it
    leaves the kernel that computes it, and is kept in f32 inside a kernel. The kernels are evaluated one by one, in
    plan order, each on its own members: a node may be a member of several instructions (a value the plan computes
    again in every kernel that uses it instead of passing it through memory), and every kernel then works on its own,
    unrounded copy. A member may also stand for its value in another layout (a plan that cancels transpositions computes a
    pointwise op on the untransposed operands and leaves the SwapDims out): element by element that is the same
    arithmetic, so the op is evaluated as recorded and the SwapDims, a member of no kernel, is read through.
    Returns {output node id: storage array}."""
    by_id = {n["id"]: n for n in nodes}
    # ops that compute the same thing may be one op of the plan (it then names the first of them): every id is read
    # through `canon`
    canon, seen = {}, {}
    for n in nodes:
        i = n["id"]
        canon[i] = i
        if n["node"] != "op":
            continue
        key = (tuple(canon[p] for p in n["inputs"]), repr(sorted((k, repr(v)) for k, v in n.items() if k not in ("id", "inputs"))))
        canon[i] = seen.setdefault(key, i)

    class _Through(dict):
        def __getitem__(self, k):
            k = canon[k]
            if not dict.__contains__(self, k) and by_id[k].get("op") in ("swap_dims", "reshape", "broadcast"):
                # A plan may have taken a transposition out (the ops behind it then run on the untransposed tensor and
                # the plan names them, not the SwapDims) or folded a shape op into a neighbour: such ops only move
                # values, so they are read through, from whatever holds their operand.
                # (not kept: a later kernel may compute the operand afresh, and must then see its own copy)
                return _eval_op(by_id[k], desc, self)
            if not dict.__contains__(self, k) and k in unnamed:
                shape, dtype = desc[k]
                return nm.from_storage(nm.to_storage(_eval_op(by_id[k], desc, stored), dtype), dtype, shape)
            return dict.__getitem__(self, k)

        def __contains__(self, k):
            return dict.__contains__(self, canon[k])

        def __setitem__(self, k, v):
            dict.__setitem__(self, canon[k], v)

    # What a kernel writes to memory: the members that another kernel (or an Output) reads without computing them
    # itself. A shape op that no kernel holds is read through, so the need passes on to its operand.
    computed = {canon[m] for instrs, _ in plan_steps for _, members in instrs for m in members}
    needed, unnamed = set(), set()

    def need(i, inside):
        i = canon[i]
        if i in inside or by_id[i]["node"] == "input":
            return
        if i in computed:
            needed.add(i)
        else:
            # A shape op that no kernel holds is read through. So is, rounded to its storage type, any other op that no
            # kernel names: a rewrite of the plan's may have merged it with an op that computes the same values from
            # other nodes (the op applied before a broadcast instead of after it) and names only that one.
            if by_id[i].get("op") not in ("swap_dims", "reshape", "broadcast"):
                unnamed.add(i)
            for j in by_id[i]["inputs"]:
                need(j, set())

    for instrs, _ in plan_steps:
        for _, members in instrs:
            inside = {canon[m] for m in members}
            for m in members:
                for j in by_id[m]["inputs"]:
                    need(j, inside)
    for n in nodes:
        if n["node"] == "output":
            need(n["from"], set())

    desc, stored = {}, _Through()
    for n in nodes:  # descriptors of everything; values of the inputs
        i = n["id"]
        if n["node"] == "input":
            desc[i] = (list(n["shape"]), n["dtype"])
            stored[i] = nm.from_storage(inputs[i], n["dtype"], n["shape"])
        elif n["node"] == "output":
            desc[i] = desc[n["from"]]
        else:
            desc[i] = infer(n, desc)
    for instrs, _ in plan_steps:
        for _, members in instrs:
            inside = set(members)
            local = _Through(stored)  # what memory holds, overlaid by this kernel's own values
            for m in sorted(inside):
                local[m] = _eval_op(by_id[m], desc, local)
                assert list(local[m].shape) == list(desc[m][0]), (by_id[m], local[m].shape)
            for m in inside:
                if canon[m] in needed:
                    shape, dtype = desc[m]
                    stored[m] = nm.from_storage(nm.to_storage(local[m], dtype), dtype, shape)
    return {n["id"]: nm.to_storage(stored[n["from"]], desc[n["id"]][1]) for n in nodes if n["node"] == "output"}

