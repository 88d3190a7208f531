"""The graphs of the reference's own autodiff / loss / matmul / convolution tests (helium/tests/autodiff.rs,
helium/tests/loss.rs, helium/tests/tensor_ops.rs:172-318,379-397), recorded the way the reference's front end records
them; the vectors come from tests/golden/*.json. Shared by the CPU tests (oracle) and the GPU tests (HIP path)."""
import json
import os

import numpy as np

from harness import autodiff as ad
from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
AUTODIFF = json.load(open(os.path.join(GOLDEN, "autodiff.json")))["cases"]
TENSOR_OPS = json.load(open(os.path.join(GOLDEN, "tensor_ops.json")))


def record_autodiff(case):
    """Returns (Graph, {name: Raw}) for one case of autodiff.json."""
    G = ad.Graph()
    name = case["name"]
    if "op" in case:  # max_* / min_*: Param(from_constant) (autodiff.rs:157-221)
        a = ad.Param(G.constant(case["constants"]["a"], [1]))
        b = ad.Param(G.constant(case["constants"]["b"], [1]))
        result = getattr(a.value, case["op"])(b) * 2.0
        grads = result.backward()
        return G, {"a": grads[a.id], "b": grads[b.id]}
    if name.startswith("bce_loss"):
        prediction = G.constant(case["prediction"], [1, 1])
        target = G.constant(case["target"], [1, 1])
        return G, {"loss": ad.binary_cross_entropy_loss(prediction, target).raw}
    params = {k: G.param(v, case.get("param_shape")) for k, v in case["params"].items()}
    inputs = {k: G.tensor(v, case.get("input_shape")) for k, v in case["inputs"].items()}
    if name == "simple":
        result = params["p"].value * 3.0
    elif name == "autodiff_scalar":
        x = inputs["x"] * params["p1"]
        x = x.pow_scalar(2.0)
        result = x * params["p2"]
    elif name == "reduce_sum":
        result = (inputs["x"] * params["p"]).reduce_sum(1) * 3.0
    elif name == "reduce_mean":
        result = (inputs["x"] * params["p"]).reduce_mean(1) * 3.0
    elif name == "broadcast":
        x = inputs["x"]
        result = (params["p"].value.broadcast_to(x.shape) * x).reduce_sum(3)
    elif name == "reduce_min":
        x = inputs["x"]
        result = (params["p"].value.broadcast_to(x.shape) * x).reduce_min(1)
    elif name == "reduce_max":
        x = inputs["x"]
        result = (params["p"].value.broadcast_to(x.shape) * x).reduce_max(1)
    elif name == "relu":
        result = (inputs["x"] * params["p"]).relu().reduce_sum(1)
    else:
        raise ValueError(name)
    grads = result.backward()
    return G, {k: grads[p.id] for k, p in params.items()}


def record_matmul(case):
    """tensor_ops.rs:172-318: operands are uploaded as written and transposed in the graph where the test does."""
    G = ad.Graph()

    def operand(key):
        if key + "_fill" in case:
            value, shape = case[key + "_fill"]
            t = G.tensor(np.full(shape, value, dtype=np.float32), dtype=case["dtype"])
        else:
            t = G.tensor(np.array(case[key], dtype=np.float32), dtype=case["dtype"])
        return t.transpose() if case["transpose_" + key] else t
    a, b = operand("a"), operand("b")
    out = a.matmul(b, case["precision"])
    if case["transpose_out"]:
        out = out.transpose()
    expected = (np.full(case["expected_fill"][1], case["expected_fill"][0]) if "expected_fill" in case
                else np.array(case["expected"])).astype(np.float32)
    return G, out.raw, expected


def record_conv(case):
    G = ad.Graph()
    x = G.tensor(case["image"]).reshape(case["image_shape"])
    w = G.tensor(case["filter"]).reshape(case["filter_shape"])
    return G, x.conv2d(w, case["params"]).raw


def gradient_descent_step(guess, target=1001.0, learning_rate=1e-4):
    """One iteration of autodiff.rs:121-145. Returns (Graph, error Raw, new guess Raw)."""
    G = ad.Graph()
    p = G.param([guess])
    result = p.value.pow_scalar(2.0)
    error = (result - target).pow_scalar(2.0)
    grads = error.backward()
    gradient = ad.Tensor(grads[p.id])
    new_guess = p.value.detach() - gradient * learning_rate
    return G, error.raw, new_guess.raw


def evaluate_on_oracle(G, raws):
    """{name: f32 array (flat)} of the recorded nodes, evaluated by the oracle with every node in one kernel."""
    val, _ = oracle_ir.evaluate(G.g.nodes, G.feeds)
    return {k: np.asarray(val[r.node], dtype=np.float32).reshape(-1) for k, r in raws.items()}


def evaluate_on_device(G, raws):
    """The same through plan generation and execute_graph on the GPU."""
    from helium_amd.backend import Tensor, execute_graph

    outs = {k: G.g.new_output(r.node) for k, r in raws.items()}
    by_id = {n["id"]: n for n in G.g.nodes}
    tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in G.feeds.items()}
    got = execute_graph(G.g, tensors)
    res = {}
    for k, o in outs.items():
        shape, dtype = G.g.descriptor(o)
        res[k] = nm.from_storage(got[o].to_numpy(), dtype, shape).astype(np.float32).reshape(-1)
    return res
