"""GPU parity of whole fusion-IR graphs run through the fusion search and its kernels, against the oracle."""
import numpy as np
import pytest

import helium_amd as ha
from helium_amd import configs
from helium_amd import fusion_search as fs
from oracle import fusion_ir as oracle
from oracle import numerics as nm

pytestmark = pytest.mark.gpu


def two_layer_graph(n=256):
    """Two chained GEMMs with pointwise work between and after them and a column reduction."""
    g = ha.fusion.OpGraph()
    x = g.producer([1, n, n]); w1 = g.producer([1, n, n]); w2 = g.producer([1, n, n])
    b1 = g.producer([1, 1, n], "f32")
    h = g.unary(g.binary(g.matmul(x, w1), g.broadcast(b1, 1, n), "add"), "relu")
    y = g.matmul(h, w2)
    s = g.reduction(g.unary(y, "tanh"), "columns")
    t = g.binary(h, y, "add")
    outs = {"s": g.consumer(s, "f32"), "t": g.consumer(t, "bf16")}
    rng = np.random.default_rng(12)
    inputs = {x: configs.bf16_rne(rng.standard_normal((1, n, n)).astype(np.float32)),
              w1: configs.bf16_rne((rng.standard_normal((1, n, n)) * 0.06).astype(np.float32)),
              w2: configs.bf16_rne((rng.standard_normal((1, n, n)) * 0.06).astype(np.float32)),
              b1: rng.standard_normal((1, 1, n)).astype(np.float32)}
    return g, inputs, outs


def run_plan(g, inputs, plan):
    by_id = {n["id"]: n for n in g.nodes}
    prod = {i: ha.DeviceBuffer.from_numpy(a) for i, a in inputs.items()}
    cons = {}
    for n in g.nodes:
        if n["op"] == "consumer":
            numel = int(np.prod(n["shape"]))
            cons[n["id"]] = ha.DeviceBuffer(max(256, numel * (4 if n["dtype"] == "f32" else 2)))
    plan.execute(prod, cons)
    ha.device.synchronize()
    out = {}
    for i, b in cons.items():
        n = by_id[i]
        out[i] = b.to_numpy(np.float32 if n["dtype"] == "f32" else np.uint16)[: int(np.prod(n["shape"]))]
    return out


def boundary_values(g, plan):
    """Nodes whose value crosses a kernel boundary, with the dtype they are stored in."""
    by_id = {n["id"]: n for n in g.nodes}
    mat = {}
    for f in plan.fusions:
        inside = set(f["mainloop"] + f["epilogue"] + f["aux"] + ([f["anchor"]] if f["core"] else []))
        for n in g.nodes:
            if n["id"] in inside:
                continue
            for k in ("a", "b", "x", "lhs", "rhs"):
                src = n.get(k)
                if src in inside and n["op"] != "consumer":
                    mat[src] = "f32" if by_id[src]["op"] == "reduction" else "bf16"
    return mat


@pytest.mark.parametrize("objective,subdivided", [(fs.MAXIMAL, False), (fs.MIN_NAIVE_COST, False), (fs.MIN_ANALYTICAL_COST, False),
                                                  (fs.MIN_NAIVE_COST, True), (fs.MIN_ANALYTICAL_COST, True)])
def test_two_layer_graph_through_the_search(gpu, objective, subdivided):
    g, inputs, outs = two_layer_graph()
    plan = fs.FusionPlan(g, objective, subdivided=subdivided)
    print(plan.text, flush=True)
    got = run_plan(g, inputs, plan)
    val, _ = oracle.evaluate(g.nodes, inputs, round_mainloop_to="bf16", materialize=boundary_values(g, plan))
    t = nm.bf16_bits_to_f32(got[outs["t"]]).astype(np.float64)
    want_t = val[outs["t"]].reshape(-1).astype(np.float64)
    assert (np.abs(t - want_t) <= 2e-2 * np.maximum(np.abs(want_t), 0.25)).all(), float(np.abs(t - want_t).max())
    s = got[outs["s"]].astype(np.float64)
    want_s = val[outs["s"]].reshape(-1).astype(np.float64)
    assert np.abs(s - want_s).max() <= 2e-2 * np.abs(want_s).max() + 1e-2


def test_readme_graph_found_by_the_search_matches_the_hand_fed_fusion(gpu):
    size = 256
    g, outs = configs.c4_graph(size)
    inputs = configs.c4_inputs(g, size)
    want = oracle.outputs(g.nodes, inputs, round_mainloop_to="bf16")
    leaf_of = {}
    for name, node in outs.items():
        leaf_of[g.consumer(node, "f32")] = node
    plan = fs.FusionPlan(g, fs.MIN_NAIVE_COST)
    assert len(plan.fusions) == 1
    got = run_plan(g, inputs, plan)
    for c, node in leaf_of.items():
        a, b = got[c].astype(np.float64), want[node].reshape(-1).astype(np.float64)
        assert np.abs(a - b).max() <= 1e-3 * np.abs(b).max(), (node, float(np.abs(a - b).max()))


def test_merged_plan_with_a_kernel_feeding_a_mainloop(gpu):
    """Searched by subdivision: a row reduction (a kernel of its own) feeds a broadcast that is fused into the Matmul's
    mainloop, and the Matmul's epilogue reads a value of the other subdivision."""
    n = 128
    g = ha.fusion.OpGraph()
    a = g.producer([1, n, n]); w = g.producer([1, n, n]); b = g.producer([1, n, n])
    nb = g.unary(b, "neg")
    r = g.reduction(g.unary(a, "tanh"), "rows")
    x = g.binary(a, g.broadcast(r, 2, n), "mul")
    y = g.binary(g.matmul(x, w), nb, "add")
    out = g.consumer(y, "bf16")
    rng = np.random.default_rng(3)
    inputs = {a: configs.bf16_rne((rng.standard_normal((1, n, n)) * 0.3).astype(np.float32)),
              w: configs.bf16_rne((rng.standard_normal((1, n, n)) * 0.1).astype(np.float32)),
              b: configs.bf16_rne(rng.standard_normal((1, n, n)).astype(np.float32))}
    plan = fs.FusionPlan(g, fs.MIN_NAIVE_COST, subdivided=True)
    print(plan.text, flush=True)
    assert len(plan.fusions) == 2
    got = run_plan(g, inputs, plan)
    val, _ = oracle.evaluate(g.nodes, inputs, round_mainloop_to="bf16", materialize=boundary_values(g, plan))
    t = nm.bf16_bits_to_f32(got[out]).astype(np.float64)
    want = val[out].reshape(-1).astype(np.float64)
    assert (np.abs(t - want) <= 2e-2 * np.maximum(np.abs(want), 0.25)).all(), float(np.abs(t - want).max())
