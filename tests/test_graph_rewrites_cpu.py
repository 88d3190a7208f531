"""The rewrites a graph goes through before it is planned (ir.cpp: transposes_cancelled, broadcasts_hoisted, rematerialized), checked on
the CPU: the graph a plan is made of is read back through the C ABI (he_plan_graph, he_graph_node_op) and evaluated by
the oracle next to the graph as recorded. Both must give the same outputs - exactly where only data moves, to rounding
where a reduction walks its operand in another order - and the transpositions that undo each other must be gone.

The recorded graphs are what the reference's front end writes for these computations: a reduction over leading dims as
SwapDims + Reduce (batch_norm.rs:41-46), a SwapDims answered by a SwapDims in the backward pass and the gradient of a
broadcast as a chain of swaps in front of a Reduce (tensor.rs; harness/autodiff.py restates them)."""
import numpy as np
import pytest

from harness import autodiff as ad
from helium_amd import ir
from harness import resnet
from helium_amd.backend import OPT_CANCEL_TRANSPOSES, OPT_HOIST_BROADCASTS, OPT_REMATERIALIZE, Plan, set_option
from oracle import helium_ir as oracle_ir
from oracle import numerics as nm


@pytest.fixture(params=["transposes only", "all rewrites"])
def rewrites(request):
    set_option(OPT_REMATERIALIZE, 0 if request.param == "transposes only" else 1)
    set_option(OPT_HOIST_BROADCASTS, 0 if request.param == "transposes only" else 1)
    set_option(OPT_CANCEL_TRANSPOSES, 1)
    yield request.param
    set_option(OPT_REMATERIALIZE, 1)
    set_option(OPT_HOIST_BROADCASTS, 1)


def _feeds(g, seed=3):
    rng = np.random.default_rng(seed)
    return {n["id"]: nm.to_storage(rng.standard_normal(n["shape"]).astype(np.float32), n["dtype"]) for n in g.nodes if n["node"] == "input"}


def _both(g, feeds):
    """(outputs of the graph as recorded, outputs of the graph its plan is made of, that graph's nodes), outputs keyed by
    the recorded Output node."""
    plan = Plan(g)
    planned = plan.graph()
    want, _ = oracle_ir.evaluate(g.nodes, feeds)
    planned_feeds = {n["id"]: feeds[n["origin"]] for n in planned.nodes if n["node"] == "input"}
    got, _ = oracle_ir.evaluate(planned.nodes, planned_feeds)
    outs_want = {n["id"]: want[n["id"]] for n in g.nodes if n["node"] == "output"}
    outs_got = {n["origin"]: got[n["id"]] for n in planned.nodes if n["node"] == "output"}
    assert set(outs_want) == set(outs_got)
    return outs_want, outs_got, planned.nodes, plan


def _swaps(nodes):
    return [n for n in nodes if n.get("op") == "swap_dims"]


def test_a_swap_that_undoes_a_swap_is_gone(rewrites):
    g = ir.OpGraph()
    x = g.new_input([3, 4, 5], "f32")
    y = g.swap_dims(g.unary(g.swap_dims(x, 0, 2), "exp"), 2, 0)
    g.new_output(g.binary(y, x, "add"))
    want, got, nodes, _ = _both(g, _feeds(g))
    assert not _swaps(nodes)
    for o in want:
        np.testing.assert_array_equal(want[o], got[o])


def test_swaps_move_through_pointwise_ops_broadcasts_constants_compare_and_select(rewrites):
    """The backward pass of a relu and a per-channel scale, both recorded on the transposed tensor."""
    g = ir.OpGraph()
    x = g.new_input([6, 2, 3, 4], "f32")  # NHWC
    scale = g.new_input([4], "f32")
    xt = g.swap_dims(x, 0, 3)             # CHWN
    s = g.broadcast(g.reshape(scale, [4, 1, 1, 1]), 4, [(1, 2), (2, 3), (3, 6)])
    zero = g.constant(0.0, "f32", [4, 2, 3, 6])
    mask = g.compare(xt, zero, "gt")
    y = g.select(zero, g.binary(xt, s, "mul"), mask)
    y = g.binary(y, g.constant(2.0, "f32", [4, 2, 3, 6]), "pow")
    g.new_output(g.swap_dims(y, 3, 0))
    want, got, nodes, _ = _both(g, _feeds(g))
    assert not _swaps(nodes)
    for o in want:
        np.testing.assert_array_equal(want[o], got[o])


def test_a_broadcast_whose_source_has_to_be_transposed_itself(rewrites):
    g = ir.OpGraph()
    x = g.new_input([5, 9, 3], "f32")
    v = g.new_input([5, 1, 3], "f32")
    xt = g.swap_dims(x, 0, 2)                                           # [3, 9, 5]
    vt = g.broadcast(g.swap_dims(v, 0, 2), 3, [(1, 9)])                 # [3, 1, 5] -> [3, 9, 5]
    g.new_output(g.swap_dims(g.binary(xt, vt, "mul"), 0, 2))
    want, got, nodes, _ = _both(g, _feeds(g))
    assert not [n for n in _swaps(nodes) if int(np.prod(n["shape"])) > 15]
    for o in want:
        np.testing.assert_array_equal(want[o], got[o])


def test_a_swap_that_would_only_move_is_left_alone(rewrites):
    g = ir.OpGraph()
    x = g.new_input([3, 4], "f32")
    y = g.new_input([4, 3], "f32")
    g.new_output(g.swap_dims(g.binary(g.swap_dims(x, 0, 1), y, "mul"), 0, 1))
    want, got, nodes, _ = _both(g, _feeds(g))
    assert len(_swaps(nodes)) == 2
    for o in want:
        np.testing.assert_array_equal(want[o], got[o])


def test_the_chain_of_swaps_in_front_of_a_reduction_becomes_the_shortest_one(rewrites):
    """The gradient of a [C] -> [N,H,W,C] broadcast as tensor.rs records it: the dims reversed by two swaps, then a
    Reduce over three of them. One swap does."""
    g = ir.OpGraph()
    flow = g.new_input([6, 2, 3, 4], "f32")
    t = g.swap_dims(g.swap_dims(flow, 0, 3), 1, 2)
    g.new_output(g.reduce(t, "sum", 3))
    # global average pooling as model.rs:81-83 writes it
    pooled = g.reduce(g.swap_dims(g.swap_dims(flow, 2, 3), 1, 2), "mean", 2)
    g.new_output(pooled)
    # kept dims that are already in front need no swap at all
    g.new_output(g.reduce(g.swap_dims(flow, 2, 3), "max", 2))
    want, got, nodes, _ = _both(g, _feeds(g))
    swaps = _swaps(nodes)
    assert len(swaps) == 2, swaps
    for o in want:
        np.testing.assert_allclose(got[o], want[o], rtol=1e-6, atol=1e-6)


def test_pointwise_ops_on_broadcasts_alone_are_applied_before_the_broadcast():
    """batch_norm.rs:56 as recorded: (variance.broadcast_to(x.shape) + 1e-3).sqrt() and the division by it."""
    g = ir.OpGraph()
    x = g.new_input([6, 5, 5, 8], "bf16")
    var = g.new_input([8], "bf16")
    mean = g.new_input([8], "bf16")
    axes = [(0, 6), (1, 5), (2, 5)]
    deviation = g.unary(g.binary(g.broadcast(var, 4, axes), g.constant(1e-3, "bf16", [6, 5, 5, 8]), "add"), "sqrt")
    centred = g.binary(x, g.unary(g.broadcast(mean, 4, axes), "neg"), "add")
    g.new_output(g.binary(centred, g.unary(deviation, "recip"), "mul"))
    # broadcasts along different axes meet in the smallest shape that holds both: [6,1,1,1] and [8] in [6,1,1,8]
    other = g.broadcast(g.new_input([6, 1, 1, 1], "bf16"), 4, [(1, 5), (2, 5), (3, 8)])
    g.new_output(g.binary(other, g.broadcast(var, 4, axes), "mul"))
    want, got, nodes, _ = _both(g, _feeds(g))
    full = [n for n in nodes if n.get("op") in ("unary", "binary") and int(np.prod(n["shape"])) == 6 * 5 * 5 * 8]
    assert sorted((n["op"], n["fn"]) for n in full) == [("binary", "add"), ("binary", "mul")], full
    small = [n for n in nodes if n.get("op") in ("unary", "binary") and int(np.prod(n["shape"])) == 8]
    assert sorted(n["fn"] for n in small) == ["add", "neg", "recip", "sqrt"]
    assert [n["shape"] for n in nodes if n.get("op") == "binary" and int(np.prod(n["shape"])) == 48] == [[6, 1, 1, 8]]
    for o in want:
        np.testing.assert_array_equal(want[o], got[o])


def test_a_reduction_of_a_broadcast_along_reduced_dims_walks_the_small_tensor():
    g = ir.OpGraph()
    x = g.new_input([10, 16, 1, 1], "bf16")
    full = g.broadcast(x, 4, [(2, 7), (3, 7)])
    g.new_output(g.reduce(full, "sum", 3))
    g.new_output(g.reduce(full, "mean", 3))
    g.new_output(g.reduce(full, "max", 2))
    # a broadcast along a kept dim is left alone
    g.new_output(g.reduce(g.broadcast(g.new_input([1, 16, 7, 7], "bf16"), 4, [(0, 10)]), "sum", 3))
    want, got, nodes, _ = _both(g, _feeds(g))
    by_id = {n["id"]: n for n in nodes}
    sizes = sorted(int(np.prod(by_id[n["inputs"][0]]["shape"])) for n in nodes if n.get("op") == "reduce")
    assert sizes == [160, 160, 160, 10 * 16 * 49], sizes
    for o in want:
        np.testing.assert_allclose(got[o], want[o], rtol=1e-6)


def _batch_norm_backward_graph(dtype):
    G = ad.Graph()
    rng = np.random.default_rng(5)
    bn = resnet.BatchNorm2d(G, 8)
    x = G.param(rng.standard_normal([4, 3, 5, 8]).astype(np.float32))
    y = bn.forward(x.value.to_data_type(dtype)).relu()
    loss = (y * y).reduce_sum(4).reshape([1])
    grads = loss.backward()
    for p in [x] + bn.parameters():
        G.g.new_output(grads[p.id].node)
    G.g.new_output(bn.running_mean.raw.node)
    G.g.new_output(bn.running_variance.raw.node)
    return G


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_batch_norm_backward_has_no_transposition_left_but_the_ones_reductions_fold(rewrites, dtype):
    G = _batch_norm_backward_graph(dtype)
    g = G.g
    g.optimize()
    recorded = [n for n in g.nodes]
    want, got, nodes, plan = _both(g, G.feeds)
    by_id = {n["id"]: n for n in nodes}
    consumers = {}
    for n in nodes:
        for i in n.get("inputs", []):
            consumers.setdefault(i, []).append(n)
    # what is left of the recorded swaps feeds reductions only, through pointwise ops
    def ends_in_reductions(i):
        users = consumers.get(i, [])
        return bool(users) and all(u["op"] == "reduce" or (u["op"] in ("unary", "binary", "change_dtype") and ends_in_reductions(u["id"])) for u in users)
    left = [n for n in _swaps(nodes) if int(np.prod(n["shape"])) > 8]
    assert len(left) < len([n for n in _swaps(recorded) if int(np.prod(n["shape"])) > 8])
    assert all(ends_in_reductions(n["id"]) for n in left), [n for n in left if not ends_in_reductions(n["id"])]
    assert not any(kind == "permute" for instrs, _ in plan.steps for kind, _ in instrs)
    tol = 1e-5 if dtype == "f32" else 2e-2
    for o in want:
        scale = max(float(np.abs(want[o]).max()), 1e-30)
        assert float(np.abs(got[o].astype(np.float64) - want[o]).max()) <= tol * scale, o


def test_training_step_outputs_survive_the_rewrites(rewrites):
    """The whole training step (f32, so that where a value is rounded does not matter): the graph the plan is made of
    computes what the recorded graph computes."""
    r = resnet.record_training_step(2, 32, width=8, num_classes=16, dtype="f32")
    g = r["graph"].g
    g.optimize()
    want, got, nodes, plan = _both(g, r["graph"].feeds)
    assert len(want) == len(r["carried"]) + 2
    for o in want:
        scale = max(float(np.abs(want[o]).max()), 1e-30)
        assert float(np.abs(got[o].astype(np.float64) - want[o]).max()) <= 2e-4 * scale, o
    assert not any(kind == "permute" for instrs, _ in plan.steps for kind, _ in instrs)
    # the plan names its kernels' members by recorded nodes: the oracle, evaluating those kernels one by one on the
    # recorded graph, arrives at the same outputs (this is how the GPU tests get their expected values)
    by_id = {n["id"]: n for n in g.nodes}
    stepwise = oracle_ir.plan_outputs(g.nodes, r["graph"].feeds, plan.steps)
    for o in want:
        dtype = by_id[by_id[o]["from"]]["dtype"]
        have = nm.from_storage(stepwise[o].reshape(-1), dtype, [stepwise[o].size]).astype(np.float64)
        scale = max(float(np.abs(want[o]).max()), 1e-30)
        assert float(np.abs(have - want[o].reshape(-1)).max()) <= 2e-4 * scale, o
