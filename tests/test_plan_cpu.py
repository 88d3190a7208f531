"""Plan generation (helium/src/backend/plan_generation.rs) through the C ABI.

The expected plans of the named cases are worked out by hand from the reference text (slot order of the greedy
fusion, Kahn levels, delay_computations, release lists); the same cases then pin oracle/plan.py, which in turn
checks the library on seeded random graphs together with the invariants the reference asserts in debug builds
(plan_generation.rs:418-445)."""
import numpy as np
import pytest

import helium_amd as ha
from helium_amd.backend import (OPT_CANCEL_TRANSPOSES, OPT_FOLD_SWAP_INTO_REDUCE, OPT_FUSE_MATMUL_EPILOGUE, OPT_HOIST_BROADCASTS,
                                OPT_REMATERIALIZE, Plan,
                                set_option, stats)
from oracle import plan as oracle_plan


@pytest.fixture
def reference_grouping():
    """The reference's rules: a matmul instruction never fuses (cudnn_graph.rs:319-321), a SwapDims of more
    than 1M elements is always a permute instruction (cuda.rs:38-41), and the graph is planned as recorded (no value
    is computed twice, every SwapDims stays; a Constant is a kernel of its own, pointwise.rs:181)."""
    set_option(OPT_FUSE_MATMUL_EPILOGUE, 0)
    set_option(OPT_FOLD_SWAP_INTO_REDUCE, 0)
    set_option(OPT_REMATERIALIZE, 0)
    set_option(OPT_CANCEL_TRANSPOSES, 0)
    set_option(OPT_HOIST_BROADCASTS, 0)
    yield
    set_option(OPT_FUSE_MATMUL_EPILOGUE, 1)
    set_option(OPT_FOLD_SWAP_INTO_REDUCE, 1)
    set_option(OPT_REMATERIALIZE, 1)
    set_option(OPT_CANCEL_TRANSPOSES, 1)
    set_option(OPT_HOIST_BROADCASTS, 1)


def linear_layer():
    g = ha.ir.OpGraph()
    x = g.new_input([256, 512], "f32"); w = g.new_input([512, 512], "f32"); b = g.new_input([512], "f32")
    mm = g.matmul(x, w, "tf32_f32")
    bb = g.broadcast(b, 2, [(0, 256)])
    y = g.unary(g.binary(mm, bb, "add"), "relu")
    r = g.reduce(g.swap_dims(y, 0, 1), "sum", 1)
    g.new_output(y); g.new_output(r)
    # broadcast+add+relu fuse; the swap cannot join them (a Broadcast was counted first, pointwise.rs:156-162) and
    # starts a second kernel that takes the reduction
    return g, [([("gemm", [3])], []), ([("pointwise", [4, 5, 6])], [0, 1]), ([("pointwise", [7, 8])], [2, 3]), ([], [])]


def second_path_blocks_fusion():
    g = ha.ir.OpGraph()
    a = g.new_input([64, 64], "f32"); w = g.new_input([64, 64], "f32")
    u = g.unary(a, "exp"); m = g.matmul(u, w, "f32_f32"); v = g.binary(u, m, "add")
    g.new_output(v)
    # exp and add are fusible, but exp -> matmul -> add is a second path (plan_generation.rs:195-217)
    return g, [([("pointwise", [2])], []), ([("gemm", [3])], [0]), ([("pointwise", [4])], [1]), ([], [2, 3])]


def constant_is_delayed():
    g = ha.ir.OpGraph()
    x = g.new_input([32, 32], "f32"); w = g.new_input([32, 32], "f32")
    m1 = g.matmul(x, w, "f32_f32"); m2 = g.matmul(m1, w, "f32_f32")
    c = g.constant(1.0, "f32", [32, 32])
    g.new_output(g.binary(m2, c, "add"))
    # the constant is ready at step 0 but first read at step 2, so it moves to step 1 (:325-353)
    return g, [([("gemm", [2])], []), ([("gemm", [3]), ("pointwise", [4])], [0]), ([("pointwise", [5])], [1, 2]),
               ([], [3, 4])]


def large_swaps_chain():
    g = ha.ir.OpGraph()
    x = g.new_input([64, 56, 56, 256], "bf16")
    g.new_output(g.swap_dims(g.swap_dims(x, 2, 3), 1, 2))
    return g, [([("permute", [1, 2])], []), ([], [0])]


def two_reduction_depths():
    g = ha.ir.OpGraph()
    a = g.new_input([64, 64], "f32")
    t = g.unary(a, "tanh")
    r1 = g.reduce(t, "sum", 2)
    r2 = g.reduce(g.swap_dims(t, 0, 1), "sum", 1)
    g.new_output(r1); g.new_output(r2)
    # the chain takes the first reduction and the swap; the second reduction has another depth (pointwise.rs:163-179)
    return g, [([("pointwise", [1, 2, 3])], []), ([("pointwise", [4])], [0]), ([], [3])]


NAMED = [linear_layer, second_path_blocks_fusion, constant_is_delayed, large_swaps_chain, two_reduction_depths]


@pytest.mark.parametrize("make", NAMED, ids=lambda f: f.__name__)
def test_hand_derived_plans(reference_grouping, make):
    g, want = make()
    assert oracle_plan.generate_plan(g.nodes) == want
    assert Plan(g).steps == want


def random_graph(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.choice([8, 1024, 1100]))  # 1100² > 1,000,000: swaps become permute instructions
    g = ha.ir.OpGraph()
    vals = [(g.new_input([n, n], "f32"), [n, n]) for _ in range(int(rng.integers(1, 4)))]
    for _ in range(int(rng.integers(3, 22))):
        kind = rng.choice(["unary", "binary", "swap", "reduce", "matmul", "constant", "broadcast", "cast"],
                          p=[0.3, 0.25, 0.12, 0.1, 0.06, 0.04, 0.08, 0.05])
        x, shape = vals[int(rng.integers(len(vals)))]
        if kind == "unary":
            vals.append((g.unary(x, str(rng.choice(["exp", "relu", "neg", "tanh"]))), shape))
        elif kind == "binary":
            same = [v for v in vals if v[1] == shape]
            y, _ = same[int(rng.integers(len(same)))]
            vals.append((g.binary(x, y, str(rng.choice(["add", "mul", "max"]))), shape))
        elif kind == "swap" and len(shape) == 2:
            vals.append((g.swap_dims(x, 0, 1), shape[::-1]))
        elif kind == "reduce" and len(shape) >= 1:
            d = int(rng.integers(1, len(shape) + 1))
            vals.append((g.reduce(x, str(rng.choice(["sum", "max"])), d), shape[: len(shape) - d] or [1]))
        elif kind == "matmul" and shape == [n, n] and n <= 1024:
            sq = [v for v in vals if v[1] == [n, n]]
            y, _ = sq[int(rng.integers(len(sq)))]
            vals.append((g.matmul(x, y, "f32_f32"), [n, n]))
        elif kind == "constant":
            vals.append((g.constant(2.0, "f32", [n, n]), [n, n]))
        elif kind == "broadcast" and shape == [n]:
            vals.append((g.broadcast(x, 2, [(0, n)]), [n, n]))
        elif kind == "cast":
            vals.append((g.unary(g.change_data_type(x, "bf16"), "neg"), shape))
    consumed = {i for nd in g.nodes if nd["node"] == "op" for i in nd["inputs"]}
    ops = [nd["id"] for nd in g.nodes if nd["node"] == "op"]
    for i in ops:
        if i not in consumed and rng.random() < 0.85 or rng.random() < 0.1:  # a few sinks stay dead on purpose
            g.new_output(i)
    return g


def check_invariants(g, steps):
    og = oracle_plan.Graph(g.nodes)
    ops = [nd["id"] for nd in g.nodes if nd["node"] == "op"]
    placed = [n for instrs, _ in steps for _, nodes in instrs for n in nodes]
    assert sorted(placed) == sorted(ops), "every op belongs to exactly one instruction"
    assert steps[-1][0] == [] and steps[0][1] == []
    ready = {nd["id"] for nd in g.nodes if nd["node"] == "input"}
    freed = set()
    for instrs, released in steps:
        for t in released:
            assert t in ready and t not in freed and not og.feeds_output(t)
            freed.add(t)
        produced = set()
        for _, nodes in instrs:
            inside = set(nodes)
            for n in nodes:
                for p in og.inbound[n]:
                    if p not in inside:
                        assert p in ready and p not in freed, f"node {n} reads {p} before it exists / after its release"
            produced |= inside
        ready |= produced
    # every tensor some instruction reads from outside is freed at some step unless it feeds an output
    for instrs, _ in steps:
        for _, nodes in instrs:
            inside = set(nodes)
            for n in nodes:
                for p in og.inbound[n]:
                    if p not in inside:
                        assert p in freed or og.feeds_output(p), f"tensor {p} is never released"


@pytest.mark.parametrize("seed", range(60))
def test_random_graphs_match_the_restatement(reference_grouping, seed):
    g = random_graph(seed)
    got = Plan(g).steps
    assert got == oracle_plan.generate_plan(g.nodes)
    check_invariants(g, got)


def test_matmul_takes_the_ops_that_can_run_on_its_accumulators():
    # default grouping of this backend. Worked out by hand: the matmul (slot 1) takes the add, the bias broadcast
    # (slot 2) then joins as an epilogue operand, the relu follows; the swap alone cannot run on accumulators and
    # starts a second instruction, which takes the reduction; swap + reduce together are a column reduction of the
    # product, so the second look at the product's dependents merges the two instructions.
    g, _ = linear_layer()
    want = [([("gemm", [3, 4, 5, 6, 7, 8])], []), ([], [0, 1, 2])]
    assert Plan(g).steps == want

    def runs_on_accumulators(instr):
        ops = [instr.g.nodes[n]["op"] for n in instr.nodes]
        return ops.count("swap_dims") == ops.count("reduce")   # a transposition only together with its reduction

    assert oracle_plan.generate_plan(g.nodes, gemm_epilogue=runs_on_accumulators) == want


def test_ops_feeding_a_matmul_operand_stay_outside_it():
    g, want = second_path_blocks_fusion()
    # exp feeds the Matmul's A operand: no merge with it; the add after the Matmul reads exp's tensor and joins
    assert Plan(g).steps == [([("pointwise", [2])], []), ([("gemm", [3, 4])], [0]), ([], [1, 2])]


def test_row_sums_join_the_matmul():
    g = ha.ir.OpGraph()
    a = g.new_input([3, 64, 32], "bf16"); b = g.new_input([3, 32, 48], "bf16")
    y = g.unary(g.matmul(a, b, "bf16_f32"), "relu")
    g.new_output(y); g.new_output(g.reduce(y, "sum", 1)); g.new_output(g.reduce(y, "max", 1))
    # the Sum folds into the epilogue; Max is not a reduction the GEMM epilogue offers and stays a kernel of its own
    assert Plan(g).steps == [([("gemm", [2, 3, 5])], []), ([("pointwise", [7])], [0, 1]), ([], [])]


def test_plan_cache_returns_the_same_plan_for_an_equal_graph():
    before = stats()
    a, _ = linear_layer()
    b, _ = linear_layer()
    pa, pb = Plan(a), Plan(b)
    after = stats()
    assert pa.text == pb.text
    assert after["plan_cache_hits"] + after["plan_cache_misses"] >= before["plan_cache_hits"] + before["plan_cache_misses"]


def batch_norm_graph(shape):
    from harness import frontend

    g = ha.ir.OpGraph()
    rec = frontend.Recorder(g)
    c = shape[3]
    x = g.new_input(list(shape), "bf16")
    stats_in = [g.new_input([c], "f32") for _ in range(4)]
    y, new_mean, new_var = frontend.batch_norm_train(rec, x, *stats_in)
    for v in (y, new_mean, new_var):
        g.new_output(v)
    return g


def test_batch_norm_statistics_skip_the_permute():
    """BatchNorm2d::forward (batch_norm.rs:32-72) at [64,56,56,256]: the reference's plan transposes 51M elements
    and reads the transposed tensor twice; with the transposition folded into the reductions, one kernel reads x
    once for both statistics."""
    g = batch_norm_graph([64, 56, 56, 256])
    kinds = [[k for k, _ in instrs] for instrs, _ in Plan(g).steps]
    assert kinds[0] == ["pointwise"] and "permute" not in sum(kinds, [])
    swap = next(n["id"] for n in g.nodes if n.get("op") == "swap_dims")
    reduces = [n["id"] for n in g.nodes if n.get("op") == "reduce"]
    first = Plan(g).steps[0][0][0][1]
    assert swap in first and all(r in first for r in reduces)


def test_batch_norm_reference_plan_has_the_permute(reference_grouping):
    g = batch_norm_graph([64, 56, 56, 256])
    steps = Plan(g).steps
    assert [k for k, _ in steps[0][0]] == ["permute"]
    assert sorted(k for k, _ in steps[1][0]) == ["pointwise", "pointwise"]  # the two statistics read xt separately
    assert oracle_plan.generate_plan(g.nodes) == steps


def test_batch_norm_statistics_join_the_convolution_that_feeds_them():
    """conv -> BatchNorm2d (a resnet block's first half): the per-channel means of y and y^2 are column reductions of the
    implicit GEMM, so the convolution's instruction takes the SwapDims, the square and both reductions; the rest of
    the batch norm needs the finished statistics and stays outside."""
    from harness import frontend

    g = ha.ir.OpGraph()
    rec = frontend.Recorder(g)
    x = g.new_input([64, 56, 56, 64], "bf16"); w = g.new_input([64, 3, 3, 64], "bf16")
    conv = g.conv(x, w, {"in_channels": 64, "out_channels": 64, "kernel_size": [3, 3]})
    outs = frontend.batch_norm_train(rec, conv, *[g.new_input([64], "f32") for _ in range(4)])
    for v in outs:
        g.new_output(v)
    plan = Plan(g)
    steps = plan.steps
    kind, members = steps[0][0][0]
    by_id = {n["id"]: n for n in g.nodes}
    assert kind == "gemm" and len(steps[0][0]) == 1
    assert sorted(by_id[m]["op"] for m in members) == ["binary", "broadcast", "conv", "reduce", "reduce", "swap_dims"]
    assert all(k == "pointwise" for instrs, _ in steps[1:] for k, _ in instrs)
    # (the invariants hold on the graph the plan is made of: the backend's rewrites add and drop ops)
    check_invariants(plan.graph(), plan.planned_steps())


def linear_backward_graph(rows=64, inner=96, cols=80, dtype="f32", precision="f32_f32"):
    """The two products of a linear layer's backward pass as the front end records them:
    dW = x^T dy and dX = dy w^T (transpositions as SwapDims of the matrix dims)."""
    g = ha.ir.OpGraph()
    x = g.new_input([rows, inner], dtype); w = g.new_input([inner, cols], dtype); dy = g.new_input([rows, cols], dtype)
    xt = g.swap_dims(x, 0, 1)
    dw = g.matmul(xt, dy, precision)
    wt = g.swap_dims(w, 0, 1)
    dx = g.matmul(dy, wt, precision)
    names = {"x": x, "w": w, "dy": dy, "xt": xt, "wt": wt, "dw": dw, "dx": dx, "dw_out": g.new_output(dw), "dx_out": g.new_output(dx)}
    return g, names


def test_transposed_matmul_operands_join_the_gemm_instruction():
    g, n = linear_backward_graph()
    instrs = [i for step, _ in Plan(g).steps for i in step]
    assert sorted(instrs) == sorted([("gemm", [n["xt"], n["dw"]]), ("gemm", [n["wt"], n["dx"]])]), instrs


def test_transposed_matmul_operands_reference_grouping(reference_grouping):
    g, n = linear_backward_graph()
    steps = Plan(g).steps
    assert oracle_plan.generate_plan(g.nodes) == steps
    kinds = sorted(k for step, _ in steps for k, _ in step)
    assert kinds == ["gemm", "gemm", "pointwise", "pointwise"], steps


def conv_graph(kind, image=(2, 8, 8, 16), oc=32, kernel=(3, 3), dtype="bf16", filter_shape=None):
    g = ha.ir.OpGraph()
    params = {"in_channels": image[3], "out_channels": oc, "kernel_size": list(kernel)}
    fshape = filter_shape or [oc, kernel[0], kernel[1], image[3]]
    flow_shape = [image[0], image[1], image[2], oc]
    if kind == "conv":
        x = g.new_input(list(image), dtype); w = g.new_input(fshape, dtype)
        out = g.conv(x, w, params)
    elif kind == "data":
        dy = g.new_input(flow_shape, dtype); w = g.new_input(fshape, dtype)
        out = g.conv_backward_data(dy, w, params, image[1:3])
    else:
        dy = g.new_input(flow_shape, dtype); x = g.new_input(list(image), dtype)
        out = g.conv_backward_filter(dy, x, params)
    g.new_output(out)
    return g, out


@pytest.mark.parametrize("kind,shape", [("conv", [2, 8, 8, 32]), ("data", [2, 8, 8, 16]), ("filter", [32, 3, 3, 16])])
def test_convolution_ops_are_gemm_instructions(kind, shape):
    """Descriptors as op.rs:123-173 infers them, and one Gemm instruction per convolution op (the reference hands
    them to cuDNN, cuda.rs:55-58)."""
    g, out = conv_graph(kind)
    assert g.descriptor(out) == (shape, "bf16")
    assert [k for step, _ in Plan(g).steps for k, _ in step] == ["gemm"]


def test_convolution_output_size_follows_the_reference_formula():
    """compute_output_size (conv.rs:51-73): Same keeps the size, Valid subtracts kernel/2, Full adds kernel/2,
    then the stride divides (rounding down)."""
    for mode, stride, want in [("same", 1, 9), ("same", 2, 4), ("valid", 1, 8), ("valid", 2, 4), ("full", 1, 10), ("full", 3, 3)]:
        g = ha.ir.OpGraph()
        x = g.new_input([1, 9, 9, 8], "f32"); w = g.new_input([4, 3, 3, 8], "f32")
        y = g.conv(x, w, {"in_channels": 8, "out_channels": 4, "kernel_size": [3, 3], "stride": [stride, stride], "padding_mode": mode})
        assert g.descriptor(y)[0] == [1, want, want, 4], (mode, stride)


def test_unsupported_convolutions_fail_with_a_message():
    """What the implicit-GEMM instructions cannot run is refused when the kernel is made, not computed wrongly:
    a filter whose shape contradicts the parameters, a filter type that differs from the image's, and a data
    gradient over a channel count that does not fill 16-byte chunks."""
    g, out = conv_graph("conv", filter_shape=[32, 5, 3, 16])
    with pytest.raises(ha.HeliumError, match="do not match"):
        ha.backend.matmul_kernel(g, [out])
    g = ha.ir.OpGraph()
    x = g.new_input([1, 8, 8, 16], "bf16"); w = g.new_input([8, 3, 3, 16], "f32")
    out = g.conv(x, w, {"in_channels": 16, "out_channels": 8, "kernel_size": [3, 3]})
    with pytest.raises(ha.HeliumError, match="same type"):
        ha.backend.matmul_kernel(g, [out])
    g, out = conv_graph("data", image=(1, 8, 8, 3))
    with pytest.raises(ha.HeliumError, match="16-byte chunks"):
        ha.backend.matmul_kernel(g, [out])
    # (the filter gradient takes any channel count: its image operand is then gathered element by element)
    g, out = conv_graph("filter", image=(1, 8, 8, 3))
    assert "direct=" in ha.backend.matmul_kernel(g, [out]).description
