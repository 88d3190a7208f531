"""GPU parity tests of the backend slice through the C ABI: tensors, plans and execute_graph
(helium/src/backend.rs:40-80, helium/src/cuda.rs:155-260) against the oracle on the same seeded inputs."""
import threading

import numpy as np
import pytest

import helium_amd as ha
from helium_amd import configs
from helium_amd.backend import Plan, Tensor, execute_graph, stats
from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

import test_plan_cpu as plans
from helpers import assert_storage_close

pytestmark = pytest.mark.gpu


def run_graph(g, host_inputs):
    """Uploads, executes, downloads. Returns ({output node: storage array}, plan steps)."""
    by_id = {n["id"]: n for n in g.nodes}
    tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in host_inputs.items()}
    outs = execute_graph(g, tensors)
    return {o: t.to_numpy() for o, t in outs.items()}, Plan(g).steps


def check_against_oracle(g, host_inputs, got, steps, max_ulps=2, rel=1e-3, matmul_rel=None):
    want = oracle_ir.plan_outputs(g.nodes, host_inputs, steps)
    _, desc = oracle_ir.evaluate(g.nodes, host_inputs)
    by_id = {n["id"]: n for n in g.nodes}
    assert sorted(got) == sorted(want)
    for o in want:
        src = by_id[by_id[o]["from"]]
        dtype = desc[o][1]
        if matmul_rel is not None:
            a = nm.from_storage(got[o], dtype, [got[o].size]).astype(np.float64)
            b = nm.from_storage(want[o].reshape(-1), dtype, [want[o].size]).astype(np.float64)
            scale = np.maximum(np.abs(b), np.abs(b).mean())
            assert (np.abs(a - b) <= matmul_rel * scale + 1e-6).all(), (o, np.abs(a - b).max())
        else:
            is_sum = src.get("op") == "reduce" and src["fn"] in ("sum", "mean")
            assert_storage_close(got[o], want[o].reshape(-1), dtype, f"output {o}", max_ulps=max_ulps,
                                 reduce_rel=rel if is_sum else None)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16", "u32", "bool"])
def test_tensor_upload_download_round_trip(gpu, dtype):
    rng = np.random.default_rng(5)
    n = 100_003
    if dtype == "bool":
        host = rng.integers(0, 2**32, (n + 31) // 32, dtype=np.uint32)
    elif dtype == "u32":
        host = rng.integers(0, 2**32, n, dtype=np.uint32)
    elif dtype == "f32":
        host = rng.standard_normal(n).astype(np.float32)
    else:
        host = rng.integers(0, 2**16, n).astype(np.uint16)
    t = Tensor.from_numpy(host, dtype, n)
    assert t.len == n and t.dtype == dtype
    assert np.array_equal(t.to_numpy(), host)


def seeded_inputs(g, seed):
    rng = np.random.default_rng(seed)
    return {n["id"]: nm.to_storage(rng.uniform(-1, 1, n["shape"]).astype(np.float32), n["dtype"])
            for n in g.nodes if n["node"] == "input"}


@pytest.mark.parametrize("make", [plans.linear_layer, plans.second_path_blocks_fusion, plans.constant_is_delayed,
                                  plans.two_reduction_depths], ids=lambda f: f.__name__)
def test_named_plans_execute(gpu, make):
    g, _ = make()
    host = seeded_inputs(g, 7)
    got, steps = run_graph(g, host)
    has_mm = any(n.get("op") == "matmul" for n in g.nodes)
    check_against_oracle(g, host, got, steps, matmul_rel=1e-4 if has_mm else None)


def test_large_swap_chain_runs_as_one_permute_and_is_bit_exact(gpu):
    g, want_plan = plans.large_swaps_chain()
    x = configs.permute_input("C2a")
    got, steps = run_graph(g, {0: x})
    assert steps == want_plan
    (out,) = got.values()
    assert np.array_equal(out.reshape(64, 256, 56, 56), np.transpose(x, (0, 3, 1, 2)))


def live_nodes(nodes):
    """The nodes OpGraph::optimize keeps (helium-ir/src/opgraph.rs:165-191): those an Output node reaches."""
    by_id = {n["id"]: n for n in nodes}
    stack = [n["id"] for n in nodes if n["node"] == "output"]
    seen = set()
    while stack:
        i = stack.pop()
        if i in seen:
            continue
        seen.add(i)
        n = by_id[i]
        stack += [n["from"]] if n["node"] == "output" else list(n.get("inputs", []))
    return [n for n in nodes if n["id"] in seen]


@pytest.mark.parametrize("grouping", ["reference", "default"])
@pytest.mark.parametrize("seed", range(24))
def test_random_graphs_execute(gpu, seed, grouping):
    """Random graphs of 8x8, 1024x1024 and 1100x1100 tensors through plan generation and the executor: steps with several
    instructions on several streams, scoped block reuse, and (from 1,000,000 elements) SwapDims chains that run as
    permute instructions in the middle of a graph. With the reference's grouping rules (and its use of one stream per
    instruction of a step) the plan the library runs must
    be the one the CPU restatement of plan_generation.rs derives, and that plan - not the library's - tells the oracle
    where values are rounded to their storage type."""
    from helium_amd.backend import (OPT_CANCEL_TRANSPOSES, OPT_FOLD_SWAP_INTO_REDUCE, OPT_FUSE_MATMUL_EPILOGUE, OPT_HOIST_BROADCASTS,
                                    OPT_REMATERIALIZE, OPT_STREAM_FAN_OUT, set_option)
    from oracle import plan as oracle_plan

    g = plans.random_graph(seed)
    n = g.nodes[0]["shape"][0]
    if not any(nd["node"] == "output" for nd in g.nodes):
        pytest.skip("graph without outputs")
    nodes = live_nodes(g.nodes)
    g.optimize()
    # large extents: small operands keep a first product well inside f32 (a product of exp'ed values then overflows to
    # infinity on both sides alike)
    rng = np.random.default_rng(seed)
    scale = 1.0 if n == 8 else 1.0 / 32
    host = {nd["id"]: (rng.uniform(-1, 1, nd["shape"]) * scale).astype(np.float32) for nd in nodes if nd["node"] == "input"}
    reference = grouping == "reference"
    set_option(OPT_FUSE_MATMUL_EPILOGUE, 0 if reference else 1)
    set_option(OPT_FOLD_SWAP_INTO_REDUCE, 0 if reference else 1)
    set_option(OPT_REMATERIALIZE, 0 if reference else 1)
    set_option(OPT_CANCEL_TRANSPOSES, 0 if reference else 1)
    set_option(OPT_HOIST_BROADCASTS, 0 if reference else 1)
    # the reference puts every instruction of a step on a stream of its own (cuda.rs:190-221); by default only steps
    # where that pays do
    set_option(OPT_STREAM_FAN_OUT, 2 if reference else 1)
    try:
        got, steps = run_graph(g, host)
        if reference and any(len(instrs) > 1 for instrs, _ in steps):
            assert stats()["streams_used"] > 1
    finally:
        set_option(OPT_STREAM_FAN_OUT, 1)
        set_option(OPT_FUSE_MATMUL_EPILOGUE, 1)
        set_option(OPT_FOLD_SWAP_INTO_REDUCE, 1)
        set_option(OPT_REMATERIALIZE, 1)
        set_option(OPT_CANCEL_TRANSPOSES, 1)
        set_option(OPT_HOIST_BROADCASTS, 1)
    set_option(OPT_HOIST_BROADCASTS, 1)
    if reference:
        want_steps = oracle_plan.generate_plan(nodes)
        assert steps == want_steps
        steps = want_steps
        if n * n > 1_000_000 and any(nd.get("op") == "swap_dims" for nd in nodes):
            assert any(k == "permute" for instrs, _ in steps for k, _ in instrs)
    # chains of exp/tanh over matmuls amplify 1-ulp differences; the bound here is on the whole graph
    want = oracle_ir.plan_outputs(nodes, host, steps)
    _, desc = oracle_ir.evaluate(nodes, host)
    assert sorted(got) == sorted(want)
    for o in want:
        a = nm.from_storage(got[o], desc[o][1], [got[o].size]).astype(np.float64)
        b = nm.from_storage(want[o].reshape(-1), desc[o][1], [want[o].size]).astype(np.float64)
        fin = np.isfinite(b)
        assert np.array_equal(np.isfinite(a), fin), (o, steps)
        assert np.allclose(a[fin], b[fin], rtol=2e-2 if desc[o][1] == "bf16" else 1e-3, atol=1e-5), (o, steps)


def test_random_graphs_cover_concurrent_steps_and_permute_instructions():
    """What the random cases above are there for: plans with several instructions in one step and plans with a permute
    instruction are among them (the plans are generated without a device)."""
    multi = permute = 0
    for seed in range(24):
        g = plans.random_graph(seed)
        g.optimize()
        kinds = [[k for k, _ in instrs] for instrs, _ in Plan(g).steps]
        multi += any(len(k) > 1 for k in kinds)
        permute += any("permute" in k for k in kinds)
    assert multi >= 12 and permute >= 8, (multi, permute)


@pytest.mark.parametrize("fuse", [1, 0], ids=["matmul_takes_its_epilogue", "reference_grouping"])
def test_config1_linear_layer(gpu, fuse):
    from helium_amd.backend import (OPT_CANCEL_TRANSPOSES, OPT_FOLD_SWAP_INTO_REDUCE, OPT_FUSE_MATMUL_EPILOGUE, OPT_HOIST_BROADCASTS,
                                    OPT_REMATERIALIZE, OPT_STREAM_FAN_OUT, set_option)

    g, names = configs.c1_ir_graph()
    host = configs.c1_inputs(names, batched=False)
    options = (OPT_FUSE_MATMUL_EPILOGUE, OPT_FOLD_SWAP_INTO_REDUCE, OPT_REMATERIALIZE, OPT_CANCEL_TRANSPOSES, OPT_HOIST_BROADCASTS)
    for option in options:
        set_option(option, fuse)
    try:
        got, steps = run_graph(g, host)
    finally:
        for option in options:
            set_option(option, 1)
    # (the reference's rule keeps the column sums' SwapDims out of the kernel that broadcasts the bias, pointwise.rs:150-160)
    assert [k for instrs, _ in steps for k, _ in instrs] == (["gemm"] if fuse else ["gemm", "pointwise", "pointwise"])
    val, _ = oracle_ir.evaluate(g.nodes, host)
    y = got[names["y"]].reshape(256, 512).astype(np.float64)
    want = val[names["y"]].astype(np.float64)
    assert (np.abs(y - want) <= 1e-4 * np.maximum(np.abs(want), 1.0)).all()
    cs = got[names["colsum"]].astype(np.float64)
    want_cs = want.sum(axis=0)
    assert (np.abs(cs - want_cs) <= 1e-3 * np.abs(want_cs) + 1e-4).all()


@pytest.mark.parametrize("precision,dtype,rel", [("f32_f32", "f32", 1e-4), ("tf32_f32", "f32", 1e-4),
                                                 ("bf16_f32", "bf16", 1e-2), ("f16_f32", "f16", 1e-2),
                                                 ("f16_f16", "f16", 1e-2), ("bf16_f32", "f32", 1e-2)])
def test_matmul_precisions(gpu, precision, dtype, rel):
    rng = np.random.default_rng(9)
    m, k, n = 384, 520, 264
    g = ha.ir.OpGraph()
    a, b = g.new_input([m, k], dtype), g.new_input([k, n], dtype)
    g.new_output(g.matmul(a, b, precision))
    host = {a: nm.to_storage(rng.uniform(-1, 1, (m, k)).astype(np.float32), dtype),
            b: nm.to_storage(rng.uniform(-1, 1, (k, n)).astype(np.float32), dtype)}
    got, steps = run_graph(g, host)
    check_against_oracle(g, host, got, steps, matmul_rel=rel)


def test_outputs_feed_the_next_graph_and_inputs_stay_intact(gpu):
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (300, 70)).astype(np.float32)
    g1 = ha.ir.OpGraph(); i1 = g1.new_input([300, 70], "f32"); o1 = g1.new_output(g1.unary(i1, "exp"))
    g2 = ha.ir.OpGraph(); i2 = g2.new_input([300, 70], "f32"); o2 = g2.new_output(g2.reduce(g2.unary(i2, "neg"), "sum", 1))
    tx = Tensor.from_numpy(x, "f32")
    mid = execute_graph(g1, {i1: tx})[o1]
    out = execute_graph(g2, {i2: mid})[o2].to_numpy()
    assert np.array_equal(tx.to_numpy(), x.reshape(-1))
    want = -np.exp(x.astype(np.float64)).sum(axis=1)
    assert np.allclose(out, want, rtol=1e-5)


def test_a_step_of_many_small_kernels_fans_out_over_streams(gpu):
    """The executor's own rule (HE_OPT_STREAM_FAN_OUT = 1): sixteen independent kernels over 1 MB each in one step are
    worth the joins and run on several streams; two are not and share one. (Kernels of 65,536 elements or fewer would be
    merged into one launch instead.)"""
    for count, fans in ((16, True), (2, False)):
        g = ha.ir.OpGraph()
        xs = [g.new_input([512, 512], "f32") for _ in range(count)]
        # (two ops per branch that do not fuse across branches: each branch is an instruction of its own)
        outs = [g.new_output(g.unary(g.unary(x, "exp"), "relu")) for x in xs]
        rng = np.random.default_rng(count)
        host = {x: rng.uniform(-1, 1, (512, 512)).astype(np.float32) for x in xs}
        got, steps = run_graph(g, host)
        assert max(len(instrs) for instrs, _ in steps) == count, steps
        assert (stats()["streams_used"] > 1) == fans, stats()
        check_against_oracle(g, host, got, steps)


def test_four_threads_execute_concurrently(gpu):
    # helium/tests/stress_test.rs:16-17: any thread may call execute_graph
    g, names = configs.c1_ir_graph(64, 96, 80)
    host = configs.c1_inputs(names, 64, 96, 80, batched=False)
    ref, _ = run_graph(g, host)
    misses_before = stats()["plan_cache_misses"]
    errors = []

    def worker():
        try:
            for _ in range(20):
                got, _ = run_graph(g, host)
                for o in ref:
                    if o == names["y"]:
                        assert np.array_equal(got[o], ref[o])
                    else:
                        assert np.allclose(got[o], ref[o], rtol=1e-5)
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=worker) for _ in range(4)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors, errors[0]
    s = stats()
    # the plan made by the first execution is reused by all 80 later ones, and freed blocks go round
    assert s["plan_cache_misses"] == misses_before and s["pool_reuses"] > 0


@pytest.mark.parametrize("fold, shape", [(1, [8, 36, 36, 128]), (0, [8, 36, 36, 128]), (1, [16, 48, 48, 128])],
                         ids=["statistics_without_permute", "reference_grouping", "channel_arithmetic_rides_on_the_fold_launch"])
def test_batch_norm_train_step(gpu, fold, shape):
    """BatchNorm2d::forward in Train mode + Relu (helium/src/modules/batch_norm.rs:32-72) above the 1M-element
    SwapDims threshold, planned both ways: with the transposition folded into the statistics kernel and as the
    reference plans it (permute, then two reductions). Above 2M elements (the third case: 4.7M) the statistics fold in a
    second launch, which then also does the per-channel arithmetic behind them."""
    from harness import frontend
    from helium_amd.backend import OPT_FOLD_SWAP_INTO_REDUCE, set_option

    g = ha.ir.OpGraph()
    rec = frontend.Recorder(g)
    x = g.new_input(shape, "bf16")
    params = [g.new_input([shape[3]], "f32") for _ in range(4)]
    y, new_mean, new_var = frontend.batch_norm_train(rec, x, *params)
    for v in (y, new_mean, new_var):
        g.new_output(v)
    rng = np.random.default_rng(77)
    host = {x: nm.to_storage((rng.standard_normal(shape) * 1.5 + 0.3).astype(np.float32), "bf16"),
            params[0]: rng.standard_normal(shape[3]).astype(np.float32),
            params[1]: rng.uniform(0.5, 2.0, shape[3]).astype(np.float32),
            params[2]: rng.uniform(0.5, 1.5, shape[3]).astype(np.float32),
            params[3]: rng.standard_normal(shape[3]).astype(np.float32), **rec.scalars}
    set_option(OPT_FOLD_SWAP_INTO_REDUCE, fold)
    try:
        got, steps = run_graph(g, host)
    finally:
        set_option(OPT_FOLD_SWAP_INTO_REDUCE, 1)
    kinds = [k for instrs, _ in steps for k, _ in instrs]
    assert ("permute" in kinds) == (fold == 0), steps
    if int(np.prod(shape)) > (1 << 21):
        plan = Plan(g)
        assert "carries=" in plan.kernel(0).description, plan.kernel(0).description
        with pytest.raises(ha.HeliumError, match="launches nothing"):
            plan.kernel(1)
    want = oracle_ir.plan_outputs(g.nodes, host, steps)
    _, desc = oracle_ir.evaluate(g.nodes, host)
    for o in want:
        a = nm.from_storage(got[o], desc[o][1], [got[o].size]).astype(np.float64)
        b = nm.from_storage(want[o].reshape(-1), desc[o][1], [want[o].size]).astype(np.float64)
        # statistics: f32 sums of 10k bf16 terms in a different order; y: bf16 output of a chain that divides by
        # sqrt(variance), so one bf16 step of y (2^-8 relative) plus the statistics' error
        tol = 2e-2 if desc[o][1] == "bf16" else 1e-3
        assert np.allclose(a, b, rtol=tol, atol=tol), (o, np.abs(a - b).max())


def test_residual_block_forward(gpu):
    """BasicBlock::forward in Train mode (resnet-train/src/model.rs:155-165) through execute_graph: the first convolution's
    instruction takes its bias and the second batch norm's statistics, the second one its bias and the shortcut add."""
    from harness import frontend

    shape = [4, 12, 10, 64]
    c = shape[3]
    rng = np.random.default_rng(41)
    g = ha.ir.OpGraph()
    rec = frontend.Recorder(g)
    x = g.new_input(shape, "bf16")
    bn1 = [g.new_input([c], "f32") for _ in range(4)]
    bn2 = [g.new_input([c], "f32") for _ in range(4)]
    k1, b1 = g.new_input([c, 3, 3, c], "bf16"), g.new_input([c], "bf16")
    k2, b2 = g.new_input([c, 3, 3, c], "bf16"), g.new_input([c], "bf16")
    out, stats = frontend.basic_block_forward(rec, x, bn1, k1, b1, bn2, k2, b2)
    outs = [g.new_output(out)] + [g.new_output(v) for v in stats]
    host = {x: nm.to_storage((rng.standard_normal(shape) * 1.2 + 0.2).astype(np.float32), "bf16")}
    for bn in (bn1, bn2):
        host.update({bn[0]: rng.standard_normal(c).astype(np.float32), bn[1]: rng.uniform(0.5, 2.0, c).astype(np.float32),
                     bn[2]: rng.uniform(0.5, 1.5, c).astype(np.float32), bn[3]: (rng.standard_normal(c) * 0.5).astype(np.float32)})
    for k, b in ((k1, b1), (k2, b2)):
        host[k] = nm.to_storage((rng.standard_normal((c, 3, 3, c)) * 0.06).astype(np.float32), "bf16")
        host[b] = nm.to_storage((rng.standard_normal(c) * 0.1).astype(np.float32), "bf16")
    host.update(rec.scalars)
    got, steps = run_graph(g, host)
    gemms = [members for instrs, _ in steps for kind, members in instrs if kind == "gemm"]
    by_id = {n["id"]: n for n in g.nodes}
    assert len(gemms) == 2 and sorted(by_id[m]["op"] for m in gemms[0]).count("reduce") == 2, steps
    assert [by_id[m]["op"] for m in gemms[1]].count("binary") == 2, steps   # bias and shortcut
    want = oracle_ir.plan_outputs(g.nodes, host, steps)
    _, desc = oracle_ir.evaluate(g.nodes, host)
    for o in outs:
        a = nm.from_storage(got[o], desc[o][1], [got[o].size]).astype(np.float64)
        b = nm.from_storage(want[o].reshape(-1), desc[o][1], [want[o].size]).astype(np.float64)
        tol = 4e-2 if desc[o][1] == "bf16" else 2e-3
        assert np.allclose(a, b, rtol=tol, atol=tol), (o, np.abs(a - b).max())


@pytest.mark.parametrize("image,oc", [((8, 28, 28, 64), 64), ((4, 30, 26, 32), 128), ((64, 14, 14, 64), 64)])
def test_convolution_takes_the_batch_norm_statistics_of_its_output(gpu, image, oc):
    """conv -> BatchNorm2d(train) -> relu through execute_graph: the convolution's kernel also folds its output per
    channel (mean of y and of y^2, written SwapDims + Reduce), the rest of the batch norm runs as pointwise kernels.
    The last case has batch = channels: the Reduce's input then has the output's own shape."""
    from harness import frontend

    rng = np.random.default_rng(31)
    g = ha.ir.OpGraph()
    rec = frontend.Recorder(g)
    fshape = [oc, 3, 3, image[3]]
    x = g.new_input(list(image), "bf16"); w = g.new_input(fshape, "bf16")
    conv = g.conv(x, w, {"in_channels": image[3], "out_channels": oc, "kernel_size": [3, 3]})
    params = [g.new_input([oc], "f32") for _ in range(4)]
    y, new_mean, new_var = frontend.batch_norm_train(rec, conv, *params)
    for v in (y, new_mean, new_var):
        g.new_output(v)
    host = {x: nm.to_storage(rng.standard_normal(image).astype(np.float32), "bf16"),
            w: nm.to_storage((rng.standard_normal(fshape) * 0.1).astype(np.float32), "bf16"),
            params[0]: rng.standard_normal(oc).astype(np.float32), params[1]: rng.uniform(0.5, 2.0, oc).astype(np.float32),
            params[2]: rng.uniform(0.5, 1.5, oc).astype(np.float32), params[3]: rng.standard_normal(oc).astype(np.float32),
            **rec.scalars}
    got, steps = run_graph(g, host)
    first = steps[0][0]
    assert len(first) == 1 and first[0][0] == "gemm" and len(first[0][1]) == 6, steps
    assert all(k == "pointwise" for instrs, _ in steps[1:] for k, _ in instrs), steps
    want = oracle_ir.plan_outputs(g.nodes, host, steps)
    _, desc = oracle_ir.evaluate(g.nodes, host)
    for o in want:
        a = nm.from_storage(got[o], desc[o][1], [got[o].size]).astype(np.float64)
        b = nm.from_storage(want[o].reshape(-1), desc[o][1], [want[o].size]).astype(np.float64)
        tol = 3e-2 if desc[o][1] == "bf16" else 1e-3
        assert np.allclose(a, b, rtol=tol, atol=tol), (o, np.abs(a - b).max())


@pytest.mark.parametrize("image,oc,kernel,stride,mode,dtype", [
    ((4, 28, 28, 64), 64, (3, 3), (1, 1), "same", "bf16"),     # a resnet block convolution
    ((2, 30, 30, 64), 128, (3, 3), (2, 2), "same", "bf16"),    # the strided first convolution of a stage
    ((2, 30, 30, 64), 128, (1, 1), (2, 2), "same", "bf16"),    # its 1x1 shortcut
    ((2, 33, 31, 3), 32, (7, 7), (2, 2), "same", "bf16"),      # three-channel input
    ((1, 17, 19, 16), 24, (3, 3), (1, 1), "valid", "f32"),
])
def test_convolution_runs_as_an_implicit_gemm(gpu, image, oc, kernel, stride, mode, dtype):
    """Op::Conv (NHWC image, [out, kh, kw, in] filter) through execute_graph: one GEMM instruction whose A operand
    is gathered from the image; parity against the oracle's direct cross-correlation in float64."""
    rng = np.random.default_rng(9)
    g = ha.ir.OpGraph()
    fshape = [oc, kernel[0], kernel[1], image[3]]
    x = g.new_input(list(image), dtype); w = g.new_input(fshape, dtype)
    y = g.conv(x, w, {"in_channels": image[3], "out_channels": oc, "kernel_size": list(kernel), "stride": list(stride),
                      "padding_mode": mode})
    out = g.new_output(g.unary(y, "relu"))
    host = {x: nm.to_storage(rng.uniform(-1, 1, image).astype(np.float32), dtype),
            w: nm.to_storage((rng.uniform(-1, 1, fshape) * 0.2).astype(np.float32), dtype)}
    got, steps = run_graph(g, host)
    assert [k for instrs, _ in steps for k, _ in instrs] == ["gemm"], steps   # the relu runs on the accumulators
    want = oracle_ir.plan_outputs(g.nodes, host, steps)[out]
    a = nm.from_storage(got[out], dtype, [got[out].size]).astype(np.float64)
    b = nm.from_storage(want.reshape(-1), dtype, [want.size]).astype(np.float64)
    tol = 1e-4 if dtype == "f32" else 1e-2
    assert (np.abs(a - b) <= tol * np.maximum(np.abs(b), 1.0)).all(), float(np.abs(a - b).max())


@pytest.mark.parametrize("image,oc,kernel,stride,dtype", [
    ((4, 28, 28, 64), 64, (3, 3), (1, 1), "bf16"),
    ((2, 30, 30, 64), 128, (3, 3), (2, 2), "bf16"),
    ((2, 30, 30, 64), 128, (1, 1), (2, 2), "bf16"),
    ((1, 17, 19, 16), 24, (3, 3), (1, 1), "f32"),
    # classes of pixels that no tap reaches (zeroed by the fill), the last pixel among them
    ((1, 7, 7, 8), 8, (3, 3), (4, 4), "bf16"),
])
def test_convolution_backward_data_runs_as_an_implicit_gemm(gpu, image, oc, kernel, stride, dtype):
    """Op::ConvBackwardData through execute_graph against the oracle's adjoint of the forward convolution, and the
    adjoint identity itself on the device results: <conv(x, w), dy> = <x, conv_backward_data(dy, w)>."""
    rng = np.random.default_rng(12)
    params = {"in_channels": image[3], "out_channels": oc, "kernel_size": list(kernel), "stride": list(stride)}
    out_hw = oracle_ir.conv_output_size(params, image[1:3], kernel)
    flow_shape, fshape = [image[0], out_hw[0], out_hw[1], oc], [oc, kernel[0], kernel[1], image[3]]
    g = ha.ir.OpGraph()
    x = g.new_input(list(image), dtype); dy = g.new_input(flow_shape, dtype); w = g.new_input(fshape, dtype)
    y_out = g.new_output(g.conv(x, w, params))
    dx_out = g.new_output(g.conv_backward_data(dy, w, params, image[1:3]))
    host = {x: nm.to_storage(rng.uniform(-1, 1, image).astype(np.float32), dtype),
            dy: nm.to_storage(rng.uniform(-1, 1, flow_shape).astype(np.float32), dtype),
            w: nm.to_storage((rng.uniform(-1, 1, fshape) * 0.2).astype(np.float32), dtype)}
    got, steps = run_graph(g, host)
    assert sorted(k for instrs, _ in steps for k, _ in instrs) == ["gemm", "gemm"], steps
    want = oracle_ir.plan_outputs(g.nodes, host, steps)
    tol = 1e-4 if dtype == "f32" else 1e-2
    for o in (y_out, dx_out):
        a = nm.from_storage(got[o], dtype, [got[o].size]).astype(np.float64)
        b = nm.from_storage(want[o].reshape(-1), dtype, [want[o].size]).astype(np.float64)
        assert (np.abs(a - b) <= tol * np.maximum(np.abs(b), 1.0)).all(), (o, float(np.abs(a - b).max()))
    y = nm.from_storage(got[y_out], dtype, flow_shape).astype(np.float64)
    dx = nm.from_storage(got[dx_out], dtype, list(image)).astype(np.float64)
    xs = nm.from_storage(host[x], dtype, list(image)).astype(np.float64)
    dys = nm.from_storage(host[dy], dtype, flow_shape).astype(np.float64)
    lhs, rhs = (y * dys).sum(), (xs * dx).sum()
    scale = np.sqrt((y * y).sum() * (dys * dys).sum())
    assert abs(lhs - rhs) <= (1e-5 if dtype == "f32" else 5e-3) * scale, (lhs, rhs, scale)


@pytest.mark.parametrize("image,oc,kernel,stride,dtype", [
    ((8, 28, 28, 64), 64, (3, 3), (1, 1), "bf16"),
    ((4, 30, 30, 64), 128, (3, 3), (2, 2), "bf16"),
    ((4, 30, 30, 64), 128, (1, 1), (2, 2), "bf16"),
    ((2, 17, 19, 16), 24, (3, 3), (1, 1), "f32"),
])
def test_convolution_backward_filter_runs_as_a_split_k_gemm(gpu, image, oc, kernel, stride, dtype):
    """Op::ConvBackwardFilter through execute_graph against the oracle, and the identity that ties it to the
    forward op on the device results: <conv(x, w), dy> = <w, conv_backward_filter(dy, x)>."""
    rng = np.random.default_rng(13)
    params = {"in_channels": image[3], "out_channels": oc, "kernel_size": list(kernel), "stride": list(stride)}
    out_hw = oracle_ir.conv_output_size(params, image[1:3], kernel)
    flow_shape, fshape = [image[0], out_hw[0], out_hw[1], oc], [oc, kernel[0], kernel[1], image[3]]
    g = ha.ir.OpGraph()
    x = g.new_input(list(image), dtype); dy = g.new_input(flow_shape, dtype); w = g.new_input(fshape, dtype)
    y_out = g.new_output(g.conv(x, w, params))
    dw_out = g.new_output(g.conv_backward_filter(dy, x, params))
    host = {x: nm.to_storage(rng.uniform(-1, 1, image).astype(np.float32), dtype),
            dy: nm.to_storage((rng.uniform(-1, 1, flow_shape) * 0.1).astype(np.float32), dtype),
            w: nm.to_storage((rng.uniform(-1, 1, fshape) * 0.2).astype(np.float32), dtype)}
    got, steps = run_graph(g, host)
    assert sorted(k for instrs, _ in steps for k, _ in instrs) == ["gemm", "gemm"], steps
    want = oracle_ir.plan_outputs(g.nodes, host, steps)
    tol = 1e-4 if dtype == "f32" else 1e-2
    for o in (y_out, dw_out):
        a = nm.from_storage(got[o], dtype, [got[o].size]).astype(np.float64)
        b = nm.from_storage(want[o].reshape(-1), dtype, [want[o].size]).astype(np.float64)
        assert (np.abs(a - b) <= tol * np.maximum(np.abs(b), 1.0)).all(), (o, float(np.abs(a - b).max()))
    y = nm.from_storage(got[y_out], dtype, flow_shape).astype(np.float64)
    dw = nm.from_storage(got[dw_out], dtype, fshape).astype(np.float64)
    ws = nm.from_storage(host[w], dtype, fshape).astype(np.float64)
    dys = nm.from_storage(host[dy], dtype, flow_shape).astype(np.float64)
    lhs, rhs = (y * dys).sum(), (ws * dw).sum()
    scale = np.sqrt((y * y).sum() * (dys * dys).sum())
    assert abs(lhs - rhs) <= (1e-5 if dtype == "f32" else 5e-3) * scale, (lhs, rhs, scale)


@pytest.mark.parametrize("dtype,precision", [("f32", "f32_f32"), ("bf16", "bf16_f32")])
def test_linear_layer_backward_products(gpu, dtype, precision):
    """dW = x^T dy and dX = dy w^T through execute_graph: two GEMM instructions that read the untransposed
    operands, no permute and no pointwise transposition in the plan."""
    g, n = plans.linear_backward_graph(512, 384, 640, dtype, precision)
    rng = np.random.default_rng(15)
    host = {n["x"]: nm.to_storage(rng.uniform(-1, 1, (512, 384)).astype(np.float32), dtype),
            n["w"]: nm.to_storage(rng.uniform(-1, 1, (384, 640)).astype(np.float32), dtype),
            n["dy"]: nm.to_storage(rng.uniform(-1, 1, (512, 640)).astype(np.float32), dtype)}
    got, steps = run_graph(g, host)
    assert sorted(k for instrs, _ in steps for k, _ in instrs) == ["gemm", "gemm"], steps
    check_against_oracle(g, host, got, steps, matmul_rel=1e-4 if dtype == "f32" else 1e-2)
