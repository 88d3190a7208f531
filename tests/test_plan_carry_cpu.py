"""A small pointwise instruction that reads the column reductions of a large one rides on the launch that folds them
(plan.cpp: Instr::carry, emit.cpp: the fold launch evaluates the carried program once per column). The plan keeps both
instructions; the large one's kernel takes the small one's tensors as arguments. Run on the CPU (tests/cpu_emul.py)."""
import numpy as np
import pytest

import helium_amd as ha
from helium_amd.backend import Plan
from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

from helpers import assert_storage_close, broadcast_to, run_tile_kernel_cpu, scalar_tensor


def batch_norm_like(rows, channels, dtype, rng):
    """Per-channel sums of x and x*x (written as SwapDims + Reduce), the per-channel arithmetic behind them, and the
    pass that applies it: three instructions."""
    g = ha.ir.OpGraph()
    inputs = {}

    def inp(shape, dt, values):
        i = g.new_input(list(shape), dt)
        inputs[i] = nm.to_storage(np.asarray(values).reshape(shape), dt)
        return i

    x = inp([rows, channels], dtype, rng.standard_normal(rows * channels))
    gamma = inp([channels, 1], "f32", rng.uniform(0.5, 2.0, channels))
    xt = g.swap_dims(x, 0, 1)
    s1 = g.reduce(xt, "sum", 1)
    s2 = g.reduce(g.binary(xt, xt, "mul"), "sum", 1)

    def scalar(value):
        b, s, host = scalar_tensor(g, value, [channels, 1])
        inputs[s] = host
        return b

    mean = g.binary(s1, scalar(1.0 / rows), "mul")
    ex2 = g.binary(s2, scalar(1.0 / rows), "mul")
    var = g.binary(ex2, g.unary(g.binary(mean, mean, "mul"), "neg"), "add")
    inv = g.unary(g.unary(g.binary(var, scalar(1e-3), "add"), "sqrt"), "recip")
    scale = g.binary(gamma, inv, "mul")
    shift = g.unary(g.binary(mean, scale, "mul"), "neg")
    y = g.binary(g.binary(x, broadcast_to(g, g.reshape(scale, [channels]), [channels], [rows, channels]), "mul"),
                 broadcast_to(g, g.reshape(shift, [channels]), [channels], [rows, channels]), "add")
    g.new_output(y)
    g.new_output(mean)
    return g, inputs, dict(s1=s1, s2=s2, mean=mean, scale=scale, shift=shift, y=y)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_per_channel_arithmetic_rides_on_the_fold_launch(dtype, monkeypatch):
    monkeypatch.setenv("HELIUM_HIP_FOLD_COLUMNS_MIN", "0")   # reorder the reductions at a size the emulation can afford
    monkeypatch.setenv("HELIUM_HIP_REDUCE", "twopass")       # ... and fold them in a second launch, as large kernels do
    rng = np.random.default_rng(77)
    g, inputs, names = batch_norm_like(600, 72, dtype, rng)
    g.optimize()
    plan = Plan(g)
    instrs = [i for step, _ in plan.planned_steps() for i in step]
    assert [kind for kind, _ in instrs] == ["pointwise"] * 3, plan.text
    pg = plan.graph()
    origin = {n["id"]: n["origin"] for n in pg.nodes}
    large = plan.kernel(0)
    assert "carries=" in large.description, large.description
    with pytest.raises(ha.HeliumError, match="launches nothing"):
        plan.kernel(1)
    # the large kernel's arguments: its own, then what the small instruction reads from elsewhere and writes
    out_nodes = [origin[a["node"]] for a in large.args if a["is_output"]]
    assert names["s1"] in out_nodes and names["s2"] in out_nodes and names["mean"] in out_nodes and len(out_nodes) >= 4, (out_nodes, names)
    val, _ = oracle_ir.evaluate(g.nodes, inputs)
    by_id = {n["id"]: n for n in g.nodes}
    planned_inputs = {n["id"]: inputs[origin[n["id"]]] for n in pg.nodes if n["node"] == "input"}
    got = run_tile_kernel_cpu(large, planned_inputs, "pointwise_kernel")
    assert len(got) == len(out_nodes)
    for node, data in got.items():
        o = origin[node]
        want = np.asarray(val[o], dtype=np.float32).reshape(-1)
        is_sum = by_id[o].get("op") == "reduce"
        rel = 2e-2 if dtype == "bf16" else 1e-4
        g32 = nm.from_storage(data, by_id[o]["dtype"], want.shape).reshape(-1)
        assert np.allclose(g32, want, rtol=rel, atol=rel * np.abs(want).max()), (o, is_sum, g32[:4], want[:4])


def test_without_the_option_every_instruction_launches_for_itself(monkeypatch):
    from helium_amd.backend import OPT_REMATERIALIZE, set_option

    monkeypatch.setenv("HELIUM_HIP_FOLD_COLUMNS_MIN", "0")
    monkeypatch.setenv("HELIUM_HIP_REDUCE", "twopass")
    g, inputs, names = batch_norm_like(600, 72, "f32", np.random.default_rng(5))
    g.optimize()
    set_option(OPT_REMATERIALIZE, 0)
    try:
        plan = Plan(g)
        n = sum(len(step) for step, _ in plan.planned_steps())
        for i in range(n):
            try:
                assert "carries=" not in plan.kernel(i).description
            except ha.HeliumError as e:
                assert "permute" in str(e)
    finally:
        set_option(OPT_REMATERIALIZE, 1)


def product_with_statistics(rows, inner, channels, rng):
    """y = x w with the per-channel sums of y and y*y in the product's epilogue, the arithmetic behind them, and the pass
    that applies it."""
    g = ha.ir.OpGraph()
    inputs = {}

    def inp(shape, dt, values):
        i = g.new_input(list(shape), dt)
        inputs[i] = nm.to_storage(np.asarray(values).reshape(shape), dt)
        return i

    x = inp([rows, inner], "f32", rng.standard_normal(rows * inner) * 0.5)
    w = inp([inner, channels], "f32", rng.standard_normal(inner * channels) * 0.2)
    gamma = inp([channels, 1], "f32", rng.uniform(0.5, 2.0, channels))
    y = g.matmul(x, w, "f32_f32")
    yt = g.swap_dims(y, 0, 1)
    s1 = g.reduce(yt, "sum", 1)
    s2 = g.reduce(g.binary(yt, yt, "mul"), "sum", 1)

    def scalar(value):
        b, s, host = scalar_tensor(g, value, [channels, 1])
        inputs[s] = host
        return b

    mean = g.binary(s1, scalar(1.0 / rows), "mul")
    ex2 = g.binary(s2, scalar(1.0 / rows), "mul")
    var = g.binary(ex2, g.unary(g.binary(mean, mean, "mul"), "neg"), "add")
    inv = g.unary(g.unary(g.binary(var, scalar(1e-3), "add"), "sqrt"), "recip")
    scale = g.binary(gamma, inv, "mul")
    z = g.binary(y, broadcast_to(g, g.reshape(scale, [channels]), [channels], [rows, channels]), "mul")
    g.new_output(z)
    g.new_output(mean)
    return g, inputs, dict(y=y, s1=s1, s2=s2, mean=mean)


def test_per_channel_arithmetic_rides_on_a_products_fold_launch():
    import test_gemm_cpu as gemm

    rng = np.random.default_rng(3)
    g, inputs, names = product_with_statistics(300, 64, 72, rng)
    g.optimize()
    plan = Plan(g)
    instrs = [i for step, _ in plan.planned_steps() for i in step]
    assert [kind for kind, _ in instrs] == ["gemm", "pointwise", "pointwise"], plan.text
    pg = plan.graph()
    origin = {n["id"]: n["origin"] for n in pg.nodes}
    k = plan.kernel(0)
    assert k.description.startswith("gemm") and "carries=" in k.description and "reduce_counters=0" in k.description, k.description
    with pytest.raises(ha.HeliumError, match="launches nothing"):
        plan.kernel(1)
    planned_inputs = {n["id"]: inputs[origin[n["id"]]] for n in pg.nodes if n["node"] == "input"}
    got = gemm._run_one_product(k, planned_inputs)
    val, _ = oracle_ir.evaluate(g.nodes, inputs)
    by_id = {n["id"]: n for n in g.nodes}
    seen = {origin[node] for node in got}
    assert {names["y"], names["s1"], names["s2"], names["mean"]} <= seen and len(seen) >= 5, (seen, names)
    for node, data in got.items():
        o = origin[node]
        want = np.asarray(val[o], dtype=np.float32).reshape(-1)
        g32 = nm.from_storage(data, by_id[o]["dtype"], want.shape).reshape(-1)
        assert np.allclose(g32, want, rtol=1e-4, atol=1e-4 * np.abs(want).max()), (o, g32[:4], want[:4])
