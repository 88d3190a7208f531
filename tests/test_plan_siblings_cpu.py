"""Kernels that reduce over one index space and share an input merge into one pass over it, also when each writes a
full-size tensor beside its reductions (plan.cpp: the sibling pass after the greedy fusion). Run on the CPU
(tests/cpu_emul.py)."""
import numpy as np
import pytest

import helium_amd as ha
from helium_amd.backend import Plan
from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

from helpers import run_tile_kernel_cpu


def two_gradients(rows, channels, dtype, rng):
    """dy * x and dy - z, each written out and summed per channel: nothing orders the two, both read dy."""
    g = ha.ir.OpGraph()
    inputs = {}

    def inp(values):
        i = g.new_input([rows, channels], dtype)
        inputs[i] = nm.to_storage(np.asarray(values).reshape(rows, channels), dtype)
        return i

    dy, x, z = (inp(rng.standard_normal(rows * channels)) for _ in range(3))
    a = g.binary(dy, x, "mul")
    b = g.binary(dy, g.unary(z, "neg"), "add")
    sa = g.reduce(g.swap_dims(a, 0, 1), "sum", 1)
    sb = g.reduce(g.swap_dims(b, 0, 1), "sum", 1)
    for o in (a, b, sa, sb):
        g.new_output(o)
    return g, inputs


def planned(plan):
    return [i for step, _ in plan.planned_steps() for i in step]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_siblings_with_full_size_outputs_share_one_pass(dtype, monkeypatch):
    monkeypatch.setenv("HELIUM_HIP_REDUCE", "twopass")
    g, inputs = two_gradients(1100, 64, dtype, np.random.default_rng(3))
    g.optimize()
    plan = Plan(g)
    assert [kind for kind, _ in planned(plan)] == ["pointwise"], plan.text
    kernel = plan.kernel(0)
    assert sum(a["is_output"] for a in kernel.args) == 4, kernel.description
    pg = plan.graph()
    origin = {n["id"]: n["origin"] for n in pg.nodes}
    val, _ = oracle_ir.evaluate(g.nodes, inputs)
    by_id = {n["id"]: n for n in g.nodes}
    got = run_tile_kernel_cpu(kernel, {n["id"]: inputs[origin[n["id"]]] for n in pg.nodes if n["node"] == "input"}, "pointwise_kernel")
    assert len(got) == 4
    for node, data in got.items():
        o = origin[node]
        want = np.asarray(val[o], dtype=np.float32).reshape(-1)
        have = nm.from_storage(data, by_id[o]["dtype"], want.shape).reshape(-1)
        if by_id[o].get("op") == "reduce":
            rel = 2e-2 if dtype == "bf16" else 1e-4
            assert np.allclose(have, want, rtol=rel, atol=rel * np.abs(want).max()), (o, have[:4], want[:4])
        else:
            want = nm.from_storage(nm.to_storage(want, by_id[o]["dtype"]), by_id[o]["dtype"], want.shape).reshape(-1)
            assert np.array_equal(have, want), (o, have[:4], want[:4])


def test_the_size_limit_of_zero_merges_kernels_of_reductions_only(monkeypatch):
    monkeypatch.setenv("HELIUM_HIP_SIBLING_MAX", "0")
    g, _ = two_gradients(1100, 64, "f32", np.random.default_rng(4))
    g.optimize()
    assert [kind for kind, _ in planned(Plan(g))] == ["pointwise"] * 2


def test_planned_as_recorded_the_siblings_stay_apart():
    from helium_amd.backend import OPT_REMATERIALIZE, set_option

    g, _ = two_gradients(1100, 64, "f32", np.random.default_rng(5))
    g.optimize()
    set_option(OPT_REMATERIALIZE, 0)
    try:
        assert len(planned(Plan(g))) >= 2
    finally:
        set_option(OPT_REMATERIALIZE, 1)
