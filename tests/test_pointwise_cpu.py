"""CPU-side tests of the pointwise/reduction path: the oracle against the reference's known answers, and every
generated kernel run on the CPU (threads + barriers, AddressSanitizer) against the oracle."""
import numpy as np
import pytest

from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

import pointwise_cases
from helpers import assert_storage_close, reduction_fills, run_tile_kernel_cpu

import helium_amd as ha

CASES = pointwise_cases.all_cases()


@pytest.mark.parametrize("case", [c for c in CASES if c.expected], ids=lambda c: c.name)
def test_oracle_matches_reference_known_answers(case):
    val, desc = oracle_ir.evaluate(case.g.nodes, case.inputs)
    for leaf, want in case.expected.items():
        got = np.asarray(val[leaf], dtype=np.float32).reshape(-1)
        # approx::assert_ulps_eq defaults (epsilon = f32::EPSILON, 4 ulps); the op chain uses epsilon 1e-6
        eps = 1e-6 if case.name == "complex_operation_chain" else np.finfo(np.float32).eps
        assert nm.ulps_close(got, want.reshape(-1), max_ulps=4, epsilon=eps).all(), (case.name, got[:4], want[:4])


@pytest.mark.parametrize("case", CASES, ids=lambda c: c.name)
def test_generated_kernel_on_cpu_matches_oracle(case, monkeypatch):
    for name, value in case.env.items():
        monkeypatch.setenv(name, value)
    # what the reference's fusion rule admits (pointwise.rs:121-186); the generator itself accepts more
    from helium_amd.backend import OPT_REMATERIALIZE, set_option

    has_constant = any(n.get("op") == "constant" for n in case.g.nodes if n["id"] in case.nodes)
    set_option(OPT_REMATERIALIZE, 0)
    try:
        # a Constant is an instruction of its own that the reference's rule never merges (pointwise.rs:181)
        assert ha.kernels.pointwise_supports(case.g, case.nodes) == (case.admitted_by_fusion_rule and not has_constant), case.name
    finally:
        set_option(OPT_REMATERIALIZE, 1)
    # ... and an immediate of the kernel that uses it when values may be computed where they are used; the count of
    # broadcasts and transpositions (pointwise.rs:150-160) is then not applied either: the generator walks them all
    assert ha.kernels.pointwise_supports(case.g, case.nodes), case.name
    kernel = ha.TileKernel.pointwise(case.g, case.nodes)
    assert [a["node"] for a in kernel.args if a["is_output"]] == sorted(case.leaves)
    assert case.describes is None or case.describes in kernel.description, kernel.description
    want = oracle_ir.kernel_outputs(case.g.nodes, case.inputs, case.leaves)
    got = run_tile_kernel_cpu(kernel, case.inputs, "pointwise_kernel", reduction_fills(case.g.nodes, case.leaves))
    by_id = {n["id"]: n for n in case.g.nodes}
    for leaf in case.leaves:
        is_reduce = by_id[leaf].get("op") == "reduce"
        rel = (case.reduce_rel or 1e-5) if is_reduce and by_id[leaf]["fn"] in ("sum", "mean") else None
        assert_storage_close(got[leaf], want[leaf].reshape(-1), by_id[leaf]["dtype"], f"{case.name} leaf {leaf}: {kernel.description}",
                             reduce_rel=rel)
        if leaf in case.expected:
            g32 = nm.from_storage(got[leaf], by_id[leaf]["dtype"], case.expected[leaf].shape)
            assert nm.ulps_close(g32, case.expected[leaf], max_ulps=4, epsilon=1e-6).all()


@pytest.mark.parametrize("case", [c for c in CASES if c.env], ids=lambda c: c.name)
def test_reordered_cases_also_run_in_the_reduce_own_index_space(case):
    """Below 1M elements a SwapDims + Reduce kernel iterates in the Reduce's index space (strided reads, rows folded
    by one wave): the same cases without the override."""
    kernel = ha.TileKernel.pointwise(case.g, case.nodes)
    want = oracle_ir.kernel_outputs(case.g.nodes, case.inputs, case.leaves)
    got = run_tile_kernel_cpu(kernel, case.inputs, "pointwise_kernel", reduction_fills(case.g.nodes, case.leaves))
    for leaf in case.leaves:
        assert_storage_close(got[leaf], want[leaf].reshape(-1), "f32", f"{case.name} leaf {leaf}: {kernel.description}",
                             reduce_rel=case.reduce_rel)
