"""GPU parity tests of the pointwise/reduction instruction through the C ABI, against the oracle."""
import numpy as np
import pytest

from oracle import helium_ir as oracle_ir
from oracle import numerics as nm

import pointwise_cases
from helpers import assert_storage_close, run_tile_kernel_gpu

import helium_amd as ha

pytestmark = pytest.mark.gpu
CASES = pointwise_cases.all_cases()


@pytest.mark.parametrize("case", CASES, ids=lambda c: c.name)
def test_kernel_matches_oracle(gpu, case):
    kernel = ha.TileKernel.pointwise(case.g, case.nodes)
    print(f"{case.name}: {kernel.description}", flush=True)
    want = oracle_ir.kernel_outputs(case.g.nodes, case.inputs, case.leaves)
    got = run_tile_kernel_gpu(kernel, case.inputs)
    by_id = {n["id"]: n for n in case.g.nodes}
    for leaf in case.leaves:
        is_sum = by_id[leaf].get("op") == "reduce" and by_id[leaf]["fn"] in ("sum", "mean")
        # elementwise: 2 ulp in f32 (approx::assert_ulps_eq form); sums: 1e-3 relative
        assert_storage_close(got[leaf], want[leaf].reshape(-1), by_id[leaf]["dtype"], f"{case.name} leaf {leaf}",
                             max_ulps=2, reduce_rel=1e-3 if is_sum else None)
        if leaf in case.expected:
            g32 = nm.from_storage(got[leaf], by_id[leaf]["dtype"], case.expected[leaf].shape)
            assert nm.ulps_close(g32, case.expected[leaf], max_ulps=4, epsilon=1e-6).all()


def test_kernel_can_be_relaunched_with_fresh_reduction_outputs(gpu):
    # the launch re-initialises reduction outputs itself, so a second run must not accumulate onto the first
    case = next(c for c in CASES if c.name == "reduce_large_all")
    kernel = ha.TileKernel.pointwise(case.g, case.nodes)
    a = run_tile_kernel_gpu(kernel, case.inputs)
    b = run_tile_kernel_gpu(kernel, case.inputs)
    leaf = case.leaves[0]
    assert a[leaf][0] == b[leaf][0] == np.float32(300000.0)
