"""Anchor-less fusion-IR kernels run on the CPU (threads + barriers, AddressSanitizer) against the oracle, with
shapes that spread every kind of reduction over several blocks: the partial results then meet in the kernel's
scratch and the block that arrives last writes the output."""
import re

import numpy as np
import pytest

import helium_amd as ha
from helium_amd import configs
from oracle import fusion_ir as oracle

from helpers import run_tile_kernel_cpu


def all_reductions_graph(shape, seed):
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(seed)
    x = g.producer(shape, "bf16"); y = g.producer(shape, "f32")
    v = g.binary(g.unary(x, "gelu"), y, "drelu")
    outs = [g.consumer(g.reduction(v, d), "f32") for d in ("rows", "columns", "item", "batch")]
    outs.append(g.consumer(v, "bf16"))
    inputs = {x: configs.bf16_rne(rng.standard_normal(shape).astype(np.float32)),
              y: rng.standard_normal(shape).astype(np.float32)}
    return g, inputs, outs


@pytest.mark.parametrize("shape", [(3, 50, 36), (2, 300, 200), (1, 1100, 24), (4, 7, 1300)])
def test_all_reduction_depths_across_blocks(shape):
    g, inputs, outs = all_reductions_graph(list(shape), 5)
    kernel = ha.TileKernel.auxiliary(g)
    got = run_tile_kernel_cpu(kernel, inputs, "fused_auxiliary")
    want = oracle.outputs(g.nodes, inputs)
    for leaf in outs[:4]:
        assert np.allclose(got[leaf], want[leaf].reshape(-1), rtol=1e-3, atol=1e-4), (leaf, kernel.description)
    full = outs[4]
    assert np.all(np.abs(got[full].astype(np.int32) - want[full].reshape(-1).astype(np.int32)) <= 1)


@pytest.mark.parametrize("mode", ["ticket", "twopass"])
def test_both_ways_of_combining_blocks(monkeypatch, mode):
    """Short launches fold the blocks' partials in the block that arrives last (tickets), long ones in a second
    small launch; the override picks either for a shape the emulation can afford. Neither needs a pre-filled
    output."""
    monkeypatch.setenv("HELIUM_HIP_REDUCE", mode)
    g, inputs, outs = all_reductions_graph([2, 200, 200], 9)
    kernel = ha.TileKernel.auxiliary(g)
    assert "fills=[]" in kernel.description
    assert ("finalize_grid=0" in kernel.description) == (mode == "ticket"), kernel.description
    got = run_tile_kernel_cpu(kernel, inputs, "fused_auxiliary")
    want = oracle.outputs(g.nodes, inputs)
    for leaf in outs[:4]:
        assert np.allclose(got[leaf], want[leaf].reshape(-1), rtol=1e-3, atol=1e-4), (leaf, kernel.description)


def test_scratch_is_used_when_blocks_share_an_output():
    g, _, _ = all_reductions_graph([2, 300, 200], 5)
    d = ha.TileKernel.auxiliary(g).description
    floats, counters = map(int, re.search(r"ws_floats=(\d+) ws_counters=(\d+)", d).groups())
    assert floats > 0 and counters > 0, d


@pytest.mark.parametrize("rows,cols,axis", [(100, 72, 2), (33, 260, 1), (600, 256, 2)])
def test_c3_chain_on_cpu(rows, cols, axis):
    g, inputs, _ = configs.c3_chain(rows, cols, bias_axis=axis)
    kernel = ha.TileKernel.auxiliary(g)
    got = run_tile_kernel_cpu(kernel, inputs, "fused_auxiliary")
    want = oracle.outputs(g.nodes, inputs)
    assert set(got) == set(want)
    for leaf, w in want.items():
        a = got[leaf].astype(np.float64)
        w = w.reshape(-1).astype(np.float64)
        assert np.all(np.abs(a - w) <= 1e-3 * np.maximum(np.abs(w), 1e-6)), (leaf, kernel.description)
