"""GPU parity tests of anchor-less fusion-IR kernels (pointwise chain + reductions) against the oracle."""
import numpy as np
import pytest

import helium_amd as ha
from helium_amd import configs
from oracle import fusion_ir as oracle

from helpers import run_tile_kernel_gpu

pytestmark = pytest.mark.gpu


def check(graph, inputs, rel=1e-3):
    kernel = ha.TileKernel.auxiliary(graph)
    print(kernel.description, flush=True)
    got = run_tile_kernel_gpu(kernel, inputs)
    want = oracle.outputs(graph.nodes, inputs)
    assert set(got) == set(want)
    for leaf, w in want.items():
        g = got[leaf].astype(np.float64)
        w = w.reshape(-1).astype(np.float64)
        assert np.all(np.abs(g - w) <= rel * np.maximum(np.abs(w), 1e-6)), (leaf, g[:4], w[:4])


@pytest.mark.parametrize("rows,cols,axis", [(64, 128, 2), (100, 72, 2), (33, 260, 1), (512, 4096, 2), (4096, 4096, 2),
                                            (4096, 4096, 1)])
def test_c3_chain_with_both_reductions(gpu, rows, cols, axis):
    g, inputs, _ = configs.c3_chain(rows, cols, bias_axis=axis)
    check(g, inputs)


def test_all_reduction_depths_and_a_full_size_output(gpu):
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(5)
    x = g.producer([3, 50, 36], "bf16"); y = g.producer([3, 50, 36], "f32")
    v = g.binary(g.unary(x, "gelu"), y, "drelu")
    outs = [g.consumer(g.reduction(v, d), "f32") for d in ("rows", "columns", "item", "batch")]
    outs.append(g.consumer(v, "bf16"))
    inputs = {x: configs.bf16_rne(rng.standard_normal((3, 50, 36)).astype(np.float32)),
              y: rng.standard_normal((3, 50, 36)).astype(np.float32)}
    kernel = ha.TileKernel.auxiliary(g)
    got = run_tile_kernel_gpu(kernel, inputs)
    want = oracle.outputs(g.nodes, inputs)
    for leaf in outs[:4]:
        assert np.allclose(got[leaf], want[leaf].reshape(-1), rtol=1e-3, atol=1e-5), leaf
    full = outs[4]
    assert np.all(np.abs(got[full].astype(np.int32) - want[full].reshape(-1).astype(np.int32)) <= 1)


def test_every_fusion_ir_pointwise_op(gpu):
    rng = np.random.default_rng(6)
    for fn, const, lo, hi in [("neg", 0, -2, 2), ("relu", 0, -2, 2), ("gelu", 0, -3, 3), ("tanh", 0, -4, 4),
                              ("exp", 0, -5, 5), ("ln", 0, 0.01, 9), ("sqrt", 0, 0, 9), ("add_constant", 1.5, -2, 2),
                              ("mul_constant", -0.25, -2, 2), ("pow_constant", 2.0, -2, 2), ("pow_constant", 1.5, 0.1, 4)]:
        g = ha.fusion.OpGraph()
        x = g.producer([2, 9, 20], "f32")
        out = g.consumer(g.unary(x, fn, const), "f32")
        inputs = {x: rng.uniform(lo, hi, (2, 9, 20)).astype(np.float32)}
        got = run_tile_kernel_gpu(ha.TileKernel.auxiliary(g), inputs)[out]
        want = oracle.outputs(g.nodes, inputs)[out].reshape(-1)
        from oracle import numerics as nm
        assert nm.ulps_close(got, want, max_ulps=2).all(), fn
    for fn in ("add", "sub", "mul", "div", "pow", "drelu"):
        g = ha.fusion.OpGraph()
        x = g.producer([2, 9, 20], "f32"); y = g.producer([2, 9, 20], "f32")
        out = g.consumer(g.binary(x, y, fn), "f32")
        inputs = {x: rng.uniform(0.1, 3, (2, 9, 20)).astype(np.float32), y: rng.uniform(-2, 2, (2, 9, 20)).astype(np.float32)}
        got = run_tile_kernel_gpu(ha.TileKernel.auxiliary(g), inputs)[out]
        want = oracle.outputs(g.nodes, inputs)[out].reshape(-1)
        from oracle import numerics as nm
        assert nm.ulps_close(got, want, max_ulps=2).all(), fn


def test_transposed_producer_and_broadcast_constant(gpu):
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(7)
    x = g.producer([2, 24, 40], "f32"); y = g.producer([2, 40, 24], "f32")
    k = g.constant([2, 40, 24], 0.5)
    v = g.binary(g.binary(g.transpose(x), y, "mul"), k, "add")
    out = g.consumer(v, "f32")
    inputs = {x: rng.standard_normal((2, 24, 40)).astype(np.float32), y: rng.standard_normal((2, 40, 24)).astype(np.float32)}
    got = run_tile_kernel_gpu(ha.TileKernel.auxiliary(g), inputs)[out]
    want = oracle.outputs(g.nodes, inputs)[out].reshape(-1)
    assert np.array_equal(got, want)


def test_repeated_launches_reuse_the_scratch_and_agree_bit_for_bit(gpu):
    """A short launch combines its blocks' partial sums through scratch memory in block order: the arrival
    counters must be back at zero after every launch, and the sums do not depend on which block finished last."""
    g = ha.fusion.OpGraph()
    rng = np.random.default_rng(21)
    shape = [2, 700, 520]
    x = g.producer(shape, "f32")
    v = g.unary(x, "tanh")
    outs = [g.consumer(g.reduction(v, d), "f32") for d in ("columns", "item", "batch")]
    inputs = {x: rng.standard_normal(shape).astype(np.float32)}
    kernel = ha.TileKernel.auxiliary(g)
    assert "fills=[]" in kernel.description, kernel.description
    want = oracle.outputs(g.nodes, inputs)
    first = run_tile_kernel_gpu(kernel, inputs)
    for leaf in outs:
        assert np.allclose(first[leaf], want[leaf].reshape(-1), rtol=1e-3, atol=1e-4), leaf
    for _ in range(4):
        again = run_tile_kernel_gpu(kernel, inputs)
        for leaf in outs:
            assert np.array_equal(first[leaf], again[leaf]), leaf
