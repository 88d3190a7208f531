"""GPU parity tests of the fused GEMM through the C ABI against the oracle (f32-accumulated reference on the
rounded operands). Tolerance: approx::relative_eq(epsilon 1e-3, max_relative 1e-2), the reference's own
(helium-kernel-generator/tests/matmul.rs:140-147); reductions 1e-3 relative."""
import numpy as np
import pytest

import helium_amd as ha
from oracle import fusion_ir as oracle
from oracle import numerics as nm

import gemm_cases
from helpers import run_tile_kernel_gpu

pytestmark = pytest.mark.gpu


def check(g, inputs, outs, mma="bf16", rel=1e-2, eps=1e-3):
    k = ha.TileKernel.fused(g)
    print(k.description, flush=True)
    got = run_tile_kernel_gpu(k, inputs)
    want = oracle.outputs(g.nodes, inputs, round_mainloop_to=mma)
    assert sorted(got) == sorted(outs)
    dt = {a["node"]: a["dtype"] for a in k.args if a["is_output"]}
    for node in outs:
        gv, wv = got[node], want[node].reshape(-1)
        if dt[node] == "bf16":
            gv, wv = nm.bf16_bits_to_f32(gv), nm.bf16_bits_to_f32(wv)
        gv, wv = gv.astype(np.float64), wv.astype(np.float64)
        ok = (np.abs(gv - wv) <= eps) | (np.abs(gv - wv) <= rel * np.maximum(np.abs(gv), np.abs(wv)))
        assert ok.all(), (node, float(np.abs(gv - wv).max()), k.description)
    return k


@pytest.mark.parametrize("m,n,k,batch", [(256, 256, 64, 1), (512, 768, 320, 1), (100, 100, 100, 1), (3, 3, 3, 1),
                                         (300, 520, 136, 3), (1024, 1024, 1024, 1), (257, 263, 129, 2)])
def test_plain_gemm(gpu, m, n, k, batch):
    g, inputs, outs = gemm_cases.plain(m, n, k, batch=batch, seed=m + n)
    check(g, inputs, outs)


def test_reference_small_cases(gpu):
    # helium/tests/tensor_ops.rs:190-212: [[1,2],[3,4]]^2 = [7,10,15,22] in bf16
    g = ha.fusion.OpGraph()
    a = g.producer([1, 2, 2], "bf16"); b = g.producer([1, 2, 2], "bf16")
    out = g.consumer(g.matmul(a, b), "f32")
    x = ha.configs.bf16_rne(np.array([1, 2, 3, 4], dtype=np.float32))
    got = run_tile_kernel_gpu(ha.TileKernel.fused(g), {a: x, b: x})[out]
    assert got.tolist() == [7.0, 10.0, 15.0, 22.0]
    # tensor_ops.rs:250-318: batched 2 x [3,2]x[2,3] (the test multiplies the transposes)
    g = ha.fusion.OpGraph()
    a = g.producer([2, 3, 2], "bf16"); b = g.producer([2, 2, 3], "bf16")
    out = g.consumer(g.matmul(a, b), "f32")
    A = np.arange(1, 13, dtype=np.float32).reshape(2, 2, 3).transpose(0, 2, 1)
    B = np.arange(1, 13, dtype=np.float32).reshape(2, 3, 2).transpose(0, 2, 1)
    got = run_tile_kernel_gpu(ha.TileKernel.fused(g), {a: ha.configs.bf16_rne(A), b: ha.configs.bf16_rne(B)})[out]
    want = [9, 19, 29, 12, 26, 40, 15, 33, 51, 129, 163, 197, 144, 182, 220, 159, 201, 243]
    assert got.tolist() == [float(v) for v in want]


def test_f16_and_f32_operands(gpu):
    g, inputs, outs = gemm_cases.plain(192, 200, 136, dtype="f16")
    check(g, inputs, outs, mma="f16")
    # all-f32 sources multiply as f32: 1e-4 relative
    g, inputs, outs = gemm_cases.plain(192, 200, 136, dtype="f32")
    check(g, inputs, outs, mma=None, rel=1e-4, eps=1e-5)


def test_config1_linear_layer_as_one_fusion(gpu):
    from helium_amd import configs

    g, names = configs.c1_graph()
    k = check(g, configs.c1_inputs(names), [names["y"], names["colsum"]], mma=None, rel=1e-4, eps=1e-4)
    assert "mma=f32" in k.description


@pytest.mark.parametrize("mainloop", [False, True])
@pytest.mark.parametrize("bias_axis", [1, 2])
def test_bias_relu_epilogue_with_column_sums(gpu, mainloop, bias_axis):
    g, inputs, outs = gemm_cases.bias_relu_colsum(520, 392, 264, batch=2, mainloop=mainloop, bias_axis=bias_axis)
    check(g, inputs, outs)


def test_all_reduction_depths(gpu):
    g, inputs, outs = gemm_cases.all_reductions(300, 264, 136)
    check(g, inputs, outs)


def test_reference_test_shape_4097_cubed_is_predicated(gpu):
    # The reference's GEMM test multiplies 4097^3 matrices (helium-kernel-generator/tests/matmul.rs:165-166); a
    # thinner problem with the same ragged edges in every dim keeps the CPU oracle fast.
    g, inputs, outs = gemm_cases.plain(4097, 513, 257, seed=9)
    check(g, inputs, outs)


def test_4096_cubed_plain(gpu):
    g, inputs, outs = gemm_cases.plain(4096, 4096, 4096, seed=3, scale=0.02)
    check(g, inputs, outs, eps=1e-4)


def check_reductions_and_full(g, inputs, rel_full=1e-2, rel_red=1e-3):
    k = ha.TileKernel.fused(g)
    print(k.description, flush=True)
    got = run_tile_kernel_gpu(k, inputs)
    want = oracle.outputs(g.nodes, inputs, round_mainloop_to="bf16")
    for a in k.args:
        if not a["is_output"]:
            continue
        gv, wv = got[a["node"]], want[a["node"]].reshape(-1)
        if a["dtype"] == "bf16":
            gv, wv = nm.bf16_bits_to_f32(gv).astype(np.float64), nm.bf16_bits_to_f32(wv).astype(np.float64)
            ok = (np.abs(gv - wv) <= 1e-3) | (np.abs(gv - wv) <= rel_full * np.maximum(np.abs(gv), np.abs(wv)))
            assert ok.all(), (a["node"], float(np.abs(gv - wv).max()))
        else:
            gv, wv = gv.astype(np.float64), wv.astype(np.float64)
            assert np.abs(gv - wv).max() <= rel_red * np.abs(wv).max(), (a["node"], float(np.abs(gv - wv).max()), float(np.abs(wv).max()))


@pytest.mark.parametrize("size,mainloop,full", [(256, False, False), (384, True, True), (1024, True, True), (4096, False, False),
                                                (4096, True, True)])
def test_c4_readme_fusion(gpu, size, mainloop, full):
    from helium_amd import configs

    g, outs = configs.c4_graph(size, mainloop=mainloop, full_size_outputs=full)
    check_reductions_and_full(g, configs.c4_inputs(g, size))


@pytest.mark.parametrize("size", [384, 4096])
def test_c4_with_biases_along_the_rows(gpu, size):
    """The headline configuration words its biases [1,4096,1]: broadcast along the columns, their gradients sums over
    each row (the README's own listing has them [1,1,4096])."""
    from helium_amd import configs

    g, outs = configs.c4_graph(size, bias_rows=True)
    check_reductions_and_full(g, configs.c4_inputs(g, size))


@pytest.mark.parametrize("size", [512, 4096])
def test_c5a_mainloop_and_epilogue(gpu, size):
    from helium_amd import configs

    g, names = configs.c5a_graph(size)
    check_reductions_and_full(g, configs.c5a_inputs(names, size))


@pytest.mark.parametrize("m,n,k,batch,scaled", [(256, 256, 128, 1, False), (512, 768, 320, 1, False), (100, 100, 100, 2, False),
                                                (257, 263, 129, 1, True), (1024, 1024, 1024, 1, True), (4096, 4096, 512, 1, False)])
def test_b_operand_stored_transposed(gpu, m, n, k, batch, scaled):
    """C = A * Bt^T with Bt stored [n][k]: the B tile is staged and read like A's (chunks along k), straight from
    global memory into LDS when Bt is used as it is, through registers when a mainloop op works on it first."""
    g, inputs, outs = gemm_cases.transposed_b(m, n, k, batch=batch, scaled=scaled)
    kernel = check(g, inputs, outs)
    assert "NVB=8" in kernel.description or k % 8, kernel.description


def test_b_operand_stored_transposed_f32(gpu):
    g, inputs, outs = gemm_cases.transposed_b(192, 200, 136, dtype="f32")
    check(g, inputs, outs, mma=None, rel=1e-4, eps=1e-5)


@pytest.mark.parametrize("m,n,k,batch,both", [(256, 256, 128, 1, False), (512, 768, 320, 1, False), (100, 100, 100, 2, False),
                                              (257, 263, 129, 1, True), (1024, 1024, 1024, 1, True), (4096, 4096, 512, 1, False)])
def test_a_operand_stored_transposed(gpu, m, n, k, batch, both):
    """C = At^T * B with At stored [k][m]: the A tile is staged and read like a [k][n] B tile (chunks along m,
    transposing LDS reads); with `both`, B is stored [n][k] as well (the TT product)."""
    g, inputs, outs = gemm_cases.transposed_a(m, n, k, batch=batch, both=both)
    check(g, inputs, outs)


def test_a_operand_stored_transposed_f32(gpu):
    g, inputs, outs = gemm_cases.transposed_a(192, 200, 136, dtype="f32")
    check(g, inputs, outs, mma=None, rel=1e-4, eps=1e-5)
