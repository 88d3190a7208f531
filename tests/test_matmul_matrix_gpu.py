"""The reference's GEMM test matrix (helium-kernel-generator/tests/matmul.rs:24-190, `matmul_no_fusion`): every
combination of operand A / operand B / output storage type out of {f32, bf16, f16} under every Precision, through the
MatmulGenerator boundary (he_matmul_kernel_create on the subgraph {Matmul, ChangeDataType}). As there, operands are
uniform in [0, 1), the expectation is the product of the *unrounded* f32 matrices, and the bar is
approx::relative_eq(epsilon 1e-3, max_relative 1e-2) (matmul.rs:140-147). The whole matrix runs at a ragged reduced
size with every element checked; the reference's own 4097^3 runs for one case per multiplicand type and for mixed
operand types, checked on sampled rows and columns."""
import itertools

import numpy as np
import pytest

from oracle import numerics as nm

import gemm_cases
from helpers import run_tile_kernel_gpu

pytestmark = pytest.mark.gpu


def _f32(storage, dtype, shape):
    return nm.from_storage(storage, dtype, shape).astype(np.float64)


def _check(got, want, what):
    d = np.abs(got - want)
    ok = (d <= 1e-3) | (d <= 1e-2 * np.maximum(np.abs(got), np.abs(want)))
    assert ok.all(), (what, int((~ok).sum()), float(d.max()))


@pytest.mark.parametrize("precision", gemm_cases.MATMUL_PRECISIONS)
def test_matmul_no_fusion_every_type_combination(gpu, precision):
    m, n, k = 129, 257, 193
    for dtype_a, dtype_b, out_dtype in itertools.product(gemm_cases.MATMUL_DTYPES, repeat=3):
        g, kernel, host, out = gemm_cases.ir_matmul(m, n, k, dtype_a, dtype_b, precision, out_dtype)
        rng = np.random.default_rng(7)  # the unrounded operands ir_matmul drew
        a, b = rng.random((m, k), dtype=np.float32).astype(np.float64), rng.random((k, n), dtype=np.float32).astype(np.float64)
        got = _f32(run_tile_kernel_gpu(kernel, host)[out], out_dtype, (m, n))
        _check(got, a @ b, (dtype_a, dtype_b, precision, out_dtype, kernel.description))


@pytest.mark.parametrize("dtype_a,dtype_b,precision,out_dtype", [
    ("bf16", "bf16", "bf16_f32", "bf16"), ("f16", "f16", "f16_f32", "f16"), ("f32", "f32", "f32_f32", "f32"),
    ("f32", "bf16", "bf16_f32", "f32"), ("bf16", "f16", "f16_f16", "bf16"), ("f16", "f32", "tf32_f32", "f16")])
def test_matmul_no_fusion_at_the_reference_size(gpu, dtype_a, dtype_b, precision, out_dtype):
    size = 4097
    g, kernel, host, out = gemm_cases.ir_matmul(size, size, size, dtype_a, dtype_b, precision, out_dtype)
    print(kernel.description, flush=True)
    rng = np.random.default_rng(7)
    a, b = rng.random((size, size), dtype=np.float32), rng.random((size, size), dtype=np.float32)
    got = _f32(run_tile_kernel_gpu(kernel, host)[out], out_dtype, (size, size))
    pick = np.unique(np.concatenate([[0, 1, 255, 256, 4095, 4096], np.random.default_rng(8).integers(0, size, 40)]))
    _check(got[pick], a[pick].astype(np.float64) @ b.astype(np.float64), ("rows", kernel.description))
    _check(got[:, pick], a.astype(np.float64) @ b[:, pick].astype(np.float64), ("columns", kernel.description))
