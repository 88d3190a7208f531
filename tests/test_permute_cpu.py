"""CPU-side tests of the permute instruction: oracle vs the reference's golden vectors, plan/stride logic,
and the generated kernel's index arithmetic run on the CPU under AddressSanitizer."""
import json
import os
import re

import numpy as np
import pytest

from oracle import permute as oracle
from helium_amd import PermuteDims
from helium_amd.permute import reference_output_strides

from cpu_emul import run_kernel

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "tensor_ops.json")))


@pytest.mark.parametrize("case", GOLDEN["permute"], ids=lambda c: c["name"])
def test_oracle_matches_reference_vectors(case):
    x = np.array(case["input"], dtype=np.float32).reshape(case["shape"])
    swaps = [tuple(s) for s in case["swaps"]]
    got = oracle.swap_dims_sequence(x, swaps)
    assert got.reshape(-1).tolist() == case["expected"]
    # the transpose form agrees with the sequential form
    perm = oracle.permutation_from_swaps(x.ndim, swaps)
    assert np.array_equal(oracle.permute(x, perm), got)


@pytest.mark.parametrize("case", GOLDEN["permute_strides"], ids=lambda c: c["ref"])
def test_reference_stride_known_answers(case):
    swaps = [tuple(s) for s in case["swaps"]]
    assert oracle.reference_output_strides(case["shape"], swaps) == case["expected"]
    assert reference_output_strides(case["shape"], swaps) == case["expected"]


def test_reference_kernel_walk_is_a_transpose_for_correct_strides():
    rng = np.random.default_rng(1)
    for shape, swaps in [((3, 4), [(0, 1)]), ((2, 3, 4), [(0, 2)]), ((2, 3, 4, 5), [(1, 3)]),
                         ((2, 3, 4, 5), [(3, 2), (2, 1)]), ((2, 3, 4), [(0, 1), (1, 2), (0, 2)])]:
        x = rng.integers(0, 1 << 20, size=shape).astype(np.uint32)
        want = oracle.swap_dims_sequence(x, swaps)
        got = oracle.reference_kernel_walk(x, oracle.correct_output_strides(shape, swaps))
        assert np.array_equal(got, want.reshape(-1)), (shape, swaps)


def test_reference_stride_quirk_is_the_inverse_permutation():
    # NHWC -> NCHW written as swaps (2,3),(1,2) is a 3-cycle: the reference's stride routine yields the
    # layout of the inverse permutation, which is why the kernels here take a permutation instead.
    shape, swaps = (2, 3, 4, 5), [(2, 3), (1, 2)]
    x = np.arange(np.prod(shape), dtype=np.uint32).reshape(shape)
    quirk = oracle.reference_kernel_walk(x, oracle.reference_output_strides(shape, swaps))
    perm = oracle.permutation_from_swaps(4, swaps)
    inverse = tuple(np.argsort(perm))
    assert np.array_equal(quirk, oracle.permute(x, inverse).reshape(-1))
    assert not np.array_equal(quirk, oracle.permute(x, perm).reshape(-1))


def _emulate(shape, perm, dtype, np_dtype):
    p = PermuteDims(shape, dtype, perm=perm)
    desc = p.description
    grid = int(re.search(r"grid=(\d+)", desc).group(1))
    threads = int(re.search(r"threads=(\d+)", desc).group(1))
    rng = np.random.default_rng(abs(hash((shape, perm))) % (1 << 32))
    x = rng.integers(0, np.iinfo(np_dtype).max, size=shape, dtype=np_dtype)
    (got,) = run_kernel(p.source, "permute_dims", grid, threads,
                        [(x, False), (np.empty(p.out_shape, dtype=np_dtype), True)])
    assert np.array_equal(got, oracle.permute(x, perm)), desc
    return desc


EMUL_CASES = [
    # tile variant: vector widths 8/4/2/1, ragged edges, middle dims, 3-cycles
    ((72, 40), (1, 0), "bf16", np.uint16),
    ((24, 130), (1, 0), "bf16", np.uint16),
    ((33, 17), (1, 0), "bf16", np.uint16),
    ((3, 20, 28), (0, 2, 1), "bf16", np.uint16),
    ((2, 12, 3, 16), (0, 3, 1, 2), "bf16", np.uint16),
    ((4, 6, 5, 8), (3, 1, 2, 0), "f32", np.uint32),
    ((70, 36), (1, 0), "f32", np.uint32),
    ((5, 7, 3), (2, 1, 0), "f32", np.uint32),
    # rows / copy variants
    ((5, 7, 24), (1, 0, 2), "bf16", np.uint16),
    ((6, 4, 9), (1, 0, 2), "f32", np.uint32),
    ((10, 12), (0, 1), "bf16", np.uint16),
]


@pytest.mark.parametrize("shape,perm,dtype,np_dtype", EMUL_CASES, ids=lambda v: str(v) if isinstance(v, tuple) else None)
def test_generated_kernel_on_cpu(shape, perm, dtype, np_dtype):
    _emulate(shape, perm, dtype, np_dtype)


def test_plan_collapses_adjacent_dims():
    d = PermuteDims((64, 56, 56, 256), "bf16", perm=(0, 3, 1, 2)).description
    assert "collapsed=[64x3136x256]" in d and "variant=tile" in d and "VA=8 VB=8" in d
    d = PermuteDims((32, 128, 28, 28), "bf16", perm=(0, 2, 3, 1)).description
    assert "collapsed=[32x128x784]" in d
    d = PermuteDims((1, 2, 2, 1), "f32", swaps=[(0, 3)]).description
    assert "variant=copy" in d


def test_invalid_arguments_are_rejected():
    from helium_amd import HeliumError

    with pytest.raises(HeliumError):
        PermuteDims((4, 4), "f32", perm=(0, 0))
    with pytest.raises(HeliumError):
        PermuteDims((4, 4), "bool", perm=(1, 0))
