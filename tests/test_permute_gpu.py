"""GPU parity tests of the permute instruction through the C ABI: bit-exact against the numpy oracle."""
import json
import os

import numpy as np
import pytest

from oracle import permute as oracle
from helium_amd import DeviceBuffer, PermuteDims

pytestmark = pytest.mark.gpu
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "tensor_ops.json")))


def run(shape, dtype, np_dtype, perm=None, swaps=None, x=None, seed=0):
    rng = np.random.default_rng(seed)
    if x is None:
        x = rng.integers(0, np.iinfo(np_dtype).max, size=shape, dtype=np_dtype, endpoint=True)
    p = PermuteDims(shape, dtype, perm=perm, swaps=swaps)
    print(f"permute {shape} {dtype} perm={p.perm}: {p.description}", flush=True)
    src = DeviceBuffer.from_numpy(x)
    dst = DeviceBuffer(x.nbytes)
    dst.fill_u8(0xEE)
    p.execute(src, dst)
    return x, dst.to_numpy(np_dtype, p.out_shape), p


@pytest.mark.parametrize("case", GOLDEN["permute"], ids=lambda c: c["name"])
def test_reference_vectors(gpu, case):
    x = np.array(case["input"], dtype=np.float32).reshape(case["shape"])
    _, got, _ = run(tuple(case["shape"]), "f32", np.uint32, swaps=[tuple(s) for s in case["swaps"]],
                    x=x.view(np.uint32))
    assert got.view(np.float32).reshape(-1).tolist() == case["expected"]


BASELINE_CASES = [
    ("C2a_nhwc_to_nchw", (64, 56, 56, 256), (0, 3, 1, 2)),
    ("C2b_transpose_4096", (4096, 4096), (1, 0)),
    ("C2c_perm_0231", (32, 128, 28, 28), (0, 2, 3, 1)),
]


@pytest.mark.parametrize("name,shape,perm", BASELINE_CASES, ids=[c[0] for c in BASELINE_CASES])
def test_baseline_configs_bit_exact(gpu, name, shape, perm):
    # bf16 values are N(0,1) rounded to nearest even, as the benchmark uses; compared as bit patterns.
    rng = np.random.default_rng(20)
    f = rng.standard_normal(size=shape, dtype=np.float32).view(np.uint32)
    bf16 = ((f + 0x7FFF + ((f >> 16) & 1)) >> 16).astype(np.uint16)
    x, got, p = run(shape, "bf16", np.uint16, perm=perm, x=bf16)
    assert np.array_equal(got, oracle.permute(x, perm))
    # size-independent property: permuting back with the inverse permutation restores the input
    inv = tuple(int(i) for i in np.argsort(perm))
    back = PermuteDims(p.out_shape, "bf16", perm=inv)
    a, b = DeviceBuffer.from_numpy(got), DeviceBuffer(x.nbytes)
    back.execute(a, b)
    assert np.array_equal(b.to_numpy(np.uint16, shape), x)


def test_resnet_style_swaps_nhwc_to_nchw(gpu):
    # written as the reference's model does: swap_dims(2,3) then swap_dims(1,2) (resnet-train/src/model.rs:79-80)
    shape, swaps = (8, 14, 14, 96), [(2, 3), (1, 2)]
    x, got, _ = run(shape, "bf16", np.uint16, swaps=swaps, seed=3)
    assert np.array_equal(got, oracle.swap_dims_sequence(x, swaps))


RAGGED = [
    ((1000, 1003), (1, 0), "bf16", np.uint16),
    ((129, 257), (1, 0), "f32", np.uint32),
    ((7, 130, 66), (0, 2, 1), "bf16", np.uint16),
    ((3, 5, 300, 12), (3, 1, 2, 0), "f32", np.uint32),
    ((2048, 16, 16, 32), (3, 1, 2, 0), "f32", np.uint32),  # the reference benchmark's swap(0,3), scaled down
    ((6, 50, 70, 24), (2, 0, 1, 3), "bf16", np.uint16),    # rows variant
    ((16, 3, 224, 224), (0, 2, 3, 1), "bf16", np.uint16),  # NCHW -> NHWC with 3 channels
    ((16, 224, 224, 3), (0, 3, 1, 2), "f32", np.uint32),
    ((5, 1, 9, 1), (3, 2, 1, 0), "bf16", np.uint16),
    ((1, 1), (1, 0), "f32", np.uint32),
]


@pytest.mark.parametrize("shape,perm,dtype,np_dtype", RAGGED, ids=lambda v: str(v) if isinstance(v, tuple) else None)
def test_ragged_and_odd_shapes(gpu, shape, perm, dtype, np_dtype):
    x, got, _ = run(shape, dtype, np_dtype, perm=perm, seed=len(shape))
    assert np.array_equal(got, oracle.permute(x, perm))


def test_f16_and_u32_take_the_same_path(gpu):
    x, got, _ = run((33, 65), "f16", np.uint16, perm=(1, 0))
    assert np.array_equal(got, oracle.permute(x, (1, 0)))
    x, got, _ = run((33, 65), "u32", np.uint32, perm=(1, 0))
    assert np.array_equal(got, oracle.permute(x, (1, 0)))


def test_empty_tensor_is_a_no_op(gpu):
    p = PermuteDims((0, 5), "f32", perm=(1, 0))
    p.execute(DeviceBuffer(16), DeviceBuffer(16))


def test_the_reference_benchmark_at_full_size(gpu):
    """helium/examples/permute_dim_benchmark.rs:13-41: f32 [2048,128,128,32], swap_dims(0, 3) - 4.3 GB in, 4.3 GB out.
    Input element i holds the value i, so the whole output is checked against the closed form of its index, slices of
    it against the oracle's permute of the same slices of the input, and permuting twice must restore the input."""
    from helium_amd import configs

    shape, perm = configs.PERM_REF_SHAPE, configs.PERM_REF_PERM
    numel = int(np.prod(shape))
    p = PermuteDims(shape, "f32", perm=perm)
    print(f"permute {shape} f32 perm={perm}: {p.description}", flush=True)
    x = np.arange(numel, dtype=np.uint32)
    src = DeviceBuffer.from_numpy(x)
    dst = DeviceBuffer(x.nbytes)
    dst.fill_u8(0xEE)
    p.execute(src, dst)
    chunk = 1 << 24
    for start in range(0, numel, chunk):  # the whole output, 64 MiB at a time
        got = dst.read(start * 4, np.uint32, chunk)
        assert np.array_equal(got, configs.perm_ref_expected(np.arange(start, start + chunk, dtype=np.uint64))), start
    # slices against the oracle: output[:, a, b, :] is the permute of input[:, a, b, :] (dims 1 and 2 stay in place)
    xs = x.reshape(shape)
    rng = np.random.default_rng(9)
    for a, b in rng.integers(0, 128, size=(6, 2)):
        want = oracle.permute(np.ascontiguousarray(xs[:, a:a + 1, b:b + 1, :]), perm)[:, 0, 0, :]
        rows = [dst.read((((i3 * 128 + int(a)) * 128 + int(b)) * 2048) * 4, np.uint32, 2048) for i3 in range(32)]
        assert np.array_equal(np.stack(rows), want), (a, b)
    del xs
    back = DeviceBuffer(x.nbytes)
    PermuteDims(p.out_shape, "f32", perm=perm).execute(dst, back)   # swap_dims(0, 3) undoes itself
    for start in range(0, numel, chunk):
        assert np.array_equal(back.read(start * 4, np.uint32, chunk), x[start:start + chunk]), start
