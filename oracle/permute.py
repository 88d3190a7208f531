"""Oracle for the permute instruction (kernel K1). Test infrastructure only.

Pinned by: helium/tests/tensor_ops.rs:343-458 (transpose, swap_dims, chained swaps, singleton swaps — all in
tests/golden/tensor_ops.json), the stride known-answers of helium/src/cuda/instr/permute_dims.rs:180-187, and
`reference_kernel_walk` below checked against numpy.transpose by brute force on small shapes.
"""
import numpy as np


def permutation_from_swaps(rank, swaps):
    """Sequential SwapDims (helium-ir/src/opgraph/op.rs:102-110: each swap exchanges two extents of the current
    shape) expressed as a numpy.transpose axes tuple: out.shape[i] == in.shape[perm[i]]."""
    perm = list(range(rank))
    for a, b in swaps:
        perm[a], perm[b] = perm[b], perm[a]
    return tuple(perm)


def swap_dims_sequence(x, swaps):
    """What a chain of SwapDims computes, one swap at a time (the semantics the reference's pointwise path
    implements, helium/src/cuda/instr/pointwise/jit.rs:435-459,807-851, pinned by tensor_ops.rs:423-434)."""
    for a, b in swaps:
        x = np.swapaxes(x, a, b)
    return np.ascontiguousarray(x)


def permute(x, perm):
    return np.ascontiguousarray(np.transpose(x, perm))


def reference_output_strides(shape, swaps):
    """compute_output_strides exactly as written (helium/src/cuda/instr/permute_dims.rs:159-171).

    For compositions of swaps that are not involutions this returns the strides of the INVERSE permutation
    (the unit test's [4096, 1, 256, 64] encodes that); see `correct_output_strides` for the strides that
    sequential SwapDims imply.
    """
    rank = len(shape)
    permutation = list(range(rank))
    for a, b in swaps:
        permutation[a], permutation[b] = permutation[b], permutation[a]
    strides = [1] * rank
    stride = 1
    for i in reversed(range(rank)):
        j = permutation.index(i)
        strides[j] = stride
        stride *= shape[j]
    return strides


def correct_output_strides(shape, swaps):
    """Output stride of every INPUT axis under sequential-swap semantics."""
    perm = permutation_from_swaps(len(shape), swaps)
    out_shape = [shape[p] for p in perm]
    packed = [1] * len(shape)
    for i in reversed(range(len(shape) - 1)):
        packed[i] = packed[i + 1] * out_shape[i + 1]
    strides = [0] * len(shape)
    for pos, axis in enumerate(perm):
        strides[axis] = packed[pos]
    return strides


def reference_kernel_walk(x, out_strides):
    """The reference permute kernel's addressing, element by element
    (helium/src/cuda/instr/permute_dims/jit.rs:62-106): for y over the product of all dims but the last and
    x over the last dim, coord[i] = (y / s_i) % dims[i] with s_i = out_stride[i], divided by the last extent
    when it exceeds the last axis' own output stride; the element goes to sum(out_stride * coord).
    Pure-Python loops: small inputs only."""
    dims = list(x.shape)
    n = len(dims)
    flat = x.reshape(-1)
    out = np.zeros_like(flat)
    in_strides = [1] * n
    for i in reversed(range(n - 1)):
        in_strides[i] = in_strides[i + 1] * dims[i + 1]
    total_y = int(np.prod(dims[:-1], dtype=np.int64))
    for gy in range(total_y):
        for gx in range(dims[-1]):
            coords = [0] * n
            coords[n - 1] = gx
            for i in range(n - 1):
                stride = out_strides[i]
                if stride > out_strides[n - 1]:
                    stride //= dims[n - 1]
                coords[i] = (gy // stride) % dims[i]
            out_index = sum(s * c for s, c in zip(out_strides, coords))
            in_index = sum(s * c for s, c in zip(in_strides, coords))
            out[out_index] = flat[in_index]
    return out
