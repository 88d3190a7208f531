"""Storage-format helpers shared by the oracle modules. Test infrastructure only.

bf16 / f16 tensors are carried as uint16 bit patterns, Bool tensors as bitsets packed little-end first in uint32
words (helium-ir/src/data_type.rs:159-167,243-251). Conversions follow the `half` crate's round-to-nearest-even
(the host-side rounding the reference uses, Cargo.lock: half 2.6.0).
"""
import numpy as np


def f32_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounded = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, ((u >> 16) | 0x0040).astype(np.uint16), rounded)
    return rounded


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def pack_bool(bits):
    bits = np.ascontiguousarray(bits, dtype=bool).reshape(-1)
    padded = np.zeros((len(bits) + 31) // 32 * 32, dtype=bool)
    padded[: len(bits)] = bits
    return np.packbits(padded.reshape(-1, 32), axis=1, bitorder="little").view(np.uint32).reshape(-1)


def unpack_bool(words, count):
    return np.unpackbits(np.ascontiguousarray(words, dtype=np.uint32).view(np.uint8), bitorder="little")[:count].astype(bool)


def to_storage(values, dtype):
    """Math-domain array (float32 / uint32 / bool) -> storage array of `dtype`."""
    if dtype == "f32":
        return np.ascontiguousarray(values, dtype=np.float32)
    if dtype == "bf16":
        return f32_to_bf16_bits(values)
    if dtype == "f16":
        return f32_to_f16_bits(values)
    if dtype == "u32":
        return np.ascontiguousarray(values, dtype=np.uint32)
    if dtype == "bool":
        return pack_bool(values)
    raise ValueError(dtype)


def from_storage(storage, dtype, shape):
    """Storage array -> math-domain array (float32 for every float type)."""
    count = int(np.prod(shape, dtype=np.int64))
    if dtype == "f32":
        return np.asarray(storage, dtype=np.float32).reshape(shape)
    if dtype == "bf16":
        return bf16_bits_to_f32(storage).reshape(shape)
    if dtype == "f16":
        return f16_bits_to_f32(storage).reshape(shape)
    if dtype == "u32":
        return np.asarray(storage, dtype=np.uint32).reshape(shape)
    if dtype == "bool":
        return unpack_bool(storage, count).reshape(shape)
    raise ValueError(dtype)


NP_STORAGE = {"f32": np.float32, "bf16": np.uint16, "f16": np.uint16, "u32": np.uint32, "bool": np.uint32}


def ulp_diff(a, b):
    """Distance in units in the last place between two float32 arrays (sign-magnitude ordered)."""
    a = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7FFFFFFF), a)
    b = np.where(b < 0, -(b & 0x7FFFFFFF), b)
    return np.abs(a - b)


def ulps_close(got, want, max_ulps=2, epsilon=np.finfo(np.float32).eps):
    """The reference tests' criterion, approx::assert_ulps_eq: |a-b| <= epsilon or within max_ulps
    (helium/tests/tensor_ops.rs uses the macro's defaults, epsilon = f32::EPSILON and 4 ulps; here 2 ulps)."""
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    both_nan = np.isnan(got) & np.isnan(want)
    same_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    with np.errstate(invalid="ignore"):
        close = (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= epsilon) | (ulp_diff(got, want) <= max_ulps)
    return close | both_nan | same_inf
