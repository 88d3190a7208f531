"""Generates and compiles (hiprtc, gfx950) the kernels of the benchmark configurations into the on-disk
kernel cache, so that a GPU run starts without JIT latency. Needs no GPU."""
import time

from .permute import PermuteDims

PERMUTES = [
    ((64, 56, 56, 256), (0, 3, 1, 2), "bf16"),
    ((4096, 4096), (1, 0), "bf16"),
    ((32, 128, 28, 28), (0, 2, 3, 1), "bf16"),
]


def prebuild_kernels(verbose=True):
    t0 = time.time()
    n = 0
    for shape, perm, dtype in PERMUTES:
        PermuteDims(shape, dtype, perm=perm)
        n += 1
    if verbose:
        print(f"prebuilt {n} kernels in {time.time() - t0:.1f}s")
    return n
