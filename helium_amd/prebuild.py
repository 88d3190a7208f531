"""Generates and compiles (hiprtc, gfx950) the kernels of the benchmark configurations into the on-disk
kernel cache, so that a GPU run starts without JIT latency. Needs no GPU."""
import time

from . import configs
from .kernels import TileKernel
from .permute import PermuteDims


def prebuild_kernels(verbose=True):
    t0 = time.time()
    n = 0
    for shape, perm in list(configs.PERMUTES.values()) + [((8192, 8192), (0, 1))]:
        PermuteDims(shape, "bf16", perm=perm)
        n += 1
    g, _, _ = configs.c3_chain(make_inputs=False)
    TileKernel.auxiliary(g)
    for mainloop, full in ((False, False), (True, True)):
        g, _ = configs.c4_graph(4096, mainloop=mainloop, full_size_outputs=full)
        TileKernel.fused(g)
        n += 1
    for g in (configs.c5a_graph(4096)[0], configs.c1_graph()[0]):
        TileKernel.fused(g)
        n += 1
    if verbose:
        print(f"prebuilt {n + 1} kernels in {time.time() - t0:.1f}s")
    return n + 1
