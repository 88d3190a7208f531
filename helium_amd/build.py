"""Builds libhelium_hip.so (the C-ABI backend library) in-tree with hipcc.

The library's GPU kernels are generated at run time and compiled with hiprtc for gfx950, so this step builds
host code only.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhelium_hip.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def sources():
    """Host C++ (.cpp) and the one file with device data (.hip, compiled for gfx950)."""
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".cpp", ".hip")))


def build(verbose=True, jobs=8):
    """Compiles every csrc/*.cpp and links libhelium_hip.so. Always recompiles."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    flags = ["-O2", "-g0", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-c++20-extensions",
             "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include"]
    procs = []
    objs = []
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if src.endswith(".hip"):
            cmd = [hipcc, "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                   *[f for f in flags if f != "-D__HIP_PLATFORM_AMD__"], "-c", src, "-o", obj]
        else:
            cmd = [hipcc, "-x", "c++", *flags, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd)))
        if len(procs) >= jobs:
            _wait(procs)
    _wait(procs)
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-o", LIB, *objs, f"-L{ROCM}/lib", "-lamdhip64", "-lhiprtc", "-lpthread", "-ldl",
            f"-Wl,-rpath,{ROCM}/lib", "-Wl,--no-undefined"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    return LIB


def _wait(procs):
    while procs:
        src, p = procs.pop(0)
        if p.wait() != 0:
            raise RuntimeError(f"compilation of {src} failed")


if __name__ == "__main__":
    build()
