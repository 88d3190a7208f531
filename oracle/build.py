"""Builds the C part of the oracle (test infrastructure): oracle/libc4_cpu.so from oracle/c4_cpu.c with gcc + OpenMP.
The target is x86-64-v3 (AVX2 + FMA), not the build host's own CPU: the library is built here and runs on the host
cores of the GPU box."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libc4_cpu.so")


def build(verbose=False):
    cmd = ["gcc", "-O3", "-march=x86-64-v3", "-fopenmp", "-shared", "-fPIC", "-Wall", "-Wextra",
           os.path.join(HERE, "c4_cpu.c"), "-o", LIB, "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
