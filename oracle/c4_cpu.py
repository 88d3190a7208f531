"""ctypes binding of oracle/c4_cpu.c (test infrastructure): the README fusion (README.md:33-79) on the host cores.
Used by tests/test_oracle_cpu.py (against the numpy oracle) and by bench.py's cpu_baseline leg."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(HERE, "libc4_cpu.so")
        if not os.path.exists(path):
            from . import build

            build.build()
        _lib = C.CDLL(path)
        _lib.c4_cpu.restype = C.c_int
        _lib.c4_cpu.argtypes = [C.c_void_p] * 9 + [C.c_int] * 4 + [C.c_void_p] * 3
        _lib.c4_cpu_threads.restype = C.c_int
    return _lib


def threads():
    return int(lib().c4_cpu_threads())


def c4(inputs, size, mainloop=False):
    """inputs: {README node id: storage array} as helium_amd.configs.c4_inputs makes them (bf16 bit patterns for the
    [1,size,size] tensors, f32 for the biases n6 / n8). Returns {39: loss [1], 58: db8 [size], 87: db6 [size]} (f32)."""
    def ptr(a, dtype):
        a = np.ascontiguousarray(a, dtype=dtype)
        keep.append(a)
        return a.ctypes.data_as(C.c_void_p)

    keep = []
    loss, db8, db6 = np.zeros(1, np.float32), np.zeros(size, np.float32), np.zeros(size, np.float32)
    a = inputs[22 if mainloop else 1]
    rc = lib().c4_cpu(ptr(a, np.uint16), ptr(inputs[2], np.uint16), ptr(inputs[6], np.float32), ptr(inputs[8], np.float32),
                      ptr(inputs[9], np.uint16), ptr(inputs[11], np.uint16), ptr(inputs[13], np.uint16), ptr(inputs[24], np.uint16),
                      ptr(inputs[26], np.uint16), size, size, size, int(mainloop), loss.ctypes.data_as(C.c_void_p),
                      db8.ctypes.data_as(C.c_void_p), db6.ctypes.data_as(C.c_void_p))
    if rc != 0:
        raise MemoryError("c4_cpu could not allocate its work arrays")
    return {39: loss, 58: db8, 87: db6}
