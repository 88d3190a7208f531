"""ctypes loader for libhelium_hip.so — the only way Python code in this package reaches the GPU.

There is no fallback: if the library is missing, importing this module raises. The signatures below restate
include/helium_hip.h; tests/test_abi.py checks that every function the header declares is exported.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhelium_hip.so")


class HeliumError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"[helium_hip status {code}] {msg}")
        self.code = code


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built. Run `python -m helium_amd.build` (or __graft_entry__.build()); "
            "this package has no CPU fallback."
        )
    return C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)


lib = _load()

OK, ERR_INVALID, ERR_HIP, ERR_RTC, ERR_UNSUPPORTED, ERR_INTERNAL = range(6)
F16, BF16, F32, U32, BOOL = range(5)
DTYPES = {"f16": F16, "bf16": BF16, "f32": F32, "u32": U32, "bool": BOOL}
DTYPE_NAMES = {v: k for k, v in DTYPES.items()}

vp = C.c_void_p
i32, i64, u32, u64 = C.c_int32, C.c_int64, C.c_uint32, C.c_uint64
sz = C.c_size_t
P = C.POINTER

lib.he_last_error.restype = C.c_char_p
lib.he_version.restype = C.c_char_p
lib.he_target_arch.restype = C.c_char_p


def check(status):
    if status != 0:
        raise HeliumError(status, lib.he_last_error().decode(errors="replace"))


def _sig(name, *argtypes, restype=C.c_int):
    fn = getattr(lib, name)
    fn.argtypes = list(argtypes)
    fn.restype = restype
    return fn


# ---- device shim ---------------------------------------------------------------------------------------
_sig("he_init", C.c_int)
_sig("he_device_count", P(C.c_int))
_sig("he_device_attr", C.c_int, C.c_int, P(i64))
_sig("he_device_arch", C.c_int, C.c_char_p, sz)
_sig("he_device_synchronize")
_sig("he_stream_create", P(vp))
_sig("he_stream_destroy", vp)
_sig("he_stream_synchronize", vp)
HOST_FN = C.CFUNCTYPE(None, vp)
_sig("he_stream_host_callback", vp, HOST_FN, vp)
_sig("he_stream_raw", vp, restype=vp)
_sig("he_event_create", P(vp))
_sig("he_event_destroy", vp)
_sig("he_event_record", vp, vp)
_sig("he_event_wait", vp, vp)
_sig("he_event_synchronize", vp)
_sig("he_event_elapsed_ms", vp, vp, P(C.c_float))
_sig("he_malloc", P(vp), sz)
_sig("he_free", vp)
_sig("he_host_alloc", P(vp), sz)
_sig("he_host_free", vp)
_sig("he_memcpy_h2d_async", vp, vp, sz, vp)
_sig("he_memcpy_d2h_async", vp, vp, sz, vp)
_sig("he_memcpy_d2d_async", vp, vp, sz, vp)
_sig("he_memset_d8_async", vp, C.c_uint8, sz, vp)
_sig("he_memset_d16_async", vp, C.c_uint16, sz, vp)
_sig("he_memset_d32_async", vp, u32, sz, vp)
_sig("he_rtc_compile", C.c_char_p, C.c_char_p, P(C.c_char_p), C.c_int, P(vp), P(sz))
_sig("he_rtc_free", vp)
_sig("he_rtc_stats", P(u64))
_sig("he_module_load", P(vp), vp, sz)
_sig("he_module_unload", vp)
_sig("he_module_get_function", vp, C.c_char_p, P(vp))
_sig("he_launch", vp, P(u32), P(u32), u32, vp, P(vp))

# ---- permute ---------------------------------------------------------------------------------------------
_sig("he_permute_create", P(vp), P(i64), P(i32), C.c_int, C.c_int)
_sig("he_permute_create_from_swaps", P(vp), P(i64), C.c_int, P(i32), C.c_int, C.c_int)
_sig("he_permute_destroy", vp)
_sig("he_permute_execute", vp, vp, vp, vp)
_sig("he_permute_source", vp, restype=C.c_char_p)
_sig("he_permute_describe", vp, restype=C.c_char_p)
_sig("he_permute_reference_output_strides", P(i64), C.c_int, P(i32), C.c_int, P(i64))


def arr(ctype, values):
    values = list(values)
    return (ctype * max(len(values), 1))(*values)
