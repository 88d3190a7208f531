"""The C-ABI library loads and exports every function include/helium_hip.h declares (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "helium_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(he_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    from helium_amd import _ffi

    names = declared_functions()
    assert len(names) > 30
    missing = [n for n in names if not hasattr(_ffi.lib, n)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    from helium_amd import _ffi

    unbound = [n for n in declared_functions() if getattr(_ffi.lib, n).argtypes is None
               and n not in ("he_last_error", "he_version", "he_target_arch", "he_device_synchronize")]
    assert not unbound, unbound


def test_version_and_arch():
    from helium_amd import _ffi

    assert _ffi.lib.he_target_arch() == b"gfx950"
    assert b"helium-hip" in _ffi.lib.he_version()


def test_rtc_compiles_for_gfx950_without_a_gpu():
    from helium_amd import device

    code = device.rtc_compile('extern "C" __global__ void k(float* p) { p[threadIdx.x] = 1.0f; }', "abi_probe")
    assert code[:4] == b"\x7fELF"


def test_rtc_reports_compile_errors():
    import pytest
    from helium_amd import HeliumError, device

    with pytest.raises(HeliumError) as e:
        device.rtc_compile('extern "C" __global__ void k(float* p) { p[0] = undefined_symbol; }', "abi_bad")
    assert "undefined_symbol" in str(e.value)
